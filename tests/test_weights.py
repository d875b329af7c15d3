"""Weights: binding by name, the one error that lists everything, the safetensors reader's
refusals, random-weights mode."""
import json
import os
import struct

import pytest
import numpy as np
import torch

import tiny_configs as tc
from fllm_amd.registry import model_spec_from_config
from fllm_amd.weights import (SafetensorsError, SafetensorsFile, WeightsError, check_tensors, expected_tensors,
                              load_checkpoint, open_checkpoint, random_tensors, write_random_model, write_safetensors)


def test_expected_tensors_of_llama():
    _, spec = model_spec_from_config(tc.TINY_A)
    required, optional, _ = expected_tensors(spec)
    assert required["model.embed_tokens.weight"] == (256, 64)
    assert required["lm_head.weight"] == (256, 64)
    assert required["model.layers.1.self_attn.k_proj.weight"] == (32, 64)
    assert required["model.layers.0.mlp.down_proj.weight"] == (64, 176)
    assert required["model.norm.weight"] == (64,)
    assert len(required) == 3 + 2 * 9
    assert optional["model.layers.0.self_attn.q_proj.bias"] == (64,)
    _, tied = model_spec_from_config(tc.TINY_B)
    assert "lm_head.weight" not in expected_tensors(tied)[0]


def test_one_error_lists_missing_unexpected_and_wrong_shapes():
    _, spec = model_spec_from_config(tc.TINY_A)
    shapes = {n: tuple(s) for n, s in expected_tensors(spec)[0].items()}
    del shapes["model.norm.weight"]
    del shapes["model.layers.0.mlp.up_proj.weight"]
    shapes["model.layers.0.self_attn.q_proj.weight"] = (64, 63)
    shapes["model.layers.7.mlp.up_proj.weight"] = (176, 64)
    shapes["model.rotary_emb.inv_freq"] = (8,)            # known, ignorable
    with pytest.raises(WeightsError) as info:
        check_tensors(spec, shapes)
    e = info.value
    assert e.missing == ["model.layers.0.mlp.up_proj.weight", "model.norm.weight"]
    assert e.unexpected == ["model.layers.7.mlp.up_proj.weight"]
    assert e.wrong_shape == [("model.layers.0.self_attn.q_proj.weight", (64, 63), (64, 64))]
    text = str(e)
    for needle in ("missing tensors (2)", "unexpected tensors (1)", "wrong shapes (1)", "expected [64, 64]"):
        assert needle in text


def test_tied_checkpoint_may_hold_a_head(tmp_path):
    _, spec = model_spec_from_config(tc.TINY_B)
    tensors = random_tensors(spec, 1, torch.float32)
    tensors["lm_head.weight"] = torch.zeros(512, 160)
    check_tensors(spec, {n: tuple(t.shape) for n, t in tensors.items()})


def test_random_model_folder_round_trip(tmp_path):
    spec = write_random_model(str(tmp_path), tc.TINY_A, seed=3, dtype="bfloat16")
    assert sorted(os.listdir(tmp_path)) == ["config.json", "model.safetensors"]
    loaded = load_checkpoint(str(tmp_path), spec)
    again = random_tensors(spec, 3, torch.bfloat16)
    assert set(loaded) == set(again)
    for n in again:
        assert loaded[n].dtype == torch.bfloat16 and torch.equal(loaded[n], again[n])
    other = random_tensors(spec, 4, torch.bfloat16)
    assert not torch.equal(other["model.norm.weight"], again["model.norm.weight"])
    exact = random_tensors(spec, 3, torch.float32)
    assert torch.equal(exact["model.norm.weight"].to(torch.bfloat16), again["model.norm.weight"])
    w = exact["model.layers.0.mlp.up_proj.weight"]
    assert abs(w.std().item() - 0.02) < 0.002 and abs(w.mean().item()) < 0.002
    n = exact["model.norm.weight"]
    assert 0.9 <= n.min().item() and n.max().item() <= 1.1


def test_stored_types_are_kept(tmp_path):
    _, spec = model_spec_from_config(tc.TINY_A)
    tensors = random_tensors(spec, 1, torch.bfloat16)
    tensors["model.norm.weight"] = tensors["model.norm.weight"].float()       # a tensor stored in 32-bit stays so
    os.makedirs(tmp_path, exist_ok=True)
    write_safetensors(str(tmp_path / "model.safetensors"), tensors)
    loaded = load_checkpoint(str(tmp_path), spec)
    assert loaded["model.norm.weight"].dtype == torch.float32
    assert loaded["lm_head.weight"].dtype == torch.bfloat16


def _write_raw(path, header, data=b""):
    raw = json.dumps(header).encode()
    with open(path, "wb") as fh:
        fh.write(struct.pack("<Q", len(raw)) + raw + data)


@pytest.mark.parametrize("header,data,text", [
    ({"a": {"dtype": "F32", "shape": [2], "data_offsets": [0, 8]}}, b"\0" * 12, "trailing bytes"),
    ({"a": {"dtype": "F32", "shape": [2], "data_offsets": [4, 12]}}, b"\0" * 12, "gap"),
    ({"a": {"dtype": "F32", "shape": [2], "data_offsets": [0, 8]}, "b": {"dtype": "F32", "shape": [2], "data_offsets": [4, 12]}},
     b"\0" * 12, "overlaps"),
    ({"a": {"dtype": "F32", "shape": [3], "data_offsets": [0, 8]}}, b"\0" * 8, "needs 12"),
    ({"a": {"dtype": "F32", "shape": [2], "data_offsets": [0, 8]}}, b"\0" * 4, "past the end"),
    ({"a": {"dtype": "F32", "shape": [2], "data_offsets": [8, 0]}}, b"\0" * 8, "start > end"),
    ({"a": {"dtype": "Q4", "shape": [2], "data_offsets": [0, 8]}}, b"\0" * 8, "unsupported dtype"),
    ({"a": {"dtype": "F32", "shape": [-2], "data_offsets": [0, 8]}}, b"\0" * 8, "invalid shape"),
])
def test_reader_refusals(tmp_path, header, data, text):
    path = str(tmp_path / "x.safetensors")
    _write_raw(path, header, data)
    with pytest.raises(SafetensorsError, match=text):
        SafetensorsFile(path)


def test_reader_refuses_broken_headers(tmp_path):
    path = str(tmp_path / "x.safetensors")
    with open(path, "wb") as fh:
        fh.write(b"\x01\x02")
    with pytest.raises(SafetensorsError, match="truncated"):
        SafetensorsFile(path)
    with open(path, "wb") as fh:
        fh.write(struct.pack("<Q", 1000) + b"{}")
    with pytest.raises(SafetensorsError, match="past the end"):
        SafetensorsFile(path)
    with open(path, "wb") as fh:
        fh.write(struct.pack("<Q", 2) + b"[]")
    with pytest.raises(SafetensorsError, match="not a JSON object"):
        SafetensorsFile(path)


def test_sharded_checkpoint(tmp_path):
    _, spec = model_spec_from_config(tc.TINY_A)
    tensors = random_tensors(spec, 1, torch.float32)
    names = sorted(tensors)
    half = len(names) // 2
    shards = {"model-00001-of-00002.safetensors": names[:half], "model-00002-of-00002.safetensors": names[half:]}
    for shard, held in shards.items():
        write_safetensors(str(tmp_path / shard), {n: tensors[n] for n in held})
    with open(tmp_path / "model.safetensors.index.json", "w") as fh:
        json.dump({"weight_map": {n: s for s, held in shards.items() for n in held}}, fh)
    loaded = load_checkpoint(str(tmp_path), spec)
    assert all(torch.equal(loaded[n], tensors[n]) for n in names)
    with open(tmp_path / "model.safetensors.index.json", "w") as fh:
        json.dump({"weight_map": {names[0]: "../evil.safetensors"}}, fh)
    with pytest.raises(SafetensorsError, match="plain file name"):
        open_checkpoint(str(tmp_path))


def _scalar_random_value(seed, name, index, norm_weight):
    """The generator's specification (the module text of fllm_amd/weights/random_init.py) written out for ONE element
    with Python integers and NumPy float32 scalars, every operation rounded on its own."""
    import hashlib
    import math
    f = np.float32
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    k = [int.from_bytes(digest[:4], "little"), int.from_bytes(digest[4:8], "little")]
    c = [index & 0xFFFFFFFF, index >> 32, 0, 0]
    for _ in range(10):
        left, right = 0xD2511F53 * c[0], 0xCD9E8D57 * c[2]
        c = [((right >> 32) ^ c[1] ^ k[0]) & 0xFFFFFFFF, right & 0xFFFFFFFF, ((left >> 32) ^ c[3] ^ k[1]) & 0xFFFFFFFF, left & 0xFFFFFFFF]
        k = [(k[0] + 0x9E3779B9) & 0xFFFFFFFF, (k[1] + 0xBB67AE85) & 0xFFFFFFFF]
    w0, w1 = c[0], c[1]
    if norm_weight:
        u = (f(w0 >> 9) + f(0.5)) / f(2 ** 23)
        return f(1.0) + (u * f(0.2) - f(0.1))
    v = 2 * (w0 >> 9) + 1
    e = v.bit_length()                       # v = m 2^e with m in [1/2, 1)
    m = f(v) / f(2.0 ** e)
    if m < f(math.sqrt(0.5)):
        m, e = m * f(2.0), e - 1
    s = (m - f(1.0)) / (m + f(1.0))
    s2 = s * s
    series = f(1.0 / 9.0)
    for t in (1.0 / 7.0, 1.0 / 5.0, 1.0 / 3.0, 1.0):
        series = series * s2 + f(t)
    log_u = f(e - 24) * f(math.log(2.0)) + (f(2.0) * s) * series
    radius = np.sqrt(max(f(-2.0) * log_u, f(0.0)))
    angle = w1 >> 9
    quadrant, j = angle >> 21, angle & ((1 << 21) - 1)
    x = ((f(j) + f(0.5)) / f(2 ** 21)) * f(math.pi / 2)
    x2 = x * x
    sine = f(-1.0 / math.factorial(11))
    for n in (9, 7, 5, 3):
        sine = sine * x2 + f((-1.0) ** (n // 2) / math.factorial(n))
    sine = x * (sine * x2 + f(1.0))
    cosine = f(1.0 / math.factorial(12))
    for n in (10, 8, 6, 4, 2):
        cosine = cosine * x2 + f((-1.0) ** (n // 2) / math.factorial(n))
    cosine = cosine * x2 + f(1.0)
    turn = [cosine, -sine, -cosine, sine][quadrant]
    return f(0.02) * (radius * turn)


def test_random_generator_follows_its_specification():
    from fllm_amd.parts.base import INIT_MATRIX, INIT_NORM
    from fllm_amd.weights.random_init import random_tensor
    count = (1 << 20) + 37                                          # longer than one piece of the host's evaluation
    for kind, norm_weight in ((INIT_MATRIX, False), (INIT_NORM, True)):
        t = random_tensor("model.some.weight", (count,), kind, 5, torch.float32)
        for i in list(range(40)) + [1 << 20, (1 << 20) - 1, count - 1]:
            want = _scalar_random_value(5, "model.some.weight", i, norm_weight)
            assert t[i].item() == float(want), (kind, i)
        # an element depends on (seed, name, index) only: not on the tensor's size or shape
        small = random_tensor("model.some.weight", (7, 11), kind, 5, torch.float32)
        assert torch.equal(small.reshape(-1), t[:77])
        assert not torch.equal(random_tensor("model.other.weight", (77,), kind, 5, torch.float32), t[:77])
        # bfloat16 is the float32 value rounded to nearest even
        assert torch.equal(random_tensor("model.some.weight", (77,), kind, 5, torch.bfloat16), t[:77].to(torch.bfloat16))
    # what the distribution is meant to be
    z = random_tensor("w", (1 << 18,), INIT_MATRIX, 9, torch.float32).double() / 0.02
    assert abs(z.mean()) < 0.01 and abs(z.std() - 1) < 0.01 and abs((z ** 4).mean() - 3) < 0.1 and abs((z ** 3).mean()) < 0.05
    assert 0.66 < (z.abs() < 1).double().mean() < 0.70 and z.abs().max() > 4.0
    u = random_tensor("w", (1 << 18,), INIT_NORM, 9, torch.float32).double()
    assert 0.9 <= u.min() < 0.9001 and 1.0999 < u.max() <= 1.1 and abs(u.mean() - 1) < 1e-3 and abs(u.std() - 0.2 / 12 ** 0.5) < 1e-3


def test_nested_language_model_names(tmp_path):
    """rust/checkpoint/src/plan.rs:2624-2650: `model.language_model.X` is `model.X`, `language_model.model.X` and
    `language_model.lm_head.X` lose their first part, any other `language_model.X` is `model.X`; vision towers are
    left aside."""
    from safetensors.torch import save_file
    _, spec = model_spec_from_config(tc.TINY_A)
    tensors = random_tensors(spec, 2, torch.float32)
    with open(tmp_path / "config.json", "w") as fh:
        json.dump(tc.TINY_A, fh)
    for form in (lambda n: "model.language_model." + n[len("model."):] if n.startswith("model.") else n,
                 lambda n: "language_model." + n,
                 lambda n: "language_model." + n[len("model."):] if n.startswith("model.") else "language_model." + n):
        stored = {form(n): t for n, t in tensors.items()}
        stored["vision_tower.patch.weight"] = torch.zeros(3, 3)
        stored["model.visual.blocks.0.weight"] = torch.zeros(2)
        assert set(stored) != set(tensors)
        save_file(stored, str(tmp_path / "model.safetensors"))
        loaded = load_checkpoint(str(tmp_path), spec)
        assert set(loaded) == set(tensors) and all(torch.equal(loaded[n], tensors[n]) for n in tensors)
    stored = dict(tensors)
    stored["language_model.model.norm.weight"] = tensors["model.norm.weight"].clone()
    save_file(stored, str(tmp_path / "model.safetensors"))
    with pytest.raises(ValueError, match="both stand for 'model.norm.weight'"):
        load_checkpoint(str(tmp_path), spec)
