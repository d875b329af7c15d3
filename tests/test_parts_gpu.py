"""Each part alone on the GPU against the plain implementation's function for it."""
import math

import numpy as np
import pytest
import torch

import plain_llama as P
from fllm_amd.config.spec import PartSpec
from fllm_amd.engine.context import CacheBinding, StepContext
from fllm_amd.parts import Runtime
from fllm_amd.registry import part_class

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module", params=["float32", "bfloat16"])
def rt(request):
    from fllm_amd.kernels import Ops
    return Runtime(torch.device(DEV), {"float32": torch.float32, "bfloat16": torch.bfloat16}[request.param], Ops(), 512)


def tol(rt):
    return 3e-5 if rt.dtype == torch.float32 else 3e-2


def weights_for(role, spec, seed, dtype):
    g = torch.Generator().manual_seed(seed)
    shapes = part_class(role, spec.kind).tensor_shapes(spec)
    out = {}
    for key in spec.tensors:
        name = key.lstrip("?")
        shape, kind = shapes[name]
        t = torch.randn(shape, generator=g) * (0.1 if kind != "norm" else 0.1)
        if kind == "norm":
            t = 1.0 + t
        out[name] = t.to(dtype).to(torch.float32) if dtype == torch.bfloat16 else t
    return out


def whole_prompt_context(rows, page_size=16, first=0):
    """One request, `rows` tokens from position `first`, pages in reverse order."""
    pages = -(-(first + rows) // page_size)
    table = torch.arange(pages - 1, -1, -1, dtype=torch.int32, device=DEV).view(1, pages)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    return StepContext(num_rows=rows, num_segments=1, ids=i32([0] * rows), row_pos=i32(list(range(first, first + rows))),
                       row_seg=i32([0] * rows), seg_start=i32([0, rows]), slots=i32([0]), logit_rows=i32([rows - 1]),
                       tables=[table], seg_rows=[rows], seg_pos_start=[first], seg_slots=[0], max_context=first + rows,
                       uniform_rows=rows == 1), pages


def compare(got, want, rt, what):
    got = got.detach().double().cpu().numpy()
    assert np.abs(got - want).max() <= tol(rt) * max(1.0, np.abs(want).max()), \
        f"{what}: max error {np.abs(got - want).max():.3e}, scale {np.abs(want).max():.3e}"


def test_rms_norm_part(rt):
    spec = PartSpec("rms", {"size": 200, "eps": 3e-6}, {"weight": "w"})
    w = weights_for("norm", spec, 1, rt.dtype)
    part = part_class("norm", "rms")(spec, w, rt)
    x = torch.randn(7, 200, generator=torch.Generator().manual_seed(2)) * 2
    want = P.rms_norm(x.double().numpy(), w["weight"].double().numpy(), 3e-6)
    compare(part.forward(None, x.to(DEV)), want, rt, "rms norm")
    rows = torch.tensor([6, 0], dtype=torch.int32, device=DEV)
    compare(part.forward(None, x.to(DEV), rows=rows), want[[6, 0]], rt, "rms norm with row selection")


@pytest.mark.parametrize("params", [
    {"dims": 16, "theta": 10000.0, "scaling": "none"},
    {"dims": 32, "theta": 500000.0, "scaling": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
     "original_max_position": 64},
    {"dims": 24, "theta": 50000.0, "scaling": "linear", "factor": 2.0},
])
def test_rotary_tables(rt, params):
    part = part_class("position", "rotary")(PartSpec("rotary", dict(params, max_position=300)), {}, rt)
    kind = {"none": "default"}.get(params["scaling"], params["scaling"])
    scaling = {"factor": params.get("factor"), "low_freq_factor": params.get("low_freq_factor"),
               "high_freq_factor": params.get("high_freq_factor"),
               "original_max_position_embeddings": params.get("original_max_position")}
    cos, sin = P.rope_tables(range(300), params["dims"], params["theta"], kind, scaling)
    assert part.cos.shape == (300, params["dims"] // 2)
    assert np.abs(part.cos.double().cpu().numpy() - cos).max() < 2e-6
    assert np.abs(part.sin.double().cpu().numpy() - sin).max() < 2e-6


def test_gated_mlp_part(rt):
    spec = PartSpec("gated_mlp", {"hidden_size": 72, "intermediate_size": 200, "activation": "silu"},
                    {"gate": "g", "up": "u", "down": "d", "?down_bias": "db"})
    w = weights_for("feed_forward", spec, 3, rt.dtype)
    part = part_class("feed_forward", "gated_mlp")(spec, w, rt)
    x = torch.randn(11, 72, generator=torch.Generator().manual_seed(4)).to(rt.dtype)
    residual = torch.randn(11, 72, generator=torch.Generator().manual_seed(5))
    n = lambda k: w[k].double().numpy()
    want = residual.double().numpy() + P.gated_mlp(x.double().numpy(), n("gate"), n("up"), n("down"), down_bias=n("down_bias"))
    out = residual.to(DEV)
    part.forward(None, x.to(DEV), out)
    compare(out, want, rt, "gated mlp")


@pytest.mark.parametrize("heads,kv_heads,head_dim,window,rows,first", [(4, 2, 16, None, 37, 0), (5, 1, 32, None, 70, 0),
                                                                       (8, 2, 64, 24, 90, 0), (6, 3, 48, None, 20, 0)])
def test_attention_part(rt, heads, kv_heads, head_dim, window, rows, first):
    hidden = 96
    position = {"kind": "rotary", "dims": head_dim, "theta": 10000.0, "scaling": "none", "max_position": 512}
    spec = PartSpec("attention", {"hidden_size": hidden, "num_heads": heads, "num_kv_heads": kv_heads, "head_dim": head_dim,
                                  "scale": head_dim ** -0.5, "window": window, "position": position},
                    {"q": "q", "k": "k", "v": "v", "o": "o", "?q_bias": "qb", "?v_bias": "vb"})
    w = weights_for("mixer", spec, 6, rt.dtype)
    part = part_class("mixer", "attention")(spec, w, rt)
    need = part.cache_need()
    assert (need.kv_heads, need.k_dim, need.v_dim, need.window) == (kv_heads, head_dim, head_dim, window)
    ctx, pages = whole_prompt_context(rows)
    binding = CacheBinding(group=0, k_pages=torch.zeros(pages, kv_heads, head_dim // 8, 16, 8, dtype=rt.dtype, device=DEV),
                           v_pages=torch.zeros(pages, kv_heads, head_dim, 16, dtype=rt.dtype, device=DEV), page_size=16,
                           writes=True)
    x = torch.randn(rows, hidden, generator=torch.Generator().manual_seed(7)).to(rt.dtype)
    residual = torch.zeros(rows, hidden, device=DEV)
    part.forward(ctx, x.to(DEV), residual, binding)
    weights = {f"p.self_attn.{k}_proj.weight": w[k].double().numpy() for k in "qkvo"}
    weights["p.self_attn.q_proj.bias"] = w["q_bias"].double().numpy()
    weights["p.self_attn.v_proj.bias"] = w["v_bias"].double().numpy()
    sizes = {"heads": heads, "kv_heads": kv_heads, "head_dim": head_dim, "rope_dims": head_dim, "theta": 10000.0,
             "rope_kind": "default", "rope_scaling": {}, "windows": [window]}
    want = P.attention_layer(x.double().numpy(), weights, "p", sizes, 0, np.arange(rows))
    compare(residual, want, rt, "attention part")


def test_embedding_and_head_parts(rt):
    spec = PartSpec("table", {"vocab_size": 300, "hidden_size": 40, "scale": 1.0}, {"weight": "e"})
    w = weights_for("embedding", spec, 8, rt.dtype)
    emb = part_class("embedding", "table")(spec, w, rt)
    ids = torch.tensor([0, 299, 5, 5], dtype=torch.int32, device=DEV)
    compare(emb.forward(None, ids), w["weight"].double().numpy()[[0, 299, 5, 5]], rt, "embedding")
    head = part_class("head", "linear")(PartSpec("linear", {"vocab_size": 300, "hidden_size": 40}, {"weight": "e"}), w, rt)
    assert head.weight.data_ptr() == emb.table.data_ptr()          # a tied head shares the table
    h = torch.randn(3, 40, generator=torch.Generator().manual_seed(9)).to(rt.dtype)
    logits = head.forward(None, h.to(DEV))
    assert logits.dtype == torch.float32
    compare(logits, h.double().numpy() @ w["weight"].double().numpy().T, rt, "head")
