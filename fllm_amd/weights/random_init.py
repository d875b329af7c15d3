"""Random-weights mode: a model folder (config.json, model.safetensors) from a configuration and
a seed.

Distributions: matrices, embedding and biases N(0, 0.02); norm weights 1 + U(-0.1, 0.1).  (The
reference's own generator, rust/engine/src/tiny_model.rs:44-60 and :118-140, draws uniform
weights from one xorshift stream in the order of the tensors; here an element's value depends on the seed,
its tensor's name and its index alone, so tensors can be made in any order, in pieces, and on the device.)

The generator, specified once; `random_tensor` below evaluates it with NumPy on the host and the kernel library's
`fllm_random_fill` (csrc/random_fill.hip) on the device, bit for bit alike, because every step is an integer operation
or ONE correctly rounded float32 operation (+, -, *, /, sqrt; nothing fused, no library logarithm or cosine):

* key (k0, k1) = the first eight bytes of sha256("<seed>:<tensor name>"), little endian, low word first.
* element i (row-major): (w0, w1, _, _) = Philox-4x32-10(counter (i mod 2^32, i div 2^32, 0, 0), key).
* norm weights: 1 + (u * 0.2 - 0.1) with u = ((w0 >> 9) + 0.5) / 2^23.
* the others: Box-Muller, 0.02 * sqrt(-2 ln u1) * cos(2 pi u2).  u1 = v / 2^24 with the odd integer
  v = 2 (w0 >> 9) + 1 = m * 2^e, m in [sqrt(1/2), sqrt 2): ln u1 = (e - 24) ln 2 + 2 s (1 + s^2/3 + s^4/5 + s^6/7 + s^8/9),
  s = (m - 1) / (m + 1).  The angle: the two top bits of w1 >> 9 name the quadrant, the other 21 bits j the place in
  it, x = ((j + 0.5) / 2^21) (pi / 2); sine and cosine of x by their Taylor polynomials (degrees 11 and 12, Horner),
  and the quadrant turns them into cos(2 pi u2).
* bfloat16 tensors are the float32 values rounded to nearest, ties to even.
"""
from __future__ import annotations

import hashlib
import json
import os
from typing import Any, Dict, Tuple

import numpy as np
import torch

from ..config.spec import ModelSpec
from ..parts.base import INIT_BIAS, INIT_MATRIX, INIT_NORM
from ..registry import model_spec_from_config
from .loader import expected_tensors
from .safetensors_io import write_safetensors


def _f32(bits: int) -> np.float32:
    return np.array([bits], dtype=np.uint32).view(np.float32)[0]


# float32 constants by their bits, the same words as in csrc/random_fill.hip
_LN2, _HALF_PI, _SQRT_HALF = _f32(0x3F317218), _f32(0x3FC90FDB), _f32(0x3F3504F3)
_LOG_TERMS = [_f32(b) for b in (0x3DE38E39, 0x3E124925, 0x3E4CCCCD, 0x3EAAAAAB)]                 # 1/9, 1/7, 1/5, 1/3
_SIN_TERMS = [_f32(b) for b in (0xB2D7322B, 0x3638EF1D, 0xB9500D01, 0x3C088889, 0xBE2AAAAB)]     # -1/11! ... -1/3!
_COS_TERMS = [_f32(b) for b in (0x310F76C7, 0xB493F27E, 0x37D00D01, 0xBAB60B61, 0x3D2AAAAB, 0xBF000000)]   # 1/12! ... -1/2!
KIND_CODES = {INIT_MATRIX: 0, INIT_BIAS: 0, INIT_NORM: 1}
_CHUNK = 1 << 20


def tensor_key(seed: int, name: str) -> Tuple[int, int]:
    digest = hashlib.sha256(f"{seed}:{name}".encode("utf-8")).digest()
    return int.from_bytes(digest[:4], "little"), int.from_bytes(digest[4:8], "little")


def _philox_words(first: int, count: int, key: Tuple[int, int]):
    """The first two output words of Philox-4x32-10 for the counters (i, 0, 0), i = first .. first + count - 1."""
    mask = np.uint64(0xFFFFFFFF)
    index = np.arange(first, first + count, dtype=np.uint64)
    c = [index & mask, index >> np.uint64(32), np.zeros(count, np.uint64), np.zeros(count, np.uint64)]
    k0, k1 = key
    for _ in range(10):
        left = np.uint64(0xD2511F53) * c[0]
        right = np.uint64(0xCD9E8D57) * c[2]
        c = [((right >> np.uint64(32)) ^ c[1] ^ np.uint64(k0)) & mask, right & mask,
             ((left >> np.uint64(32)) ^ c[3] ^ np.uint64(k1)) & mask, left & mask]
        k0, k1 = (k0 + 0x9E3779B9) & 0xFFFFFFFF, (k1 + 0xBB67AE85) & 0xFFFFFFFF
    return c[0], c[1]


def _horner(x2: np.ndarray, terms, last: np.float32) -> np.ndarray:
    acc = np.full_like(x2, terms[0])
    for t in terms[1:]:
        acc = acc * x2 + t                       # two float32 operations, each rounded
    return acc * x2 + last


def _values(first: int, count: int, key: Tuple[int, int], kind: int) -> np.ndarray:
    """float32 values of the elements first .. first + count - 1 of a tensor."""
    w0, w1 = _philox_words(first, count, key)
    one, half, two = np.float32(1.0), np.float32(0.5), np.float32(2.0)
    if kind == 1:
        u = ((w0 >> np.uint64(9)).astype(np.float32) + half) / np.float32(8388608.0)
        return one + (u * np.float32(0.2) - np.float32(0.1))
    v = ((w0 >> np.uint64(9)) * np.uint64(2) + np.uint64(1)).astype(np.float32)       # odd, below 2^24: exact
    m, e = np.frexp(v)                                                               # v = m 2^e, m in [1/2, 1)
    low = m < _SQRT_HALF
    m = np.where(low, m * two, m).astype(np.float32)
    e = np.where(low, e - 1, e)
    s = (m - one) / (m + one)
    log_u = (e - 24).astype(np.float32) * _LN2 + (two * s) * _horner(s * s, _LOG_TERMS, one)
    radius = np.sqrt(np.maximum(np.float32(-2.0) * log_u, np.float32(0.0)))
    bits = w1 >> np.uint64(9)
    quadrant = (bits >> np.uint64(21)).astype(np.int64)
    j = (bits & np.uint64((1 << 21) - 1)).astype(np.float32)
    x = ((j + half) / np.float32(2097152.0)) * _HALF_PI
    x2 = x * x
    sine = x * _horner(x2, _SIN_TERMS, one)
    cosine = _horner(x2, _COS_TERMS, one)
    turn = np.choose(quadrant, [cosine, -sine, -cosine, sine])
    return (np.float32(0.02) * (radius * turn)).astype(np.float32)


def _host_tensor(shape, key, kind: int) -> torch.Tensor:
    total = int(np.prod(shape)) if len(shape) else 1
    out = np.empty(total, dtype=np.float32)
    with np.errstate(over="ignore"):                 # the 32 x 32 bit products wrap in 64 bits on purpose
        for first in range(0, total, _CHUNK):
            n = min(_CHUNK, total - first)
            out[first:first + n] = _values(first, n, key, kind)
    return torch.from_numpy(out).reshape(tuple(shape))


def random_tensor(name: str, shape, kind: str, seed: int, dtype: torch.dtype, device="cpu", ops=None) -> torch.Tensor:
    """The tensor `name` of the random model `seed`: the same bits wherever it is made.  On a GPU the kernel
    library fills it in place (no host copy: models of many gigabytes)."""
    if kind not in KIND_CODES:
        raise ValueError(f"unknown init kind {kind!r}")
    key = tensor_key(seed, name)
    if torch.device(device).type == "cpu":
        return _host_tensor(shape, key, KIND_CODES[kind]).to(dtype)
    if ops is None:
        from ..kernels import Ops
        ops = Ops()
    out = torch.empty(tuple(shape), dtype=dtype, device=device)
    ops.random_fill(out, key, KIND_CODES[kind])
    return out


def random_tensors(spec: ModelSpec, seed: int, dtype: torch.dtype, device="cpu",
                   with_optional: bool = False, ops=None) -> Dict[str, torch.Tensor]:
    """Every required tensor of the model (and the optional ones on request) by checkpoint name."""
    required, optional, init = expected_tensors(spec)
    names = dict(required)
    if with_optional:
        names.update(optional)
    return {n: random_tensor(n, shape, init[n], seed, dtype, device, ops) for n, shape in names.items()}


def write_random_model(model_dir: str, config: Dict[str, Any], seed: int, dtype: str = "float32",
                       with_optional: bool = False) -> ModelSpec:
    """Writes `config` as config.json and seeded random tensors as model.safetensors."""
    torch_dtype = {"float32": torch.float32, "bfloat16": torch.bfloat16, "float16": torch.float16}[dtype]
    _, spec = model_spec_from_config(config)
    os.makedirs(model_dir, exist_ok=True)
    cfg = dict(config)
    cfg.setdefault("torch_dtype", dtype)
    with open(os.path.join(model_dir, "config.json"), "w", encoding="utf-8") as fh:
        json.dump(cfg, fh, indent=1)
    write_safetensors(os.path.join(model_dir, "model.safetensors"),
                      random_tensors(spec, seed, torch_dtype, with_optional=with_optional))
    return spec
