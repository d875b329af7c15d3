"""Attention over the paged cache.

q, k, v = one product with the concatenated projection matrix; rotary on q and k; k and v stored
in the pages of the row's request; every row attends to the keys of its request at positions
[pos - window + 1, pos] (all from 0 without a window), heads grouped over the key/value heads
(h -> h / (heads / kv_heads)); output projection added to the residual stream
(rust/engine/src/rust_decoder.rs:8827-8835 projections, :8895-8898 rotary, :8955-8963 cache write,
:6065-6166 scores, mask, softmax and output, :9025 and :9059 projection and residual).
"""
from __future__ import annotations

import torch

from ..config.spec import PartSpec
from ..registry import part_class, register_part
from .base import INIT_BIAS, INIT_MATRIX, KVNeed, Mixer


class PagedAttention(Mixer):
    graph_safe = True      # forward launches kernels only: no per-step decision on the host

    @classmethod
    def tensor_shapes(cls, spec):
        h, nh, nkv, d = spec["hidden_size"], spec["num_heads"], spec["num_kv_heads"], spec["head_dim"]
        return {
            "q": ((nh * d, h), INIT_MATRIX), "k": ((nkv * d, h), INIT_MATRIX), "v": ((nkv * d, h), INIT_MATRIX),
            "o": ((h, nh * d), INIT_MATRIX),
            "q_bias": ((nh * d,), INIT_BIAS), "k_bias": ((nkv * d,), INIT_BIAS), "v_bias": ((nkv * d,), INIT_BIAS),
            "o_bias": ((h,), INIT_BIAS),
        }

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        self.hidden = int(spec["hidden_size"])
        self.heads = int(spec["num_heads"])
        self.kv_heads = int(spec["num_kv_heads"])
        self.head_dim = int(spec["head_dim"])
        self.scale = float(spec["scale"])
        self.window = spec.get("window")
        if self.heads % self.kv_heads != 0:
            raise ValueError(f"head count {self.heads} is not a multiple of key/value head count {self.kv_heads}")
        if self.window is not None and self.window <= 0:
            raise ValueError("an attention window must be positive")
        position = spec.get("position")
        self.position = None
        if position is not None:
            position = dict(position)
            kind = position.pop("kind")
            self.position = part_class("position", kind)(PartSpec(kind, position), {}, rt)
        # one matrix for q, k and v: the normed input is read once
        self.w_qkv = torch.cat([rt.matrix(weights["q"]), rt.matrix(weights["k"]), rt.matrix(weights["v"])], dim=0).contiguous()
        self.w_o = rt.matrix(weights["o"])
        biases = [weights.get(n) for n in ("q_bias", "k_bias", "v_bias")]
        self.b_qkv = None
        if any(b is not None for b in biases):
            sizes = (self.heads * self.head_dim, self.kv_heads * self.head_dim, self.kv_heads * self.head_dim)
            self.b_qkv = torch.cat([rt.vector(b) if b is not None else torch.zeros(n, dtype=torch.float32, device=rt.device)
                                    for b, n in zip(biases, sizes)]).contiguous()
        self.b_o = rt.vector(weights["o_bias"]) if weights.get("o_bias") is not None else None

    def cache_need(self):
        return KVNeed(self.kv_heads, self.head_dim, self.window)

    def forward(self, ctx, h, residual, binding):
        rt, ops = self.rt, self.rt.ops
        rows = h.shape[0]
        nh, nkv, d = self.heads, self.kv_heads, self.head_dim
        qkv = rt.empty((rows, (nh + 2 * nkv) * d))
        ops.linear(h, self.w_qkv, qkv, bias=self.b_qkv)
        tables = ctx.tables[binding.group]
        if self.position is not None:
            cos, sin, dims, pairing = self.position.cos, self.position.sin, self.position.dims, self.position.pairing
        else:
            cos, sin, dims, pairing = ctx.no_rotation(rt)
        ops.rope_kv_store(qkv, ctx.row_pos, ctx.row_seg, tables, cos, sin,
                          binding.k_pages if binding.writes else None, binding.v_pages if binding.writes else None,
                          nh, nkv, d, dims, pairing, binding.page_size)
        out = rt.empty((rows, nh * d))
        ops.attention(qkv[:, : nh * d], binding.k_pages, binding.v_pages, tables, ctx.row_pos, ctx.row_seg, ctx.seg_start,
                      out, nh, nkv, d, binding.page_size, self.scale, self.window, ctx.max_context,
                      uniform_rows=1 if ctx.uniform_rows else 0,
                      workspace=ctx.attention_workspace(rt, rows, nh, nkv, d))
        ops.linear(out, self.w_o, residual, bias=self.b_o, accumulate=True)


register_part("mixer", "attention", PagedAttention)
