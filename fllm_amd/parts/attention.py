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
from .base import INIT_BIAS, INIT_MATRIX, KVNeed, Mixer, add_and_prepare, fused_form, take_prepared


class PagedAttention(Mixer):
    graph_safe = True      # forward launches kernels only: no per-step decision on the host
    KEY_CHUNK = 8          # values of a key that lie together in a page (csrc/common.h, key_offset)

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
        if self.head_dim % self.KEY_CHUNK != 0:
            raise ValueError(f"head size {self.head_dim}: the attention kernels store keys in chunks of {self.KEY_CHUNK} values, "
                             f"head sizes come in steps of {self.KEY_CHUNK}")
        if spec.get("value_head_dim") not in (None, self.head_dim):
            raise ValueError(f"this attention's kernels read keys and values of one width: values of "
                             f"{spec.get('value_head_dim')} beside keys of {self.head_dim} need a mixer of their own")
        position = spec.get("position")
        self.position = None
        if position is not None:
            position = dict(position)
            kind = position.pop("kind")
            self.position = part_class("position", kind)(PartSpec(kind, position), {}, rt)
        # Rotary with the checkpoint's pairing (l, l + dims/2): the rows of the q and k projections are
        # reordered inside every head so that the partners sit next to each other (2l, 2l + 1), the
        # pairing the kernels rotate.  q . k does not change when both are reordered alike
        # (the reference's importer does the same: rust/checkpoint/src/convert.rs:2713-2745).
        self.pairing = 1
        order_q = order_k = None
        if self.position is not None and self.position.pairing == 0:
            order_q = self._pair_order(self.heads, self.head_dim, self.position.dims).to(rt.device)
            order_k = self._pair_order(self.kv_heads, self.head_dim, self.position.dims).to(rt.device)
        elif self.position is not None:
            self.pairing = self.position.pairing
        reorder = lambda t, order: t if order is None or t is None else t.index_select(0, order)
        # one matrix for q, k and v: the normed input is read once
        self.w_qkv = torch.cat([reorder(rt.matrix(weights["q"]), order_q), reorder(rt.matrix(weights["k"]), order_k),
                                rt.matrix(weights["v"])], dim=0).contiguous()
        self.w_o = rt.matrix(weights["o"])
        rt.tile_for_decode(self.w_o)
        rt.tile_for_decode(self.w_qkv, priority=1)
        biases = [reorder(None if weights.get("q_bias") is None else rt.vector(weights["q_bias"]), order_q),
                  reorder(None if weights.get("k_bias") is None else rt.vector(weights["k_bias"]), order_k),
                  None if weights.get("v_bias") is None else rt.vector(weights["v_bias"])]
        self.b_qkv = None
        if any(b is not None for b in biases):
            sizes = (self.heads * self.head_dim, self.kv_heads * self.head_dim, self.kv_heads * self.head_dim)
            self.b_qkv = torch.cat([b if b is not None else torch.zeros(n, dtype=torch.float32, device=rt.device)
                                    for b, n in zip(biases, sizes)]).contiguous()
        self.b_o = rt.vector(weights["o_bias"]) if weights.get("o_bias") is not None else None

    @staticmethod
    def _pair_order(heads: int, head_dim: int, rope_dims: int) -> torch.Tensor:
        """New row -> old row: inside every head, row 2l comes from l and row 2l + 1 from l + rope_dims/2."""
        half = rope_dims // 2
        one = []
        for l in range(half):
            one += [l, l + half]
        one += list(range(rope_dims, head_dim))
        return torch.tensor([h * head_dim + j for h in range(heads) for j in one], dtype=torch.long)

    def cache_need(self):
        # keys and values of one width, keys in chunks of 8 values (16 bytes in bfloat16): what the kernels take
        return KVNeed(self.kv_heads, self.head_dim, self.head_dim, self.window, key_chunk=self.KEY_CHUNK)

    def forward(self, ctx, h, residual, binding, branch=None):
        rt, ops = self.rt, self.rt.ops
        rows = h.shape[0]
        nh, nkv, d = self.heads, self.kv_heads, self.head_dim
        qkv = rt.empty((rows, (nh + 2 * nkv) * d))
        ops.linear(h, self.w_qkv, qkv, bias=self.b_qkv)
        tables = ctx.tables[binding.group]
        if self.position is not None:
            cos, sin, dims, pairing = self.position.cos, self.position.sin, self.position.dims, self.pairing
        else:
            cos, sin, dims, pairing = ctx.no_rotation(rt)
        ops.rope_kv_store(qkv, ctx.row_pos, ctx.row_seg, tables, cos, sin,
                          binding.k_pages if binding.writes else None, binding.v_pages if binding.writes else None,
                          nh, nkv, d, dims, pairing, binding.page_size)
        self._attend_and_project(ctx, qkv[:, : nh * d], residual, binding, branch=branch)

    def forward_from_residual(self, ctx, residual, norm, binding) -> bool:
        """Decode-sized steps in bfloat16: the norm before the mixer, the q/k/v product, rotary and the
        cache store are one kernel.  False: not taken, the block runs norm and `forward`."""
        rt, ops = self.rt, self.rt.ops
        rows = residual.shape[0]
        prologue = getattr(norm, "fused_prologue", lambda: None)()
        form = fused_form(ops, rows, self.hidden, self.w_qkv) if hasattr(ops, "norm_qkv_rope_store") else None
        if rt.dtype != torch.bfloat16 or self.pairing != 1 or prologue is None or form is None or self.head_dim % 4 != 0:
            return False
        norm_scale, norm_eps = prologue
        nh, nkv, d = self.heads, self.kv_heads, self.head_dim
        if self.position is not None:
            cos, sin, dims = self.position.cos, self.position.sin, self.position.dims
        else:
            cos, sin, dims, _ = ctx.no_rotation(rt)
        q = rt.empty((rows, nh * d))
        prepared = take_prepared(ctx, norm, residual)      # the sum before this norm may have computed its first steps
        if prepared is None and form == "chunks":
            prepared = ops.prepare_norm(residual, norm_scale)
        ops.norm_qkv_rope_store(residual, norm_scale, norm_eps, self.w_qkv, q, ctx.row_pos, ctx.row_seg,
                                ctx.tables[binding.group], cos, sin, binding.k_pages if binding.writes else None,
                                binding.v_pages if binding.writes else None, nh, nkv, d, dims, binding.page_size,
                                bias=self.b_qkv, **({"prepared": prepared} if prepared is not None else {}))
        self._attend_and_project(ctx, q, residual, binding)
        return True

    def forward_branch(self, ctx, h, binding):
        """The mixer's output as a tensor of its own instead of a sum into the residual stream, when
        that lets the block fold the residual add into the next norm (large bfloat16 steps whose
        products go to the GEMM library, which has no residual epilogue).  None: not taken."""
        rt, ops = self.rt, self.rt.ops
        rows = h.shape[0]
        start = getattr(ops, "library_gemm_from", None)
        if rt.dtype != torch.bfloat16 or start is None or rows < start or self.b_o is not None:
            return None
        branch = rt.empty((rows, self.hidden))
        self.forward(ctx, h, None, binding, branch=branch)
        return branch

    SPLIT_SINGLE_ROWS_FROM = 3072      # context length (measured: equal cost at about 4,000 keys)

    def _attend_and_project(self, ctx, q, residual, binding, branch=None):
        rt, ops = self.rt, self.rt.ops
        rows = q.shape[0]
        nh, nkv, d = self.heads, self.kv_heads, self.head_dim
        tables = ctx.tables[binding.group]
        out = rt.empty((rows, nh * d))
        # Single rows behind portions of prompts: with long contexts they go to the kernel that splits a context over
        # workgroups (a second launch); with short ones they ride along in the portions' launch, which is faster then.
        single_from = ctx.single_rows_from()
        if 0 < single_from < ctx.num_segments and ctx.single_max_context < self.SPLIT_SINGLE_ROWS_FROM:
            single_from = ctx.num_segments
        slopes = getattr(self.position, "score_slopes", None)      # a position encoding may bias scores by distance
        if slopes is not None:
            ops.attention(q, binding.k_pages, binding.v_pages, tables, ctx.row_pos, ctx.row_seg, ctx.seg_start,
                          out, nh, nkv, d, binding.page_size, self.scale, self.window, ctx.max_context, head_slopes=slopes)
        else:
            ops.attention(q, binding.k_pages, binding.v_pages, tables, ctx.row_pos, ctx.row_seg, ctx.seg_start,
                          out, nh, nkv, d, binding.page_size, self.scale, self.window, ctx.max_context,
                          single_from=single_from,
                          workspace=ctx.attention_workspace(rt, rows, nh, nkv, d))
        if branch is not None:
            ops.linear(out, self.w_o, branch, bias=self.b_o)
        elif not add_and_prepare(ctx, ops, out, self.w_o, residual, self.b_o):
            ops.linear(out, self.w_o, residual, bias=self.b_o, accumulate=True)


register_part("mixer", "attention", PagedAttention)
