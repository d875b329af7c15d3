"""Gated feed-forward: x += W_down (silu(W_gate n) * W_up n), silu(g) = g / (1 + exp(-g))
(rust/engine/src/rust_decoder.rs:8328-8352, :1645; rust/engine/src/cpu_elementwise.rs:3-43).
Gate and up are one product with the concatenated matrix."""
from __future__ import annotations

import torch

from ..registry import register_part
from .base import INIT_BIAS, INIT_MATRIX, FeedForward, add_and_prepare, fused_form, take_prepared


class GatedMLP(FeedForward):
    graph_safe = True      # forward launches kernels only: no per-step decision on the host

    @classmethod
    def tensor_shapes(cls, spec):
        h, i = spec["hidden_size"], spec["intermediate_size"]
        return {"gate": ((i, h), INIT_MATRIX), "up": ((i, h), INIT_MATRIX), "down": ((h, i), INIT_MATRIX),
                "gate_bias": ((i,), INIT_BIAS), "up_bias": ((i,), INIT_BIAS), "down_bias": ((h,), INIT_BIAS)}

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        if spec.get("activation", "silu") not in ("silu", "swish"):
            raise ValueError(f"unsupported activation {spec.get('activation')!r}; the gated feed-forward uses silu")
        self.hidden = int(spec["hidden_size"])
        self.inter = int(spec["intermediate_size"])
        self.w_gate_up = torch.cat([rt.matrix(weights["gate"]), rt.matrix(weights["up"])], dim=0).contiguous()
        self.w_down = rt.matrix(weights["down"])
        rt.tile_for_decode(self.w_down)
        rt.tile_for_decode(self.w_gate_up, gate_up=True, priority=1)
        gb, ub = weights.get("gate_bias"), weights.get("up_bias")
        self.b_gate_up = None
        if gb is not None or ub is not None:
            zeros = lambda: torch.zeros(self.inter, dtype=torch.float32, device=rt.device)
            self.b_gate_up = torch.cat([rt.vector(gb) if gb is not None else zeros(),
                                        rt.vector(ub) if ub is not None else zeros()]).contiguous()
        self.b_down = rt.vector(weights["down_bias"]) if weights.get("down_bias") is not None else None

    def forward_from_residual(self, ctx, residual, norm) -> bool:
        """Decode-sized steps in bfloat16: norm, gate/up product and activation are one kernel.
        False: not taken, the block runs norm and `forward`."""
        rt, ops = self.rt, self.rt.ops
        rows = residual.shape[0]
        prologue = getattr(norm, "fused_prologue", lambda: None)()
        form = fused_form(ops, rows, self.hidden, self.w_gate_up, gate_up=True) if hasattr(ops, "norm_gate_up_swiglu") else None
        if rt.dtype != torch.bfloat16 or prologue is None or form is None:
            return False
        norm_scale, norm_eps = prologue
        act = rt.empty((rows, self.inter))
        prepared = take_prepared(ctx, norm, residual)      # the sum before this norm may have computed its first steps
        if prepared is None and form == "chunks":
            prepared = ops.prepare_norm(residual, norm_scale)
        ops.norm_gate_up_swiglu(residual, norm_scale, norm_eps, self.w_gate_up, act, bias=self.b_gate_up,
                                **({"prepared": prepared} if prepared is not None else {}))
        if not add_and_prepare(ctx, ops, act, self.w_down, residual, self.b_down):
            ops.linear(act, self.w_down, residual, bias=self.b_down, accumulate=True)
        return True

    def _own_products(self, rows: int) -> bool:
        """17 to 128 rows: the kernel library may prefer its own products to the GEMM library's (it does when both matrices
        have their tile-major copies)."""
        own = getattr(self.rt.ops, "own_feed_forward", None)
        return own is not None and self.rt.dtype == torch.bfloat16 and own(rows, self.w_gate_up, self.w_down)

    def forward_branch(self, ctx, h):
        """The output as a tensor of its own instead of a sum into the residual stream (large bfloat16
        steps whose products go to the GEMM library, which has no residual epilogue): the block lets
        the sum ride on the next norm.  None: not taken."""
        rt, ops = self.rt, self.rt.ops
        rows = h.shape[0]
        start = getattr(ops, "library_gemm_from", None)
        if rt.dtype != torch.bfloat16 or start is None or rows < start or self.b_down is not None:
            return None
        if self._own_products(rows):
            return None          # `forward` runs the own products, which add into the residual stream themselves
        act = rt.empty((rows, self.inter))
        if (getattr(ops, "prefers_own_gate_up", None) is not None and ops.prefers_own_gate_up(rows, self.w_gate_up)
                and self.hidden % 8 == 0 and h.stride(0) % 8 == 0):
            ops.gate_up_swiglu(h, self.w_gate_up, act, bias=self.b_gate_up)     # the activation as the product's epilogue
        else:
            gate_up = rt.empty((rows, 2 * self.inter))
            ops.linear(h, self.w_gate_up, gate_up, bias=self.b_gate_up)
            ops.swiglu(gate_up, act)
        out = rt.empty((rows, self.hidden))
        ops.linear(act, self.w_down, out)
        return out

    def forward(self, ctx, h, residual):
        rt, ops = self.rt, self.rt.ops
        rows = h.shape[0]
        start = getattr(ops, "library_gemm_from", None)
        if (rt.dtype == torch.bfloat16 and self.hidden % 8 == 0 and h.stride(0) % 8 == 0
                and (self._own_products(rows) or (rows <= getattr(ops, "GATE_UP_SWIGLU_ROWS", 0) and (start is None or rows < start)))):
            # decode batches that the hand-written products serve: the activation is the epilogue of the gate/up product
            act = rt.empty((rows, self.inter))
            ops.gate_up_swiglu(h, self.w_gate_up, act, bias=self.b_gate_up)
            ops.linear(act, self.w_down, residual, bias=self.b_down, accumulate=True)
            return
        gate_up = rt.empty((rows, 2 * self.inter))
        ops.linear(h, self.w_gate_up, gate_up, bias=self.b_gate_up)
        act = rt.empty((rows, self.inter))
        ops.swiglu(gate_up, act)
        ops.linear(act, self.w_down, residual, bias=self.b_down, accumulate=True)


register_part("feed_forward", "gated_mlp", GatedMLP)
