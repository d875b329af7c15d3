"""RMSNorm: y = x * (rsqrt(mean(x^2) + eps) * w), in float32, the product in the reference's
order (rust/engine/src/rust_decoder.rs:1481-1490; cuda/elementwise.cu:18-54)."""
from __future__ import annotations

from ..registry import register_part
from .base import INIT_NORM, Norm


class RMSNorm(Norm):
    @classmethod
    def tensor_shapes(cls, spec):
        return {"weight": ((spec["size"],), INIT_NORM)}

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        self.size = int(spec["size"])
        self.eps = float(spec["eps"])
        if not self.eps > 0.0:
            raise ValueError("RMSNorm needs a positive eps")
        self.weight = rt.vector(weights["weight"])

    def forward(self, ctx, x, out=None, rows=None):
        count = x.shape[0] if rows is None else rows.numel()
        if out is None:
            out = self.rt.empty((count, self.size))
        return self.rt.ops.rmsnorm(x, self.weight, self.eps, out, rows=rows)

    def fused_prologue(self):
        return self.weight, self.eps

    def add_forward(self, ctx, x, branch, out=None):
        """x += branch, then the norm of the sum: one pass over the row."""
        if out is None:
            out = self.rt.empty((x.shape[0], self.size))
        return self.rt.ops.add_rmsnorm(x, branch, self.weight, self.eps, out)


register_part("norm", "rms", RMSNorm)
