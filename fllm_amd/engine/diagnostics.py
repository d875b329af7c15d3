"""Layer-by-layer diagnostics of a forward pass, for finding the layer at which a model goes wrong.

With a `LayerCheck` switched on, every layer of a step runs twice on the same input: once with the plain kernels
(one float32 chain per output element, no matrix cores, no GEMM library) and once with the kernels that serving uses;
the residual streams that come out are compared, and for each layer one line says how far they are apart, the
largest value, a checksum and whether a NaN or Inf appeared.  In float32 mode both runs use the same kernels and the
line holds the statistics only.  The reference has the same aids in its decoder: a second run of every device layer by
its host code on the same input (rust/engine/src/rust_decoder.rs:4759, :4809, :6425), sums of buffers (:833-857) and
a scan of the residual stream for NaN, Inf and range (:877-917).
"""
from __future__ import annotations

import sys
from dataclasses import dataclass
from typing import IO, List, Optional

import torch


@dataclass
class LayerReport:
    step: int
    entry: int                 # index in the run order
    layer: int                 # index of the layer's weights
    rows: int
    largest: float             # max |residual| after the layer
    checksum: float            # sum of the residual stream after the layer, in float64
    bad_values: int            # NaN or Inf
    distance: Optional[float]  # max |serving - plain| / max |plain| ; None when there was no second run

    def line(self) -> str:
        far = "-" if self.distance is None else f"{self.distance:.3e}"
        return (f"[layer-check] step {self.step} entry {self.entry} layer {self.layer} rows {self.rows}: "
                f"distance to the plain kernels {far}, largest |x| {self.largest:.4e}, checksum {self.checksum:.6f}, "
                f"NaN/Inf {self.bad_values}")


class LayerCheck:
    """`steps`: how many forward passes are checked (then the check switches itself off).  `limit`: a distance above
    which a layer counts as suspect (reported in `suspects`)."""

    def __init__(self, steps: int = 2, limit: float = 5e-2, out: Optional[IO[str]] = None):
        self.steps_left = int(steps)
        self.limit = float(limit)
        self.out = out if out is not None else sys.stderr
        self.reports: List[LayerReport] = []
        self.step = 0

    @property
    def active(self) -> bool:
        return self.steps_left > 0

    def suspects(self) -> List[LayerReport]:
        return [r for r in self.reports if r.bad_values or (r.distance is not None and r.distance > self.limit)]

    # ---- called by Model.forward ----------------------------------------------------------
    def run_block(self, model, block, ctx, x: torch.Tensor, binding, entry_index: int, layer_index: int) -> None:
        """Runs `block` on the residual stream `x` in place (everything added), after a run with the plain kernels on
        a copy of it."""
        ops = model.rt.ops
        stateful = binding.state is not None          # a second run would advance the state twice
        plain = None
        if model.rt.dtype == torch.bfloat16 and not stateful and hasattr(ops, "set_fast_kernels"):
            plain = x.clone()
            library_from = getattr(ops, "library_gemm_from", None)
            ops.set_fast_kernels(False)
            ops.library_gemm_from = None
            try:
                self._run(model, block, ctx, plain, binding)
            finally:
                ops.set_fast_kernels(True)
                ops.library_gemm_from = library_from
        self._run(model, block, ctx, x, binding)       # second, so that the cache keeps what serving writes
        distance = None
        if plain is not None:
            scale = float(plain.abs().max())
            distance = float((x - plain).abs().max()) / scale if scale > 0 else float((x - plain).abs().max())
        finite = torch.isfinite(x)
        bad = int(x.numel() - int(finite.sum()))
        clean = torch.where(finite, x, torch.zeros_like(x))
        report = LayerReport(self.step, entry_index, layer_index, x.shape[0], float(clean.abs().max()) if x.numel() else 0.0,
                             float(clean.double().sum()), bad, distance)
        self.reports.append(report)
        print(report.line(), file=self.out, flush=True)

    @staticmethod
    def _run(model, block, ctx, x, binding) -> None:
        if getattr(block, "takes_pending", False):
            pending = block.forward(ctx, x, binding, None)
            if pending is not None:
                model.rt.ops.add_residual(x, pending)
        else:
            block.forward(ctx, x, binding)

    def end_step(self) -> None:
        self.step += 1
        self.steps_left -= 1
        if self.steps_left == 0:
            suspects = self.suspects()
            if suspects:
                first = suspects[0]
                print(f"[layer-check] first suspect: step {first.step}, run entry {first.entry} (layer {first.layer})",
                      file=self.out, flush=True)
            else:
                print(f"[layer-check] {len(self.reports)} layer runs checked, none beyond {self.limit:g}", file=self.out, flush=True)
