"""Rotary position encoding: the cos/sin tables the attention kernels index by position.

inv[l] = 1 / theta^(2l/dims) in float32, divided by a per-lane divisor when the scaling has one;
phase = position * inv[l] in float32; cos and sin are evaluated in float64 and stored as float32
(rust/engine/src/rope.rs:28-68).  `linear` scaling divides the position (rope.rs:53-62);
`llama3` scaling gives per-lane divisors computed in float64 (rust/checkpoint/src/plan.rs:1478-1505).
"""
from __future__ import annotations

import math
from typing import Tuple

import torch

from ..registry import register_part
from .base import Part

PAIR_HALF, PAIR_INTERLEAVED = 0, 1


def llama3_divisors(dims: int, theta: float, factor: float, low: float, high: float, original: float):
    """float64 per-lane divisors, returned as a float32 tensor [dims/2]."""
    out = []
    low_wavelength = original / low
    high_wavelength = original / high
    for i in range(dims // 2):
        frequency = 1.0 / (theta ** ((2 * i) / dims))
        wavelength = 2.0 * math.pi / frequency
        if wavelength < high_wavelength:
            scale = 1.0
        elif wavelength > low_wavelength:
            scale = factor
        else:
            smooth = (original / wavelength - low) / (high - low)
            scale = 1.0 / ((1.0 - smooth) / factor + smooth)
        out.append(scale)
    return torch.tensor(out, dtype=torch.float64).to(torch.float32)


class Rotary(Part):
    role = "position"

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        self.dims = int(spec["dims"])
        self.theta = float(spec["theta"])
        self.pairing = {"half": PAIR_HALF, "interleaved": PAIR_INTERLEAVED}[spec.get("pairing", "half")]
        self.scaling = spec.get("scaling", "none")
        if self.dims % 2 != 0 or self.dims <= 0:
            raise ValueError("rotary dims must be even and positive")
        positions = int(min(rt.max_context, spec.get("max_position", rt.max_context)))
        key = ("rotary", self.dims, self.theta, self.scaling, spec.get("factor"), spec.get("low_freq_factor"),
               spec.get("high_freq_factor"), spec.get("original_max_position"), positions)
        tables = rt.shared.get(key)
        if tables is None:
            tables = tuple(t.to(rt.device) for t in self._build(positions))
            rt.shared[key] = tables
        self.cos, self.sin = tables
        self.positions = positions

    def _build(self, positions: int) -> Tuple[torch.Tensor, torch.Tensor]:
        half = self.dims // 2
        lanes = torch.arange(half, dtype=torch.float32)
        exponent = (lanes * 2.0) / float(self.dims)                      # float32, as `(lane*2) as f32 / dims as f32`
        # float32 powf of float32 operands, correctly rounded: evaluated in float64, rounded once
        base = torch.tensor(self.theta, dtype=torch.float32).double()
        inv = 1.0 / torch.pow(base, exponent.double()).to(torch.float32)
        if self.scaling == "llama3":
            s = self.spec
            inv = inv / llama3_divisors(self.dims, self.theta, float(s["factor"]), float(s["low_freq_factor"]),
                                        float(s["high_freq_factor"]), float(s["original_max_position"]))
        scale = 1.0
        if self.scaling == "linear":
            scale = 1.0 / float(self.spec["factor"])
        elif self.scaling not in ("none", "llama3"):
            raise ValueError(f"unknown rotary scaling {self.scaling!r}")
        pos = torch.arange(positions, dtype=torch.float32) * torch.tensor(scale, dtype=torch.float32)
        phase = (pos[:, None] * inv[None, :]).to(torch.float64)          # float32 product, then widened
        return torch.cos(phase).to(torch.float32).contiguous(), torch.sin(phase).to(torch.float32).contiguous()


register_part("position", "rotary", Rotary)
