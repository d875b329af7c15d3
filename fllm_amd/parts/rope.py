"""Rotary position encoding: the cos/sin tables the attention kernels index by position.

inv[l] = 1 / theta^(2l/dims) in float32, divided by a per-lane divisor when the scaling has one;
phase = position * inv[l] in float32; cos and sin are evaluated in float64 and stored as float32
(rust/engine/src/rope.rs:28-68).  `linear` scaling divides the position (rope.rs:53-62);
`llama3` scaling gives per-lane divisors computed in float64 (rust/checkpoint/src/plan.rs:1478-1505).
`yarn` mixes, lane by lane, the plain angle with the angle of a position divided by the factor and multiplies
cos and sin by a magnitude (rope.rs:70-110); `longrope` divides the frequencies by one of two lists of
per-lane factors, the long one when the tables reach beyond the original context, and multiplies cos and sin
by its attention factor (rope.rs:30-36, :58-61).  All of it in float32 up to the phase, as the reference.
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
        key = ("rotary", self.dims, self.theta, self.scaling, positions) + tuple(
            tuple(v) if isinstance(v, (list, tuple)) else v
            for v in (spec.get(k) for k in ("factor", "low_freq_factor", "high_freq_factor", "original_max_position",
                                            "extrapolation", "attention", "beta_fast", "beta_slow", "truncate",
                                            "short_factor", "long_factor")))
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
        f32 = lambda v: torch.tensor(float(v), dtype=torch.float32)
        if self.scaling == "yarn":
            return self._build_yarn(positions, inv)
        scale, magnitude = f32(1.0), None
        if self.scaling == "linear":
            scale = f32(1.0) / f32(self.spec["factor"])
        elif self.scaling == "longrope":
            s = self.spec
            longer = positions > int(s["original_max_position"])
            factors = torch.tensor(list(s["long_factor"] if longer else s["short_factor"]), dtype=torch.float32)
            if factors.numel() != half:
                raise ValueError(f"longrope factors must have {half} entries")
            inv = inv / factors
            magnitude = f32(s["attention"])
        elif self.scaling not in ("none", "llama3"):
            raise ValueError(f"unknown rotary scaling {self.scaling!r}")
        pos = torch.arange(positions, dtype=torch.float32) * scale
        phase = (pos[:, None] * inv[None, :]).to(torch.float64)          # float32 product, then widened
        cos, sin = torch.cos(phase).to(torch.float32), torch.sin(phase).to(torch.float32)
        if magnitude is not None:
            cos, sin = cos * magnitude, sin * magnitude
        return cos.contiguous(), sin.contiguous()

    def _build_yarn(self, positions: int, inv: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
        """rope.rs:70-110, every step in float32 as there.  The lanes below `low` keep their angle, the lanes
        above `high` get the angle of position / factor, the lanes between a mix of both."""
        s = self.spec
        f32 = lambda v: torch.tensor(float(v), dtype=torch.float32)
        half = self.dims // 2
        factor, extrapolation = f32(s["factor"]), f32(s.get("extrapolation", 1.0))
        base, original, dims = f32(self.theta), f32(int(s["original_max_position"])), f32(self.dims)
        # the checkpoint's factor stands in for the built-in 1 + 0.1 ln(factor): plan.rs:1460-1476
        attention = f32(1.0)
        if s.get("attention") is not None:
            attention = f32(float(s["attention"]) / (0.1 * math.log(float(s["factor"])) + 1.0))
        scale = f32(1.0) / factor

        def correction_dim(rotations):                                   # rope.rs:15-18
            return dims * torch.log(original / (f32(rotations) * f32(2.0) * f32(math.pi))) / (f32(2.0) * torch.log(base))

        low, high = correction_dim(s.get("beta_fast", 32.0)), correction_dim(s.get("beta_slow", 1.0))
        if s.get("truncate", True):
            low, high = torch.floor(low), torch.ceil(high)
        low, high = torch.clamp(low, min=0.0), torch.clamp(high, max=float(self.dims) - 1.0)
        lanes = torch.arange(half, dtype=torch.float32)
        ramp = f32(1.0) - torch.clamp((lanes - low) / torch.clamp(high - low, min=0.001), 0.0, 1.0)   # rope.rs:20-23
        pos = torch.arange(positions, dtype=torch.float32)
        extrapolated = pos[:, None] * inv[None, :]
        interpolated = scale * extrapolated
        if float(extrapolation) != 0.0:
            mix = (ramp * extrapolation)[None, :]
            theta = interpolated * (f32(1.0) - mix) + extrapolated * mix
            magnitude = attention * (f32(1.0) + f32(0.1) * torch.log(f32(1.0) / scale))
        else:
            theta, magnitude = interpolated, attention
        phase = theta.to(torch.float64)
        cos, sin = torch.cos(phase).to(torch.float32) * magnitude, torch.sin(phase).to(torch.float32) * magnitude
        return cos.contiguous(), sin.contiguous()


register_part("position", "rotary", Rotary)
