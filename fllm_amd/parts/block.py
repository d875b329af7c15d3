"""Arrangement of parts in a layer.  `prenorm`: x += mixer(norm(x)); x += feed_forward(norm(x))
(rust/engine/src/rust_decoder.rs:8764-8766, :9059-9088)."""
from __future__ import annotations

from ..registry import register_part
from .base import Block


class PreNormBlock(Block):
    def __init__(self, spec, weights, rt, mixer=None, feed_forward=None, norms=None):
        super().__init__(spec, weights, rt)
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.mixer_norm = norms["mixer"]
        self.feed_forward_norm = norms["feed_forward"]

    def forward(self, ctx, residual, binding):
        h = self.mixer_norm.forward(ctx, residual)
        self.mixer.forward(ctx, h, residual, binding)
        h = self.feed_forward_norm.forward(ctx, residual)
        self.feed_forward.forward(ctx, h, residual)


register_part("block", "prenorm", PreNormBlock)
