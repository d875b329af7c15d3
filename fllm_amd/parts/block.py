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
        # a part may take the residual stream and the norm before it in one fused kernel
        h = None
        fused = getattr(self.mixer, "forward_from_residual", None)
        if fused is None or not fused(ctx, residual, self.mixer_norm, binding):
            h = self.mixer_norm.forward(ctx, residual)
            # a mixer may hand back its output instead of adding it: the add then rides on the next norm
            as_branch = getattr(self.mixer, "forward_branch", None)
            add_norm = getattr(self.feed_forward_norm, "add_forward", None)
            branch = as_branch(ctx, h, binding) if as_branch is not None and add_norm is not None else None
            if branch is not None:
                h = add_norm(ctx, residual, branch)
                self.feed_forward.forward(ctx, h, residual)
                return
            self.mixer.forward(ctx, h, residual, binding)
        fused = getattr(self.feed_forward, "forward_from_residual", None)
        if fused is None or not fused(ctx, residual, self.feed_forward_norm):
            h = self.feed_forward_norm.forward(ctx, residual)
            self.feed_forward.forward(ctx, h, residual)


register_part("block", "prenorm", PreNormBlock)
