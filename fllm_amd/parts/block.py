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
        self.feed_forward_norm = norms["feed_forward"] if feed_forward is not None else None

    def first_norm(self):
        return self.mixer_norm

    takes_pending = True     # forward accepts a branch that the block before has not added yet, and may hand one on

    def forward(self, ctx, residual, binding, pending=None):
        """Runs the layer on the residual stream.  `pending`: the output of the block before, still
        to be added; the return value is this block's own such output, or None when everything has
        been added.  Where a sum can ride on the norm that follows it, it costs no pass of its own."""
        ops = self.rt.ops
        # a norm prepared ahead: what the block before left for this block's first norm, and the norms that this
        # block's own sums are read by (the feed-forward's; the first norm of the block after)
        incoming, ctx.prepared = getattr(ctx, "prepared", None), None
        after = getattr(ctx, "next_norm", None)
        try:
            return self._forward(ctx, residual, binding, pending, incoming, after)
        finally:
            ctx.then_norm = None
            left = getattr(ctx, "prepared", None)
            if left is not None and (after is None or left[0] is not after):
                ctx.prepared = None          # nothing outlives the sum it was made from

    def _forward(self, ctx, residual, binding, pending, incoming, after):
        ops = self.rt.ops
        add_mixer_norm = getattr(self.mixer_norm, "add_forward", None)
        add_ff_norm = getattr(self.feed_forward_norm, "add_forward", None) if self.feed_forward is not None else None
        # a part may take the residual stream and the norm before it in one fused kernel
        fused = getattr(self.mixer, "forward_from_residual", None)
        if pending is not None:
            if add_mixer_norm is None:
                ops.add_residual(residual, pending)
                pending = None
            else:
                fused = None     # the fused kernels read the finished residual stream: the sum rides on the norm instead
        if fused is not None and pending is None:
            ctx.prepared = incoming
        ctx.then_norm = self.feed_forward_norm if self.feed_forward is not None else after
        taken = fused is not None and fused(ctx, residual, self.mixer_norm, binding)
        ctx.then_norm = None
        if not taken:
            ctx.prepared = None
            if pending is not None:
                h = add_mixer_norm(ctx, residual, pending)
            else:
                h = self.mixer_norm.forward(ctx, residual)
            # a mixer may hand back its output instead of adding it: the add then rides on the next norm
            as_branch = getattr(self.mixer, "forward_branch", None)
            branch = as_branch(ctx, h, binding) if as_branch is not None and add_ff_norm is not None else None
            if branch is not None:
                h = add_ff_norm(ctx, residual, branch)
                ff_branch = getattr(self.feed_forward, "forward_branch", None)
                out = ff_branch(ctx, h) if ff_branch is not None else None
                if out is None:
                    self.feed_forward.forward(ctx, h, residual)
                return out
            self.mixer.forward(ctx, h, residual, binding)
        if self.feed_forward is None:
            return None                  # a layer of a mixer alone
        left = getattr(ctx, "prepared", None)
        if left is not None and left[0] is not self.feed_forward_norm:
            ctx.prepared = None
        fused = getattr(self.feed_forward, "forward_from_residual", None)
        ctx.then_norm = after
        taken = fused is not None and fused(ctx, residual, self.feed_forward_norm)
        ctx.then_norm = None
        if not taken:
            ctx.prepared = None
            h = self.feed_forward_norm.forward(ctx, residual)
            self.feed_forward.forward(ctx, h, residual)
        return None


register_part("block", "prenorm", PreNormBlock)
