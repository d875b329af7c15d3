"""Token embedding (x[r] = scale * E[ids[r]], rust/engine/src/rust_decoder.rs:8605-8616) and
the output head (logits = W h, float32; :8685)."""
from __future__ import annotations

import torch

from ..registry import register_part
from .base import INIT_MATRIX, Part


class TokenEmbedding(Part):
    role = "embedding"

    @classmethod
    def tensor_shapes(cls, spec):
        return {"weight": ((spec["vocab_size"], spec["hidden_size"]), INIT_MATRIX)}

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        self.table = rt.matrix(weights["weight"])
        self.scale = float(spec.get("scale", 1.0))
        self.hidden = int(spec["hidden_size"])

    def forward(self, ctx, ids):
        out = self.rt.empty((ids.numel(), self.hidden), torch.float32)
        return self.rt.ops.embed(ids, self.table, out, self.scale)


class LinearHead(Part):
    role = "head"

    @classmethod
    def tensor_shapes(cls, spec):
        return {"weight": ((spec["vocab_size"], spec["hidden_size"]), INIT_MATRIX)}

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        self.weight = rt.matrix(weights["weight"])
        self.vocab = int(spec["vocab_size"])
        rt.tile_for_decode(self.weight, priority=2)      # read once a step of up to 16 rows: after the layers' copies

    def forward(self, ctx, h):
        logits = self.rt.empty((h.shape[0], self.vocab), torch.float32)
        return self.rt.ops.linear(h, self.weight, logits)


register_part("embedding", "table", TokenEmbedding)
register_part("head", "linear", LinearHead)
