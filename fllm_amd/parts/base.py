"""What every part must offer.

A part is built from a `PartSpec` (its sizes and constants), the tensors the spec names, and the
runtime (device, precision, kernel library).  It never sees the model configuration.

Roles and their interfaces:

  norm          forward(ctx, x_f32[R,H], out=None, rows=None) -> normed[R or len(rows), H] in the
                compute dtype; `rows` (int32 device tensor) selects rows first.  Optional:
                add_forward(ctx, x, branch, out=None) adds `branch` to x first (one pass over the row), and
                fused_prologue() -> (scale_f32[H], eps) when the norm is x * rsqrt(mean(x^2) + eps) * scale for some
                vector `scale` (None otherwise): parts that have a kernel which norms its input on the way in ask the
                norm for these instead of asking what kind of norm it is.
  position      what the mixer's kernels take: for the attention mixer float32 device tables `cos` and `sin`
                [positions, dims/2], `dims` (lanes of a head that are rotated; 0 with empty tables: none) and `pairing`
                (0: lanes l and l + dims/2, 1: lanes 2l and 2l + 1).  Optional: `score_slopes`, a float32 device
                vector [heads]: every score gets score_slopes[head] * (key position - row position) added (an
                encoding that biases scores by distance; such layers run the plain attention kernel).
  mixer         cache_need() / state_need() say what the cache manager must keep for it (keys and values of widths
                of their own; one state tensor or several named ones); portion_multiple() on which multiples of
                tokens a prompt may be cut;
                forward(ctx, h[R,H], residual_f32[R,H], binding) adds its output to `residual`.
                State of fixed size: `binding.state[slot]` (`binding.state[name][slot]` when the mixer named several)
                belongs to one live request (slot = ctx.seg_slots[s] on the
                host, ctx.slots[s] on the device).  The step function hands it over filled with zeros at the first
                step of a request it has not seen before (also one that was freed and is fed again from position 0),
                touches it at no other time, and runs a request's rows in position order, `seg_pos_start[s]` being the
                number of tokens the request held before this step; so the state a mixer finds is the one it left after
                position seg_pos_start[s] - 1.
  feed_forward  forward(ctx, h[R,H], residual_f32[R,H]) adds its output to `residual`.
  block         forward(ctx, residual_f32[R,H], binding) runs norms, mixer and feed-forward.  It is built with
                mixer=, feed_forward= (None for a layer without one), norms= (by the names the layer's spec
                uses) and, only when the spec lists any, extras= (further parts by name).  A block
                with `takes_pending = True` is called as forward(ctx, residual, binding, pending): `pending`
                is a branch [R,H] that the block before left for it to add (or None), and it returns its
                own such branch or None.
                A norm prepared ahead (optional, for blocks and parts that want it): before a block runs a part whose
                sum into `residual` is read next by a norm it knows, it names that norm in `ctx.then_norm` (for the
                part that ends the block: `ctx.next_norm`, which whoever runs the blocks sets to the first norm of the
                block after).  A part whose last kernel can compute that norm's first steps on the way out does so and
                leaves `ctx.prepared = (norm, residual, payload)` (`leave_prepared`); the part that applies `norm` to
                that very `residual` next asks `take_prepared(ctx, norm, residual)` and gets the payload or None.  A
                block clears what its parts did not take, so nothing outlives the sum it was made from.
  embedding     forward(ctx, ids[R]) -> residual_f32[R,H].
  head          forward(ctx, h[L,H]) -> logits_f32[L,V].

The residual stream is float32 in every precision mode; `h` is in the compute dtype.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Optional, Tuple

import torch

from ..config.spec import PartSpec

# how random-weights mode fills a tensor
INIT_MATRIX = "matrix"     # N(0, 0.02)
INIT_NORM = "norm"         # 1 + U(-0.1, 0.1)
INIT_BIAS = "bias"         # N(0, 0.02)


@dataclass(frozen=True)
class KVNeed:
    """Per token, keys of `kv_heads` heads of `k_dim` values and values of as many heads of `v_dim` (`k_dim` when left
    out; 0: the mixer caches keys alone); `window` keys back (the token itself included) or all of them when None.
    The pages are shaped from both widths; what a mixer's kernels can read is the mixer's matter.  `key_chunk`: 0 stores
    a token's keys together ([page][kv_head][token][k_dim]); n > 0 stores them in chunks of n values, chunk by chunk over
    the tokens of a page ([page][kv_head][k_dim / n][token][n]), the order this library's attention kernels read."""
    kv_heads: int
    k_dim: int
    v_dim: Optional[int] = None
    window: Optional[int] = None
    key_chunk: int = 0

    def __post_init__(self):
        if self.v_dim is None:
            object.__setattr__(self, "v_dim", self.k_dim)
        if self.kv_heads <= 0 or self.k_dim <= 0 or self.v_dim < 0:
            raise ValueError(f"a cache of {self.kv_heads} heads with keys of {self.k_dim} and values of {self.v_dim}")
        if self.key_chunk < 0 or (self.key_chunk and self.k_dim % self.key_chunk != 0):
            raise ValueError(f"keys of {self.k_dim} values cannot be stored in chunks of {self.key_chunk}")

    def key_page_shape(self, page_size: int) -> Tuple[int, ...]:
        """Shape of the keys of one key/value head in one page."""
        if self.key_chunk:
            return (self.k_dim // self.key_chunk, page_size, self.key_chunk)
        return (page_size, self.k_dim)


@dataclass(frozen=True)
class StateNeed:
    """A fixed-size tensor per live request (shape without the request dimension)."""
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


class Part:
    role = ""

    @classmethod
    def tensor_shapes(cls, spec: PartSpec) -> Dict[str, Tuple[Tuple[int, ...], str]]:
        """Own parameter name -> (shape, init kind).  Names that `spec.tensors` lists with a
        leading '?' are optional in a checkpoint."""
        return {}

    def __init__(self, spec: PartSpec, weights: Dict[str, torch.Tensor], rt):
        self.spec = spec
        self.rt = rt


class Mixer(Part):
    role = "mixer"

    def cache_need(self) -> Optional[KVNeed]:
        return None

    def state_need(self):
        """None, one `StateNeed` (then `binding.state[slot]` is the request's tensor), or a dict of named ones of any
        shapes and types (then `binding.state[name][slot]`)."""
        return None

    def portion_multiple(self) -> int:
        """A portion of a prompt that does not end the prompt must hold a multiple of this many tokens (a mixer whose
        kernels work on fixed chunks of positions); 1: any cut.  The scheduler cuts accordingly and the step function
        refuses other cuts."""
        return 1

    def forward(self, ctx, h, residual, binding) -> None:
        raise NotImplementedError


class FeedForward(Part):
    role = "feed_forward"

    def forward(self, ctx, h, residual) -> None:
        raise NotImplementedError


class Norm(Part):
    role = "norm"

    def forward(self, ctx, x, out=None, rows=None):
        raise NotImplementedError

    def fused_prologue(self):
        """(scale, eps) if the norm is x * rsqrt(mean(x^2) + eps) * scale with a float32 device vector `scale`,
        so that a kernel can apply it to the rows it reads; None if it is anything else."""
        return None


class Block(Part):
    role = "block"

    def first_norm(self):
        """The norm this block applies to the residual stream first, if whoever ends the block before may prepare it
        (`ctx.next_norm`); None: the block says nothing, and nothing is prepared for it."""
        return None


def take_prepared(ctx, norm, residual):
    """What the part before left for `norm` applied to `residual`, or None; whatever was left is gone afterwards."""
    left = getattr(ctx, "prepared", None)
    if left is None:
        return None
    ctx.prepared = None
    return left[2] if left[0] is norm and left[1] is residual else None


def leave_prepared(ctx, norm, residual, payload) -> None:
    ctx.prepared = (norm, residual, payload)


def fused_form(ops, rows: int, width: int, w, gate_up: bool = False):
    """Which of the kernel library's fused kernels serve a product of `rows` rows with the matrix `w` behind a norm of
    `width`: "resident" (the norm is folded in or prepared), "chunks" (more rows: the norm must be prepared,
    `ops.prepare_norm` does it where the product before has not) or None."""
    ask = getattr(ops, "fused_form", None)
    if ask is not None:
        return ask(rows, width, w, gate_up=gate_up)
    return "resident" if ops.fused_decode_supported(rows, width) else None


def add_and_prepare(ctx, ops, x, w, residual, bias) -> bool:
    """residual += x @ w.T (+ bias) in the kernel that also prepares `ctx.then_norm`, where the kernel library has one
    for this size and that norm says what it multiplies by (`fused_prologue`); the result is left for the norm's
    reader.  False: nothing was done, the caller adds as usual."""
    norm = getattr(ctx, "then_norm", None)
    prepare = getattr(ops, "linear_add_prepare", None)
    prologue = getattr(norm, "fused_prologue", lambda: None)() if norm is not None else None
    if prepare is None or prologue is None or residual is None:
        return False
    rows, width = residual.shape
    if not (ops.prepares_norm(rows, width, w) if rows > 16 else ops.prepares_norm(rows, width)):
        return False
    if x.dtype != torch.bfloat16 or x.stride(0) % 8 != 0 or x.shape[1] % 8 != 0:
        return False
    leave_prepared(ctx, norm, residual, prepare(x, w, residual, prologue[0], bias=bias))
    return True
