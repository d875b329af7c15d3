"""What parts get to work with: the device, the compute precision and the kernel library."""
from __future__ import annotations

import weakref
from typing import Any, Dict

import torch


class Runtime:
    """`dtype` is the compute precision: float32 (everything in true 32-bit) or bfloat16
    (matrices, activations and pages in bfloat16; residual stream, norms, softmax, rotary angles
    and logits in float32).  `ops` is the kernel library (`fllm_amd.kernels.Ops`)."""

    def __init__(self, device: torch.device, dtype: torch.dtype, ops, max_context: int, decode_weight_tiles="auto"):
        if dtype not in (torch.float32, torch.bfloat16):
            raise ValueError(f"compute dtype must be float32 or bfloat16, not {dtype}")
        self.device = torch.device(device)
        self.dtype = dtype
        self.ops = ops
        self.max_context = int(max_context)
        # second copies of some weight matrices in the order decode steps read them (`tile_for_decode`): True, False, or
        # "auto": as long as they leave half of the free memory to the cache
        self.decode_weight_tiles = decode_weight_tiles
        self._tile_requests = None            # a list while a model is being built
        # weak: a placed tensor lives as long as a part holds it (pieces of a concatenated matrix are freed)
        self._placed = weakref.WeakValueDictionary()
        self.shared: Dict[Any, Any] = {}      # tables several parts share (rotary tables)

    def _place(self, t: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
        key = (t.data_ptr(), tuple(t.shape), t.dtype, dtype)
        hit = self._placed.get(key)
        if hit is None:
            hit = t.to(device=self.device, dtype=dtype).contiguous()
            self._placed[key] = hit
        return hit

    def matrix(self, t: torch.Tensor) -> torch.Tensor:
        """A weight matrix or table on the device in the compute dtype.  The same checkpoint
        tensor is placed once (a tied head shares the embedding's copy)."""
        return self._place(t, self.dtype)

    def vector(self, t: torch.Tensor) -> torch.Tensor:
        """Norm weights and biases: float32 (exact for both storage types)."""
        return self._place(t, torch.float32)

    def tile_for_decode(self, w: torch.Tensor, gate_up: bool = False, priority: int = 0) -> None:
        """For a matrix that decode steps stream: lets the kernel library keep a tile-major copy beside it, where it has
        such kernels and the memory is there (288 GB a device are laid out for bandwidth: the copy costs the matrix's
        bytes again and takes a fifth off such a product at 8 rows).  `gate_up`: w is [gate; up], see the library.
        `priority`: while a model is being built the copies are only asked for, and made when it is whole
        (`tiles_for_model`), the lower numbers first: 0 for copies that every decode step reads (output and down
        projections), 1 for the layers' other matrices, 2 for the vocabulary projection (once a step)."""
        make = getattr(self.ops, "tile_for_decode", None)
        if not self.decode_weight_tiles or make is None or self.dtype != torch.bfloat16 or not w.is_cuda:
            return
        if self._tile_requests is not None:
            self._tile_requests.append((priority, len(self._tile_requests), w, gate_up))
            return
        if self.decode_weight_tiles == "auto":
            free, _ = torch.cuda.mem_get_info(self.device)
            if w.numel() * w.element_size() > free // 20:
                return                                    # the device is filling up
        make(w, gate_up=True) if gate_up else make(w)

    def collect_tile_requests(self) -> None:
        """From here on `tile_for_decode` only notes what is asked for, until `tiles_for_model`."""
        self._tile_requests = []

    def tiles_for_model(self) -> int:
        """Makes the copies that the parts of a model asked for, now that all its weights are on the device: in the order
        of their priorities, and under "auto" within half of the memory that is free now (the other half is the
        cache's).  A copy that does not fit is left out and smaller ones behind it may still be made, so a model too
        large for all copies keeps those that every step reads.  Returns the bytes copied."""
        requests, self._tile_requests = sorted(self._tile_requests or [], key=lambda r: r[:2]), None
        make = getattr(self.ops, "tile_for_decode", None)
        if not requests or make is None:
            return 0
        budget = None
        if self.decode_weight_tiles == "auto":
            torch.cuda.empty_cache()          # what placing the weights left in the allocator's hands counts as free
            free, _ = torch.cuda.mem_get_info(self.device)
            budget = free // 2
        made = 0
        for _, _, w, gate_up in requests:
            size = w.numel() * w.element_size()
            if budget is not None and size > budget:
                continue
            if make(w, gate_up=True) if gate_up else make(w):
                made += size
                if budget is not None:
                    budget -= size
        return made

    def forget_host_tensors(self) -> None:
        self._placed.clear()

    def empty(self, shape, dtype=None) -> torch.Tensor:
        return torch.empty(shape, dtype=dtype or self.dtype, device=self.device)
