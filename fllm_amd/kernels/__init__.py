"""The kernel library seen from Python: `Ops` wraps the C ABI of csrc/api.h.

Every method checks on the host that tensors are on the GPU, dense, of the element type and the
shape the kernel assumes, before anything is launched.  There is no other implementation: if the
library cannot be loaded or built, constructing `Ops` raises.
"""
from __future__ import annotations

import ctypes
import weakref
from typing import Dict, NamedTuple, Optional, Sequence, Tuple

import torch

from . import build as _build

F32, BF16 = 0, 1
_DTYPE_CODE = {torch.float32: F32, torch.bfloat16: BF16}
OUT_STORE, OUT_STORE_F32, OUT_ADD_F32 = 0, 1, 2


class KernelError(RuntimeError):
    pass


class SampleRow(ctypes.Structure):
    _fields_ = [("temperature", ctypes.c_float), ("top_p", ctypes.c_float), ("top_k", ctypes.c_int32),
                ("min_p", ctypes.c_float), ("seed", ctypes.c_uint64), ("draw", ctypes.c_uint64)]


class PreparedNorm(NamedTuple):
    """What `Ops.linear_add_prepare` leaves for the RMSNorm that reads the residual stream next: the rows times the
    norm's weight in bfloat16, and every row's sum of squares in `parts` parts a row."""
    x: torch.Tensor
    ssq: torch.Tensor
    parts: int


class AdjustLists(ctypes.Structure):
    """FllmAdjustLists: device addresses of the lists that the row records of `adjust_logits` point into."""
    _fields_ = [(name, ctypes.c_void_p) for name in ("seen_ids", "seen_counts", "bias_ids", "bias_values", "blocked_ids",
                                                     "allowed_ids", "if_last", "then_blocked")]


SAMPLE_ROW_BYTES = ctypes.sizeof(SampleRow)
ADJUST_ROW_WORDS = 14         # int32 words of one FllmAdjustRow
assert SAMPLE_ROW_BYTES == 32

_lib = None


ABI_VERSION = 11


def load_library(build_if_missing: bool = True):
    """The loaded library; builds it first when there is none that matches the sources."""
    global _lib
    if _lib is not None:
        return _lib
    path = _build.find_library()
    if path is None:
        if not build_if_missing:
            raise KernelError("the HIP kernel library is not built (run `python -m fllm_amd.kernels.build`)")
        path = _build.build()
    try:
        lib = ctypes.CDLL(path)
    except OSError as exc:
        raise KernelError(f"cannot load the HIP kernel library {path}: {exc}") from None
    c_int, c_void, c_float, c_size = ctypes.c_int, ctypes.c_void_p, ctypes.c_float, ctypes.c_size_t
    lib.fllm_last_error.restype = ctypes.c_char_p
    lib.fllm_abi_version.restype = c_int
    if lib.fllm_abi_version() != ABI_VERSION:
        raise KernelError(f"the HIP kernel library {path} has interface version {lib.fllm_abi_version()}, this package needs "
                          f"{ABI_VERSION}: build it again (python -m fllm_amd.kernels.build)")
    sig = {
        "fllm_embed": [c_void, c_void, c_void, c_int, c_int, c_int, c_int, c_float, c_void],
        "fllm_rmsnorm": [c_void, c_void, c_void, c_void, c_int, c_int, c_float, c_int, c_void],
        "fllm_linear": [c_void, c_int, c_void, c_void, c_void, c_int, c_int, c_int, c_int, c_int, c_int, c_void],
        "fllm_swiglu": [c_void, c_void, c_int, c_int, c_int, c_void],
        "fllm_add_residual": [c_void, c_void, c_int, c_int, c_int, c_void],
        "fllm_add_rmsnorm": [c_void, c_void, c_int, c_void, c_void, c_int, c_int, c_float, c_int, c_void],
        "fllm_rope_kv_store": [c_void, c_void, c_void, c_void, c_int, c_void, c_void, c_int, c_void, c_void, c_int,
                               c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void],
        "fllm_attention": [c_void, c_int, c_void, c_void, c_void, c_int, c_void, c_void, c_void, c_int, c_void, c_int,
                           c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_int, c_int, c_void, c_size, c_void],
        "fllm_attention_sloped": [c_void, c_int, c_void, c_void, c_void, c_int, c_void, c_void, c_void, c_int, c_void, c_int,
                                  c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_int, c_void, c_void],
        "fllm_norm_linear": [c_void, c_void, c_float, c_void, c_void, c_void, c_int, c_int, c_int, c_void],
        "fllm_norm_gate_up_swiglu": [c_void, c_void, c_float, c_void, c_void, c_void, c_int, c_int, c_int, c_void],
        "fllm_norm_qkv_rope_store": [c_void, c_void, c_float, c_void, c_void, c_void, c_void, c_void, c_void, c_int, c_void,
                                     c_void, c_int, c_void, c_void, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void],
        "fllm_argmax": [c_void, c_void, c_int, c_int, c_void],
        "fllm_gate_up_swiglu": [c_void, c_int, c_void, c_void, c_void, c_int, c_int, c_int, c_void],
        "fllm_linear_add_normed": [c_void, c_int, c_void, c_void, c_void, c_int, c_int, c_int, c_void, c_void, c_void, c_void, c_void, c_void],
        "fllm_tile_weights": [c_void, c_void, c_int, c_int, c_void],
        "fllm_tile_weights_gate_up": [c_void, c_void, c_int, c_int, c_void],
        "fllm_gate_up_swiglu_tiled": [c_void, c_int, c_void, c_void, c_void, c_void, c_int, c_int, c_int, c_void],
        "fllm_linear_add_tiled": [c_void, c_int, c_void, c_void, c_void, c_void, c_int, c_int, c_int, c_int, c_void],
        "fllm_linear_f32_tiled": [c_void, c_int, c_void, c_void, c_void, c_void, c_int, c_int, c_int, c_int, c_void],
        "fllm_scaled_gate_up_swiglu": [c_void, c_void, c_int, c_float, c_void, c_void, c_void, c_int, c_int, c_int, c_void, c_void],
        "fllm_scaled_qkv_rope_store": [c_void, c_void, c_int, c_float, c_void, c_void, c_void, c_void, c_void, c_void, c_int, c_void,
                                       c_void, c_int, c_void, c_void, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void, c_void],
        "fllm_prepare_norm": [c_void, c_void, c_void, c_void, c_int, c_int, c_void],
        "fllm_carry_ids": [c_void, c_void, c_void, c_int, c_int, c_void],
        "fllm_sample": [c_void, c_void, c_void, c_void, c_int, c_int, c_int, c_void],
        "fllm_adjust_logits": [c_void, c_int, c_int, c_void, c_void, c_void, c_void],
        "fllm_logprobs": [c_void, c_int, c_int, c_void, c_int, c_void, c_int, c_void, c_void, c_void],
        "fllm_logprobs_processed": [c_void, c_int, c_int, c_void, c_int, c_void, c_void, c_int, c_void, c_void, c_void],
    }
    for name, args in sig.items():
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = c_int
    lib.fllm_fused_decode_supported.argtypes = [c_int, c_int]
    lib.fllm_fused_decode_supported.restype = c_int
    lib.fllm_set_option.argtypes = [ctypes.c_char_p, c_int]
    lib.fllm_set_option.restype = c_int
    lib.fllm_set_device_workspace.argtypes = [c_void, c_size]
    lib.fllm_set_device_workspace.restype = c_int
    lib.fllm_probe_read.argtypes = [c_void, c_size, c_void, c_int, c_void]
    lib.fllm_probe_read.restype = c_int
    lib.fllm_probe_mfma_bf16.argtypes = [c_void, c_int, c_int, c_void]
    lib.fllm_probe_mfma_bf16.restype = ctypes.c_double
    lib.fllm_random_fill.argtypes = [c_void, ctypes.c_uint64, ctypes.c_uint32, ctypes.c_uint32, c_int, c_int, c_void]
    lib.fllm_random_fill.restype = c_int
    lib.fllm_weight_tiles_supported.argtypes = [c_int, c_int]
    lib.fllm_weight_tiles_supported.restype = c_int
    lib.fllm_weight_tiles_elements.argtypes = [c_int, c_int]
    lib.fllm_weight_tiles_elements.restype = c_size
    lib.fllm_weight_tiles_elements_gate_up.argtypes = [c_int, c_int]
    lib.fllm_weight_tiles_elements_gate_up.restype = c_size
    lib.fllm_set_fast_kernels.argtypes = [c_int]
    lib.fllm_set_fast_kernels.restype = None
    lib.fllm_attention_workspace_bytes.argtypes = [c_int, c_int, c_int, c_int, c_int]
    lib.fllm_attention_workspace_bytes.restype = c_size
    _lib = lib
    return lib


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelError(msg)


def _dense(t: torch.Tensor, name: str, dtype=None, shape=None) -> None:
    # (every launch checks its operands: the messages are put together only when a check fails)
    if not t.is_cuda:
        raise KernelError(f"{name} must be on the GPU")
    if not t.is_contiguous():
        raise KernelError(f"{name} must be contiguous")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name} must be {dtype}, is {t.dtype}")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise KernelError(f"{name} must have shape {tuple(shape)}, has {tuple(t.shape)}")


class Ops:
    """Launches kernels on the current torch stream of the tensors' device.

    `library_gemm_from`: bfloat16 products of at least this many rows (prompt portions, large decode batches) go
    to the vendor's GEMM library through `torch.matmul`, as the reference sends its prompt-sized dense products
    to a library (rust/engine/cuda/cublaslt_gemm.cu:1-20).  None: every product runs the hand-written kernels.
    `fused_decode_rows`: up to this many rows a step uses the kernels that fold the norm, rotary, cache store and
    activation into the product (the kernels take up to 64 rows; beyond 16 the library products with separate small
    kernels are faster at the sizes measured)."""

    def __init__(self, library_gemm_from: Optional[int] = 17, fused_decode_rows: int = 16):
        if not torch.cuda.is_available():
            raise KernelError("no GPU is visible: the engine runs on gfx950 only")
        self.lib = load_library()
        self.library_gemm_from = library_gemm_from
        self.fused_decode_rows = int(fused_decode_rows)
        self._device_workspace(torch.cuda.current_device())

    _WORKSPACE_BYTES = 192 << 20
    _workspaces = {}         # device index -> tensor; lives as long as the process: the library keeps its address

    def _device_workspace(self, device: int) -> None:
        """Hands the library the memory in which workgroups of one kernel meet (counters, partial sums): once per device."""
        if device in Ops._workspaces:
            return
        with torch.cuda.device(device):
            buf = torch.zeros(Ops._WORKSPACE_BYTES, dtype=torch.uint8, device=f"cuda:{device}")
            torch.cuda.synchronize()
            self._check(self.lib.fllm_set_device_workspace(_ptr(buf), buf.numel()))
        Ops._workspaces[device] = buf

    # ---- tile-major copies of weights for decode steps --------------------------------------------------
    _tiles: Dict[int, Tuple[tuple, torch.Tensor]] = {}     # address of a weight matrix -> (its shape, its tile-major copy)

    def tile_for_decode(self, w: torch.Tensor, gate_up: bool = False) -> bool:
        """Keeps beside `w` (bfloat16 [N, K] on the GPU) a copy in the order in which the products of decode steps read
        it (`fllm_tile_weights`): `linear(..., accumulate=True)`, `linear_add_prepare`, the forms behind a prepared norm
        and `linear` with float32 logits find it by the matrix's address and use it for steps of up to 64 rows (sums into a
        float32 `out` and `gate_up_swiglu`: up to 128).  `gate_up`: w is [gate; up] and the copy holds 8 gate rows and the
        same 8 up rows a tile (`fllm_tile_weights_gate_up`), for `norm_gate_up_swiglu` and `gate_up_swiglu`.  The copy is
        given up with `w`.  False: nothing was made (another type or place, a shape the kernels do not take tiles of)."""
        if not (w.is_cuda and w.dtype == torch.bfloat16 and w.dim() == 2 and w.is_contiguous()):
            return False
        N, K = w.shape
        if not self.lib.fllm_weight_tiles_supported(N, K) or (gate_up and N % 2 != 0):
            return False
        key = w.data_ptr()
        kind = (N, K, bool(gate_up))
        if key in Ops._tiles and Ops._tiles[key][0] == kind:
            return True
        with torch.cuda.device(w.device):
            if gate_up:
                tiles = torch.empty(int(self.lib.fllm_weight_tiles_elements_gate_up(N // 2, K)), dtype=torch.bfloat16, device=w.device)
                self._check(self.lib.fllm_tile_weights_gate_up(_ptr(w), _ptr(tiles), N // 2, K, self._stream()))
            else:
                tiles = torch.empty(int(self.lib.fllm_weight_tiles_elements(N, K)), dtype=torch.bfloat16, device=w.device)
                self._check(self.lib.fllm_tile_weights(_ptr(w), _ptr(tiles), N, K, self._stream()))
        Ops._tiles[key] = (kind, tiles)
        weakref.finalize(w, Ops._tiles.pop, key, None)
        return True

    def _tiles_of(self, w: torch.Tensor, gate_up: bool = False) -> Optional[torch.Tensor]:
        held = Ops._tiles.get(w.data_ptr())
        return held[1] if held is not None and held[0] == (w.shape[0], w.shape[1], bool(gate_up)) else None

    # 17 to 128 rows beside the GEMM library: with the tile-major copies the own products of the feed-forward (gate/up
    # with its SwiGLU epilogue, down with the residual sum) are faster than the library's products and the SwiGLU kernel
    # (measured at the 8B sizes, 64 / 32 rows: gate/up 48 / 44 us against 55 / 53, down 34 / 28 against 40 / 31; at the 1B
    # sizes, 67 MB of gate and up weights, the library is 3 % of a 64-row step ahead, hence the same floor on the bytes
    # as for `prefers_own_gate_up`)
    def own_feed_forward(self, rows: int, w_gate_up: torch.Tensor, w_down: torch.Tensor) -> bool:
        """Whether a bfloat16 step of 17 to 128 rows whose products would go to the GEMM library should take
        `gate_up_swiglu` and `linear(..., accumulate=True)` for its feed-forward instead: when both matrices have their
        tile-major copies."""
        return (self.library_gemm_from is not None and self.library_gemm_from <= rows <= self.GATE_UP_SWIGLU_TILED_ROWS and bool(Ops._tiles)
                and (rows <= 64 or (w_gate_up.shape[1] % 256 == 0 and w_down.shape[1] % 256 == 0))
                and w_gate_up.numel() * w_gate_up.element_size() >= self.OWN_GATE_UP_BYTES
                and self._tiles_of(w_gate_up, gate_up=True) is not None and self._tiles_of(w_down) is not None)

    def set_fast_kernels(self, on: bool) -> None:
        """Off: bfloat16 calls run the plain kernels (tests compare the two)."""
        self.lib.fllm_set_fast_kernels(1 if on else 0)

    def set_option(self, name: str, value: int) -> None:
        """Switches a kernel variant, for measurements and for tests that compare variants."""
        self._check(self.lib.fllm_set_option(name.encode(), int(value)))

    def _check(self, code: int) -> None:
        if code != 0:
            raise KernelError(self.lib.fllm_last_error().decode("utf-8", "replace"))

    _streams = {}            # device index -> the stream on which this process launches the kernels of that device

    @staticmethod
    def _stream() -> int:
        """The current stream.  Kernels of one device meet in that device's workspace (counters that each launch leaves
        at zero, partial results behind them), so launches on one device must not overlap: all of them go to one stream
        (a stream that is capturing a graph stands for the stream the graph will be replayed on).  A launch on a second
        stream of the same device is refused."""
        raw = getattr(torch._C, "_cuda_getCurrentRawStream", None)
        if raw is not None:               # the handle without a Stream object around it (a launch asks for it every time)
            device = torch.cuda.current_device()
            handle = raw(device)
        else:
            stream = torch.cuda.current_stream()
            handle, device = stream.cuda_stream, stream.device_index
        seen = Ops._streams.get(device)
        if seen is None:
            if not torch.cuda.is_current_stream_capturing():
                Ops._streams[device] = handle
        elif handle != seen and not torch.cuda.is_current_stream_capturing():
            raise KernelError(f"kernels of device {device} were launched on stream {seen:#x} before and are now asked for on "
                              f"stream {handle:#x}: they share the device workspace and must stay on one stream")
        return handle

    def random_fill(self, out: torch.Tensor, key, kind: int) -> torch.Tensor:
        """Fills `out` with the random tensor of `key` (two 32-bit words): kind 0 normal numbers of deviation 0.02, kind 1
        norm weights; the generator of `fllm_amd.weights.random_init`."""
        _dense(out, "out")
        _need(out.dtype in _DTYPE_CODE, f"out dtype {out.dtype} unsupported")
        with torch.cuda.device(out.device):
            self._check(self.lib.fllm_random_fill(_ptr(out), out.numel(), int(key[0]), int(key[1]), int(kind),
                                                  _DTYPE_CODE[out.dtype], self._stream()))
        return out

    def embed(self, ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
        rows = ids.numel()
        vocab, width = table.shape
        _dense(ids, "ids", torch.int32)
        _dense(table, "table")
        _need(table.dtype in _DTYPE_CODE, f"table dtype {table.dtype} unsupported")
        _dense(out, "out", torch.float32, (rows, width))
        self._check(self.lib.fllm_embed(_ptr(ids), _ptr(table), _ptr(out), rows, width, vocab, _DTYPE_CODE[table.dtype],
                                        float(scale), self._stream()))
        return out

    def rmsnorm(self, x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor,
                rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        width = x.shape[-1]
        _dense(x, "x", torch.float32)
        _dense(weight, "weight", torch.float32, (width,))
        count = x.shape[0] if rows is None else rows.numel()
        if rows is not None:
            _dense(rows, "rows", torch.int32)
        _dense(out, "out", None, (count, width))
        _need(out.dtype in _DTYPE_CODE, f"out dtype {out.dtype} unsupported")
        self._check(self.lib.fllm_rmsnorm(_ptr(x), _ptr(rows), _ptr(weight), _ptr(out), count, width, float(eps),
                                          _DTYPE_CODE[out.dtype], self._stream()))
        return out

    def add_rmsnorm(self, x: torch.Tensor, branch: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor) -> torch.Tensor:
        """x += branch (float32 sum, in place), out = rmsnorm(x): the residual add and the norm after it in one pass."""
        rows, width = x.shape
        _dense(x, "x", torch.float32)
        _dense(branch, "branch", None, (rows, width))
        _need(branch.dtype in _DTYPE_CODE, f"branch dtype {branch.dtype} unsupported")
        _dense(weight, "weight", torch.float32, (width,))
        _dense(out, "out", None, (rows, width))
        _need(out.dtype in _DTYPE_CODE, f"out dtype {out.dtype} unsupported")
        self._check(self.lib.fllm_add_rmsnorm(_ptr(x), _ptr(branch), _DTYPE_CODE[branch.dtype], _ptr(weight), _ptr(out), rows,
                                              width, float(eps), _DTYPE_CODE[out.dtype], self._stream()))
        return out

    def linear(self, x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, bias: Optional[torch.Tensor] = None,
               accumulate: bool = False) -> torch.Tensor:
        """out = x @ w.T (+ bias); `accumulate` adds into a float32 `out` instead of storing."""
        _need(x.dim() == 2 and w.dim() == 2 and out.dim() == 2, "linear takes matrices")
        M, K = x.shape
        N = w.shape[0]
        _need(w.shape[1] == K, f"w has {w.shape[1]} columns, x has {K}")
        _need(x.is_cuda and w.is_cuda and out.is_cuda, "linear operands must be on the GPU")
        _need(x.dtype == w.dtype and x.dtype in _DTYPE_CODE, f"x is {x.dtype}, w is {w.dtype}")
        _need(x.stride(1) == 1 and out.stride(1) == 1 and w.is_contiguous(), "linear operands must be row-major")
        _need(tuple(out.shape) == (M, N), f"out must have shape {(M, N)}, has {tuple(out.shape)}")
        if accumulate:
            _need(out.dtype == torch.float32, "accumulate needs a float32 out")
            mode = OUT_ADD_F32
        elif out.dtype == x.dtype:
            mode = OUT_STORE
        else:
            _need(out.dtype == torch.float32, f"out must be {x.dtype} or float32")
            mode = OUT_STORE_F32
        if bias is not None:
            _dense(bias, "bias", torch.float32, (N,))
        ldx = x.stride(0) if M > 1 else K
        ldo = out.stride(0) if M > 1 else N
        tiles = (self._tiles_of(w) if Ops._tiles and ((mode == OUT_ADD_F32 and M <= self.ADD_KERNEL_ROWS) or (mode == OUT_STORE_F32 and M <= 64))
                 else None)
        if tiles is not None and ldx % 8 == 0 and K % 8 == 0 and (M <= 64 or K % 256 == 0):
            entry = self.lib.fllm_linear_add_tiled if mode == OUT_ADD_F32 else self.lib.fllm_linear_f32_tiled
            self._check(entry(_ptr(x), ldx, _ptr(w), _ptr(tiles), _ptr(bias), _ptr(out), ldo, M, N, K, self._stream()))
            return out
        if (self.library_gemm_from is not None and M >= self.library_gemm_from and x.dtype == torch.bfloat16
                and bias is None):
            if mode == OUT_STORE:
                torch.matmul(x, w.t(), out=out)
            elif mode == OUT_STORE_F32:
                torch.mm(x, w.t(), out_dtype=torch.float32, out=out)     # bfloat16 operands, float32 sums stored as they are
            else:
                self.add_residual(out, torch.matmul(x, w.t()))
            return out
        self._check(self.lib.fllm_linear(_ptr(x), ldx, _ptr(w), _ptr(bias), _ptr(out), ldo, M, N, K, _DTYPE_CODE[x.dtype],
                                         mode, self._stream()))
        return out

    # ---- fused forms of decode steps (bfloat16, at most 64 rows) ---------------------------------
    def fused_decode_supported(self, rows: int, width: int) -> bool:
        """Whether a step of `rows` rows should take the fused forms: the kernels can (1..64 rows, widths in steps of 8)
        and `fused_decode_rows` lets them."""
        return rows <= self.fused_decode_rows and self._fused_kernels_take(rows, width)

    def _fused_kernels_take(self, rows: int, width: int) -> bool:
        return bool(self.lib.fllm_fused_decode_supported(int(rows), int(width)))

    def _fused_operands(self, x, norm_weight, w, bias, n_rows_w):
        M, K = x.shape
        _dense(x, "x", torch.float32)
        _dense(norm_weight, "norm_weight", torch.float32, (K,))
        _dense(w, "w", torch.bfloat16, (n_rows_w, K))
        if bias is not None:
            _dense(bias, "bias", torch.float32, (n_rows_w,))
        _need(self._fused_kernels_take(M, K), f"the fused decode kernels take 1..64 rows and widths in steps of 8, not {M} x {K}")
        return M, K

    def norm_linear(self, x, norm_weight, eps, w, out, bias=None):
        """out = rmsnorm(x) @ w.T (+ bias); x float32 [M, K], w bfloat16 [N, K], out bfloat16 [M, N]."""
        N = w.shape[0]
        M, K = self._fused_operands(x, norm_weight, w, bias, N)
        _dense(out, "out", torch.bfloat16, (M, N))
        self._check(self.lib.fllm_norm_linear(_ptr(x), _ptr(norm_weight), float(eps), _ptr(w), _ptr(bias), _ptr(out), M, N, K,
                                              self._stream()))
        return out

    PREPARED_NORM_ROWS = 16
    CHUNK_KERNEL_ROWS = 64   # what those kernels take behind a prepared norm
    ADD_KERNEL_ROWS = 128    # and as sums into the residual stream or with the SwiGLU epilogue (beyond 64 rows from the tile-major
                             # copies only): the feed-forward of steps of up to 128 rows, whose down projection the GEMM library
                             # runs on half of the device (96 / 128 rows of the 8B sizes: 39 / 53 us against 63 / 75)
    CHUNK_ROWS = 48          # steps of 17 to this many rows take the fused forms of the kernels that pass the activations through
                             # LDS in chunks (measured at the 8B sizes: 4 to 5 % of a step at 17 and 32 rows, 1 % at 48; from 49
                             # rows on the library's q/k/v and output products beside the own feed-forward are 1 % faster)

    def fused_form(self, rows: int, width: int, w: torch.Tensor, gate_up: bool = False) -> Optional[str]:
        """Which fused kernels serve a product of `rows` rows with the matrix `w` behind an RMSNorm of `width`:
        "resident" (up to `fused_decode_rows` rows), "chunks" (17 to 64 rows: they need the norm prepared, by
        `linear_add_prepare` or `prepare_norm`, and the tile-major copy of `w`) or None."""
        if self.fused_decode_supported(rows, width):
            return "resident"
        if (self.fused_decode_rows < rows <= self.CHUNK_ROWS and (self.library_gemm_from is None or rows >= self.library_gemm_from)
                and self.fused_decode_rows >= self.PREPARED_NORM_ROWS and width % 256 == 0 and Ops._tiles
                and self._tiles_of(w, gate_up=gate_up) is not None):
            return "chunks"
        return None

    def prepares_norm(self, rows: int, width: int, w: Optional[torch.Tensor] = None) -> bool:
        """Whether `linear_add_prepare` serves a sum into a residual stream of this size: the fused forms are in use,
        up to 16 rows, or up to 64 with the tile-major copy of the matrix `w`; widths in steps of 16."""
        if width % 16 != 0:
            return False
        if rows <= self.PREPARED_NORM_ROWS:
            return self.fused_decode_supported(rows, width)
        return w is not None and self.fused_form(rows, w.shape[1], w) == "chunks"      # the product's own width counts

    def prepare_norm(self, x: torch.Tensor, norm_weight: torch.Tensor) -> PreparedNorm:
        """What `linear_add_prepare` leaves for an RMSNorm, from float32 rows that no such product wrote (a model's first
        layer): the rows times the norm's weight in bfloat16 and each row's sum of squares as one part."""
        M, K = x.shape
        _dense(x, "x", torch.float32)
        _dense(norm_weight, "norm_weight", torch.float32, (K,))
        xn = torch.empty((M, K), dtype=torch.bfloat16, device=x.device)
        ssq = torch.empty((M,), dtype=torch.float32, device=x.device)
        self._check(self.lib.fllm_prepare_norm(_ptr(x), _ptr(norm_weight), _ptr(xn), _ptr(ssq), M, K, self._stream()))
        return PreparedNorm(xn, ssq, 1)

    def linear_add_prepare(self, x, w, residual, next_norm_weight, bias=None) -> PreparedNorm:
        """residual += x @ w.T (+ bias) as `linear(..., accumulate=True)` does, and in the same kernel what the RMSNorm
        with weight `next_norm_weight` that reads `residual` next would compute first (fllm_linear_add_normed): hand the
        result to `norm_gate_up_swiglu` / `norm_qkv_rope_store` as `prepared`.  x bfloat16 [M <= 64, K], w bfloat16 [N, K],
        residual float32 [M, N], N a multiple of 16."""
        M, K = x.shape
        N = w.shape[0]
        _need(x.is_cuda and x.dtype == torch.bfloat16 and x.dim() == 2 and x.stride(1) == 1, "x must be bfloat16 rows on the GPU")
        _dense(w, "w", torch.bfloat16, (N, K))
        _dense(residual, "residual", torch.float32, (M, N))
        _dense(next_norm_weight, "next_norm_weight", torch.float32, (N,))
        if bias is not None:
            _dense(bias, "bias", torch.float32, (N,))
        _need(1 <= M <= self.ADD_KERNEL_ROWS and N % 16 == 0 and K % 8 == 0,
              f"linear_add_prepare takes 1..128 rows, N in steps of 16 and K in steps of 8, not {M} x {N} x {K}")
        xn = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
        ssq = torch.empty((M * (N // 8),), dtype=torch.float32, device=x.device)
        parts = ctypes.c_int(0)
        self._check(self.lib.fllm_linear_add_normed(_ptr(x), x.stride(0) if M > 1 else K, _ptr(w), _ptr(bias), _ptr(residual), M, N,
                                                    K, _ptr(next_norm_weight), _ptr(xn), _ptr(ssq), ctypes.addressof(parts),
                                                    _ptr(self._tiles_of(w)) if Ops._tiles else None, self._stream()))
        return PreparedNorm(xn, ssq, int(parts.value))

    def _prepared_operands(self, prepared: PreparedNorm, w, bias, n_rows_w):
        M, K = prepared.x.shape
        _dense(prepared.x, "prepared.x", torch.bfloat16)
        _dense(prepared.ssq, "prepared.ssq", torch.float32)
        _need(prepared.parts >= 1 and prepared.ssq.numel() >= M * prepared.parts, "prepared.ssq is shorter than rows x parts")
        _dense(w, "w", torch.bfloat16, (n_rows_w, K))
        if bias is not None:
            _dense(bias, "bias", torch.float32, (n_rows_w,))
        _need(1 <= M <= self.CHUNK_KERNEL_ROWS and K % 8 == 0, f"a prepared norm serves 1..64 rows and widths in steps of 8, not {M} x {K}")
        return M, K

    def _chunk_tiles(self, M: int, K: int, w: torch.Tensor, gate_up: bool = False) -> Optional[torch.Tensor]:
        """The tile-major copy that a prepared norm of more than 16 rows needs; up to 16 rows the kernel streams it
        where there is one and the launch it chooses can."""
        tiles = self._tiles_of(w, gate_up=gate_up) if Ops._tiles else None
        if M <= self.PREPARED_NORM_ROWS:
            return tiles
        _need(tiles is not None and K % 256 == 0,
              f"a prepared norm of {M} rows needs the tile-major copy of the matrix (tile_for_decode) and a width in steps of 256, not {K}")
        return tiles

    def norm_gate_up_swiglu(self, x, norm_weight, eps, w_gate_up, out, bias=None, prepared: Optional[PreparedNorm] = None):
        """out = silu(rmsnorm(x) @ gate.T) * (rmsnorm(x) @ up.T); w_gate_up = [gate; up], out bfloat16 [M, I].
        `prepared`: what `linear_add_prepare` left for this norm, in place of x and norm_weight."""
        two_i = w_gate_up.shape[0]
        _need(two_i % 2 == 0, "w_gate_up needs an even number of rows")
        if prepared is not None:
            M, K = self._prepared_operands(prepared, w_gate_up, bias, two_i)
            _dense(out, "out", torch.bfloat16, (M, two_i // 2))
            self._check(self.lib.fllm_scaled_gate_up_swiglu(_ptr(prepared.x), _ptr(prepared.ssq), prepared.parts, float(eps),
                                                            _ptr(w_gate_up), _ptr(bias), _ptr(out), M, two_i // 2, K,
                                                            _ptr(self._chunk_tiles(M, K, w_gate_up, gate_up=True)), self._stream()))
            return out
        M, K = self._fused_operands(x, norm_weight, w_gate_up, bias, two_i)
        _dense(out, "out", torch.bfloat16, (M, two_i // 2))
        self._check(self.lib.fllm_norm_gate_up_swiglu(_ptr(x), _ptr(norm_weight), float(eps), _ptr(w_gate_up), _ptr(bias),
                                                      _ptr(out), M, two_i // 2, K, self._stream()))
        return out

    GATE_UP_SWIGLU_ROWS = 64          # from the matrix as the checkpoint has it
    GATE_UP_SWIGLU_TILED_ROWS = 128   # from its tile-major copy, widths in steps of 256
    # Beside the GEMM library: up to this many rows, and from this many bytes of gate and up weights on, the own
    # product with the SwiGLU epilogue is faster than the library's product and a SwiGLU kernel behind it (measured at
    # 17 and 32 rows: 6.5 and 4.6 us a layer at 235 MB of weights; slower at 64 rows, and at 67 MB of weights).
    OWN_GATE_UP_ROWS = 32
    OWN_GATE_UP_BYTES = 128 << 20

    def prefers_own_gate_up(self, rows: int, w_gate_up: torch.Tensor) -> bool:
        """Whether a bfloat16 step of `rows` rows whose products go to the GEMM library should still take
        `gate_up_swiglu` for its gate/up product."""
        return (self.library_gemm_from is not None and self.library_gemm_from <= rows <= self.OWN_GATE_UP_ROWS
                and w_gate_up.numel() * w_gate_up.element_size() >= self.OWN_GATE_UP_BYTES)

    def gate_up_swiglu(self, x, w_gate_up, out, bias=None):
        """out = silu(x @ gate.T) * (x @ up.T) for up to 64 bfloat16 rows, up to 128 with the tile-major copy of w_gate_up
        ([gate; up]); out bfloat16 [M, I]."""
        M, K = x.shape
        two_i = w_gate_up.shape[0]
        _need(two_i % 2 == 0, "w_gate_up needs an even number of rows")
        _need(x.dtype == torch.bfloat16 and x.is_cuda and x.stride(1) == 1, "x must be bfloat16 rows on the GPU")
        _dense(w_gate_up, "w_gate_up", torch.bfloat16, (two_i, K))
        if bias is not None:
            _dense(bias, "bias", torch.float32, (two_i,))
        _dense(out, "out", torch.bfloat16, (M, two_i // 2))
        _need(1 <= M <= self.GATE_UP_SWIGLU_TILED_ROWS and K % 8 == 0, f"gate_up_swiglu takes 1..128 rows and widths in steps of 8, not {M} x {K}")
        tiles = self._tiles_of(w_gate_up, gate_up=True) if M >= 17 and Ops._tiles else None
        _need(M <= 64 or (tiles is not None and K % 256 == 0 and x.stride(0) % 8 == 0),
              f"gate_up_swiglu takes more than 64 rows only with the tile-major copy of the matrix and widths in steps of 256, not {M} x {K}")
        if tiles is not None and x.stride(0) % 8 == 0:
            self._check(self.lib.fllm_gate_up_swiglu_tiled(_ptr(x), x.stride(0), _ptr(w_gate_up), _ptr(tiles), _ptr(bias), _ptr(out), M,
                                                           two_i // 2, K, self._stream()))
            return out
        self._check(self.lib.fllm_gate_up_swiglu(_ptr(x), x.stride(0) if M > 1 else K, _ptr(w_gate_up), _ptr(bias), _ptr(out), M,
                                                 two_i // 2, K, self._stream()))
        return out

    def norm_qkv_rope_store(self, x, norm_weight, eps, w_qkv, q_out, row_pos, row_seg, tables, cos, sin, k_pages, v_pages,
                            heads, kv_heads, head_dim, rope_dims, page_size, bias=None, prepared: Optional[PreparedNorm] = None):
        """q, k, v = rmsnorm(x) @ w_qkv.T; rotary on pairs (2l, 2l+1) of q and k; q to `q_out`
        (bfloat16 [M, heads * head_dim]), k and v into the pages (None: not stored).
        `prepared`: what `linear_add_prepare` left for this norm, in place of x and norm_weight."""
        if prepared is not None:
            M, K = self._prepared_operands(prepared, w_qkv, bias, (heads + 2 * kv_heads) * head_dim)
        else:
            M, K = self._fused_operands(x, norm_weight, w_qkv, bias, (heads + 2 * kv_heads) * head_dim)
        _dense(q_out, "q_out", torch.bfloat16, (M, heads * head_dim))
        _dense(row_pos, "row_pos", torch.int32, (M,))
        _dense(row_seg, "row_seg", torch.int32, (M,))
        _dense(tables, "tables", torch.int32)
        _need(tables.dim() == 2, "tables must be [segments, pages]")
        _dense(cos, "cos", torch.float32)
        _dense(sin, "sin", torch.float32, tuple(cos.shape))
        _need(cos.dim() == 2 and cos.shape[1] == rope_dims // 2, f"rotary tables must be [positions, {rope_dims // 2}]")
        store = k_pages is not None
        if store:
            pages = k_pages.shape[0]
            _dense(k_pages, "k_pages", torch.bfloat16, (pages, kv_heads, head_dim // 8, page_size, 8))
            _dense(v_pages, "v_pages", torch.bfloat16, (pages, kv_heads, head_dim, page_size))
        if prepared is not None:
            self._check(self.lib.fllm_scaled_qkv_rope_store(
                _ptr(prepared.x), _ptr(prepared.ssq), prepared.parts, float(eps), _ptr(w_qkv), _ptr(bias), _ptr(q_out), _ptr(row_pos),
                _ptr(row_seg), _ptr(tables), tables.shape[1], _ptr(cos), _ptr(sin), rope_dims, _ptr(k_pages), _ptr(v_pages), M, heads,
                kv_heads, head_dim, K, page_size, 1 if store else 0, _ptr(self._chunk_tiles(M, K, w_qkv)), self._stream()))
            return q_out
        self._check(self.lib.fllm_norm_qkv_rope_store(
            _ptr(x), _ptr(norm_weight), float(eps), _ptr(w_qkv), _ptr(bias), _ptr(q_out), _ptr(row_pos), _ptr(row_seg),
            _ptr(tables), tables.shape[1], _ptr(cos), _ptr(sin), rope_dims, _ptr(k_pages), _ptr(v_pages), M, heads, kv_heads,
            head_dim, K, page_size, 1 if store else 0, self._stream()))
        return q_out

    def add_residual(self, residual: torch.Tensor, branch: torch.Tensor) -> torch.Tensor:
        """residual += branch, summed in float32."""
        _dense(residual, "residual", torch.float32)
        _dense(branch, "branch", None, tuple(residual.shape))
        _need(branch.dtype in _DTYPE_CODE and residual.dim() == 2, "add_residual takes matrices of float32 / bfloat16")
        self._check(self.lib.fllm_add_residual(_ptr(residual), _ptr(branch), residual.shape[0], residual.shape[1],
                                               _DTYPE_CODE[branch.dtype], self._stream()))
        return residual

    def swiglu(self, gate_up: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
        rows, two_i = gate_up.shape
        _need(two_i % 2 == 0, "gate_up needs an even width")
        _dense(gate_up, "gate_up")
        _need(gate_up.dtype in _DTYPE_CODE, f"dtype {gate_up.dtype} unsupported")
        _dense(out, "out", gate_up.dtype, (rows, two_i // 2))
        self._check(self.lib.fllm_swiglu(_ptr(gate_up), _ptr(out), rows, two_i // 2, _DTYPE_CODE[gate_up.dtype],
                                         self._stream()))
        return out

    def rope_kv_store(self, qkv: torch.Tensor, row_pos: torch.Tensor, row_seg: torch.Tensor, tables: torch.Tensor,
                      cos: torch.Tensor, sin: torch.Tensor, k_pages: Optional[torch.Tensor],
                      v_pages: Optional[torch.Tensor], heads: int, kv_heads: int, head_dim: int, rope_dims: int,
                      pairing: int, page_size: int) -> None:
        rows = qkv.shape[0]
        _dense(qkv, "qkv", None, (rows, (heads + 2 * kv_heads) * head_dim))
        _need(qkv.dtype in _DTYPE_CODE, f"dtype {qkv.dtype} unsupported")
        _dense(row_pos, "row_pos", torch.int32, (rows,))
        _dense(row_seg, "row_seg", torch.int32, (rows,))
        _dense(tables, "tables", torch.int32)
        _need(tables.dim() == 2, "tables must be [segments, pages]")
        half = rope_dims // 2
        _dense(cos, "cos", torch.float32)
        _dense(sin, "sin", torch.float32, tuple(cos.shape))
        _need(cos.dim() == 2 and cos.shape[1] == half, f"rotary tables must be [positions, {half}]")
        store = k_pages is not None
        num_pages = 0
        _need(head_dim % 8 == 0, f"head size {head_dim}: keys are stored in chunks of 8 values")
        if store:
            num_pages = k_pages.shape[0]
            _dense(k_pages, "k_pages", qkv.dtype, (num_pages, kv_heads, head_dim // 8, page_size, 8))
            _dense(v_pages, "v_pages", qkv.dtype, (num_pages, kv_heads, head_dim, page_size))
        self._check(self.lib.fllm_rope_kv_store(
            _ptr(qkv), _ptr(row_pos), _ptr(row_seg), _ptr(tables), tables.shape[1], _ptr(cos), _ptr(sin), cos.shape[0],
            _ptr(k_pages), _ptr(v_pages), num_pages, rows, heads, kv_heads, head_dim, rope_dims, pairing, page_size,
            _DTYPE_CODE[qkv.dtype], 1 if store else 0, self._stream()))

    def attention_workspace_bytes(self, rows: int, heads: int, kv_heads: int, head_dim: int, max_context: int) -> int:
        return int(self.lib.fllm_attention_workspace_bytes(rows, heads, kv_heads, head_dim, max_context))

    def attention(self, q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, tables: torch.Tensor,
                  row_pos: torch.Tensor, row_seg: torch.Tensor, seg_start: torch.Tensor, out: torch.Tensor, heads: int, kv_heads: int,
                  head_dim: int, page_size: int, scale: float, window: Optional[int], max_context: int,
                  uniform_rows: int = 0, workspace: Optional[torch.Tensor] = None, single_from: Optional[int] = None,
                  head_slopes: Optional[torch.Tensor] = None) -> torch.Tensor:
        """`q` may be a column slice of a wider row-major matrix (the fused qkv buffer).
        `max_context` bounds pos + 1 over the rows; the segments from `single_from` on have one row each
        (`uniform_rows` = 1 is `single_from` = 0: a decode step; by default no segment is known to).
        `head_slopes` (float32 [heads]): every score gets head_slopes[head] * (key position - row position) added, for
        position encodings that bias scores; such a call runs the plain kernel in both precisions."""
        rows = q.shape[0]
        _need(q.is_cuda and q.dim() == 2 and q.stride(1) == 1 and q.shape[1] == heads * head_dim,
              f"q must be [rows, {heads * head_dim}] with unit column stride")
        _need(q.dtype in _DTYPE_CODE, f"dtype {q.dtype} unsupported")
        num_pages = k_pages.shape[0]
        _dense(k_pages, "k_pages", q.dtype, (num_pages, kv_heads, head_dim // 8, page_size, 8))
        _dense(v_pages, "v_pages", q.dtype, (num_pages, kv_heads, head_dim, page_size))
        _dense(tables, "tables", torch.int32)
        _need(tables.dim() == 2, "tables must be [segments, pages]")
        _dense(row_pos, "row_pos", torch.int32, (rows,))
        _dense(row_seg, "row_seg", torch.int32, (rows,))
        _dense(seg_start, "seg_start", torch.int32)
        _need(seg_start.numel() >= 2, "seg_start must hold at least one segment")
        _need(tables.shape[0] >= seg_start.numel() - 1, "tables must have a row per segment")
        _dense(out, "out", q.dtype, (rows, heads * head_dim))
        ws_ptr, ws_bytes = None, 0
        if workspace is not None:
            _need(workspace.is_cuda and workspace.is_contiguous(), "workspace must be a dense GPU tensor")
            ws_ptr, ws_bytes = workspace.data_ptr(), workspace.numel() * workspace.element_size()
        q_stride = q.stride(0) if rows > 1 else heads * head_dim
        num_segs = seg_start.numel() - 1
        if head_slopes is not None:
            _dense(head_slopes, "head_slopes", torch.float32, (heads,))
            self._check(self.lib.fllm_attention_sloped(
                _ptr(q), q_stride, _ptr(k_pages), _ptr(v_pages), _ptr(tables), tables.shape[1], _ptr(row_pos), _ptr(row_seg),
                _ptr(seg_start), num_segs, _ptr(out), rows, heads, kv_heads, head_dim, page_size, num_pages, float(scale),
                int(window) if window else 0, _DTYPE_CODE[q.dtype], int(max_context), _ptr(head_slopes), self._stream()))
            return out
        if single_from is None:
            single_from = 0 if uniform_rows else num_segs
        _need(0 <= single_from <= num_segs and num_segs - single_from <= rows, f"single_from {single_from} does not fit {num_segs} segments of {rows} rows")
        self._check(self.lib.fllm_attention(
            _ptr(q), q_stride, _ptr(k_pages), _ptr(v_pages), _ptr(tables), tables.shape[1], _ptr(row_pos), _ptr(row_seg),
            _ptr(seg_start), seg_start.numel() - 1, _ptr(out), rows, heads, kv_heads, head_dim, page_size, num_pages, float(scale),
            int(window) if window else 0, _DTYPE_CODE[q.dtype], int(max_context), int(single_from), ws_ptr, ws_bytes,
            self._stream()))
        return out

    def measured_ceilings(self, read_bytes: int = 4 << 30, repeats: int = 5) -> dict:
        """What the device delivers to kernels that do nothing else: GB/s of a kernel that only reads a buffer much larger
        than the caches, TFLOP/s of a kernel that only issues bfloat16 MFMA products.  The best of `repeats` timings."""
        dev = torch.device("cuda", torch.cuda.current_device())
        props = torch.cuda.get_device_properties(dev)
        blocks = props.multi_processor_count * 8
        buf = torch.zeros(read_bytes, dtype=torch.uint8, device=dev)
        sink = torch.zeros(max(blocks, 2 * props.multi_processor_count * 512), dtype=torch.float32, device=dev)
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        best_read, best_mfma = 0.0, 0.0
        iters, mfma_blocks = 4096, 2 * props.multi_processor_count
        for _ in range(repeats + 1):
            start.record()
            self._check(self.lib.fllm_probe_read(_ptr(buf), buf.numel(), _ptr(sink), blocks, self._stream()))
            end.record()
            end.synchronize()
            best_read = max(best_read, buf.numel() / (start.elapsed_time(end) * 1e-3) / 1e9)
            start.record()
            flops = self.lib.fllm_probe_mfma_bf16(_ptr(sink), mfma_blocks, iters, self._stream())
            end.record()
            end.synchronize()
            if flops < 0:
                raise KernelError(self.lib.fllm_last_error().decode("utf-8", "replace"))
            best_mfma = max(best_mfma, flops / (start.elapsed_time(end) * 1e-3) / 1e12)
        return {"hbm_read_gbs": best_read, "mfma_bf16_tflops": best_mfma}

    def carry_ids(self, ids: torch.Tensor, source: torch.Tensor, previous: torch.Tensor) -> torch.Tensor:
        """ids[r] = previous[source[r]] where source[r] >= 0 (int32 device tensors): tokens an earlier step chose
        become this step's input without passing through the host."""
        rows = ids.numel()
        _dense(ids, "ids", torch.int32)
        _dense(source, "source", torch.int32, (rows,))
        _dense(previous, "previous", torch.int32)
        self._check(self.lib.fllm_carry_ids(_ptr(ids), _ptr(source), _ptr(previous), rows, previous.numel(), self._stream()))
        return ids

    def argmax(self, logits: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
        rows, vocab = logits.shape
        _dense(logits, "logits", torch.float32)
        _dense(out, "out", torch.int32, (rows,))
        self._check(self.lib.fllm_argmax(_ptr(logits), _ptr(out), rows, vocab, self._stream()))
        return out

    def adjust_logits(self, logits: torch.Tensor, packed: torch.Tensor, sections: Sequence[int],
                      last_tokens: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Penalties, biases, blocked and allowed ids on float32 logits [rows, vocab], in place (fllm_adjust_logits).
        `packed`: one int32 device tensor holding, one behind the other, the row records (14 words a row: the three
        penalties as float bits, then seen_off, seen_len, bias_off, bias_len, blocked_off, blocked_len, last_row,
        allowed_off, allowed_len, pairs_off, pairs_len), the seen ids, the seen counts, the bias ids, the bias values
        (float bits), the blocked ids, the allowed ids (rising within a row) and the pairs (first all "if the newest
        token is" ids, then all "block" ids); `sections`: (entries of the seen lists, of the bias lists, blocked ids,
        allowed ids, pairs), each over all rows.
        `last_tokens`: int32 device tensor that the records' last_row points into."""
        rows, vocab = logits.shape
        seen, bias, blocked, allowed, pairs = (int(n) for n in sections)
        _dense(logits, "logits", torch.float32)
        _dense(packed, "packed", torch.int32, (rows * ADJUST_ROW_WORDS + 2 * seen + 2 * bias + blocked + allowed + 2 * pairs,))
        if last_tokens is not None:
            _dense(last_tokens, "last_tokens", torch.int32)
        base = packed.data_ptr()
        at = rows * ADJUST_ROW_WORDS
        lists = AdjustLists()
        for name, count in (("seen_ids", seen), ("seen_counts", seen), ("bias_ids", bias), ("bias_values", bias),
                            ("blocked_ids", blocked), ("allowed_ids", allowed), ("if_last", pairs), ("then_blocked", pairs)):
            setattr(lists, name, base + 4 * at)
            at += count
        self._check(self.lib.fllm_adjust_logits(_ptr(logits), rows, vocab, base, ctypes.byref(lists), _ptr(last_tokens), self._stream()))
        return logits

    def logprobs(self, logits: torch.Tensor, wanted_rows: torch.Tensor, tokens: torch.Tensor, top: int,
                 values: torch.Tensor, ids: torch.Tensor) -> None:
        """Log-probabilities in the softmax of float32 logits [rows, vocab] (fllm_logprobs): for each row named in
        `wanted_rows` (int32 on the device, every one inside [0, rows): the caller's word), `values[w, 0]` is that of
        `tokens[row]` and `values[w, 1:]`, `ids[w, 1:]` are the `top` likeliest tokens, the lower id first among equals;
        `ids[w, 0]` repeats the chosen token.  A row with a NaN or +inf, or without a finite value, gives NaN."""
        rows, vocab = logits.shape
        wanted = wanted_rows.numel()
        _dense(logits, "logits", torch.float32)
        _dense(wanted_rows, "wanted_rows", torch.int32, (wanted,))
        _dense(tokens, "tokens", torch.int32, (rows,))
        _dense(values, "values", torch.float32, (wanted, 1 + top))
        _dense(ids, "ids", torch.int32, (wanted, 1 + top))
        self._check(self.lib.fllm_logprobs(_ptr(logits), rows, vocab, _ptr(wanted_rows), wanted, _ptr(tokens), int(top),
                                           _ptr(values), _ptr(ids), self._stream()))

    def logprobs_processed(self, logits: torch.Tensor, wanted_rows: torch.Tensor, tokens: torch.Tensor, params: torch.Tensor,
                           top: int, values: torch.Tensor, ids: torch.Tensor) -> None:
        """As `logprobs`, in the distribution each token was drawn from (fllm_logprobs_processed): `logits` are what the
        sampler saw (penalties and biases applied), `params` the `SampleRow` records `sample` took (uint8 [rows, 32]):
        temperature, then top-k, min-p and top-p with the sampler's ties; a greedy row is a point mass.  A chosen token
        that the filters leave out gives -inf; where fewer than `top` tokens are left, the rest of `ids` is -1."""
        rows, vocab = logits.shape
        wanted = wanted_rows.numel()
        _dense(logits, "logits", torch.float32)
        _dense(wanted_rows, "wanted_rows", torch.int32, (wanted,))
        _dense(tokens, "tokens", torch.int32, (rows,))
        _dense(params, "params", torch.uint8, (rows, SAMPLE_ROW_BYTES))
        _dense(values, "values", torch.float32, (wanted, 1 + top))
        _dense(ids, "ids", torch.int32, (wanted, 1 + top))
        self._check(self.lib.fllm_logprobs_processed(_ptr(logits), rows, vocab, _ptr(wanted_rows), wanted, _ptr(tokens), _ptr(params),
                                                     int(top), _ptr(values), _ptr(ids), self._stream()))

    def sample(self, logits: torch.Tensor, work: torch.Tensor, params: torch.Tensor, out: torch.Tensor,
               kinds: int = 7) -> torch.Tensor:
        """`params`: uint8 GPU tensor [rows, 32] holding `SampleRow` records.  `kinds`: what the caller knows of the rows,
        a sum of 1 (some have a temperature and no filter: their draw looks at every token, and several workgroups
        share such a row), 2 (some are of another kind) and 4 (some of those have a top-k of at most 64: several
        workgroups share such a row as well); 7 when nothing is known."""
        rows, vocab = logits.shape
        _dense(logits, "logits", torch.float32)
        _dense(work, "work", torch.float32, (rows, vocab))
        _dense(params, "params", torch.uint8, (rows, SAMPLE_ROW_BYTES))
        _dense(out, "out", torch.int32, (rows,))
        self._check(self.lib.fllm_sample(_ptr(logits), _ptr(work), _ptr(params), _ptr(out), rows, vocab, int(kinds), self._stream()))
        return out
