"""The argmax entry point that allocates nothing (`fllm_argmax_static`): called through ctypes, twice in a row, the
second time with a smaller input, and compared with `fllm_argmax` on the same logits."""
import ctypes

import pytest
import torch

from fllm_amd.kernels import Ops, build

pytestmark = pytest.mark.gpu


def test_argmax_without_allocation_matches_argmax():
    ops = Ops()                                       # hands the ordinary entry point its workspace
    lib = ctypes.CDLL(build.find_library())
    lib.fllm_last_error.restype = ctypes.c_char_p
    for fn in (lib.fllm_argmax_static, lib.fllm_argmax):
        fn.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
        fn.restype = ctypes.c_int
    stream = torch.cuda.current_stream().cuda_stream
    gen = torch.Generator(device="cuda").manual_seed(5)
    # a first call of both, untimed and unmeasured: the runtime loads a kernel's code at its first launch
    warm = torch.zeros((2, 64), dtype=torch.float32, device="cuda")
    warm_out = torch.zeros(2, dtype=torch.int32, device="cuda")
    assert lib.fllm_argmax_static(warm.data_ptr(), warm_out.data_ptr(), 2, 64, stream) == 0, lib.fllm_last_error()
    assert lib.fllm_argmax(warm.data_ptr(), warm_out.data_ptr(), 2, 64, stream) == 0, lib.fllm_last_error()
    torch.cuda.synchronize()
    for rows, vocab in ((24, 128256), (3, 50001), (1, 777)):          # the second and third inputs are smaller
        logits = torch.randn((rows, vocab), generator=gen, device="cuda", dtype=torch.float32)
        logits[0, vocab // 3] = float("inf")                          # not finite: never chosen
        logits[rows - 1, vocab - 1] = 50.0                            # the last column wins its row
        got = torch.full((rows,), -7, dtype=torch.int32, device="cuda")
        want = torch.full((rows,), -9, dtype=torch.int32, device="cuda")
        torch.cuda.synchronize()
        # free bytes of the whole device, as the driver counts them: an allocation by anyone in this process would show,
        # torch's own counters see only what goes through torch's allocator
        free_before, _ = torch.cuda.mem_get_info()
        assert lib.fllm_argmax_static(logits.data_ptr(), got.data_ptr(), rows, vocab, stream) == 0, lib.fllm_last_error()
        torch.cuda.synchronize()
        free_after, _ = torch.cuda.mem_get_info()
        assert free_after == free_before, f"the device has {free_before - free_after} bytes less after the call"
        assert lib.fllm_argmax(logits.data_ptr(), want.data_ptr(), rows, vocab, stream) == 0, lib.fllm_last_error()
        torch.cuda.synchronize()
        assert torch.equal(got, want), (rows, vocab)
        finite = torch.where(torch.isfinite(logits), logits, torch.full_like(logits, -float("inf")))
        assert torch.equal(got.long(), finite.argmax(dim=1))
        assert int(got[rows - 1]) == vocab - 1
    too_many = torch.zeros((257, 8), dtype=torch.float32, device="cuda")
    out = torch.zeros(257, dtype=torch.int32, device="cuda")
    assert lib.fllm_argmax_static(too_many.data_ptr(), out.data_ptr(), 257, 8, stream) != 0
    assert b"at most 256" in lib.fllm_last_error()
    del ops
