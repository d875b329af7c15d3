"""Requests that begin alike on a model whose layers keep state of their own per request: the scheduler's cuts, the
copies of the state and where they are put back, on the CPU with the plain kernels of tests/reference_ops.py (the toy
architectures are those of tests/test_toy_parts_gpu.py, which runs the same checks on the device)."""
import test_toy_parts_gpu as toys
from reference_ops import ReferenceOps


def test_state_is_copied_where_requests_part():
    toys.check_shared_beginnings(dict(device="cpu", ops=ReferenceOps()))


def test_two_state_tensors_and_portions_on_multiples():
    toys.check_two_state_tensors(dict(device="cpu", ops=ReferenceOps()))
