"""Requests that begin alike on a model whose layers keep state of their own per request: the scheduler's cuts, the
copies of the state and where they are put back, on the CPU with the plain kernels of tests/reference_ops.py (the toy
architectures are those of tests/test_toy_parts_gpu.py, which runs the same checks on the device)."""
import test_toy_parts_gpu as toys
from reference_ops import ReferenceOps


def test_state_is_copied_where_requests_part():
    toys.check_shared_beginnings(dict(device="cpu", ops=ReferenceOps()))


def test_two_state_tensors_and_portions_on_multiples():
    toys.check_two_state_tensors(dict(device="cpu", ops=ReferenceOps()))


def test_a_given_number_of_pages_is_kept_unless_a_window_bounds_it():
    """A group that keeps all keys gets the pages it was given (up to what its requests can hold at the longest
    context); a group that keeps a window gets no more than its requests can fill when steps are bounded."""
    import tiny_configs as tc
    from fllm_amd import Engine
    from fllm_amd.cache import CacheManager
    options = dict(seed=0, dtype="float32", device="cpu", ops=ReferenceOps(), max_seqs=3, max_batched_tokens=8, block_size=4)
    whole = Engine(config=tc.TINY_A, ctx=100, num_blocks=60, **options)
    assert whole.runner.pages_per_group == [60]
    assert Engine(config=tc.TINY_A, ctx=100, num_blocks=1000, **options).runner.pages_per_group == [3 * 25]
    mixed = Engine(config=tc.TINY_C, ctx=100, num_blocks=60, **options)
    windows = [key.window for key in mixed.runner.model.group_keys]
    assert sorted(windows, key=str) == [24, None]
    bound = 3 * CacheManager.window_pages_bound(24, 4, 8)
    assert mixed.runner.pages_per_group == [bound if w else 60 for w in windows] and bound < 60
