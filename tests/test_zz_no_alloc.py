"""sdx_paged_attention_static -- the entry point that allocates nothing (its partial results live in an area the library
itself holds on the GPU) -- gives the bits of sdx_paged_attention, on two calls in a row, the second with a smaller
input; it also agrees with the oracle, refuses a batch whose partial results would not fit, and leaves the handle's
memory accounting untouched."""
import numpy as np
import pytest

from gpu_util import backend, close_enough
from straydog_amd.workloads import PagedWorkload

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gpu():
    with backend() as handle:
        yield handle


def _nothing_allocated(before, after):
    """Device memory as the driver reports it has not shrunk (it may grow: memory released earlier comes back late), and the
    handle's workspace and its timing events are what they were."""
    assert after[0] >= before[0], f"the device's free memory fell by {before[0] - after[0]} bytes"
    assert after[1:] == before[1:]


def _both(gpu, work):
    """Output bytes of the scratch-argument entry point and of the static one, on the same inputs."""
    count = work.seqs * work.span * work.heads * work.dim * (2 if work.out_f16 else 4)
    gpu.write_buffer(work.out_buffer, 0, np.full(count, 0xa5, np.uint8))
    work.step()
    want = gpu.read_buffer(work.out_buffer, 0, np.uint8, count).copy()
    gpu.write_buffer(work.out_buffer, 0, np.full(count, 0x5a, np.uint8))
    used_before, state_before = gpu.memory()[0], gpu.device_state()
    gpu.paged_attention_static(work.pool, work.table_buffer.base(), work.table_stride, work.position_buffer.base(), work.max_context,
                               work.q_buffer.base(), work.q_f16, work.seqs, work.span, work.heads, work.scale, work.out_buffer.base(),
                               work.out_f16)
    got = gpu.read_buffer(work.out_buffer, 0, np.uint8, count).copy()
    # nothing allocated: neither in the handle's own accounting, nor as the driver sees the device, nor as workspace or events
    assert gpu.memory()[0] == used_before
    _nothing_allocated(state_before, gpu.device_state())
    return got, want


def test_static_entry_first_call_on_a_fresh_handle():
    # the handle's very first launch is the static entry's: whatever it sets up for itself (LDS limits) allocates nothing either
    with backend() as fresh:
        work = PagedWorkload(fresh, [900, 4100, 33], span=1, heads=32, kv_heads=4, dim=128, seed=20)
        count = work.seqs * work.span * work.heads * work.dim * 2
        state_before = fresh.device_state()
        fresh.paged_attention_static(work.pool, work.table_buffer.base(), work.table_stride, work.position_buffer.base(), work.max_context,
                                     work.q_buffer.base(), work.q_f16, work.seqs, work.span, work.heads, work.scale, work.out_buffer.base(),
                                     work.out_f16)
        got = fresh.read_buffer(work.out_buffer, 0, np.uint8, count).copy()
        _nothing_allocated(state_before, fresh.device_state())
        work.step()
        assert np.array_equal(got, fresh.read_buffer(work.out_buffer, 0, np.uint8, count))
        work.release()


def test_static_entry_equals_the_scratch_entry_twice_in_a_row(gpu, oracle):
    rng = np.random.default_rng(77)
    # first a ragged decode batch (many workgroups, many segments), then a smaller one: the area keeps the first call's
    # partial results, and the second must not read them
    large = PagedWorkload(gpu, [int(n) for n in rng.integers(300, 9000, size=12)], span=1, heads=32, kv_heads=4, dim=128, seed=21)
    small = PagedWorkload(gpu, [700, 130, 1], span=1, heads=32, kv_heads=4, dim=128, seed=22)
    for work in (large, small):
        got, want = _both(gpu, work)
        assert np.array_equal(got, want), "the static entry point's output differs from sdx_paged_attention's"
        reference = oracle.paged_attention(work.read_pool(), work.row_bytes, work.page_tokens, work.kv_heads, work.dim, work.table,
                                           work.positions, work.read_queries(), work.scale)
        close_enough(work.read_output(), reference, "static entry point vs oracle")
    large.release()
    small.release()


def test_static_entry_verify_span_and_wide_rows(gpu):
    # a verify span (three query tiles) and 256-column FP16 rows, then smaller inputs of each
    for kwargs in (dict(span=5, heads=32, kv_heads=4, dim=128), dict(span=1, heads=24, kv_heads=2, dim=256, row_bytes=512, q_f16=False, out_f16=False)):
        for lengths in ([4000, 2500, 777, 64], [300, 40]):
            work = PagedWorkload(gpu, lengths, seed=23, **kwargs)
            got, want = _both(gpu, work)
            assert np.array_equal(got, want)
            work.release()


def test_static_entry_refuses_what_does_not_fit(gpu):
    assert gpu.lib.sdx_paged_attention_static_bytes() == 16 << 20
    # 64 query rows per K/V head over many workgroups: more partial results than the area holds
    work = PagedWorkload(gpu, [2000] * 80, span=8, heads=32, kv_heads=4, dim=128, seed=24)
    with pytest.raises(RuntimeError, match="allocates nothing holds"):
        gpu.paged_attention_static(work.pool, work.table_buffer.base(), work.table_stride, work.position_buffer.base(), work.max_context,
                                   work.q_buffer.base(), work.q_f16, work.seqs, work.span, work.heads, work.scale, work.out_buffer.base(),
                                   work.out_f16)
    work.release()
    # a prefill-sized span goes to kernels that need a workspace: refused here
    work = PagedWorkload(gpu, [600], span=64, heads=32, kv_heads=4, dim=128, seed=25)
    with pytest.raises(RuntimeError, match="too many query rows"):
        gpu.paged_attention_static(work.pool, work.table_buffer.base(), work.table_stride, work.position_buffer.base(), work.max_context,
                                   work.q_buffer.base(), work.q_f16, work.seqs, work.span, work.heads, work.scale, work.out_buffer.base(),
                                   work.out_f16)
    work.release()
