"""K/V rows that are not in HBM, through the C ABI: the paged cache's host tier (park / resume on the move stream), the VRAM
stage registered with sd_kv_stage (stage / unstage), pool growth, and mapped host state (sd_host_state).  The reference's
counterparts are gpu/kv_stage.hpp:4-184, sd_kv_stage (gpu/kernels.cpp:4277-4290), sd_kv_grow (:4048-4140) and sd_host_state
(:3876-3903); its own tests of them need model bundles (tests/kv_growth*_gpu.rs), so the checks here are the properties they
assert: where rows are held changes no bit of what attention returns, and the bookkeeping refuses what it cannot do without
changing anything."""
import numpy as np
import pytest

from gpu_util import backend, close_enough
from straydog_amd import abi
from straydog_amd.backend import StraydogError

pytestmark = pytest.mark.gpu

PAGE, KVH, DIM, ROW, HEADS, CONTEXT = 64, 2, 128, 136, 8, 1024


@pytest.fixture(scope="module")
def gpu():
    with backend() as handle:
        yield handle


class Sequences:
    """Appends rows to, and attends over, sequences of one cache; keeps the float rows to check against the oracle."""

    def __init__(self, gpu, oracle, cache, seed):
        self.gpu, self.oracle, self.cache = gpu, oracle, cache
        self.rng = np.random.default_rng(seed)
        self.rows = {}

    def view(self, sequence):
        pool, table, stride = self.gpu.kv_cache_view(self.cache)
        return pool, table + sequence * stride * 4, stride

    def append(self, sequence, count, view=None, reserve=True):
        gpu = self.gpu
        k = self.rng.standard_normal((count, KVH, DIM)).astype(np.float32)
        v = self.rng.standard_normal((count, KVH, DIM)).astype(np.float32)
        have = self.rows.get(sequence, (np.zeros((0, KVH, DIM), np.float32),) * 2)
        start = have[0].shape[0]
        if reserve:
            gpu.kv_cache_reserve(self.cache, sequence, start + count)
        pool, table, stride = view or self.view(sequence)
        kb, vb, pb = gpu.upload(k), gpu.upload(v), gpu.upload(np.array([start], dtype=np.int32))
        gpu.kv_write(pool, table, stride, pb.base(), kb.base(), vb.base(), False, 1, count)
        for b in (kb, vb, pb):
            gpu.release(b)
        self.rows[sequence] = (np.concatenate([have[0], k]), np.concatenate([have[1], v]))
        return start

    def attend(self, sequence, q, view=None):
        gpu = self.gpu
        length = self.rows[sequence][0].shape[0]
        pool, table, stride = view or self.view(sequence)
        qb, pb = gpu.upload(q), gpu.upload(np.array([length - 1], dtype=np.int32))
        out = gpu.buffer(q.size * 4)
        scratch = gpu.buffer(gpu.paged_attention_scratch(1, 1, HEADS, DIM, CONTEXT))
        gpu.paged_attention(pool, table, stride, pb.base(), CONTEXT, qb.base(), False, 1, 1, HEADS, 0.09, out.base(), False, scratch)
        got = gpu.read_buffer(out, 0, np.float32, q.size).reshape(q.shape)
        for b in (qb, pb, out, scratch):
            gpu.release(b)
        return got

    def want(self, sequence, q):
        k, v = self.rows[sequence]
        length = k.shape[0]
        pages = (length + PAGE - 1) // PAGE
        host = np.zeros(self.oracle.pool_bytes(pages, KVH, PAGE, ROW), dtype=np.uint8)
        own = np.arange(pages, dtype=np.int32)[None, :]
        self.oracle.kv_write(host, ROW, PAGE, KVH, DIM, own, np.zeros(1, np.int32), k[None], v[None])
        return self.oracle.paged_attention(host, ROW, PAGE, KVH, DIM, own, np.array([length - 1], np.int32), q, 0.09)

    def query(self):
        return self.rng.standard_normal((1, 1, HEADS, DIM)).astype(np.float32)


def test_a_parked_sequence_comes_back_bit_for_bit_while_others_take_its_pages(gpu, oracle):
    cache, *_ = gpu.kv_cache(8, PAGE, KVH, DIM, ROW, 3, CONTEXT)
    s = Sequences(gpu, oracle, cache, 71)
    with pytest.raises(StraydogError, match="no host tier"):
        s.append(0, 10)
        gpu.kv_cache_park(cache, 0)
    gpu.kv_cache_host(cache, 6)
    with pytest.raises(StraydogError, match="one host tier"):
        gpu.kv_cache_host(cache, 6)
    s.append(0, 290)                                     # 300 rows: five pages, the last partial
    s.append(1, 100)
    q0, q1 = s.query(), s.query()
    before0, before1 = s.attend(0, q0), s.attend(1, q1)
    close_enough(before0, s.want(0, q0), "resident")
    assert gpu.kv_cache_usage(cache, 0) == (5, 1)
    gpu.kv_cache_park(cache, 0)
    assert gpu.kv_cache_usage(cache, 0) == (5, 6)        # its HBM pages are free at once
    assert gpu.kv_cache_residency(cache, 0) == (True, 1, 0)
    for refused in (lambda: gpu.kv_cache_reserve(cache, 0, 400), lambda: gpu.kv_cache_park(cache, 0), lambda: gpu.kv_cache_fork(cache, 0, 2, 64)):
        with pytest.raises(StraydogError, match="parked"):
            refused()
    # another sequence takes the very pages the parked rows are still leaving from, and writes them
    s.append(2, 6 * PAGE)
    assert gpu.kv_cache_usage(cache, 2) == (6, 0)
    q2 = s.query()
    close_enough(s.attend(2, q2), s.want(2, q2), "the sequence on the freed pages")
    assert np.array_equal(s.attend(1, q1), before1)
    with pytest.raises(StraydogError, match="out of pages"):
        gpu.kv_cache_resume(cache, 0)
    assert gpu.kv_cache_residency(cache, 0)[0]
    gpu.kv_cache_truncate(cache, 2, 0)
    gpu.kv_cache_resume(cache, 0)
    assert gpu.kv_cache_residency(cache, 0) == (False, 6, 0)
    assert np.array_equal(s.attend(0, q0), before0), "rows that went to host memory and back"
    s.append(0, 40)                                      # and the sequence goes on
    q = s.query()
    close_enough(s.attend(0, q), s.want(0, q), "after the return")
    # a parked sequence gives pages back too
    gpu.kv_cache_park(cache, 0)
    gpu.kv_cache_truncate(cache, 0, 100)
    s.rows[0] = (s.rows[0][0][:100], s.rows[0][1][:100])
    assert gpu.kv_cache_residency(cache, 0) == (True, 4, 0)
    gpu.kv_cache_resume(cache, 0)
    close_enough(s.attend(0, q), s.want(0, q), "shortened while parked")
    gpu.kv_cache_destroy(cache)


def test_a_parked_sequence_is_attended_from_the_stage_and_grows_there(gpu, oracle):
    cache, *_ = gpu.kv_cache(8, PAGE, KVH, DIM, ROW, 2, CONTEXT)
    s = Sequences(gpu, oracle, cache, 72)
    gpu.kv_cache_host(cache, 12)
    s.append(0, 200)
    q = s.query()
    resident = s.attend(0, q)
    gpu.kv_cache_park(cache, 0)
    with pytest.raises(StraydogError, match="no K/V stage"):
        gpu.kv_cache_stage(cache, 0, 200)
    page_bytes = 2 * KVH * PAGE * ROW
    stage_rows = 6 * page_bytes // 4096 + 1              # room for six pages
    stage = gpu.buffer(stage_rows * 4096)
    for pointer, rows in ((stage.base(), stage_rows - 1), (stage.base() + 4096, stage_rows), (stage.base(), 0)):
        with pytest.raises(StraydogError, match="invalid Straydog K/V stage"):
            gpu.kv_stage(pointer, rows)
    gpu.kv_stage(stage.base(), stage_rows)
    view = gpu.kv_cache_stage(cache, 0, 200)
    assert view[0].pages == stage.base() and view[0].page_count == 6
    assert gpu.kv_cache_residency(cache, 0) == (True, 8, 4)
    assert np.array_equal(s.attend(0, q, view), resident), "the same rows, read from the stage"
    # a second batch over the same prefix copies nothing more; rows appended through the view go back to host memory
    view = gpu.kv_cache_stage(cache, 0, 200)
    first = s.append(0, 130, view, reserve=False)        # rows 200..329: the rest of page 3, page 4, some of page 5
    gpu.kv_cache_unstage(cache, 0, first, 130)
    assert gpu.kv_cache_residency(cache, 0) == (True, 6, 6)
    q2 = s.query()
    staged = s.attend(0, q2, view)
    close_enough(staged, s.want(0, q2), "grown in the stage")
    with pytest.raises(StraydogError, match="holds fewer rows"):
        gpu.kv_cache_stage(cache, 0, 7 * PAGE)           # past the stage
    with pytest.raises(StraydogError, match="outside the stage"):
        gpu.kv_cache_unstage(cache, 0, 330, 2 * PAGE)
    # back in the pool the sequence has every row, from host memory alone (the stage is overwritten first)
    s.append(1, 64)
    gpu.kv_cache_park(cache, 1)
    gpu.kv_cache_stage(cache, 1, 64)
    assert gpu.kv_cache_residency(cache, 0)[2] == 0
    gpu.kv_cache_resume(cache, 0)
    assert np.array_equal(s.attend(0, q2), staged)
    # a released stage is forgotten
    gpu.release(stage)
    with pytest.raises(StraydogError, match="no K/V stage"):
        gpu.kv_cache_stage(cache, 1, 64)
    gpu.kv_cache_destroy(cache)


def test_a_pool_grows_in_place_of_sd_kv_grow(gpu, oracle):
    cache, *_ = gpu.kv_cache(4, PAGE, KVH, DIM, ROW, 2, CONTEXT)
    s = Sequences(gpu, oracle, cache, 73)
    s.append(0, 150)
    s.append(1, 20)
    q = s.query()
    before = s.attend(0, q)
    with pytest.raises(StraydogError, match="out of pages"):
        s.append(0, 100)
    source, out = gpu.upload(np.ones(64, np.float32)), gpu.buffer(128)
    gpu.graph_begin()
    gpu.to_bf16(source.base(), 64, out.base())
    gpu.graph_end(7, True)
    assert gpu.graph_run(7)
    for pages in (4, 2):
        with pytest.raises(StraydogError, match="invalid Straydog K/V growth"):
            gpu.kv_cache_grow(cache, pages)
    used = gpu.memory()[0]
    with pytest.raises(StraydogError, match="not enough VRAM for the K/V of this sequence"):
        gpu.kv_cache_grow(cache, 1 << 24)
    assert gpu.memory()[0] == used and np.array_equal(s.attend(0, q), before)
    gpu.kv_cache_grow(cache, 9)
    assert not gpu.graph_run(7), "graphs recorded before the pool moved are gone"
    assert gpu.kv_cache_usage(cache, 0) == (3, 5)
    assert np.array_equal(s.attend(0, q), before), "the rows moved with the pool"
    s.append(0, 300)
    q2 = s.query()
    close_enough(s.attend(0, q2), s.want(0, q2), "grown")
    q1 = s.query()
    close_enough(s.attend(1, q1), s.want(1, q1), "the other sequence")
    gpu.release(out); gpu.release(source)
    gpu.kv_cache_destroy(cache)


def test_a_pool_in_mapped_host_memory_attends_to_the_same_bits(gpu, oracle):
    assert gpu.lib.sd_host_state_supported(gpu.handle) == 1
    rng = np.random.default_rng(74)
    pages, length = 4, 230
    used = gpu.memory()[0]
    state = gpu.host_state(pages * 2 * KVH * PAGE * ROW)
    assert gpu.memory()[0] == used, "host state is outside the VRAM budget"
    pool_host = abi.KvPool(state.base(), pages, PAGE, KVH, DIM, ROW)
    pool_vram, buffer = gpu.kv_pool(pages, PAGE, KVH, DIM, ROW)
    table = np.array([[2, 0, 3, 1]], dtype=np.int32)
    k = rng.standard_normal((1, length, KVH, DIM)).astype(np.float32)
    v = rng.standard_normal((1, length, KVH, DIM)).astype(np.float32)
    q = rng.standard_normal((1, 1, HEADS, DIM)).astype(np.float32)
    tb, kb, vb, zero, qb, pb = (gpu.upload(a) for a in (table, k, v, np.zeros(1, np.int32), q, np.array([length - 1], np.int32)))
    outs = []
    for pool in (pool_vram, pool_host):
        gpu.kv_write(pool, tb.base(), 4, zero.base(), kb.base(), vb.base(), False, 1, length)
        out = gpu.buffer(q.size * 4)
        scratch = gpu.buffer(gpu.paged_attention_scratch(1, 1, HEADS, DIM, 256))
        gpu.paged_attention(pool, tb.base(), 4, pb.base(), 256, qb.base(), False, 1, 1, HEADS, 0.09, out.base(), False, scratch)
        outs.append(gpu.read_buffer(out, 0, np.float32, q.size))
        gpu.release(out); gpu.release(scratch)
    assert np.array_equal(outs[0], outs[1])
    rows_vram = gpu.read_buffer(buffer, 0, np.uint8, pages * 2 * KVH * PAGE * ROW)
    rows_host = gpu.read_buffer(state, 0, np.uint8, pages * 2 * KVH * PAGE * ROW)
    assert np.array_equal(rows_vram, rows_host)
    with pytest.raises(StraydogError, match="invalid Straydog K/V stage"):
        gpu.kv_stage(state.base(), pages * 2 * KVH * PAGE * ROW // 4096)
    for b in (tb, kb, vb, zero, qb, pb, buffer, state):
        gpu.release(b)
    assert gpu.memory()[0] == used
    # states page-locked ahead of time on a thread are taken by size, zeroed; another size is allocated on the spot
    import ctypes
    sizes = (ctypes.c_uint64 * 2)(4096, 1 << 20)
    assert gpu.lib.sd_host_states_prefetch(gpu.handle, sizes, 2) == 0
    assert gpu.lib.sd_host_states_prefetch(gpu.handle, sizes, 2) == -1 and "prefetch" in gpu.error()
    large, other, small = gpu.host_state(1 << 20), gpu.host_state(12345), gpu.host_state(4096)
    assert not gpu.read_buffer(large, 0, np.uint8, 1 << 20).any() and not gpu.read_buffer(small, 0, np.uint8, 4096).any()
    for b in (large, other, small):
        gpu.release(b)


def test_a_recorded_step_runs_after_the_page_moves_queued_before_it(gpu, oracle):
    """A decode step recorded as a graph reads the pages its sequence holds when it is replayed: a replay queued right after a
    resume (onto other pages) or a stage comes after the copies that fill them, and gives the eager call's bits."""
    context, length = 16384, 16000
    pages = context // PAGE
    cache, *_ = gpu.kv_cache(2 * pages, PAGE, KVH, DIM, ROW, 2, context)
    gpu.kv_cache_host(cache, 2 * pages)
    rng = np.random.default_rng(75)
    pool, table, stride = gpu.kv_cache_view(cache)
    gpu.kv_cache_reserve(cache, 0, length)
    k = rng.standard_normal((1, length, KVH, DIM)).astype(np.float32)
    v = rng.standard_normal((1, length, KVH, DIM)).astype(np.float32)
    q = rng.standard_normal((1, 1, HEADS, DIM)).astype(np.float32)
    kb, vb, zero, qb, pb = (gpu.upload(a) for a in (k, v, np.zeros(1, np.int32), q, np.array([length - 1], np.int32)))
    gpu.kv_write(pool, table, stride, zero.base(), kb.base(), vb.base(), False, 1, length)
    out = gpu.buffer(q.size * 4)
    scratch = gpu.buffer(gpu.paged_attention_scratch(1, 1, HEADS, DIM, context))

    def step(view):
        gpu.paged_attention(view[0], view[1], view[2], pb.base(), context, qb.base(), False, 1, 1, HEADS, 0.09, out.base(), False, scratch)

    def result():
        return gpu.read_buffer(out, 0, np.float32, q.size)

    step((pool, table, stride))
    eager = result()
    gpu.graph_begin()
    step((pool, table, stride))
    gpu.graph_end(31, True)
    for turn in range(3):
        # the sequence leaves, another takes (and writes) the pages it held, and it comes back onto other pages
        gpu.kv_cache_park(cache, 0)
        gpu.kv_cache_reserve(cache, 1, length)
        gpu.kv_write(pool, table + stride * 4, stride, zero.base(), vb.base(), kb.base(), False, 1, length)
        gpu.kv_cache_resume(cache, 0)
        gpu.write_buffer(out, 0, np.zeros(q.size, np.float32))
        assert gpu.graph_run(31)
        assert np.array_equal(result(), eager), f"replay {turn} right after a resume"
        gpu.kv_cache_truncate(cache, 1, 0)
    # the same through the stage: the view's pool is the stage, whose rows a staging refills
    gpu.kv_cache_park(cache, 0)
    page_bytes = 2 * KVH * PAGE * ROW
    stage_rows = pages * page_bytes // 4096 + 1
    stage = gpu.buffer(stage_rows * 4096)
    gpu.kv_stage(stage.base(), stage_rows)
    view = gpu.kv_cache_stage(cache, 0, length)
    step(view)
    assert np.array_equal(result(), eager), "the same rows, read from the stage"
    gpu.graph_begin()
    step(view)
    gpu.graph_end(32, True)
    gpu.kv_cache_reserve(cache, 1, 4 * PAGE)
    gpu.kv_write(pool, table + stride * 4, stride, zero.base(), vb.base(), kb.base(), False, 1, 4 * PAGE)
    for turn in range(3):
        gpu.kv_cache_park(cache, 1)
        gpu.kv_cache_stage(cache, 1, 4 * PAGE)              # the stage now holds the other sequence's first pages
        gpu.kv_cache_resume(cache, 1)
        again = gpu.kv_cache_stage(cache, 0, length)
        assert again[0].pages == view[0].pages and again[1] == view[1]
        gpu.write_buffer(out, 0, np.zeros(q.size, np.float32))
        assert gpu.graph_run(32)
        assert np.array_equal(result(), eager), f"replay {turn} right after a staging"
    gpu.release(stage)
    for b in (kb, vb, zero, qb, pb, out, scratch):
        gpu.release(b)
    gpu.kv_cache_destroy(cache)


def _selections(rng, base, rows, context, blocks=512):
    """Selection lists as the Qwen block selection leaves them: `blocks` complete blocks of four positions in block order, then
    the positions of the row's incomplete block; floats, with the counts."""
    selected = 4 * blocks + 4
    indices = np.full((rows, selected), -7.0, np.float32)
    counts = np.zeros(rows, np.float32)
    for r in range(rows):
        position = base + r
        complete = (position + 1) // 4
        chosen = np.sort(rng.choice(complete, size=min(blocks, complete), replace=False))
        listed = (chosen[:, None] * 4 + np.arange(4)[None, :]).reshape(-1)
        tail = np.arange(complete * 4, position + 1)
        entries = np.concatenate([listed, tail]).astype(np.float32)
        indices[r, :entries.size] = entries
        counts[r] = entries.size
    return indices, counts, selected


def test_a_sparse_pass_over_a_parked_sequence_gathers_the_union_of_its_selections(gpu, oracle):
    """The union gather (the reference's qsa_attention_gathered, gpu/prefill_batch.hpp:224-254): a Qwen-shaped sequence of 242K
    tokens is attended through selection lists where it lives in HBM, then parked in host memory and attended again through the
    blocks its selections name, copied into a small VRAM stage and renumbered: the same bits, for a decode row, a verification span
    and a run of prompt rows whose union the stage only holds a few rows of at a time."""
    page, kvh, dim, row, heads, context = 256, 2, 256, 272, 24, 242000
    pages = (context + page - 1) // page
    rng = np.random.default_rng(76)
    cache, *_ = gpu.kv_cache(pages + 1, page, kvh, dim, row, 2, pages * page)
    gpu.kv_cache_host(cache, pages)
    gpu.kv_cache_reserve(cache, 0, context)
    pool, table, stride = gpu.kv_cache_view(cache)
    # the rows: seeded values drawn on the device, appended a stretch at a time
    stretch = 16384
    kb, vb, pb = gpu.buffer(stretch * kvh * dim * 2), gpu.buffer(stretch * kvh * dim * 2), gpu.buffer(4)
    for at in range(0, context, stretch):
        count = min(stretch, context - at)
        gpu.fill_normal(kb.base(), count * kvh * dim, 1000 + at, 1)
        gpu.fill_normal(vb.base(), count * kvh * dim, 5000 + at, 1)
        gpu.write_buffer(pb, 0, np.array([at], np.int32))
        gpu.kv_write(pool, table, stride, pb.base(), kb.base(), vb.base(), True, 1, count)
    stage_pages = 48                                                     # 12288 positions: a decode row names 2052, five rows about 10200
    page_bytes = 2 * kvh * page * row
    stage = gpu.buffer(stage_pages * page_bytes)
    gpu.kv_stage(stage.base(), stage_pages * page_bytes // 4096)
    scale = 1.0 / 16.0
    cases = []
    for rows, base in ((1, context - 1), (5, context - 5), (40, context - 40)):
        indices, counts, selected = _selections(rng, base, rows, context)
        if rows == 5:
            # entries that do not count stay out of the union: a position after the row's own, a negative one, entries past the count
            indices[1, 3] = float(base + 1 + 3)
            indices[2, 0] = -1.0
            counts[3] = 1000.0
        q = rng.standard_normal((rows, heads, dim)).astype(np.float32)
        ib, cb, qb = gpu.upload(indices), gpu.upload(counts), gpu.upload(q)
        out = gpu.buffer(rows * heads * dim * 4)
        scratch = gpu.buffer(gpu.selected_attention_scratch(rows, kvh, selected))
        gpu.selected_attention(pool, table, context, base, ib.base(), selected, cb.base(), qb.base(), False, rows, heads, scale, out.base(), False, scratch)
        resident = gpu.read_buffer(out, 0, np.float32, rows * heads * dim)
        assert np.all(np.isfinite(resident)) and np.abs(resident).max() > 0
        cases.append((rows, base, selected, ib, cb, qb, out, scratch, resident, indices, counts))
    gpu.kv_cache_park(cache, 0)
    assert gpu.kv_cache_residency(cache, 0)[0]
    for rows, base, selected, ib, cb, qb, out, scratch, resident, indices, counts in cases:
        renumbered = gpu.buffer(rows * selected * 4)
        gpu.write_buffer(out, 0, np.zeros(rows * heads * dim, np.float32))
        first, calls = 0, 0
        while first < rows:
            taken, gathered, view, view_table, view_stride = gpu.kv_cache_gather(cache, 0, context, base, ib.base(), selected, cb.base(), first, rows - first,
                                                                                renumbered.base())
            assert 1 <= taken <= rows - first and 0 < gathered <= stage_pages * page and view.pages == stage.base()
            gpu.selected_attention(view, view_table, context, base + first, renumbered.at(first * selected * 4), selected, cb.at(first * 4),
                                   qb.at(first * heads * dim * 4), False, taken, heads, scale, out.at(first * heads * dim * 4), False, scratch)
            first += taken
            calls += 1
        assert np.array_equal(gpu.read_buffer(out, 0, np.float32, rows * heads * dim), resident), f"{rows} rows from the stage"
        assert calls == 1 if rows <= 5 else calls > 1, "the long run's union does not fit the stage at once"
        listed = gpu.read_buffer(renumbered, 0, np.float32, rows * selected).reshape(rows, selected)
        if rows == 5:
            # the lists' places follow block order, and what did not count is -1
            assert listed[1, 3] == -1.0 and listed[2, 0] == -1.0 and np.all(listed[3, 1000:] == -1.0) and np.all(listed[0, int(counts[0]):] == -1.0)
            kept = listed[0, :int(counts[0])]
            assert np.all(np.diff(kept) > 0) and np.all(kept <= indices[0, :int(counts[0])])
        for b in (renumbered, ib, cb, qb, out, scratch):
            gpu.release(b)
    # a stage too small for one row's selection takes nothing and says so
    gpu.release(stage)
    small = gpu.buffer(4 * page_bytes)
    gpu.kv_stage(small.base(), 4 * page_bytes // 4096)
    indices, counts, selected = _selections(rng, context - 1, 1, context)
    ib, cb, rb = gpu.upload(indices), gpu.upload(counts), gpu.buffer(selected * 4)
    taken, gathered, *_ = gpu.kv_cache_gather(cache, 0, context, context - 1, ib.base(), selected, cb.base(), 0, 1, rb.base())
    assert (taken, gathered) == (0, 0)
    with pytest.raises(StraydogError, match="invalid Straydog union gather"):
        gpu.kv_cache_gather(cache, 0, context, context, ib.base(), selected, cb.base(), 0, 1, rb.base())
    with pytest.raises(StraydogError, match="holds fewer rows"):
        gpu.kv_cache_gather(cache, 1, context, 0, ib.base(), selected, cb.base(), 0, 1, rb.base())
    # back in HBM the sequence is what it was
    gpu.kv_cache_resume(cache, 0)
    for b in (small, ib, cb, rb, kb, vb, pb):
        gpu.release(b)
    gpu.kv_cache_destroy(cache)
