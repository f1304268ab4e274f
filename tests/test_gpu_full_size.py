"""The BASELINE configurations at full size on the GPU, through the C ABI: the oracle on a bounded part of each, and
size-independent properties on the whole (bit-identity under a permutation of the physical pages, chunked prefill against
single-token decode, the matrix-core indexer against the all-canonical one)."""
import numpy as np
import pytest

from gpu_util import backend, close_enough


def _bf16(bits):
    return (np.asarray(bits).astype(np.uint32) << 16).view(np.float32)

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gpu():
    g = backend(48 << 30)
    yield g
    g.close()


def _oracle_rows(oracle, work, rows):
    pool = work.read_pool()
    q, got = work.read_queries()[rows], work.read_output()[rows]
    want = oracle.paged_attention(pool, work.row_bytes, work.page_tokens, work.kv_heads, work.dim, work.table[rows], work.positions[rows], q, work.scale)
    return got, want


def test_config1_ragged_decode_full_size(gpu, oracle):
    from straydog_amd import workloads
    lengths = workloads.config1_lengths()
    work = workloads.PagedWorkload(gpu, lengths, seed=1)
    work.step()
    rows = np.argsort(lengths)[[0, 1, 15, 31]]                    # the two shortest, a middle one and the longest sequence
    got, want = _oracle_rows(oracle, work, rows)
    assert np.abs(got - want).max() <= 2e-3 + 2.0 ** -11 * np.abs(want).max()        # FP16 outputs
    first = work.read_output().copy()
    work.release()
    # the same rows behind another permutation of the physical pages: the same bits
    other = workloads.PagedWorkload(gpu, lengths, seed=1, page_seed=99)
    assert not np.array_equal(other.table, work.table)
    other.step()
    assert np.array_equal(other.read_output(), first)
    other.release()


def test_config1_all_32k_and_config3_verify_full_size(gpu, oracle):
    from straydog_amd import workloads
    work = workloads.PagedWorkload(gpu, [32768] * 32, seed=2)
    work.step()
    got, want = _oracle_rows(oracle, work, np.array([0, 31]))
    assert np.abs(got - want).max() <= 2e-3 + 2.0 ** -11 * np.abs(want).max()
    work.release()
    work = workloads.PagedWorkload(gpu, [65536 + 5] * 16, span=5, seed=5)
    work.step()
    got, want = _oracle_rows(oracle, work, np.array([3]))
    assert np.abs(got - want).max() <= 2e-3 + 2.0 ** -11 * np.abs(want).max()
    # row r of the span is the single-token decode at position context + r: the verify kernel against the decode kernel
    span_out = work.read_output()
    single = workloads.PagedWorkload(gpu, [65536 + 5] * 16, span=1, seed=5)
    q = work.read_queries()
    gpu.write_buffer(single.q_buffer, 0, q[:, 4].astype(np.float16))
    single.step()
    assert np.abs(single.read_output()[:, 0] - span_out[:, 4]).max() < 1e-3
    work.release(); single.release()


def test_config2_chunked_prefill_full_size(gpu, oracle):
    from straydog_amd import workloads
    work = workloads.PrefillWorkload(gpu)
    work.step()
    out = work.read(work.out, work.tokens * work.heads * work.dim).reshape(work.tokens, work.heads, work.dim)
    q = work.read(work.q, work.tokens * work.heads * work.dim).reshape(work.tokens, work.heads, work.dim)
    pool = gpu.read_buffer(work.pool_buffer, 0, np.uint8, work.pool_buffer.size)
    # the oracle on tokens of every chunk, first and last rows included (a row attends the cache up to its own position)
    for token in (0, 1, 2047, 2048, 5000, 8191):
        want = oracle.paged_attention(pool, work.row_bytes, work.page_tokens, work.kv_heads, work.dim, work.table, np.array([token], np.int32),
                                      q[None, token:token + 1], work.scale)
        assert np.abs(out[token] - want[0, 0]).max() <= 2e-3 + 2.0 ** -11 * np.abs(want).max(), f"token {token}"
    # the cache the chunks wrote is the oracle's encoding of the same FP16 rows
    k = work.read(work.k, work.tokens * work.kv_heads * work.dim).reshape(1, work.tokens, work.kv_heads, work.dim)
    v = work.read(work.v, work.tokens * work.kv_heads * work.dim).reshape(1, work.tokens, work.kv_heads, work.dim)
    mirror = np.zeros_like(pool)
    oracle.kv_write(mirror, work.row_bytes, work.page_tokens, work.kv_heads, work.dim, work.table, np.zeros(1, np.int32), k, v)
    assert np.array_equal(mirror, pool)
    work.release()


def test_config4_sparse_path_full_size(gpu, oracle):
    from straydog_amd import workloads
    work = workloads.SparseWorkload(gpu)
    work.step_index(keep_scores=False)                             # matrix-core brackets + canonical rescoring
    fast = gpu.read_buffer(work.indices, 0, np.int32, work.batch * work.k).reshape(work.batch, work.k).copy()
    work.step_index(keep_scores=True)                              # every score canonical
    exact = gpu.read_buffer(work.indices, 0, np.int32, work.batch * work.k).reshape(work.batch, work.k)
    assert np.array_equal(fast, exact)
    assert np.all(np.diff(exact, axis=1) > 0)                      # ascending, no index twice
    # the canonical scores of one sequence against the oracle, and the oracle's top-k over them
    scores = gpu.read_buffer(work.scores, 0, np.float32, work.batch * work.context).reshape(work.batch, work.context)
    q_bits = gpu.read_buffer(work.q_index, 0, np.uint16, work.batch * work.index_heads * work.index_dim).reshape(work.batch, work.index_heads, -1)
    b = 5
    key_bits = gpu.read_buffer(work.keys, b * work.context * work.index_dim * 2, np.uint16, work.context * work.index_dim).reshape(work.context, -1)
    weights = gpu.read_buffer(work.weights, 0, np.float32, work.batch * work.index_heads).reshape(work.batch, -1)
    want = oracle.index_scores(_bf16(q_bits[b:b + 1]), _bf16(key_bits), weights[b:b + 1], np.array([work.context], np.int32), 1.0)
    assert np.array_equal(scores[b].view(np.uint32), want[0].view(np.uint32))
    assert np.array_equal(exact[b], oracle.top_k(want, work.k)[0])
    # the gather attention of that sequence against the oracle
    work.step_attention()
    out = gpu.read_buffer(work.out, b * work.heads * work.vdim * 4, np.float32, work.heads * work.vdim).reshape(work.heads, work.vdim)
    aq = _bf16(gpu.read_buffer(work.q, b * work.heads * work.kdim * 2, np.uint16, work.heads * work.kdim).reshape(1, work.heads, work.kdim))
    lat = gpu.read_buffer(work.latents, b * work.context * work.kdim * 2, np.uint16, work.context * work.kdim).reshape(work.context, work.kdim)
    want_out = oracle.latent_attention(aq, None, None, 0, lat, exact[b:b + 1], None, work.vdim, work.scale)
    close_enough(out, want_out[0], "gather attention")
    work.release()


def test_indexer_rows_longer_than_a_million_groups(gpu):
    # more segments a row than the finishing workgroup has threads (1024 segments of 1024 groups): its counts, lists and top-k go
    # the general way through global memory.  At this length the check is the size-independent one: the matrix-core path picks
    # the indices of the all-canonical path (whose scores the oracle pins at the smaller sizes), bit for bit.
    batch, groups, heads, dim, k = 2, 1_200_000, 16, 128, 2048
    q, keys, weights = gpu.buffer(batch * heads * dim * 2), gpu.buffer(batch * groups * dim * 2), gpu.buffer(batch * heads * 4)
    gpu.fill_normal(q.base(), batch * heads * dim, 31, 2)
    gpu.fill_normal(keys.base(), batch * groups * dim, 32, 2)
    gpu.fill_uniform(weights.base(), batch * heads, 33)
    visible = gpu.upload(np.array([groups, groups - 12345], dtype=np.int32))
    scores, exact, fast = gpu.buffer(batch * groups * 4), gpu.buffer(batch * k * 4), gpu.buffer(batch * k * 4)
    gpu.index_top_k(q.base(), keys.base(), weights.base(), visible.base(), batch, groups, heads, dim, 0.25, scores.base(), k, exact.base())
    gpu.index_top_k(q.base(), keys.base(), weights.base(), visible.base(), batch, groups, heads, dim, 0.25, None, k, fast.base())
    want = gpu.read_buffer(exact, 0, np.int32, batch * k).reshape(batch, k)
    got = gpu.read_buffer(fast, 0, np.int32, batch * k).reshape(batch, k)
    assert np.array_equal(got, want)
    assert np.all(np.diff(want, axis=1) > 0) and want.min() >= 0 and want[1].max() < groups - 12345
    for b in (q, keys, weights, visible, scores, exact, fast):
        gpu.release(b)
