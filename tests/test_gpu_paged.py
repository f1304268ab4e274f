"""GPU parity of the paged K/V cache path through the C ABI: sdx_kv_write (bit-exact Q8_0 / FP16 rows against the
oracle's kv_encode restatement) and sdx_paged_attention (decode and verify spans) against the oracle's fp32
attention on identical seeded inputs, within max-abs 2e-3 and relative 1e-2; plus properties that hold at any size
(page permutation leaves the output bit-identical, a verify row equals the single-token call at its position, zero
queries give the mean of the values)."""
import numpy as np
import pytest

from gpu_util import backend, close_enough, make_pool
from straydog_amd.backend import StraydogError

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gpu():
    with backend() as handle:
        yield handle


@pytest.mark.parametrize("dim,fmt", [(128, "q8"), (256, "q8"), (128, "f16"), (256, "f16")])
@pytest.mark.parametrize("input_f16", [False, True])
def test_kv_write_rows_are_bit_exact(gpu, oracle, dim, fmt, input_f16):
    rng = np.random.default_rng(100 + dim + input_f16)
    row_bytes = dim + dim // 16 if fmt == "q8" else 2 * dim
    seqs, span, kv_heads, page_tokens = 3, 5, 2, 32
    starts = np.array([0, 30, 77], dtype=np.int32)        # row runs that cross page boundaries
    pages_per = [(int(s) + span + page_tokens - 1) // page_tokens for s in starts]
    total = sum(pages_per) + 1
    order = rng.permutation(total)
    table = np.zeros((seqs, max(pages_per)), dtype=np.int32)
    at = 0
    for s in range(seqs):
        table[s, :pages_per[s]] = order[at:at + pages_per[s]]
        at += pages_per[s]
    magnitude = 10.0 ** rng.integers(-3, 3, size=(seqs, span, kv_heads, 1))
    keys = (rng.standard_normal((seqs, span, kv_heads, dim)) * magnitude).astype(np.float32)
    values = (rng.standard_normal((seqs, span, kv_heads, dim)) * magnitude).astype(np.float32)
    keys[0, 0, 0, :32] = 0.0                              # an all-zero block: zero scale, zero bytes
    keys[1, 2, 1, 5] = 500.0                              # one large value leaves the other blocks alone
    values[2, 4, 0, 64:96] = -3.0                         # a block of equal magnitudes
    if input_f16:
        keys, values = keys.astype(np.float16), values.astype(np.float16)
    host = np.zeros(oracle.pool_bytes(total, kv_heads, page_tokens, row_bytes), dtype=np.uint8)
    oracle.kv_write(host, row_bytes, page_tokens, kv_heads, dim, table, starts, keys.astype(np.float32), values.astype(np.float32))
    pool, buffer = gpu.kv_pool(total, page_tokens, kv_heads, dim, row_bytes)
    tb, pb, kb, vb = gpu.upload(table), gpu.upload(starts), gpu.upload(keys), gpu.upload(values)
    gpu.kv_write(pool, tb.base(), table.shape[1], pb.base(), kb.base(), vb.base(), input_f16, seqs, span)
    got = gpu.read_buffer(buffer, 0, np.uint8, host.size)
    assert np.array_equal(got, host)
    for b in (tb, pb, kb, vb, buffer):
        gpu.release(b)


def _run(gpu, pool, table, table_buffer, positions, q, span, heads, scale, q_f16, out_f16, max_context=None):
    seqs = len(positions)
    dim = pool.dim
    max_context = max_context or int(max(positions)) + span
    max_context = min(max(max_context, 1), table.shape[1] * pool.page_tokens)
    scratch = gpu.buffer(max(gpu.paged_attention_scratch(seqs, span, heads, dim, max_context), 4))
    qb = gpu.upload(q.astype(np.float16) if q_f16 else q.astype(np.float32))
    pb = gpu.upload(np.asarray(positions, dtype=np.int32))
    out = gpu.buffer(seqs * span * heads * dim * (2 if out_f16 else 4))
    gpu.paged_attention(pool, table_buffer.base(), table.shape[1], pb.base(), max_context, qb.base(), q_f16, seqs, span, heads, scale,
                        out.base(), out_f16, scratch)
    result = gpu.read_buffer(out, 0, np.float16 if out_f16 else np.float32, seqs * span * heads * dim).astype(np.float32)
    for b in (scratch, qb, pb, out):
        gpu.release(b)
    return result.reshape(seqs, span, heads, dim)


def test_config0_single_sequence_decode(gpu, oracle):
    # BASELINE config 0: 1 query token, 16 query heads over 2 K/V heads, head_dim 128, context 4096, fp32 q and output
    rng = np.random.default_rng(0x9e3779b97f4a7c15 & 0xffffffff)
    heads, kv_heads, dim, context, page_tokens, row_bytes = 16, 2, 128, 4096, 256, 136
    pool, buffer, host, table, tb = make_pool(gpu, oracle, rng, [context], kv_heads, dim, page_tokens, row_bytes)
    q = rng.standard_normal((1, 1, heads, dim)).astype(np.float32)
    scale = 1.0 / np.sqrt(dim)
    got = _run(gpu, pool, table, tb, [context - 1], q, 1, heads, scale, False, False)
    want = oracle.paged_attention(host, row_bytes, page_tokens, kv_heads, dim, table, np.array([context - 1], np.int32), q, scale)
    worst, relative, size = close_enough(got, want, "config 0")
    print(f"config 0: max-abs {worst:.2e}, relative L2 {relative:.2e}, output magnitude {size:.2e}")
    gpu.release(buffer); gpu.release(tb)


@pytest.mark.parametrize("dim,fmt,heads,kv_heads", [(128, "q8", 32, 4), (128, "q8", 4, 4), (128, "q8", 12, 1), (256, "q8", 24, 2),
                                                    (128, "f16", 16, 2), (256, "f16", 8, 2)])
def test_ragged_batched_decode(gpu, oracle, dim, fmt, heads, kv_heads):
    # BASELINE config 1 in small: ragged lengths around every boundary of the kernel (1 token, a step of 32, a page, a chunk)
    rng = np.random.default_rng(7 + dim + heads)
    row_bytes = dim + dim // 16 if fmt == "q8" else 2 * dim
    page_tokens = 64
    lengths = [1, 2, 31, 32, 33, 63, 64, 65, 127, 128, 129, 255, 256, 257, 700, 1500]
    pool, buffer, host, table, tb = make_pool(gpu, oracle, rng, lengths, kv_heads, dim, page_tokens, row_bytes)
    seqs = len(lengths)
    q = rng.standard_normal((seqs, 1, heads, dim)).astype(np.float16).astype(np.float32)
    scale = 1.0 / np.sqrt(dim)
    positions = [n - 1 for n in lengths]
    got = _run(gpu, pool, table, tb, positions, q, 1, heads, scale, True, True)
    want = oracle.paged_attention(host, row_bytes, page_tokens, kv_heads, dim, table, np.array(positions, np.int32), q, scale)
    for s in range(seqs):
        close_enough(got[s], want[s], f"length {lengths[s]}")
    # the same pages at other places, the table renamed with them: bit-identical output
    page_bytes = 2 * kv_heads * page_tokens * row_bytes
    pages = host.reshape(-1, page_bytes)
    perm = rng.permutation(pages.shape[0])
    moved = np.ascontiguousarray(pages[perm]).reshape(-1)
    renamed = np.argsort(perm).astype(np.int32)[table]
    gpu.write_buffer(buffer, 0, moved)
    tb2 = gpu.upload(renamed)
    again = _run(gpu, pool, renamed, tb2, positions, q, 1, heads, scale, True, True)
    assert np.array_equal(again.view(np.uint32), got.view(np.uint32))
    for b in (buffer, tb, tb2):
        gpu.release(b)


@pytest.mark.parametrize("span,heads,kv_heads", [(5, 32, 4), (8, 8, 2), (2, 16, 1), (4, 16, 1), (8, 32, 4), (7, 32, 4), (13, 8, 2), (5, 24, 2)])
def test_verify_span_rows(gpu, oracle, span, heads, kv_heads):
    # BASELINE config 3 in small: span rows attend all of the context and causally inside the span.  (Spans of 7 and 8 at eight
    # heads a group, 13 at four and 5 at twelve are the four-tile variant: 49 to 64 rows a K/V head, the last tile full, short, or
    # starting in the middle of a token's heads.)
    rng = np.random.default_rng(31 + span)
    dim, row_bytes, page_tokens = 128, 136, 64
    contexts = [0, 27, 64, 300, 1029]
    lengths = [c + span for c in contexts]
    pool, buffer, host, table, tb = make_pool(gpu, oracle, rng, lengths, kv_heads, dim, page_tokens, row_bytes)
    seqs = len(lengths)
    q = rng.standard_normal((seqs, span, heads, dim)).astype(np.float16).astype(np.float32)
    scale = 1.0 / np.sqrt(dim)
    got = _run(gpu, pool, table, tb, contexts, q, span, heads, scale, True, False)
    want = oracle.paged_attention(host, row_bytes, page_tokens, kv_heads, dim, table, np.array(contexts, np.int32), q, scale)
    close_enough(got, want, f"span {span}")
    # row r of the span is the single-token decode at position context + r
    for r in range(span):
        single = _run(gpu, pool, table, tb, [c + r for c in contexts], q[:, r:r + 1], 1, heads, scale, True, False,
                      max_context=max(lengths))
        close_enough(single[:, 0], want[:, r], f"row {r} alone")
        # (not the same bits: with several query tiles a row's sum is the sum of its weights as rounded to FP16, the ones the
        # values are multiplied by, formed by a product; the decode variant adds the weights before they are rounded)
        assert np.abs(single[:, 0] - got[:, r]).max() < 5e-4
    gpu.release(buffer); gpu.release(tb)


@pytest.mark.parametrize("dim,fmt,span,heads,kv_heads", [(128, "f16", 3, 16, 2), (128, "f16", 5, 32, 4), (128, "f16", 8, 32, 4),
                                                         (256, "q8", 2, 24, 2), (256, "f16", 2, 24, 2)])
def test_verify_span_rows_of_other_formats(gpu, oracle, dim, fmt, span, heads, kv_heads):
    # The few-rows kernel's variants of two, three and four query tiles over FP16 rows, and of two tiles over 256 columns: the
    # same walk as over Q8_0 rows of 128 columns with other row loads (and, at 128 columns, the rows' sums formed by a product).
    rng = np.random.default_rng(900 + dim + span)
    row_bytes = (dim + dim // 16) if fmt == "q8" else 2 * dim
    page_tokens = 64
    contexts = [0, 31, 64, 290, 1100]
    lengths = [c + span for c in contexts]
    pool, buffer, host, table, tb = make_pool(gpu, oracle, rng, lengths, kv_heads, dim, page_tokens, row_bytes,
                                              dtype=np.float32 if fmt == "q8" else np.float16)
    q = rng.standard_normal((len(lengths), span, heads, dim)).astype(np.float16).astype(np.float32)
    scale = 1.0 / np.sqrt(dim)
    want = oracle.paged_attention(host, row_bytes, page_tokens, kv_heads, dim, table, np.array(contexts, np.int32), q, scale)
    for q_f16, out_f16 in ((True, False), (False, True)):
        got = _run(gpu, pool, table, tb, contexts, q, span, heads, scale, q_f16, out_f16)
        close_enough(got, want, f"span {span} of {fmt} rows, {dim} columns")
    gpu.release(buffer); gpu.release(tb)


@pytest.mark.parametrize("dim,fmt,span,heads,kv_heads", [(128, "q8", 40, 32, 4), (128, "q8", 100, 8, 1), (128, "f16", 33, 16, 2),
                                                         (256, "q8", 24, 24, 2), (256, "f16", 9, 24, 2), (128, "q8", 9, 4, 4)])
@pytest.mark.parametrize("page_tokens", [64, 32])
def test_prefill_span_rows(gpu, oracle, dim, fmt, span, heads, kv_heads, page_tokens):
    # BASELINE config 2 in small: a chunk of new tokens attends the cache (which holds the chunk's own rows) causally.
    # Rows per K/V head = span * group exceed what the decode kernel's workgroup takes, so this is the many-rows kernel.
    rng = np.random.default_rng(77 + span + dim)
    # Pages of 32 tokens are shorter than the 64 keys a workgroup of the 256-column kernel takes at a time.
    row_bytes = (dim + dim // 16) if fmt == "q8" else 2 * dim
    contexts = [0, 31, 200, 517]
    lengths = [c + span for c in contexts]
    pool, buffer, host, table, tb = make_pool(gpu, oracle, rng, lengths, kv_heads, dim, page_tokens, row_bytes,
                                              dtype=np.float32 if fmt == "q8" else np.float16)
    seqs = len(lengths)
    q = rng.standard_normal((seqs, span, heads, dim)).astype(np.float16).astype(np.float32)
    scale = 1.0 / np.sqrt(dim)
    want = oracle.paged_attention(host, row_bytes, page_tokens, kv_heads, dim, table, np.array(contexts, np.int32), q, scale)
    for q_f16, out_f16 in ((True, False), (False, False), (True, True)):
        got = _run(gpu, pool, table, tb, contexts, q, span, heads, scale, q_f16, out_f16)
        if out_f16:
            assert np.abs(got - want).max() <= 2e-3 + 2.0 ** -11 * np.abs(want).max()
        else:
            close_enough(got, want, f"prefill span {span} dim {dim} {fmt}")
    # the span's last row is the single-token decode at the last position
    single = _run(gpu, pool, table, tb, [c + span - 1 for c in contexts], q[:, span - 1:], 1, heads, scale, True, False)
    got = _run(gpu, pool, table, tb, contexts, q, span, heads, scale, True, False)
    close_enough(single[:, 0], want[:, span - 1], "last row alone")
    assert np.abs(single[:, 0] - got[:, span - 1]).max() < 1e-3      # two kernels, two roundings of the FP16 weights
    gpu.release(buffer); gpu.release(tb)


@pytest.mark.parametrize("fmt", ["q8", "f16"])
def test_prefill_with_scores_that_keep_growing(gpu, oracle, fmt):
    # Keys whose scores rise along the sequence (k_t = t/8 * u + noise, queries along u) make every row's maximum outgrow its
    # reference again and again: the path that moves the references, scales what was summed and multiplies the step's scores
    # anew runs many times per row; rows of small and large magnitude sit side by side, one head has zero queries.
    rng = np.random.default_rng(91)
    dim, page_tokens, heads, kv_heads, span, context = 128, 64, 16, 2, 160, 300
    row_bytes = (dim + dim // 16) if fmt == "q8" else 2 * dim
    total = span + context
    pages = (total + page_tokens - 1) // page_tokens
    table = rng.permutation(pages + 1)[:pages].astype(np.int32).reshape(1, pages)
    host = np.zeros(oracle.pool_bytes(pages + 1, kv_heads, page_tokens, row_bytes), dtype=np.uint8)
    u = rng.standard_normal(dim).astype(np.float32)
    u /= np.linalg.norm(u)
    rise = (np.arange(total, dtype=np.float32) / 8.0)[None, :, None, None] * u[None, None, None, :]
    k = (rise + 0.3 * rng.standard_normal((1, total, kv_heads, dim))).astype(np.float16).astype(np.float32)
    v = rng.standard_normal((1, total, kv_heads, dim)).astype(np.float16).astype(np.float32)
    oracle.kv_write(host, row_bytes, page_tokens, kv_heads, dim, table, np.zeros(1, np.int32), k, v)
    pool, buffer = gpu.kv_pool(pages + 1, page_tokens, kv_heads, dim, row_bytes)
    gpu.write_buffer(buffer, 0, host)
    tb = gpu.upload(table)
    # (with Q8_0 rows the operands' FP16 rounding of values around 50 limits how sharp a softmax the 2e-3 bound can be asked
    # of: the decode kernel shows the same errors; FP16 rows carry no such rounding)
    strength = rng.choice([0.5, 4.0, 30.0] if fmt == "f16" else [0.5, 2.0, 4.0], size=(1, span, heads, 1)).astype(np.float32)
    q = (strength * u[None, None, None, :] + 0.2 * rng.standard_normal((1, span, heads, dim))).astype(np.float16).astype(np.float32)
    q[:, :, 3] = 0.0
    scale = 1.0 / np.sqrt(dim)
    want = oracle.paged_attention(host, row_bytes, page_tokens, kv_heads, dim, table, np.array([context], np.int32), q, scale)
    got = _run(gpu, pool, table, tb, [context], q, span, heads, scale, True, False)
    close_enough(got, want, f"growing scores {fmt}")
    for r in (0, 77, span - 1):                 # the decode kernel at the same rows: another route to the same numbers
        single = _run(gpu, pool, table, tb, [context + r], q[:, r:r + 1], 1, heads, scale, True, False, max_context=total)
        assert np.abs(single[:, 0] - got[:, r]).max() < 1e-3
    gpu.release(buffer); gpu.release(tb)


@pytest.mark.parametrize("fmt,span", [("q8", 5), ("q8", 8), ("f16", 3), ("f16", 8)])
def test_verify_span_with_scores_that_keep_growing(gpu, oracle, fmt, span):
    # The same rising keys under the few-rows kernel at two, three and four query tiles: a row's reference moves many times along
    # the walk, and what was summed by then -- the outputs and, with several tiles, the sums of weights a product forms -- is scaled
    # each time.  (A workgroup's share is 256 tokens here, along which a score rises by up to 16 in the exponent: a wave moves its
    # references once or twice after the first step.)
    rng = np.random.default_rng(191 + span)
    dim, page_tokens, heads, kv_heads, context = 128, 64, 16, 2, 600
    row_bytes = (dim + dim // 16) if fmt == "q8" else 2 * dim
    total = span + context
    pages = (total + page_tokens - 1) // page_tokens
    table = rng.permutation(pages + 1)[:pages].astype(np.int32).reshape(1, pages)
    host = np.zeros(oracle.pool_bytes(pages + 1, kv_heads, page_tokens, row_bytes), dtype=np.uint8)
    u = rng.standard_normal(dim).astype(np.float32)
    u /= np.linalg.norm(u)
    rise = (np.arange(total, dtype=np.float32) / 8.0)[None, :, None, None] * u[None, None, None, :]
    k = (rise + 0.3 * rng.standard_normal((1, total, kv_heads, dim))).astype(np.float16).astype(np.float32)
    v = rng.standard_normal((1, total, kv_heads, dim)).astype(np.float16).astype(np.float32)
    oracle.kv_write(host, row_bytes, page_tokens, kv_heads, dim, table, np.zeros(1, np.int32), k, v)
    pool, buffer = gpu.kv_pool(pages + 1, page_tokens, kv_heads, dim, row_bytes)
    gpu.write_buffer(buffer, 0, host)
    tb = gpu.upload(table)
    strength = rng.choice([0.5, 4.0, 30.0] if fmt == "f16" else [0.5, 2.0, 4.0], size=(1, span, heads, 1)).astype(np.float32)
    q = (strength * u[None, None, None, :] + 0.2 * rng.standard_normal((1, span, heads, dim))).astype(np.float16).astype(np.float32)
    q[:, :, 3] = 0.0
    scale = 1.0 / np.sqrt(dim)
    want = oracle.paged_attention(host, row_bytes, page_tokens, kv_heads, dim, table, np.array([context], np.int32), q, scale)
    got = _run(gpu, pool, table, tb, [context], q, span, heads, scale, True, False)
    close_enough(got, want, f"growing scores, span {span}, {fmt}")
    gpu.release(buffer); gpu.release(tb)


def test_prefill_in_chunks_equals_prefill_at_once(gpu, oracle):
    # a prompt prefilled in 4 chunks (each chunk attends the cache so far) gives the rows of one whole-prompt pass
    rng = np.random.default_rng(5)
    dim, row_bytes, page_tokens, heads, kv_heads, tokens, chunk = 128, 136, 64, 16, 2, 512, 128
    pool, buffer, host, table, tb = make_pool(gpu, oracle, rng, [tokens], kv_heads, dim, page_tokens, row_bytes)
    q = rng.standard_normal((1, tokens, heads, dim)).astype(np.float16).astype(np.float32)
    scale = 1.0 / np.sqrt(dim)
    whole = _run(gpu, pool, table, tb, [0], q, tokens, heads, scale, True, False)
    want = oracle.paged_attention(host, row_bytes, page_tokens, kv_heads, dim, table, np.zeros(1, np.int32), q, scale)
    close_enough(whole, want, "whole prompt")
    for c in range(tokens // chunk):
        part = _run(gpu, pool, table, tb, [c * chunk], q[:, c * chunk:(c + 1) * chunk], chunk, heads, scale, True, False,
                    max_context=tokens)
        assert np.array_equal(part, whole[:, c * chunk:(c + 1) * chunk])     # the same keys in the same order: the same bits
    gpu.release(buffer); gpu.release(tb)


def test_waves_of_64_rows_and_of_32(gpu, oracle):
    # The prompt kernel at 128 columns exists twice: waves of 64 query rows (queries and accumulators in the accumulation registers,
    # the default) and waves of 32.  Each meets the oracle; they agree to the rounding of the FP16 weights.  An odd number of
    # 128-row runs (the middle run is its own partner), rows past the span's end in the last run, several contexts, growing scores.
    rng = np.random.default_rng(404)
    dim, row_bytes, page_tokens, heads, kv_heads, span = 128, 136, 64, 24, 2, 203
    contexts = [0, 100, 701]
    pool, buffer, host, table, tb = make_pool(gpu, oracle, rng, [c + span for c in contexts], kv_heads, dim, page_tokens, row_bytes)
    q = (rng.standard_normal((len(contexts), span, heads, dim)) * rng.choice([0.3, 1.0, 1.5], size=(len(contexts), span, heads, 1)))
    q = q.astype(np.float16).astype(np.float32)
    scale = 1.0 / np.sqrt(dim)
    want = oracle.paged_attention(host, row_bytes, page_tokens, kv_heads, dim, table, np.array(contexts, np.int32), q, scale)
    try:
        gpu.prefill_wave_rows(32)
        narrow = _run(gpu, pool, table, tb, contexts, q, span, heads, scale, True, False)
        gpu.prefill_wave_rows(64)
        wide = _run(gpu, pool, table, tb, contexts, q, span, heads, scale, True, False)
        with pytest.raises(StraydogError, match="32 or 64 rows"):
            gpu.prefill_wave_rows(48)
    finally:
        gpu.prefill_wave_rows(64)
    close_enough(narrow, want, "waves of 32 rows")
    close_enough(wide, want, "waves of 64 rows")
    assert np.abs(narrow - wide).max() < 1e-3
    gpu.release(buffer); gpu.release(tb)


def test_many_short_sequences(gpu, oracle):
    # more sequences than a wave has lanes: the device's numbering of the work runs over several groups of 64 sequences;
    # some sequences hold a single token, some exactly a page
    rng = np.random.default_rng(404)
    dim, row_bytes, page_tokens, heads, kv_heads = 128, 136, 32, 8, 2
    lengths = [int(n) for n in rng.integers(1, 200, size=150)]
    lengths[3], lengths[64], lengths[149] = 1, 32, 64
    pool, buffer, host, table, tb = make_pool(gpu, oracle, rng, lengths, kv_heads, dim, page_tokens, row_bytes)
    seqs = len(lengths)
    q = rng.standard_normal((seqs, 1, heads, dim)).astype(np.float16).astype(np.float32)
    scale = 1.0 / np.sqrt(dim)
    positions = [n - 1 for n in lengths]
    got = _run(gpu, pool, table, tb, positions, q, 1, heads, scale, True, False)
    want = oracle.paged_attention(host, row_bytes, page_tokens, kv_heads, dim, table, np.array(positions, np.int32), q, scale)
    close_enough(got, want, "150 sequences")
    gpu.release(buffer); gpu.release(tb)


@pytest.mark.parametrize("span", [1, 3])
def test_shares_that_cross_sequences_and_heads(gpu, oracle, span):
    # the batch's tokens are cut into equal shares: one long sequence is spread over hundreds of workgroups, the short ones
    # around it are met several to a share, and a share ends anywhere (inside a sequence, at its end, between K/V heads);
    # max_context far above the longest sequence, as a server that sizes for the worst case would pass it
    rng = np.random.default_rng(808 + span)
    dim, row_bytes, page_tokens, heads, kv_heads = 128, 136, 64, 16, 4
    lengths = [int(n) for n in rng.integers(span, 600, size=20)] + [20000] + [int(n) for n in rng.integers(span, 600, size=20)]
    lengths[0], lengths[5], lengths[30] = span, 128, 129
    pool, buffer, host, table, tb = make_pool(gpu, oracle, rng, lengths, kv_heads, dim, page_tokens, row_bytes)
    seqs = len(lengths)
    q = rng.standard_normal((seqs, span, heads, dim)).astype(np.float16).astype(np.float32)
    scale = 1.0 / np.sqrt(dim)
    positions = [n - span for n in lengths]
    got = _run(gpu, pool, table, tb, positions, q, span, heads, scale, True, False, max_context=table.shape[1] * page_tokens)
    want = oracle.paged_attention(host, row_bytes, page_tokens, kv_heads, dim, table, np.array(positions, np.int32), q, scale)
    for s in range(seqs):
        close_enough(got[s], want[s], f"sequence {s} of {lengths[s]} tokens")
    gpu.release(buffer); gpu.release(tb)


def test_positions_outside_the_context_are_taken_as_its_nearest_end(gpu, oracle):
    # the positions live on the device, where the host cannot check them: a negative one counts as 0, one past max_context as
    # max_context, and the sequences beside them are not disturbed
    rng = np.random.default_rng(515)
    dim, row_bytes, page_tokens, heads, kv_heads = 128, 136, 64, 8, 2
    lengths = [300, 300, 300, 300]
    pool, buffer, host, table, tb = make_pool(gpu, oracle, rng, lengths, kv_heads, dim, page_tokens, row_bytes)
    q = rng.standard_normal((4, 1, heads, dim)).astype(np.float16).astype(np.float32)
    scale = 1.0 / np.sqrt(dim)
    max_context = 300
    given = [-7, 120, 2_000_000_000, 299]
    meant = [0, 120, 299, 299]          # (a position of max_context with a span of 1 sees all max_context tokens, as 299 does)
    got = _run(gpu, pool, table, tb, given, q, 1, heads, scale, True, False, max_context=max_context)
    want = oracle.paged_attention(host, row_bytes, page_tokens, kv_heads, dim, table, np.array(meant, np.int32), q, scale)
    for s in range(4):
        close_enough(got[s], want[s], f"position {given[s]}")
    gpu.release(buffer); gpu.release(tb)


def test_zero_queries_give_the_mean_of_the_values(gpu, oracle):
    rng = np.random.default_rng(5)
    heads, kv_heads, dim, row_bytes, page_tokens = 8, 2, 128, 136, 32
    lengths = [45, 200]
    pool, buffer, host, table, tb = make_pool(gpu, oracle, rng, lengths, kv_heads, dim, page_tokens, row_bytes)
    q = np.zeros((2, 1, heads, dim), dtype=np.float32)
    got = _run(gpu, pool, table, tb, [n - 1 for n in lengths], q, 1, heads, 0.088, False, False)
    want = oracle.paged_attention(host, row_bytes, page_tokens, kv_heads, dim, table, np.array([n - 1 for n in lengths], np.int32), q, 0.088)
    assert np.abs(got - want).max() < 1e-4
    gpu.release(buffer); gpu.release(tb)


def test_refusals(gpu):
    from straydog_amd.backend import StraydogError
    pool, buffer = gpu.kv_pool(2, 32, 1, 128, 136)
    small = gpu.buffer(64)
    with pytest.raises(StraydogError, match="outside this device's allocations"):
        gpu.paged_attention(pool, 0x1000, 1, small.base(), 32, small.base(), 0, 1, 1, 8, 0.1, small.base(), 0, small)
    with pytest.raises(StraydogError, match="scratch too small"):
        table = gpu.upload(np.zeros(4, np.int32))
        q = gpu.buffer(8 * 128 * 4)
        gpu.paged_attention(pool, table.base(), 1, table.base(), 32, q.base(), 0, 1, 1, 8, 0.1, q.base(), 0, small)
    with pytest.raises(StraydogError, match="invalid Straydog paged attention shape"):      # the scale must be positive
        gpu.paged_attention(pool, table.base(), 1, table.base(), 32, q.base(), 0, 1, 1, 8, 0.0, q.base(), 0, small)
    bad = type(pool)(buffer.pointer, 2, 33, 1, 128, 136)
    with pytest.raises(StraydogError, match="invalid Straydog K/V pool"):
        gpu.kv_write(bad, small.base(), 1, small.base(), small.base(), small.base(), False, 1, 1)


def test_the_library_kept_cache_pages_grow_fork_and_truncate(gpu, oracle):
    # sdx_kv_cache_*: sequences grow without copies, a fork shares whole pages and copies the partial one, a truncation gives pages
    # back.  What the sequences hold is checked through attention against the oracle on each sequence's own logical rows.
    from straydog_amd.backend import StraydogError
    rng = np.random.default_rng(44)
    page_tokens, kv_heads, dim, row_bytes, heads = 64, 2, 128, 136, 8
    cache, pool, table, stride = gpu.kv_cache(12, page_tokens, kv_heads, dim, row_bytes, 3, 1024)
    assert stride == 16 and gpu.kv_cache_usage(cache) == (0, 12)
    logical = {s: (np.zeros((0, kv_heads, dim), np.float32), np.zeros((0, kv_heads, dim), np.float32)) for s in range(3)}

    def append(sequence, count):
        k = rng.standard_normal((count, kv_heads, dim)).astype(np.float32)
        v = rng.standard_normal((count, kv_heads, dim)).astype(np.float32)
        start = logical[sequence][0].shape[0]
        gpu.kv_cache_reserve(cache, sequence, start + count)
        kb, vb, pb = gpu.upload(k), gpu.upload(v), gpu.upload(np.array([start], dtype=np.int32))
        gpu.kv_write(pool, table + sequence * stride * 4, stride, pb.base(), kb.base(), vb.base(), False, 1, count)
        for b in (kb, vb, pb):
            gpu.release(b)
        logical[sequence] = (np.concatenate([logical[sequence][0], k]), np.concatenate([logical[sequence][1], v]))

    def check(sequence):
        k, v = logical[sequence]
        length = k.shape[0]
        q = rng.standard_normal((1, 1, heads, dim)).astype(np.float32)
        qb, pb = gpu.upload(q), gpu.upload(np.array([length - 1], dtype=np.int32))
        out = gpu.buffer(q.size * 4)
        scratch = gpu.buffer(gpu.paged_attention_scratch(1, 1, heads, dim, 1024))
        gpu.paged_attention(pool, table + sequence * stride * 4, stride, pb.base(), 1024, qb.base(), False, 1, 1, heads, 0.09, out.base(), False, scratch)
        got = gpu.read_buffer(out, 0, np.float32, q.size).reshape(q.shape)
        # the oracle on the sequence's rows laid out in pages of its own
        pages = (length + page_tokens - 1) // page_tokens
        host = np.zeros(oracle.pool_bytes(pages, kv_heads, page_tokens, row_bytes), dtype=np.uint8)
        own = np.arange(pages, dtype=np.int32)[None, :]
        oracle.kv_write(host, row_bytes, page_tokens, kv_heads, dim, own, np.zeros(1, np.int32), k[None], v[None])
        want = oracle.paged_attention(host, row_bytes, page_tokens, kv_heads, dim, own, np.array([length - 1], np.int32), q, 0.09)
        close_enough(got, want, f"sequence {sequence} of {length} tokens")
        for b in (qb, pb, out, scratch):
            gpu.release(b)

    append(0, 200)                                   # 4 pages
    append(0, 1)
    check(0)
    assert gpu.kv_cache_usage(cache, 0) == (4, 8)
    gpu.kv_cache_fork(cache, 0, 1, 150)              # 2 whole pages shared, the third copied up to row 22
    logical[1] = (logical[0][0][:150].copy(), logical[0][1][:150].copy())
    assert gpu.kv_cache_usage(cache, 1) == (3, 7)
    append(1, 70)                                    # the fork writes on from position 150; the source's rows 150.. are untouched
    append(0, 100)
    check(0); check(1)
    assert gpu.kv_cache_usage(cache, 0) == (5, 5) and gpu.kv_cache_usage(cache, 1) == (4, 5)
    gpu.kv_cache_truncate(cache, 1, 130)             # a rewind: the fork's fourth page goes back, its copy of the third stays
    logical[1] = (logical[1][0][:130], logical[1][1][:130])
    assert gpu.kv_cache_usage(cache, 1) == (3, 6)
    append(1, 5)                                     # rows 130..134 land in the fork's own copy of page 3
    check(1); check(0)
    gpu.kv_cache_truncate(cache, 0, 0)               # the source goes: the shared pages stay with the fork
    assert gpu.kv_cache_usage(cache, 0) == (0, 9)
    check(1)
    append(2, 9 * page_tokens)                       # exactly what is free
    check(2)
    with pytest.raises(StraydogError, match="out of pages"):
        gpu.kv_cache_reserve(cache, 0, 1)
    assert gpu.kv_cache_usage(cache, 0) == (0, 0)
    with pytest.raises(StraydogError, match="max_context"):
        gpu.kv_cache_reserve(cache, 0, 1025)
    with pytest.raises(StraydogError, match="no such sequence"):
        gpu.kv_cache_reserve(cache, 3, 1)
    with pytest.raises(StraydogError, match="fork"):
        gpu.kv_cache_fork(cache, 1, 2, 10)
    gpu.kv_cache_destroy(cache)
    used, _ = gpu.memory()
    with pytest.raises(StraydogError):
        gpu.kv_cache(0, 64, 2, 128, 136, 1, 64)
    assert gpu.memory()[0] == used, "a refused cache leaves no allocation behind"


def test_a_rewind_into_a_shared_page_continues_on_a_copy(gpu, oracle):
    # a fork at a page boundary shares whole pages; when either sequence rewinds to a position inside a shared page and
    # appends, its new rows must not overwrite the rows the sibling still attends to
    from straydog_amd.backend import StraydogError
    rng = np.random.default_rng(45)
    page_tokens, kv_heads, dim, row_bytes, heads = 64, 2, 128, 136, 8
    cache, pool, table, stride = gpu.kv_cache(12, page_tokens, kv_heads, dim, row_bytes, 2, 512)
    logical = {}

    def append(sequence, count):
        k = rng.standard_normal((count, kv_heads, dim)).astype(np.float32)
        v = rng.standard_normal((count, kv_heads, dim)).astype(np.float32)
        have = logical.get(sequence, (np.zeros((0, kv_heads, dim), np.float32),) * 2)
        start = have[0].shape[0]
        gpu.kv_cache_reserve(cache, sequence, start + count)
        kb, vb, pb = gpu.upload(k), gpu.upload(v), gpu.upload(np.array([start], dtype=np.int32))
        gpu.kv_write(pool, table + sequence * stride * 4, stride, pb.base(), kb.base(), vb.base(), False, 1, count)
        for b in (kb, vb, pb):
            gpu.release(b)
        logical[sequence] = (np.concatenate([have[0], k]), np.concatenate([have[1], v]))

    def check(sequence):
        k, v = logical[sequence]
        length = k.shape[0]
        q = rng.standard_normal((1, 1, heads, dim)).astype(np.float32)
        qb, pb = gpu.upload(q), gpu.upload(np.array([length - 1], dtype=np.int32))
        out = gpu.buffer(q.size * 4)
        scratch = gpu.buffer(gpu.paged_attention_scratch(1, 1, heads, dim, 512))
        gpu.paged_attention(pool, table + sequence * stride * 4, stride, pb.base(), 512, qb.base(), False, 1, 1, heads, 0.09, out.base(), False, scratch)
        got = gpu.read_buffer(out, 0, np.float32, q.size).reshape(q.shape)
        pages = (length + page_tokens - 1) // page_tokens
        host = np.zeros(oracle.pool_bytes(pages, kv_heads, page_tokens, row_bytes), dtype=np.uint8)
        own = np.arange(pages, dtype=np.int32)[None, :]
        oracle.kv_write(host, row_bytes, page_tokens, kv_heads, dim, own, np.zeros(1, np.int32), k[None], v[None])
        want = oracle.paged_attention(host, row_bytes, page_tokens, kv_heads, dim, own, np.array([length - 1], np.int32), q, 0.09)
        close_enough(got, want, f"sequence {sequence} of {length} tokens")
        for b in (qb, pb, out, scratch):
            gpu.release(b)

    append(0, 128)                                   # two whole pages
    gpu.kv_cache_fork(cache, 0, 1, 128)              # both shared, nothing copied
    logical[1] = (logical[0][0].copy(), logical[0][1].copy())
    assert gpu.kv_cache_usage(cache, 1) == (2, 10)
    gpu.kv_cache_truncate(cache, 1, 100)             # into the shared second page: the fork takes a copy of its rows 64..99
    logical[1] = (logical[1][0][:100], logical[1][1][:100])
    assert gpu.kv_cache_usage(cache, 1) == (2, 9)
    append(1, 20)                                    # rows 100..119 of the fork
    check(1); check(0)                               # the source still reads its own rows 100..127
    gpu.kv_cache_truncate(cache, 0, 70)              # the source rewinds below the fork point: its second page is its own by now
    logical[0] = (logical[0][0][:70], logical[0][1][:70])
    append(0, 10)
    check(0); check(1)
    gpu.kv_cache_truncate(cache, 0, 30)              # into the first page, which the fork still shares
    logical[0] = (logical[0][0][:30], logical[0][1][:30])
    append(0, 3)
    check(0); check(1)
    # with no page free for the copy the rewind is refused and changes nothing
    append(1, 512 - 120)
    assert gpu.kv_cache_usage(cache, 1) == (8, 3)
    gpu.kv_cache_truncate(cache, 0, 0)
    assert gpu.kv_cache_usage(cache, 0) == (0, 4)
    gpu.kv_cache_fork(cache, 1, 0, 64)               # the first page shared again
    gpu.kv_cache_reserve(cache, 0, 320)              # takes the four free pages
    with pytest.raises(StraydogError, match="out of pages"):
        gpu.kv_cache_truncate(cache, 1, 10)          # page 0 is shared with sequence 0 and no page is left for a copy
    assert gpu.kv_cache_usage(cache, 1)[0] == 8
    check(1)
    gpu.kv_cache_destroy(cache)


def test_rows_at_positions_outside_the_table_are_not_written(gpu, oracle):
    # K/V positions are read on the device: a negative one, one past the sequence's table row, or a table entry that names no
    # page of the pool stores nothing, and the rows of the sequences beside it keep their bytes
    rng = np.random.default_rng(616)
    dim, row_bytes, page_tokens, kv_heads, seqs, span = 128, 136, 32, 2, 5, 3
    stride, pages = 2, 12
    table = np.arange(seqs * stride, dtype=np.int32).reshape(seqs, stride)
    table[4, 1] = 4000                               # names no page
    pool, buffer = gpu.kv_pool(pages, page_tokens, kv_heads, dim, row_bytes)
    before = rng.integers(0, 255, size=buffer.size, dtype=np.uint8)
    gpu.write_buffer(buffer, 0, before)
    positions = np.array([-2, 62, 10, 2_000_000_000, 31], dtype=np.int32)
    keys = rng.standard_normal((seqs, span, kv_heads, dim)).astype(np.float32)
    values = rng.standard_normal((seqs, span, kv_heads, dim)).astype(np.float32)
    tb, pb, kb, vb = gpu.upload(table), gpu.upload(positions), gpu.upload(keys), gpu.upload(values)
    gpu.kv_write(pool, tb.base(), stride, pb.base(), kb.base(), vb.base(), False, seqs, span)
    got = gpu.read_buffer(buffer, 0, np.uint8, buffer.size)
    want = before.copy()
    # what should have been stored: sequence 1 rows at 62, 63 (64 is past its table row), sequence 2 rows at 10..12, sequence 4
    # row at 31 (32 and 33 fall into the page that does not exist); sequences 0 and 3 nothing
    for s, rows in ((1, [0, 1]), (2, [0, 1, 2]), (4, [0])):
        for r in rows:
            one = np.array([[int(positions[s]) + r]], dtype=np.int32).reshape(1)
            oracle.kv_write(want, row_bytes, page_tokens, kv_heads, dim, table[s:s + 1], one, keys[s:s + 1, r:r + 1], values[s:s + 1, r:r + 1])
    assert np.array_equal(got, want)
    for b in (tb, pb, kb, vb, buffer):
        gpu.release(b)


def test_table_entries_outside_the_pool_read_inside_it(gpu, oracle):
    # a page-table entry that names no page of the pool is read as the pool's last page (never memory outside the pool); the
    # sequences beside it are not disturbed
    rng = np.random.default_rng(717)
    dim, row_bytes, page_tokens, heads, kv_heads = 128, 136, 64, 8, 2
    lengths = [200, 200, 200]
    pool, buffer, host, table, tb = make_pool(gpu, oracle, rng, lengths, kv_heads, dim, page_tokens, row_bytes, spare_pages=0)
    last = int(pool.page_count) - 1
    bad = table.copy()
    bad[1, 2] = -5
    bad[1, 3] = 1 << 30
    meant = table.copy()
    meant[1, 2] = last
    meant[1, 3] = last
    bb = gpu.upload(bad)
    q = rng.standard_normal((3, 1, heads, dim)).astype(np.float16).astype(np.float32)
    scale = 1.0 / np.sqrt(dim)
    got = _run(gpu, pool, bad, bb, [199, 199, 199], q, 1, heads, scale, True, False)
    want = oracle.paged_attention(host, row_bytes, page_tokens, kv_heads, dim, meant, np.array([199, 199, 199], np.int32), q, scale)
    for s in range(3):
        close_enough(got[s], want[s], f"sequence {s}")
    for b in (buffer, tb, bb):
        gpu.release(b)


@pytest.mark.parametrize("pages,page_tokens,kv_heads,dim,row_bytes", [(37, 64, 2, 128, 136), (5, 256, 4, 128, 136), (3, 32, 1, 256, 272), (9, 64, 3, 128, 256),
                                                                      (4, 32, 2, 256, 512)])
def test_paged_stream_probe_reads_the_whole_pool(gpu, pages, page_tokens, kv_heads, dim, row_bytes):
    # the harness probe that walks a pool in the decode kernel's order: every layout the pools take, pools smaller than the
    # launch has workgroups; it reports the pool's bytes and leaves the pool as it was
    pool, buffer = gpu.kv_pool(pages, page_tokens, kv_heads, dim, row_bytes)
    size = pages * 2 * kv_heads * page_tokens * row_bytes
    before = np.random.default_rng(pages).integers(0, 256, size=size, dtype=np.uint8)
    gpu.write_buffer(buffer, 0, before)
    assert gpu.paged_stream_probe(pool) == size
    gpu.synchronize()
    assert np.array_equal(gpu.read_buffer(buffer, 0, np.uint8, size), before)
    gpu.release(buffer)
