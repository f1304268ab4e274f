"""Seeded random shapes of sdx_paged_attention through the C ABI against the oracle: the hand-picked cases of
test_gpu_paged.py fix the boundaries somebody thought of; these draw column counts, row formats, head groupings, spans,
page sizes, batch sizes and length mixes together (a draw of 256 columns, pages of 32 tokens and a long span once found
a kernel that took a step's keys for contiguous across a page boundary).  Same bar: max-abs 2e-3 and relative 1e-2."""
import numpy as np
import pytest

from gpu_util import backend, close_enough, make_pool
from test_gpu_paged import _run

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gpu():
    with backend() as handle:
        yield handle


def _draw(draw, spans):
    dim = int(draw.choice([128, 128, 256]))
    fmt = str(draw.choice(["q8", "q8", "f16"]))
    kv_heads = int(draw.choice([1, 2, 4]))
    group = int(draw.choice([1, 4, 8, 12]))
    span = int(draw.integers(spans[0], spans[1]))
    page_tokens = int(draw.choice([32, 64, 256]))
    return dim, fmt, kv_heads, group, span, page_tokens


def _compare(gpu, oracle, case, dim, fmt, kv_heads, group, span, page_tokens, lengths, worst_case_context):
    rng = np.random.default_rng(1000 + case)
    heads, seqs = kv_heads * group, len(lengths)
    row_bytes = dim + dim // 16 if fmt == "q8" else 2 * dim
    pool, buffer, host, table, tb = make_pool(gpu, oracle, rng, lengths, kv_heads, dim, page_tokens, row_bytes)
    q = rng.standard_normal((seqs, span, heads, dim)).astype(np.float16).astype(np.float32)
    scale = 1.0 / np.sqrt(dim)
    positions = [n - span for n in lengths]
    got = _run(gpu, pool, table, tb, positions, q, span, heads, scale, True, False,
               max_context=table.shape[1] * page_tokens if worst_case_context else None)
    want = oracle.paged_attention(host, row_bytes, page_tokens, kv_heads, dim, table, np.array(positions, np.int32), q, scale)
    close_enough(got, want, f"case {case}: dim {dim} {fmt} kv {kv_heads} group {group} span {span} pages of {page_tokens}, {seqs} sequences")
    gpu.release(buffer); gpu.release(tb)


def test_decode_and_verify_shapes(gpu, oracle):
    draw = np.random.default_rng(7)
    for case in range(32):
        dim, fmt, kv_heads, group, span, page_tokens = _draw(draw, (1, 7))
        most_rows = 64 if dim == 128 else 32                 # what the few-rows kernel takes per K/V head
        if span * group > most_rows:
            span = max(1, most_rows // group)
        seqs = int(draw.integers(1, 70))
        top = int(draw.choice([40, 300, 3000]))
        lengths = [int(n) for n in draw.integers(span, top + span, size=seqs)]
        if draw.random() < 0.3:
            lengths[int(draw.integers(0, seqs))] = int(draw.integers(5000, 20000))
        _compare(gpu, oracle, case, dim, fmt, kv_heads, group, span, page_tokens, lengths, draw.random() < 0.5)


def test_prefill_span_shapes(gpu, oracle):
    draw = np.random.default_rng(11)
    for case in range(24):
        dim, fmt, kv_heads, group, span, page_tokens = _draw(draw, (6, 150))
        seqs = int(draw.integers(1, 6))
        top = int(draw.choice([40, 300, 3000]))
        lengths = [int(n) for n in draw.integers(span, top + span, size=seqs)]
        _compare(gpu, oracle, 500 + case, dim, fmt, kv_heads, group, span, page_tokens, lengths, draw.random() < 0.5)


def test_sparse_path_shapes(gpu, oracle):
    # the batched sparse path on drawn shapes.  Indexer: the matrix-core path (no scores asked for) against the all-canonical one
    # (whose scores the oracle pins bit for bit in test_gpu_ops.py), indices bit for bit -- head counts, row lengths around the
    # kernels' segment and tile sizes, k from 1 to more than the row, bands of equal scores, negative weights, large values,
    # short visible lengths.  Gather attention: drawn batch, k, head count and holes against the oracle.
    draw = np.random.default_rng(2024)
    for case in range(20):
        heads, batch = int(draw.choice([16, 32, 48, 64])), int(draw.integers(1, 5))
        groups = int(draw.choice([1, 63, 100, 1024, 1025, 3000, 4097, 7000, 20000, 66000]))
        k = int(draw.choice([1, 7, 64, 512, 2048, 4096]))
        kind = str(draw.choice(["plain", "ties", "same", "negative", "large"]))
        q = draw.standard_normal((batch, heads, 128)).astype(np.float32)
        keys = draw.standard_normal((batch, groups, 128)).astype(np.float32)
        weights = draw.random((batch, heads)).astype(np.float32)
        if kind == "ties":
            keys = keys[:, draw.integers(0, max(groups // 50, 1), size=groups), :]      # many keys equal: wide bands of equal scores
        if kind == "same":
            keys[:] = keys[:, :1, :]
        if kind == "negative":
            weights = -weights
        if kind == "large":
            keys *= 50.0; q *= 20.0
        visible = draw.integers(0, groups + 1, size=batch).astype(np.int32)
        if draw.random() < 0.5:
            visible[:] = groups
        qb, kb, wb, vb = gpu.upload(oracle.to_bf16(q)), gpu.upload(oracle.to_bf16(keys)), gpu.upload(weights), gpu.upload(visible)
        scores, exact, fast = gpu.buffer(batch * groups * 4), gpu.buffer(batch * k * 4), gpu.buffer(batch * k * 4)
        gpu.index_top_k(qb.base(), kb.base(), wb.base(), vb.base(), batch, groups, heads, 128, 0.37, scores.base(), k, exact.base())
        gpu.index_top_k(qb.base(), kb.base(), wb.base(), vb.base(), batch, groups, heads, 128, 0.37, None, k, fast.base())
        want, got = gpu.read_buffer(exact, 0, np.int32, batch * k), gpu.read_buffer(fast, 0, np.int32, batch * k)
        assert np.array_equal(got, want), f"case {case}: {heads} heads, batch {batch}, {groups} groups, k {k}, {kind}"
        for b in (qb, kb, wb, vb, scores, exact, fast):
            gpu.release(b)
    kdim, vdim = 576, 512
    for case in range(8):
        batch, heads = int(draw.choice([1, 2, 5, 16, 40])), int(draw.choice([8, 16, 32, 40, 64]))
        groups, k = int(draw.integers(50, 3000)), int(draw.choice([1, 33, 64, 100, 129, 700]))
        q_bits = oracle.to_bf16(draw.standard_normal((batch, heads, kdim)).astype(np.float32))
        lat_bits = oracle.to_bf16(draw.standard_normal((batch, groups, kdim)).astype(np.float32))
        q_vals = (q_bits.astype(np.uint32) << 16).view(np.float32).reshape(batch, heads, kdim)
        selected = draw.integers(0, groups, size=(batch, k)).astype(np.int32)          # (repeats allowed: a row listed twice counts twice)
        selected[draw.random((batch, k)) < 0.1] = -1
        selected[:, 0] = 0                                                            # (no row of the batch without a listed row)
        qb, lb, sb, out = gpu.upload(q_bits), gpu.upload(lat_bits), gpu.upload(selected), gpu.buffer(batch * heads * vdim * 4)
        scale = float(1.0 / np.sqrt(kdim))
        gpu.latent_attention(qb.base(), lb.base(), sb.base(), batch, groups, k, heads, kdim, vdim, scale, out.base())
        got = gpu.read_buffer(out, 0, np.float32, batch * heads * vdim).reshape(batch, heads, vdim)
        for b in range(batch):
            want = oracle.latent_attention(q_vals[b:b + 1], None, None, 0, lat_bits[b], selected[b:b + 1], None, vdim, scale)
            close_enough(got[b], want[0], f"gather case {case}: batch {batch}, {heads} heads, {groups} rows, k {k}, sequence {b}")
        for b in (qb, lb, sb, out):
            gpu.release(b)
