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
