"""sdx_prefill_chunk through the C ABI: a prompt chunk's K/V append and attention in one call, with the cached rows' FP16
operand tiles kept in the caller's buffer between the chunks.  It must leave the cache bytes of sdx_kv_write and give the
output bits of sdx_paged_attention on the same arguments (the reference's prompt pass writes the chunk's rows and then
attends them, gpu/kernels.cpp:79-98 and gpu/qsa_prompt_attention.hpp:220-234), whatever the chunk size, the row format, the
input type, and whatever the tile buffer holds that `valid` does not vouch for; and it agrees with the oracle."""
import numpy as np
import pytest

from gpu_util import backend, close_enough
from straydog_amd.backend import StraydogError

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gpu():
    with backend() as handle:
        yield handle


class Prompt:
    """Sequences prefilled chunk by chunk twice: by sdx_kv_write + sdx_paged_attention into one pool, by sdx_prefill_chunk into
    another (same page table), so bytes and bits can be compared after every chunk."""

    def __init__(self, gpu, rng, seqs, context, heads, kv_heads, fmt, page_tokens, input_f16):
        self.gpu, self.seqs, self.context, self.heads, self.kv_heads, self.page_tokens = gpu, seqs, context, heads, kv_heads, page_tokens
        self.dim, self.input_f16 = 128, input_f16
        self.row_bytes = 136 if fmt == "q8" else 256
        per = (context + page_tokens - 1) // page_tokens
        self.pages = seqs * per + 2
        self.table = rng.permutation(self.pages)[:seqs * per].astype(np.int32).reshape(seqs, per)
        self.pool_a, self.buffer_a = gpu.kv_pool(self.pages, page_tokens, kv_heads, self.dim, self.row_bytes)
        self.pool_b, self.buffer_b = gpu.kv_pool(self.pages, page_tokens, kv_heads, self.dim, self.row_bytes)
        self.tb = gpu.upload(self.table)
        self.tiles = gpu.buffer(gpu.prefill_tiles_bytes(seqs, kv_heads, self.dim, context))
        # the tile buffer starts as rubbish: whatever `valid` does not vouch for must be rebuilt
        gpu.write_buffer(self.tiles, 0, rng.integers(0, 256, size=min(self.tiles.size, 1 << 20), dtype=np.uint8))
        self.scale = float(1.0 / np.sqrt(self.dim))
        self.pool_size = self.pages * 2 * kv_heads * page_tokens * self.row_bytes

    def chunk(self, rng, positions, span, valid="positions", append=True):
        gpu, dim = self.gpu, self.dim
        kind = np.float16 if self.input_f16 else np.float32
        k = rng.standard_normal((self.seqs, span, self.kv_heads, dim)).astype(kind)
        v = rng.standard_normal((self.seqs, span, self.kv_heads, dim)).astype(kind)
        q = rng.standard_normal((self.seqs, span, self.heads, dim)).astype(np.float16)
        kb, vb, qb = gpu.upload(k), gpu.upload(v), gpu.upload(q)
        pb = gpu.upload(np.asarray(positions, dtype=np.int32))
        count = self.seqs * span * self.heads * dim
        out_a, out_b = gpu.buffer(count * 4), gpu.buffer(count * 4)
        scratch = gpu.buffer(max(gpu.paged_attention_scratch(self.seqs, span, self.heads, dim, self.context), 4))
        stride = self.table.shape[1]
        gpu.kv_write(self.pool_a, self.tb.base(), stride, pb.base(), kb.base(), vb.base(), self.input_f16, self.seqs, span)
        gpu.paged_attention(self.pool_a, self.tb.base(), stride, pb.base(), self.context, qb.base(), True, self.seqs, span, self.heads, self.scale,
                            out_a.base(), False, scratch)
        if not append:          # the rows are in the second cache already: the call only attends
            gpu.kv_write(self.pool_b, self.tb.base(), stride, pb.base(), kb.base(), vb.base(), self.input_f16, self.seqs, span)
        vbuf = None
        if valid == "positions":
            valid_pointer = pb.base()
        elif valid is None:
            valid_pointer = None
        else:
            vbuf = gpu.upload(np.asarray(valid, dtype=np.int32))
            valid_pointer = vbuf.base()
        gpu.prefill_chunk(self.pool_b, self.tb.base(), stride, pb.base(), self.context, kb.base() if append else None, vb.base() if append else None,
                          self.input_f16, qb.base(), True, self.seqs, span, self.heads, self.scale, out_b.base(), False, self.tiles, valid_pointer)
        a = gpu.read_buffer(out_a, 0, np.float32, count).reshape(self.seqs, span, self.heads, dim)
        b = gpu.read_buffer(out_b, 0, np.float32, count).reshape(self.seqs, span, self.heads, dim)
        for buffer in (kb, vb, qb, pb, out_a, out_b, scratch) + ((vbuf,) if vbuf else ()):
            gpu.release(buffer)
        return a, b, q.astype(np.float32)

    def pools(self):
        return (self.gpu.read_buffer(self.buffer_a, 0, np.uint8, self.pool_size), self.gpu.read_buffer(self.buffer_b, 0, np.uint8, self.pool_size))

    def release(self):
        for buffer in (self.buffer_a, self.buffer_b, self.tb, self.tiles):
            self.gpu.release(buffer)


@pytest.mark.parametrize("fmt,input_f16,page_tokens,span", [("q8", True, 64, 128), ("q8", False, 32, 100), ("f16", True, 256, 72), ("f16", False, 64, 200)])
def test_chunks_leave_the_writers_bytes_and_give_the_attentions_bits(gpu, oracle, fmt, input_f16, page_tokens, span):
    rng = np.random.default_rng(1000 * page_tokens + span + (7 if input_f16 else 0))
    prompt = Prompt(gpu, rng, seqs=2, context=5 * span + 40, heads=16, kv_heads=2, fmt=fmt, page_tokens=page_tokens, input_f16=input_f16)
    first = prompt.chunk(rng, [0, 0], 40)
    assert np.array_equal(first[0], first[1])
    # the second sequence goes back 16 positions and writes them again: from here on the two are at different positions, neither
    # a multiple of a tile's 64 keys, and the tile the rewind lands in is rebuilt in part from the cache, in part from the new rows
    base = np.array([40, 24])
    for c in range(5):
        positions = base + c * span
        a, b, q = prompt.chunk(rng, positions, span)
        assert np.array_equal(a, b), f"chunk {c}: outputs differ from sdx_paged_attention's"
        pool_a, pool_b = prompt.pools()
        assert np.array_equal(pool_a, pool_b), f"chunk {c}: cache bytes differ from sdx_kv_write's"
    # the last chunk against the oracle, on the bytes the cache holds
    positions = base + 4 * span
    want = oracle.paged_attention(pool_b, prompt.row_bytes, page_tokens, 2, 128, prompt.table, positions.astype(np.int32), q, prompt.scale)
    close_enough(b, want, "the last chunk against the oracle")
    prompt.release()


def test_what_valid_does_not_vouch_for_is_rebuilt(gpu, oracle):
    rng = np.random.default_rng(61)
    prompt = Prompt(gpu, rng, seqs=2, context=700, heads=8, kv_heads=1, fmt="q8", page_tokens=64, input_f16=True)
    a, b, _ = prompt.chunk(rng, [0, 0], 300, valid=None)                 # no vouching at all: every tile rebuilt
    assert np.array_equal(a, b)
    a, b, _ = prompt.chunk(rng, [300, 300], 100, valid=[300, 0])         # the second sequence's tiles are said to be stale
    assert np.array_equal(a, b)
    # rubbish over the tiles, and a count that vouches for nothing: the call rebuilds them from the cache
    gpu.write_buffer(prompt.tiles, 0, np.full(min(prompt.tiles.size, 1 << 20), 0xff, np.uint8))
    a, b, _ = prompt.chunk(rng, [400, 400], 100, valid=[0, 0])
    assert np.array_equal(a, b)
    # a count above the chunk's own position counts as the position; a negative one as none
    a, b, _ = prompt.chunk(rng, [500, 500], 64, valid=[9999, -5])
    assert np.array_equal(a, b)
    # rows that are in the cache already: attention only (keys and values null), tiles kept from before
    a, b, _ = prompt.chunk(rng, [564, 564], 100, append=False)
    assert np.array_equal(a, b)
    assert np.array_equal(*prompt.pools())
    prompt.release()


def test_a_short_span_and_a_single_row(gpu, oracle):
    # spans the decode kernel would take go through the same two launches here
    rng = np.random.default_rng(62)
    prompt = Prompt(gpu, rng, seqs=3, context=300, heads=32, kv_heads=4, fmt="q8", page_tokens=32, input_f16=False)
    at = 0
    for span in (130, 1, 5, 64, 33):
        a, b, q = prompt.chunk(rng, [at] * 3, span)
        close_enough(b, a, f"span {span} against the decode / prefill kernels")
        assert np.array_equal(*prompt.pools())
        at += span
    want = oracle.paged_attention(prompt.pools()[1], prompt.row_bytes, 32, 4, 128, prompt.table, np.full(3, at - 33, np.int32), q, prompt.scale)
    close_enough(b, want, "against the oracle")
    prompt.release()


def test_refusals(gpu):
    rng = np.random.default_rng(63)
    prompt = Prompt(gpu, rng, seqs=1, context=256, heads=8, kv_heads=2, fmt="q8", page_tokens=64, input_f16=True)
    k = gpu.upload(np.zeros((1, 64, 2, 128), np.float16))
    q = gpu.upload(np.zeros((1, 64, 8, 128), np.float16))
    out = gpu.buffer(64 * 8 * 128 * 4)
    pb = gpu.upload(np.zeros(1, np.int32))
    small = gpu.buffer(prompt.tiles.size - 1024)
    args = lambda tiles, keys=k.base(), values=k.base(), context=256: (prompt.pool_b, prompt.tb.base(), prompt.table.shape[1], pb.base(), context, keys, values,
                                                                      True, q.base(), True, 1, 64, 8, prompt.scale, out.base(), False, tiles, None)
    with pytest.raises(StraydogError, match="tile buffer is too small"):
        gpu.prefill_chunk(*args(small))
    with pytest.raises(StraydogError, match="invalid Straydog prefill chunk shape"):
        gpu.prefill_chunk(*args(prompt.tiles, values=None))
    with pytest.raises(StraydogError, match="invalid Straydog prefill chunk shape"):
        gpu.prefill_chunk(*args(prompt.tiles, context=100000))
    wide, wide_buffer = gpu.kv_pool(2, 64, 2, 256, 272)
    with pytest.raises(StraydogError, match="128 columns only"):
        gpu.prefill_chunk(wide, prompt.tb.base(), prompt.table.shape[1], pb.base(), 64, None, None, True, q.base(), True, 1, 16, 8, prompt.scale,
                          out.base(), False, prompt.tiles, None)
    assert gpu.prefill_tiles_bytes(1, 2, 256, 256) == 0 and gpu.prefill_tiles_bytes(3, 2, 128, 130) == 3 * 2 * 3 * 32768
    for buffer in (k, q, out, pb, small, wide_buffer):
        gpu.release(buffer)
    prompt.release()
