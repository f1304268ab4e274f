"""Pins the oracle's attention functions (CPU only).

Independent checks: a float64 numpy softmax(QK^T)V over the dequantised cache, with the derived error
bound of crates/straydog-engine/tests/attention_gpu.rs:28-31,66,81; invariants the mathematics fixes
(weights sum to one, a zero query gives the mean of the values, permuting physical pages changes
nothing, a verify row equals the single-token call at its position, one page equals the unpaged plane
layout of gpu/kernels.cpp:79-98); and brute force on tiny shapes.
"""
import numpy as np
import pytest


def _xorshift_floats(seed, count):
    # crates/straydog-engine/tests/attention_gpu.rs:10-20
    out = np.zeros(count, dtype=np.float32)
    s = seed
    mask = (1 << 64) - 1
    for i in range(count):
        s ^= (s << 13) & mask
        s ^= s >> 7
        s ^= (s << 17) & mask
        out[i] = np.float32(s >> 40) / np.float32(1 << 23) - np.float32(1.0)
    return out


def _f64_attention(q, k, v, length, scale):
    """q [heads][dim], k/v [tokens][kv][dim] float32 -> float64 [heads][dim]."""
    heads, kv_heads = q.shape[0], k.shape[1]
    out = np.zeros(q.shape, dtype=np.float64)
    for h in range(heads):
        kh = h // (heads // kv_heads)
        s = (k[:length, kh].astype(np.float64) @ q[h].astype(np.float64)) * float(np.float32(scale))
        w = np.exp(s - s.max())
        out[h] = (w / w.sum()) @ v[:length, kh].astype(np.float64)
    return out


def _build_pool(oracle, rng, seqs, lengths, kv_heads, dim, page_tokens, row_bytes):
    pages_per = [(n + page_tokens - 1) // page_tokens for n in lengths]
    total = sum(pages_per)
    order = rng.permutation(total + 3)          # a few unused pages too
    table = np.full((seqs, max(pages_per)), -1, dtype=np.int32)
    at = 0
    for s in range(seqs):
        table[s, :pages_per[s]] = order[at:at + pages_per[s]]
        at += pages_per[s]
    pool = np.zeros(oracle.pool_bytes(total + 3, kv_heads, page_tokens, row_bytes), dtype=np.uint8)
    ks, vs = [], []
    for s in range(seqs):
        k = rng.standard_normal((1, lengths[s], kv_heads, dim)).astype(np.float32)
        v = rng.standard_normal((1, lengths[s], kv_heads, dim)).astype(np.float32)
        oracle.kv_write(pool, row_bytes, page_tokens, kv_heads, dim, table[s:s + 1], np.zeros(1, np.int32), k, v)
        ks.append(k[0]); vs.append(v[0])
    return pool, table, ks, vs


def _dequant(oracle, x, dim, row_bytes):
    if row_bytes == 2 * dim:
        return x.astype(np.float16).astype(np.float32)
    return oracle.kv_q8_values(oracle.kv_q8_row(x), dim)


@pytest.mark.parametrize("dim,row_bytes", [(128, 136), (128, 256), (256, 272)])
def test_paged_attention_matches_f64_softmax(oracle, dim, row_bytes):
    rng = np.random.default_rng(10 + dim + row_bytes)
    seqs, kv_heads, heads, page_tokens = 3, 2, 8, 16
    lengths = [37, 16, 1]
    pool, table, ks, vs = _build_pool(oracle, rng, seqs, lengths, kv_heads, dim, page_tokens, row_bytes)
    q = rng.standard_normal((seqs, 1, heads, dim)).astype(np.float32)
    scale = 1.0 / np.sqrt(dim)
    positions = np.array([n - 1 for n in lengths], dtype=np.int32)
    out, out64 = oracle.paged_attention(pool, row_bytes, page_tokens, kv_heads, dim, table, positions, q, scale, wide=True)
    for s in range(seqs):
        k = _dequant(oracle, ks[s], dim, row_bytes)
        v = _dequant(oracle, vs[s], dim, row_bytes)
        want = _f64_attention(q[s, 0], k, v, lengths[s], scale)
        assert np.allclose(out64[s, 0], want, rtol=0, atol=1e-12)
        assert np.abs(out[s, 0] - want).max() < 2e-5


def test_paged_attention_page_permutation_and_span_rows(oracle):
    rng = np.random.default_rng(5)
    kv_heads, heads, dim, page_tokens, row_bytes = 2, 4, 128, 8, 136
    length, span = 45, 5
    pool, table, ks, vs = _build_pool(oracle, rng, 1, [length], kv_heads, dim, page_tokens, row_bytes)
    q = rng.standard_normal((1, span, heads, dim)).astype(np.float32)
    scale = 1.0 / np.sqrt(dim)
    first = np.array([length - span], dtype=np.int32)
    out = oracle.paged_attention(pool, row_bytes, page_tokens, kv_heads, dim, table, first, q, scale)
    # each span row is the single-token call at its position, bit for bit
    for r in range(span):
        one = oracle.paged_attention(pool, row_bytes, page_tokens, kv_heads, dim, table, first + r, q[:, r:r + 1], scale)
        assert np.array_equal(one[0, 0].view(np.uint32), out[0, r].view(np.uint32))
    # moving the pages and the table together changes nothing
    pages = pool.reshape(-1, 2 * kv_heads * page_tokens * row_bytes)
    perm = rng.permutation(pages.shape[0])
    moved = np.ascontiguousarray(pages[perm]).reshape(-1)
    inverse = np.argsort(perm).astype(np.int32)
    again = oracle.paged_attention(moved, row_bytes, page_tokens, kv_heads, dim, inverse[table], first, q, scale)
    assert np.array_equal(again.view(np.uint32), out.view(np.uint32))


def test_zero_query_gives_the_mean_of_the_values(oracle):
    rng = np.random.default_rng(6)
    kv_heads, heads, dim, page_tokens, row_bytes = 1, 2, 128, 4, 136
    pool, table, ks, vs = _build_pool(oracle, rng, 1, [11], kv_heads, dim, page_tokens, row_bytes)
    q = np.zeros((1, 1, heads, dim), dtype=np.float32)
    out = oracle.paged_attention(pool, row_bytes, page_tokens, kv_heads, dim, table, np.array([10], np.int32), q, 0.088)
    v = _dequant(oracle, vs[0], dim, row_bytes)
    assert np.allclose(out[0, 0, 0], v[:, 0].mean(axis=0), atol=1e-6)


def test_attention_sequence_is_the_dense_case_with_a_selection_list(oracle):
    # gpu/kernels.cpp:4387-4419: packed [q | k | v | indices | counts]; compare with the paged oracle over one page = the plane layout.
    rng = np.random.default_rng(7)
    context, base, steps, selected = 40, 9, 3, 16
    for row_bytes in (272, 512):
        state = np.zeros(context * 4 * row_bytes, dtype=np.uint8)
        old_k = rng.standard_normal((1, base, 2, 256)).astype(np.float32)
        old_v = rng.standard_normal((1, base, 2, 256)).astype(np.float32)
        table = np.zeros((1, 1), dtype=np.int32)
        oracle.kv_write(state, row_bytes, context, 2, 256, table, np.zeros(1, np.int32), old_k, old_v)
        q = rng.standard_normal((steps, 24, 256)).astype(np.float32)
        k = rng.standard_normal((steps, 2, 256)).astype(np.float32)
        v = rng.standard_normal((steps, 2, 256)).astype(np.float32)
        indices = np.full((steps, selected), -1.0, dtype=np.float32)
        counts = np.zeros(steps, dtype=np.float32)
        for s in range(steps):
            n = base + s + 1
            indices[s, :n] = np.arange(n)
            counts[s] = n
        packed = np.concatenate([q.ravel(), k.ravel(), v.ravel(), indices.ravel(), counts])
        got = oracle.attention_sequence(state, row_bytes, context, base, steps, selected, packed).reshape(steps, 24, 256)
        want = oracle.paged_attention(state, row_bytes, context, 2, 256, table, np.array([base], np.int32), q[None], 0.0625)[0]
        assert np.abs(got - want).max() < 1e-6
        # entries past the row's position, negative or past the context are ignored (:107-108)
        indices2 = indices.copy()
        indices2[0, base + 1:base + 4] = [base + 2, -3, context + 5]
        counts2 = counts.copy(); counts2[0] = base + 4
        packed2 = np.concatenate([q.ravel(), k.ravel(), v.ravel(), indices2.ravel(), counts2])
        again = oracle.attention_sequence(state, row_bytes, context, base, steps, selected, packed2).reshape(steps, 24, 256)
        assert np.array_equal(again[0].view(np.uint32), got[0].view(np.uint32))
        # a shorter list attends fewer keys: drop position 0 from row 1 and compare with float64
        indices3 = indices.copy()
        indices3[1, :base + 1] = np.arange(1, base + 2); counts3 = counts.copy(); counts3[1] = base + 1
        packed3 = np.concatenate([q.ravel(), k.ravel(), v.ravel(), indices3.ravel(), counts3])
        third = oracle.attention_sequence(state, row_bytes, context, base, steps, selected, packed3).reshape(steps, 24, 256)
        kk = _dequant(oracle, np.concatenate([old_k[0], k]), 256, row_bytes)
        vv = _dequant(oracle, np.concatenate([old_v[0], v]), 256, row_bytes)
        want3 = _f64_attention(q[1], kk[1:], vv[1:], base + 1, 0.0625)
        assert np.abs(third[1] - want3).max() < 2e-5


SHAPES = [(15, 4, 2, 256, 33), (16, 4, 2, 256, 33), (17, 4, 2, 256, 35), (31, 6, 2, 256, 65), (32, 4, 4, 256, 129),
          (16, 4, 2, 128, 35), (1, 2, 1, 256, 137), (17, 1, 1, 256, 1), (15, 16, 2, 256, 137)]


def _attention_gpu_case(rows, heads, kv_heads, dim, context, zero_queries=False):
    # crates/straydog-engine/tests/attention_gpu.rs:89-104
    seed = 0x9e3779b97f4a7c15 ^ rows ^ (dim << 16)
    flat = _xorshift_floats(seed, rows * heads * dim + 2 * context * kv_heads * dim)
    q = flat[:rows * heads * dim].reshape(rows, heads, dim).copy()
    if zero_queries:
        q[:] = 0
    keys = flat[rows * heads * dim:rows * heads * dim + context * kv_heads * dim].reshape(context, kv_heads, dim)
    values = flat[rows * heads * dim + context * kv_heads * dim:].reshape(context, kv_heads, dim)
    special = [0, 1, 15, 16, context - 1, context + 7]
    positions = np.array([special[r] if r < len(special) else (r * 17 + 3) % context for r in range(rows)], dtype=np.int32)
    gate = np.array([[-12.0, -1.0, 0.0, 1.0, 12.0][i % 5] for i in range(q.size)], dtype=np.float32).reshape(q.shape)
    return q, keys, values, positions, gate, np.float32(1.0 / np.sqrt(np.float32(dim)))


@pytest.mark.parametrize("shape", SHAPES[:6] + SHAPES[7:8])
def test_op_attention_within_the_derived_f64_bound(oracle, shape):
    rows, heads, kv_heads, dim, context = shape
    q, keys, values, positions, gate, scale = _attention_gpu_case(*shape)
    for gated in (None, gate):
        out = oracle.op_attention(q, keys, values, positions, scale, gated)
        want, bound = oracle.op_attention_f64(q, keys, values, positions, scale, gated)
        assert np.all(np.isfinite(out)) and np.all(np.abs(out - want) <= bound)
        # the F64 twin itself against plain numpy
        for row in (0, rows - 1):
            length = min(int(positions[row]) + 1, context)
            ref = _f64_attention(q[row], keys, values, length, scale)
            if gated is not None:
                ref = ref / (1.0 + np.exp(-gated[row].astype(np.float64)))
            assert np.allclose(want[row], ref, rtol=1e-12, atol=1e-14)


def test_op_attention_zero_queries_give_the_mean(oracle):
    q, keys, values, positions, gate, scale = _attention_gpu_case(17, 4, 2, 256, 35, zero_queries=True)
    out = oracle.op_attention(q, keys, values, positions, scale)
    for row in range(17):
        length = min(int(positions[row]) + 1, 35)
        for head in range(4):
            assert np.allclose(out[row, head], values[:length, head // 2].mean(axis=0), atol=2e-6)


def test_latent_attention_closed_form_and_special_cases(oracle):
    rng = np.random.default_rng(8)
    rows, heads, kdim, vdim, n, selections = 2, 3, 96, 64, 50, 12
    q = rng.standard_normal((rows, heads, kdim)).astype(np.float32)
    comp = rng.standard_normal((n, kdim)).astype(np.float32)
    comp_bf16 = oracle.to_bf16(comp)
    comp_wide = (comp_bf16.astype(np.uint32) << 16).view(np.float32)
    selected = np.stack([rng.permutation(n)[:selections] for _ in range(rows)]).astype(np.int32)
    selected[0, 3] = -1
    scale = 1.0 / np.sqrt(kdim)
    out, out64 = oracle.latent_attention(q, None, None, 0, comp_bf16, selected, None, vdim, scale, wide=True)
    for r in range(rows):
        rows_kept = [i for i in selected[r] if i >= 0]
        k = comp_wide[rows_kept].astype(np.float64)
        for h in range(heads):
            s = k @ q[r, h].astype(np.float64) * float(np.float32(scale))
            w = np.exp(s - s.max()); w /= w.sum()
            want = w @ k[:, :vdim]
            assert np.allclose(out64[r, h], want, rtol=1e-12, atol=1e-13)
            assert np.abs(out[r, h] - want).max() < 1e-5
    # BF16 rows and the fp32 values they stand for give the same bits (ds_state_bf16_gpu.rs:99-102)
    same = oracle.latent_attention(q, None, None, 0, comp_wide, selected, None, vdim, scale)
    assert np.array_equal(same.view(np.uint32), out.view(np.uint32))
    # one selected row: the output is that row's first vdim values
    single = np.full((rows, 4), -1, dtype=np.int32); single[:, 2] = 7
    one = oracle.latent_attention(q, None, None, 0, comp_wide, single, None, vdim, scale)
    assert np.allclose(one, np.broadcast_to(comp_wide[7, :vdim], one.shape), atol=1e-6)


def test_latent_attention_window_sink_and_rope(oracle):
    # gpu/ops.hpp:1240-1297 with a ring window and the sink in the denominator only; rope in and back out.
    rng = np.random.default_rng(9)
    rows, heads, dim, window, raw_rows, n, selections, rope_dims = 3, 2, 64, 5, 8, 20, 6, 16
    q = rng.standard_normal((rows, heads, dim)).astype(np.float32)
    raw = rng.standard_normal((raw_rows, dim)).astype(np.float32)
    comp = rng.standard_normal((n, dim)).astype(np.float32)
    positions = np.array([2, 9, 21], dtype=np.int32)
    selected = np.stack([rng.permutation(n)[:selections] for _ in range(rows)]).astype(np.int32)
    selected[1, 0] = -1
    sinks = rng.standard_normal(heads).astype(np.float32)
    freqs = (1.6e5 ** (-(2.0 * np.arange(rope_dims // 2)) / rope_dims)).astype(np.float32)
    scale = 0.11
    out, out64 = oracle.latent_attention(q, raw, positions, window, comp, selected, sinks, dim, scale, rope_dims, freqs, wide=True)
    for r in range(rows):
        p = int(positions[r])
        first = max(0, p - window + 1)
        keys = [raw[t % raw_rows] for t in range(first, p + 1)] + [comp[i] for i in selected[r] if i >= 0]
        k = np.array(keys, dtype=np.float64)
        angle = p * freqs.astype(np.float64)
        for h in range(heads):
            qq = q[r, h].astype(np.float64).copy()
            a, b = qq[dim - rope_dims::2].copy(), qq[dim - rope_dims + 1::2].copy()
            # the oracle rounds the rotated query to fp32, as the reference's op_rope does
            qq[dim - rope_dims::2] = (a * np.cos(angle) - b * np.sin(angle)).astype(np.float32)
            qq[dim - rope_dims + 1::2] = (a * np.sin(angle) + b * np.cos(angle)).astype(np.float32)
            s = k @ qq * float(np.float32(scale))
            m = max(float(sinks[h]), s.max())
            w = np.exp(s - m)
            o = (w @ k) / (w.sum() + np.exp(float(sinks[h]) - m))
            a, b = o[dim - rope_dims::2].copy(), o[dim - rope_dims + 1::2].copy()
            o[dim - rope_dims::2] = a * np.cos(-angle) - b * np.sin(-angle)
            o[dim - rope_dims + 1::2] = a * np.sin(-angle) + b * np.cos(-angle)
            assert np.allclose(out64[r, h], o, rtol=1e-11, atol=1e-12)
            assert np.abs(out[r, h] - o).max() < 1e-5
    # every selection empty and window rows only + a dominant sink: the output shrinks toward zero
    big = np.full(heads, 50.0, dtype=np.float32)
    none = np.full((rows, selections), -1, dtype=np.int32)
    small = oracle.latent_attention(q, raw, positions, window, comp, none, big, dim, scale)
    assert np.abs(small).max() < 1e-12


def test_compress_matches_f64(oracle):
    rng = np.random.default_rng(11)
    groups, ratio, dim = 7, 4, 24
    kv = rng.standard_normal((groups * ratio, dim)).astype(np.float32)
    gate = (rng.standard_normal((groups * ratio, dim)) * 3).astype(np.float32)
    got = oracle.compress(kv, gate, ratio)
    g = gate.reshape(groups, ratio, dim).astype(np.float64)
    w = np.exp(g - g.max(axis=1, keepdims=True)); w /= w.sum(axis=1, keepdims=True)
    want = (w * kv.reshape(groups, ratio, dim)).sum(axis=1)
    assert np.abs(got - want).max() < 1e-6
    assert np.array_equal(oracle.compress(kv[:groups], None, 1), kv[:groups])


def _dspark_inputs(seed=0x9e3779b97f4a7c15):
    # the generator and magnitudes of crates/straydog-engine/tests/dspark_attention_gpu.rs:9-16, 55-60
    state = [seed]

    def floats(n, scale):
        out = np.empty(n, dtype=np.float32)
        s = state[0]
        for i in range(n):
            s ^= (s << 13) & 0xffffffffffffffff
            s ^= s >> 7
            s ^= (s << 17) & 0xffffffffffffffff
            out[i] = np.float32((np.float32(s >> 40) / np.float32(1 << 24) - np.float32(0.5)) * np.float32(2.0) * np.float32(scale))
        state[0] = s
        return out
    q, ring, block, sinks = floats(5 * 64 * 512, 0.3), floats(128 * 512, 0.4), floats(5 * 512, 0.6), floats(64, 2.0)
    sinks[0::16] = 30.0
    sinks[1::16] = -30.0
    return q, ring, block, sinks


def test_dspark_known_answers_and_float64(oracle):
    # the reference's own known answers (dspark_attention_gpu.rs:101-124): zero queries, block keys of constant 1..5, a sink of 0:
    # every query sees five keys and one sink, (1+2+3+4+5)/6; a changed last key; a huge sink takes everything, a tiny one nothing
    q, ring = np.zeros(5 * 64 * 512, np.float32), np.full(128 * 512, 23.0, np.float32)
    block = np.repeat(np.arange(1, 6, dtype=np.float32), 512)
    assert np.allclose(oracle.dspark_attention(q, ring, block, np.zeros(64, np.float32), 64, 5, 0, 0), 2.5, rtol=0, atol=1e-12)
    block[4 * 512:] = 11.0
    assert np.allclose(oracle.dspark_attention(q, ring, block, np.zeros(64, np.float32), 64, 5, 0, 0), 3.5, rtol=0, atol=1e-12)
    assert np.allclose(oracle.dspark_attention(q, ring, block, np.full(64, 1000.0, np.float32), 64, 5, 0, 0), 0.0, atol=1e-12)
    assert np.allclose(oracle.dspark_attention(q, ring, block, np.full(64, -1000.0, np.float32), 64, 5, 0, 0), 4.2, rtol=0, atol=1e-12)
    # random inputs against numpy in float64, a ring that wraps
    q, ring, block, sinks = _dspark_inputs()
    heads, slots, anchor, history = 64, 3, 389, 128
    got = oracle.dspark_attention(q, ring, block, sinks, heads, slots, anchor, history).reshape(slots, heads, 512)
    keys = np.concatenate([ring.reshape(128, 512)[np.arange(anchor - history, anchor) % 128], block.reshape(5, 512)[:slots]]).astype(np.float64)
    scores = q.reshape(5, 64, 512)[:slots].astype(np.float64) @ keys.T / np.sqrt(512.0)
    top = np.maximum(scores.max(axis=-1), sinks.astype(np.float64)[None, :])
    weights = np.exp(scores - top[..., None])
    want = weights @ keys / (weights.sum(axis=-1) + np.exp(sinks.astype(np.float64)[None, :] - top))[..., None]
    assert np.allclose(got, want, rtol=1e-12, atol=1e-14)
