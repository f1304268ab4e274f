"""GPU parity of the reference ABI's attention ops, written after the reference's own model-free tests:
crates/straydog-engine/tests/attention_gpu.rs (causal GQA against an F64 reference with a derived bound, output
guards), tests/fused_gpu.rs:326-428 (top-k against its rule on adversarial ties; index_select == rope + index_scores
+ top_k bit for bit, run twice; candidates), tests/ds_state_bf16_gpu.rs (BF16 rounding; BF16-tagged rows == the FP32
values they stand for, bit for bit), and sd_attention_sequence / sd_op_sparse_attention / sd_op_compress against the
CPU oracle."""
import numpy as np
import pytest

from gpu_util import backend, close_enough
from test_oracle_attention import SHAPES, _attention_gpu_case
from test_oracle_index_topk import Random, _adversarial

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gpu():
    with backend(4 << 30) as handle:
        yield handle


def _read(gpu, buffer, dtype, count):
    return gpu.read_buffer(buffer, 0, dtype, count)


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("zero_queries", [False, True])
def test_causal_gqa_matches_f64_softmax(gpu, oracle, shape, zero_queries):
    rows, heads, kv_heads, dim, context = shape
    if zero_queries and shape != (17, 4, 2, 256, 35):
        pytest.skip("the reference runs zero queries on one shape")
    q, keys, values, positions, gate, scale = _attention_gpu_case(*shape, zero_queries=zero_queries)
    qs, ks, vs, gs, ps = (gpu.upload(x) for x in (q, keys, values, gate, positions))
    scratch = gpu.buffer(rows * heads * 64 * (dim + 2) * 4)
    guard, canary = 7, np.float32(12345.125)
    output = gpu.upload(np.full(q.size + 2 * guard, canary, dtype=np.float32))
    for gated in (False, True):
        gpu.attention(qs.base(), ks.base(), vs.base(), context, ps.base(), rows, heads, kv_heads, dim, float(scale),
                      gs.base() if gated else None, scratch, output.at(guard * 4))
        actual = _read(gpu, output, np.float32, q.size + 2 * guard)
        assert np.all(actual[:guard] == canary) and np.all(actual[guard + q.size:] == canary), "output guard"
        want, bound = oracle.op_attention_f64(q, keys, values, positions, scale, gate if gated else None)
        got = actual[guard:guard + q.size].reshape(q.shape)
        assert np.all(np.isfinite(got))
        ratio = np.abs(got - want) / bound
        assert ratio.max() <= 1.0, f"{shape} gated={gated}: error/bound {ratio.max():.3f}"
    for b in (qs, ks, vs, gs, ps, scratch, output):
        gpu.release(b)


def test_attention_refuses_bad_arguments(gpu):
    from straydog_amd.backend import StraydogError
    b = gpu.buffer(1 << 20)
    with pytest.raises(StraydogError, match="scratch too small"):
        gpu.attention(b.base(), b.base(), b.base(), 8, b.base(), 1, 2, 1, 64, 0.1, None, None, b.base())
    with pytest.raises(StraydogError, match="invalid Straydog attention shape"):
        gpu.attention(b.base(), b.base(), b.base(), 8, b.base(), 1, 3, 2, 64, 0.1, None, b, b.base())
    with pytest.raises(StraydogError, match="overflows|outside"):
        gpu.attention(b.base(), b.base(), b.base(), 1 << 62, b.base(), 1, 2, 1, 64, 0.1, None, b, b.base())
    gpu.release(b)


@pytest.mark.parametrize("row_bytes", [272, 512])
def test_attention_sequence_matches_the_oracle(gpu, oracle, row_bytes):
    rng = np.random.default_rng(70 + row_bytes)
    context, base, steps, selected = 600, 300, 5, 2052
    gpu.kv_format(row_bytes)
    state_host = np.zeros(context * 4 * row_bytes, dtype=np.uint8)
    old_k = rng.standard_normal((1, base, 2, 256)).astype(np.float32)
    old_v = rng.standard_normal((1, base, 2, 256)).astype(np.float32)
    oracle.kv_write(state_host, row_bytes, context, 2, 256, np.zeros((1, 1), np.int32), np.zeros(1, np.int32), old_k, old_v)
    state = gpu.upload(state_host)
    q = rng.standard_normal((steps, 24, 256)).astype(np.float32)
    k = rng.standard_normal((steps, 2, 256)).astype(np.float32)
    v = rng.standard_normal((steps, 2, 256)).astype(np.float32)
    indices = np.full((steps, selected), -1.0, dtype=np.float32)
    counts = np.zeros(steps, dtype=np.float32)
    for s in range(steps):
        picked = np.sort(rng.permutation(base + s + 1)[: 200 + 13 * s])
        extra = [base + s + 3, -2.0, context + 1]        # ignored: past the row's position, negative, past the context
        row = np.concatenate([picked, extra]).astype(np.float32)
        indices[s, :row.size] = row
        counts[s] = row.size
    packed = np.concatenate([q.ravel(), k.ravel(), v.ravel(), indices.ravel(), counts]).astype(np.float32)
    got = gpu.attention_sequence(state.base(), context, base, steps, selected, packed)
    want = oracle.attention_sequence(state_host, row_bytes, context, base, steps, selected, packed)
    assert np.abs(got - want).max() < 2e-5
    # the rows' K/V were written as the oracle writes them
    after = _read(gpu, state, np.uint8, state_host.size)
    assert np.array_equal(after, state_host)
    from straydog_amd.backend import StraydogError
    with pytest.raises(StraydogError, match="selection count"):
        bad = packed.copy(); bad[-1] = 0.0
        gpu.attention_sequence(state.base(), context, base, steps, selected, bad)
    with pytest.raises(StraydogError, match="workspace mismatch"):
        gpu.attention_sequence(state.base(), context, base, steps, selected, packed[:-1])
    gpu.release(state)
    gpu.kv_format(272)


def test_to_bf16_rounds_to_nearest_even(gpu, oracle):
    rng = np.random.default_rng(2)
    bits = np.concatenate([rng.integers(0, 2 ** 32, 50000, dtype=np.uint64).astype(np.uint32),
                           np.array([0, 0x80000000, 0x3f808000, 0x3f818000, 0x3f807fff, 0x3f808001, 0x7f7fffff, 0x7f800000, 0xff800000,
                                     0x7f800001, 0x7fc00000, 0xffc00001, 1, 0x8000, 0x18000], dtype=np.uint32)])
    x = gpu.upload(bits)
    out = gpu.buffer(bits.size * 2)
    gpu.to_bf16(x.base(), bits.size, out.base())
    assert np.array_equal(_read(gpu, out, np.uint16, bits.size), oracle.to_bf16(bits.view(np.float32)))
    gpu.release(x); gpu.release(out)


def test_compress_matches_the_oracle(gpu, oracle):
    rng = np.random.default_rng(3)
    groups, ratio, dim = 37, 4, 512
    kv = rng.standard_normal((groups * ratio, dim)).astype(np.float32)
    gate = (rng.standard_normal((groups * ratio, dim)) * 3).astype(np.float32)
    kb, gb, out = gpu.upload(kv), gpu.upload(gate), gpu.buffer(groups * dim * 4)
    gpu.compress(kb.base(), gb.base(), groups, ratio, dim, out.base())
    assert np.abs(_read(gpu, out, np.float32, groups * dim).reshape(groups, dim) - oracle.compress(kv, gate, ratio)).max() < 1e-6
    gpu.compress(kb.base(), None, groups, 1, dim, out.base())
    assert np.array_equal(_read(gpu, out, np.float32, groups * dim), kv[:groups].ravel())
    for b in (kb, gb, out):
        gpu.release(b)


@pytest.mark.parametrize("groups", [511, 512, 513, 600, 4096, 30000, 65536, 131072])
def test_top_k_matches_its_reference_with_many_ties(gpu, oracle, groups):
    random = Random(0x2f6b91d3c0a54e77 ^ groups)
    k, rows = 512, 2
    if groups > 30000:      # the pure-Python generator is slow: vectorise the same distribution
        rng = np.random.default_rng(groups)
        draw = rng.integers(0, 97, size=(rows, groups))
        scores = (rng.integers(0, 17, size=(rows, groups)) * 0.25 - 2.0).astype(np.float32)
        scores[draw <= 6] = -np.inf
        scores[draw == 7] = np.inf
        scores[draw == 8] = -0.0
        scores.reshape(-1)[999::1000] += np.float32(0.125)
    else:
        scores = _adversarial(random, rows, groups)
    sb, out = gpu.upload(scores), gpu.buffer(rows * k * 4)
    for _ in range(2):      # twice: nothing left over from the first run
        gpu.top_k(sb.base(), rows, groups, k, out.base())
        got = _read(gpu, out, np.int32, rows * k).reshape(rows, k)
        assert np.array_equal(got, oracle.top_k(scores, k)), groups
    gpu.release(sb); gpu.release(out)


def test_top_k_edge_cases(gpu, oracle):
    cases = [np.array([[1.0, 1.0, 1.0, 2.0, -np.inf, 1.0]], np.float32), np.full((1, 700), -np.inf, np.float32),
             np.zeros((3, 9000), np.float32), np.array([[0.0, -0.0, -1.0, np.inf]], np.float32)]
    for scores in cases:
        for k in (1, 3, 600, 2048):
            sb, out = gpu.upload(scores), gpu.buffer(scores.shape[0] * k * 4)
            gpu.top_k(sb.base(), scores.shape[0], scores.shape[1], k, out.base())
            got = _read(gpu, out, np.int32, scores.shape[0] * k).reshape(scores.shape[0], k)
            assert np.array_equal(got, oracle.top_k(scores, k)), (scores.shape, k)
            gpu.release(sb); gpu.release(out)


def _bf16_round(oracle, x):
    bits = oracle.to_bf16(x)
    return bits, (bits.astype(np.uint32) << 16).view(np.float32)


@pytest.mark.parametrize("rows,groups,heads,dim", [(1, 3000, 32, 128), (4, 2000, 64, 128), (2, 300, 5, 96), (1, 1000, 33, 40)])
def test_index_scores_are_bit_exact(gpu, oracle, rows, groups, heads, dim):
    rng = np.random.default_rng(rows * 1000 + groups)
    q = (rng.standard_normal((rows, heads, dim)) * 2).astype(np.float32)
    keys = rng.standard_normal((groups, dim)).astype(np.float32)
    weights = rng.standard_normal((rows, heads)).astype(np.float32)
    visible = np.array([groups - 3 * r for r in range(rows)], dtype=np.int32)
    scale = float(1.0 / (np.sqrt(np.float32(dim)) * np.sqrt(np.float32(heads))))
    qb, kb, wb, vb, out = gpu.upload(q), gpu.upload(keys), gpu.upload(weights), gpu.upload(visible), gpu.buffer(rows * groups * 4)
    gpu.index_scores(qb.base(), kb.base(), wb.base(), vb.base(), rows, groups, heads, dim, scale, out.base())
    got = _read(gpu, out, np.float32, rows * groups).reshape(rows, groups)
    want = oracle.index_scores(q, keys, weights, visible, scale)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # BF16-tagged keys give the bits of the FP32 values they stand for
    key_bits, key_values = _bf16_round(oracle, keys)
    hb = gpu.upload(key_bits)
    from straydog_amd.backend import tagged_bf16
    gpu.index_scores(qb.base(), tagged_bf16(hb.base()), wb.base(), vb.base(), rows, groups, heads, dim, scale, out.base())
    tagged = _read(gpu, out, np.float32, rows * groups).reshape(rows, groups)
    assert np.array_equal(tagged.view(np.uint32), oracle.index_scores(q, key_values, weights, visible, scale).view(np.uint32))
    for b in (qb, kb, wb, vb, out, hb):
        gpu.release(b)


def test_an_index_select_matches_rope_scores_and_top_k(gpu, oracle):
    # fused_gpu.rs:390-428
    random = np.random.default_rng(0xa54f)
    heads, dim, rope_dims, k = 32, 128, 64, 512
    frequencies = (np.float32(1.6e5) ** (-(2.0 * np.arange(rope_dims // 2, dtype=np.float32)) / np.float32(rope_dims))).astype(np.float32)
    fb = gpu.upload(frequencies)
    for rows, groups in [(1, 3000), (4, 2000), (1, 300)]:
        q = (random.random((rows, heads, dim)) * 4 - 2).astype(np.float32)
        keys = (random.random((groups, dim)) * 2 - 1).astype(np.float32)
        weights = (random.random((rows, heads)) * 2 - 1).astype(np.float32)
        visible = np.array([groups - 3 * r for r in range(rows)], dtype=np.int32)
        at = np.array([20000 + 7 * r for r in range(rows)], dtype=np.int32)
        scale = float(1.0 / (np.sqrt(np.float32(dim)) * np.sqrt(np.float32(heads))))
        kb, wb, vb, pb = gpu.upload(keys), gpu.upload(weights), gpu.upload(visible), gpu.upload(at)
        q1, s1, o1 = gpu.upload(q), gpu.buffer(rows * groups * 4), gpu.buffer(rows * k * 4)
        gpu.rope(q1.base(), rows, heads, dim, rope_dims, pb.base(), fb.base(), False)
        gpu.index_scores(q1.base(), kb.base(), wb.base(), vb.base(), rows, groups, heads, dim, scale, s1.base())
        gpu.top_k(s1.base(), rows, groups, k, o1.base())
        scores_1, out_1 = _read(gpu, s1, np.uint32, rows * groups), _read(gpu, o1, np.int32, rows * k)
        q2 = gpu.upload(q)
        for run in range(2):
            s2, o2 = gpu.buffer(rows * groups * 4), gpu.buffer(rows * k * 4)
            gpu.index_select(q2.base(), kb.base(), wb.base(), vb.base(), rows, groups, heads, dim, scale, (rope_dims, pb.base(), fb.base()),
                             s2.base(), k, o2.base())
            assert np.array_equal(_read(gpu, s2, np.uint32, rows * groups), scores_1), (rows, run)
            assert np.array_equal(_read(gpu, o2, np.int32, rows * k), out_1), (rows, run)
            gpu.release(s2); gpu.release(o2)
        assert np.array_equal(_read(gpu, q2, np.uint32, q.size), q.view(np.uint32).ravel()), "q unchanged"
        # and against the oracle: rotate on the host in double, then the canonical scores and the rule
        rotated = q.copy()
        for r in range(rows):
            angle = float(at[r]) * frequencies.astype(np.float64)
            a, b = rotated[r, :, dim - rope_dims::2].astype(np.float64), rotated[r, :, dim - rope_dims + 1::2].astype(np.float64)
            rotated[r, :, dim - rope_dims::2] = (a * np.cos(angle) - b * np.sin(angle)).astype(np.float32)
            rotated[r, :, dim - rope_dims + 1::2] = (a * np.sin(angle) + b * np.cos(angle)).astype(np.float32)
        rope_got = _read(gpu, q1, np.float32, q.size).reshape(q.shape)
        assert np.abs(rope_got - rotated).max() <= 2.4e-7 * 4      # within an ulp of the host's double sincos
        want_scores = oracle.index_scores(rope_got, keys, weights, visible, scale)
        assert np.array_equal(want_scores.view(np.uint32).ravel(), scores_1)
        assert np.array_equal(oracle.top_k(want_scores, k).ravel(), out_1)
        for b in (kb, wb, vb, pb, q1, s1, o1, q2):
            gpu.release(b)
    gpu.release(fb)


def test_the_two_level_indexer_matches_its_reference(gpu, oracle):
    # fused_gpu.rs:476-566
    rng = np.random.default_rng(0x1f83)
    heads, dim, k, blocks, block = 32, 128, 512, 2048, 8
    for rows, groups in [(1, 20000), (3, 23001)]:
        keys = (rng.random((groups, dim)) * 2 - 1).astype(np.float32)
        seen = np.array([16000 if r == 1 else groups - 13 * r for r in range(rows)], dtype=np.int32)
        scale = float(1.0 / (np.sqrt(np.float32(dim)) * np.sqrt(np.float32(heads))))
        q = (rng.random((rows, heads, dim)) * 4 - 2).astype(np.float32)
        weights = (rng.random((rows, heads)) * 2 - 1).astype(np.float32)
        kb, vb, qb, wb = gpu.upload(keys), gpu.upload(seen), gpu.upload(q), gpu.upload(weights)
        scores, out = gpu.buffer(rows * groups * 4), gpu.buffer(rows * k * 4)
        gpu.index_select(qb.base(), kb.base(), wb.base(), vb.base(), rows, groups, heads, dim, scale, (0, vb.base(), None), scores.base(), k, out.base())
        cand = gpu.buffer(rows * blocks * 4)
        count = (groups + block - 1) // block
        scratch = gpu.buffer(rows * count * 4)
        gpu.index_candidates(scores.base(), vb.base(), rows, groups, blocks, block, cand.base(), scratch)
        source = _read(gpu, scores, np.float32, rows * groups).reshape(rows, groups)
        chosen = _read(gpu, cand, np.int32, rows * blocks).reshape(rows, blocks)
        assert np.array_equal(chosen, oracle.index_candidates(source, seen, blocks, block))
        keep = np.zeros((rows, groups), dtype=bool)
        for r in range(rows):
            for b in chosen[r][chosen[r] >= 0]:
                keep[r, b * block:(b + 1) * block] = True
        q2 = (rng.random((rows, heads, dim)) * 4 - 2).astype(np.float32)
        w2 = (rng.random((rows, heads)) * 2 - 1).astype(np.float32)
        qb2, wb2 = gpu.upload(q2), gpu.upload(w2)
        every = oracle.index_scores(q2, keys, w2, seen, scale)
        masked = np.where(keep, every, -np.inf).astype(np.float32)
        for run in range(2):
            s3, o3 = gpu.buffer(rows * max(groups, blocks * block) * 4), gpu.buffer(rows * k * 4)
            gpu.index_select(qb2.base(), kb.base(), wb2.base(), vb.base(), rows, groups, heads, dim, scale, (0, vb.base(), None), s3.base(), k, o3.base(),
                             (cand.base(), blocks, block))
            got = _read(gpu, o3, np.int32, rows * k).reshape(rows, k)
            assert np.array_equal(got, oracle.top_k(masked, k)), (rows, run)
            gpu.release(s3); gpu.release(o3)
        if rows == 1:
            # the decode launch (fused_gpu.rs:543-564): the projection of x into the weights, then the same choice among the candidates
            width = 5120
            x = (rng.random(width) * 4 - 2).astype(np.float32)
            matrix = ((rng.random((heads, width)) * 0.1 - 0.05).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16).view(np.uint8).reshape(-1)
            formed = oracle.index_projection(matrix, 30, width, x, heads)
            masked = np.where(keep, oracle.index_scores(q2, keys, formed[None, :], seen, scale), -np.inf).astype(np.float32)
            xb, mb = gpu.upload(x), gpu.upload(matrix)
            for run in range(2):
                s3, o3, w3 = gpu.buffer(max(groups, blocks * block) * 4), gpu.buffer(k * 4), gpu.buffer(heads * 4)
                gpu.index_select_proj((mb.base(), 30, width), xb.base(), qb2.base(), kb.base(), w3.base(), vb.base(), groups, heads, dim, scale,
                                      (0, vb.base(), None), s3.base(), k, o3.base(), (cand.base(), blocks, block))
                assert np.array_equal(_read(gpu, o3, np.int32, k), oracle.top_k(masked, k).ravel()), f"run {run}: the decode launch's indices among the candidates"
                for b in (s3, o3, w3):
                    gpu.release(b)
            gpu.release(xb); gpu.release(mb)
        for b in (kb, vb, qb, wb, scores, out, cand, scratch, qb2, wb2):
            gpu.release(b)


def test_an_index_select_with_its_projection_matches_the_two_ops(gpu, oracle):
    # fused_gpu.rs:430-474: the indexer's projection of x into its weights and the row's index select in one call give the
    # weights, scores and indices of the two ops, bit for bit, twice in a row; BF16 rows and ggml Q8_0 rows.  The separate
    # projection is sdx_index_projection (the reference's is sd_op_linear); its weights are also the oracle's, bit for bit.
    from test_oracle_index_topk import _q8_0_rows
    rng = np.random.default_rng(0x510e)
    heads, dim, rope_dims, k, width, groups = 32, 128, 64, 512, 5120, 2500
    frequencies = (np.float32(1.6e5) ** (-(2.0 * np.arange(rope_dims // 2, dtype=np.float32)) / np.float32(rope_dims))).astype(np.float32)
    x = (rng.random(width) * 4 - 2).astype(np.float32)
    q = (rng.random((heads, dim)) * 4 - 2).astype(np.float32)
    keys = (rng.random((groups, dim)) * 2 - 1).astype(np.float32)
    scale = float(1.0 / (np.sqrt(np.float32(dim)) * np.sqrt(np.float32(heads))))
    fb, xb, qb, kb = (gpu.upload(a) for a in (frequencies, x, q, keys))
    pb, vb = gpu.upload(np.array([31337], dtype=np.int32)), gpu.upload(np.array([groups - 5], dtype=np.int32))
    bf16 = ((rng.random((heads, width)) * 0.1 - 0.05).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16).view(np.uint8).reshape(-1)
    q8 = _q8_0_rows(rng, heads, width)[0]
    rope = (rope_dims, pb.base(), fb.base())
    for kind, matrix in ((30, bf16), (8, q8)):
        mb = gpu.upload(matrix)
        w1, s1, o1 = gpu.buffer(heads * 4), gpu.buffer(groups * 4), gpu.buffer(k * 4)
        gpu.index_projection(mb.base(), kind, width, xb.base(), heads, w1.base())
        gpu.index_select(qb.base(), kb.base(), w1.base(), vb.base(), 1, groups, heads, dim, scale, rope, s1.base(), k, o1.base())
        weights_1, scores_1, out_1 = _read(gpu, w1, np.uint32, heads), _read(gpu, s1, np.uint32, groups), _read(gpu, o1, np.int32, k)
        assert np.array_equal(weights_1, oracle.index_projection(matrix, kind, width, x, heads).view(np.uint32)), f"kind {kind}: weights vs oracle"
        assert (out_1 >= 0).all() and len(set(out_1.tolist())) == k
        for run in range(2):
            w2, s2, o2 = gpu.buffer(heads * 4), gpu.buffer(groups * 4), gpu.buffer(k * 4)
            gpu.index_select_proj((mb.base(), kind, width), xb.base(), qb.base(), kb.base(), w2.base(), vb.base(), groups, heads, dim, scale, rope,
                                  s2.base(), k, o2.base())
            assert np.array_equal(_read(gpu, w2, np.uint32, heads), weights_1), f"kind {kind}, run {run}: weights"
            assert np.array_equal(_read(gpu, s2, np.uint32, groups), scores_1), f"kind {kind}, run {run}: scores"
            assert np.array_equal(_read(gpu, o2, np.int32, k), out_1), f"kind {kind}, run {run}: indices"
            for b in (w2, s2, o2):
                gpu.release(b)
        for b in (mb, w1, s1, o1):
            gpu.release(b)
    # refusals: a kind the projection does not take, columns that are not whole units
    from straydog_amd.backend import StraydogError
    mb = gpu.upload(bf16)
    w, s, o = gpu.buffer(heads * 4), gpu.buffer(groups * 4), gpu.buffer(k * 4)
    with pytest.raises(StraydogError, match="BF16 .kind 30. or Q8_0"):
        gpu.index_select_proj((mb.base(), 12, width), xb.base(), qb.base(), kb.base(), w.base(), vb.base(), groups, heads, dim, scale, rope, s.base(), k, o.base())
    with pytest.raises(StraydogError, match="invalid Straydog index shape"):
        gpu.index_select_proj((mb.base(), 30, 5004), xb.base(), qb.base(), kb.base(), w.base(), vb.base(), groups, heads, dim, scale, rope, s.base(), k, o.base())
    with pytest.raises(StraydogError, match="outside"):
        gpu.index_select_proj((mb.base(), 30, width), xb.at(4 * 100), qb.base(), kb.base(), w.base(), vb.base(), groups, heads, dim, scale, rope, s.base(), k, o.base())
    # a shape the selection half refuses is refused before the projection half has written the weights (gpu/kernels.cpp:5626-5640)
    marks = np.full(heads, 7.25, np.float32)
    gpu.write_buffer(w, 0, marks)
    with pytest.raises(StraydogError, match="invalid Straydog index shape"):
        gpu.index_select_proj((mb.base(), 30, width), xb.base(), qb.base(), kb.base(), w.base(), vb.base(), groups, heads, dim, scale, rope, s.base(), 0, o.base())
    with pytest.raises(StraydogError, match="outside"):
        gpu.index_select_proj((mb.base(), 30, width), xb.base(), qb.base(), kb.base(), w.base(), vb.base(), groups, heads, dim, scale, rope, s.base(), k + 1, o.base())
    assert np.array_equal(_read(gpu, w, np.float32, heads), marks)
    for b in (mb, w, s, o, fb, xb, qb, kb, pb, vb):
        gpu.release(b)


def test_sparse_attention_matches_the_oracle_and_bf16_rows_match_f32(gpu, oracle):
    # ds_state_bf16_gpu.rs:69-110 and the oracle's closed form (window ring, sink, -1 selections, rope in and out)
    rng = np.random.default_rng(11)
    from straydog_amd.backend import tagged_bf16
    for rows, heads, dim, window, raw_rows, n, selections, rope_dims in [(3, 64, 512, 128, 128, 900, 512, 64), (5, 10, 64, 5, 8, 40, 7, 16),
                                                                         (2, 32, 128, 16, 16, 64, 33, 0)]:
        q = rng.standard_normal((rows, heads, dim)).astype(np.float32)
        raw = rng.standard_normal((raw_rows, dim)).astype(np.float32)
        comp_bits, comp = _bf16_round(oracle, rng.standard_normal((n, dim)).astype(np.float32))
        positions = np.array([2, 500, 131, 77, 9][:rows], dtype=np.int32)
        selected = np.stack([rng.permutation(n)[:selections] for _ in range(rows)]).astype(np.int32)
        selected[0, ::5] = -1
        sinks = rng.standard_normal(heads).astype(np.float32)
        freqs = (1.6e5 ** (-(2.0 * np.arange(max(rope_dims // 2, 1))) / max(rope_dims, 1))).astype(np.float32)
        scale = float(1.0 / np.sqrt(dim))
        qb, rb, pb, sb, kb, fb = (gpu.upload(x) for x in (q, raw, positions, selected, sinks, freqs))
        cf, ch = gpu.upload(comp), gpu.upload(comp_bits)
        out = gpu.buffer(q.size * 4)
        results = []
        for compressed in (cf.base(), tagged_bf16(ch.base())):
            gpu.sparse_attention(qb.base(), rb.base(), raw_rows, pb.base(), window, compressed, n, sb.base(), selections, kb.base(), rows, heads,
                                 dim, scale, rope_dims, fb.base() if rope_dims else None, None, out.base())
            results.append(_read(gpu, out, np.float32, q.size).reshape(q.shape))
        assert np.array_equal(results[0].view(np.uint32), results[1].view(np.uint32)), "BF16 rows and their FP32 values differ"
        want = oracle.latent_attention(q, raw, positions, window, comp, selected, sinks, dim, scale, rope_dims, freqs if rope_dims else None)
        assert np.abs(results[0] - want).max() < 5e-5
        for b in (qb, rb, pb, sb, kb, fb, cf, ch, out):
            gpu.release(b)


@pytest.mark.parametrize("heads,groups,k", [(64, 5000, 256), (32, 3000, 2048), (16, 777, 100), (48, 20000, 512)])
def test_matrix_core_indexer_brackets_and_selects_exactly(gpu, oracle, heads, groups, k):
    # the fast indexer of the batched sparse path: every canonical score lies inside its bracket, and the indices chosen
    # from the brackets and the exact rescoring are those of the exact path, bit for bit (ties and short rows included)
    rng = np.random.default_rng(heads * 1000 + k)
    batch, dim = 4, 128
    q_bits, q_vals = _bf16_round(oracle, rng.standard_normal((batch, heads, dim)).astype(np.float32))
    keys = rng.standard_normal((batch, groups, dim)).astype(np.float32)
    keys[1, 100:400] = keys[1, 50]                  # a run of identical keys: equal scores, the tie rule decides
    keys[2] *= (rng.random((groups, 1)) * 4).astype(np.float32)     # rows of very different norms
    keys[3, ::7] = 0.0
    key_bits, key_vals = _bf16_round(oracle, keys)
    weights = rng.random((batch, heads)).astype(np.float32)
    weights[3, ::2] = 0.0
    visible = np.array([groups, groups - 37, groups, min(groups, k // 2)], dtype=np.int32)   # the last row: fewer visible than k
    qb, kb, wb, vb = gpu.upload(q_bits), gpu.upload(key_bits), gpu.upload(weights), gpu.upload(visible)
    lower, upper = gpu.buffer(batch * groups * 4), gpu.buffer(batch * groups * 4)
    for scale in (1.0, 0.37):
        gpu.index_score_bounds(qb.base(), kb.base(), wb.base(), vb.base(), batch, groups, heads, dim, scale, lower.base(), upper.base())
        low = _read(gpu, lower, np.float32, batch * groups).reshape(batch, groups)
        high = _read(gpu, upper, np.float32, batch * groups).reshape(batch, groups)
        indices = gpu.buffer(batch * k * 4)
        gpu.index_top_k(qb.base(), kb.base(), wb.base(), vb.base(), batch, groups, heads, dim, scale, None, k, indices.base())
        got = _read(gpu, indices, np.int32, batch * k).reshape(batch, k)
        for b in range(batch):
            want = oracle.index_scores(q_vals[b:b + 1], key_vals[b], weights[b:b + 1], visible[b:b + 1], scale)[0]
            seen = np.arange(groups) < visible[b]
            assert np.all(low[b][seen] <= want[seen]) and np.all(want[seen] <= high[b][seen])
            assert np.all(np.isneginf(low[b][~seen])) and np.all(np.isneginf(high[b][~seen]))
            width = (high[b][seen] - low[b][seen]).max()
            assert width < 1e-2 * max(1.0, np.abs(want[seen]).max())            # the brackets are tight, not vacuous
            assert np.array_equal(got[b], oracle.top_k(want[None, :], k)[0])
        gpu.release(indices)
    for b in (qb, kb, wb, vb, lower, upper):
        gpu.release(b)


def test_matrix_core_indexer_with_wide_bands_of_equal_scores(gpu, oracle):
    # what the brackets cannot decide is scored canonically; here that band is large: a row whose keys are all the same (every group
    # ties: the lowest indices win), a row where a few thousand identical keys straddle the cut, a row of zero keys (all scores 0,
    # brackets of zero width), next to an ordinary row -- twice in a row, the histograms the call keeps being its own to reset
    rng = np.random.default_rng(4242)
    batch, heads, dim, groups, k = 4, 64, 128, 20000, 512
    q_bits, q_vals = _bf16_round(oracle, rng.standard_normal((batch, heads, dim)).astype(np.float32))
    keys = rng.standard_normal((batch, groups, dim)).astype(np.float32)
    keys[0, :] = keys[0, 7]
    best = np.argsort(-np.abs(keys[1]).sum(axis=1))[:1]
    keys[1, 2000:5000] = keys[1, best[0]] * 3.0          # 3000 equal keys; whether they score high depends on q -- either way a wide tie
    keys[2, :] = 0.0
    key_bits, key_vals = _bf16_round(oracle, keys)
    weights = rng.random((batch, heads)).astype(np.float32)
    visible = np.array([groups, groups, groups - 11, groups], dtype=np.int32)
    qb, kb, wb, vb = gpu.upload(q_bits), gpu.upload(key_bits), gpu.upload(weights), gpu.upload(visible)
    indices = gpu.buffer(batch * k * 4)
    want = [oracle.top_k(oracle.index_scores(q_vals[b:b + 1], key_vals[b], weights[b:b + 1], visible[b:b + 1], 1.0), k)[0] for b in range(batch)]
    assert np.array_equal(want[0], np.arange(k)) and np.array_equal(want[2], np.arange(k))
    for run in range(2):
        gpu.write_buffer(indices, 0, np.full(batch * k, -7, np.int32))
        gpu.index_top_k(qb.base(), kb.base(), wb.base(), vb.base(), batch, groups, heads, dim, 1.0, None, k, indices.base())
        got = _read(gpu, indices, np.int32, batch * k).reshape(batch, k)
        for b in range(batch):
            assert np.array_equal(got[b], want[b]), (run, b)
    for b in (qb, kb, wb, vb, indices):
        gpu.release(b)


def test_batched_sparse_path_small(gpu, oracle):
    # BASELINE config 4 in small: index scores -> top-k (bit-exact) -> gather attention over BF16 latents, per sequence
    rng = np.random.default_rng(12)
    batch, groups, iheads, idim, k, heads, kdim, vdim = 3, 5000, 64, 128, 256, 64, 576, 512
    q_bits, q_vals = _bf16_round(oracle, rng.standard_normal((batch, iheads, idim)).astype(np.float32))
    key_bits, key_vals = _bf16_round(oracle, rng.standard_normal((batch, groups, idim)).astype(np.float32))
    weights = rng.random((batch, iheads)).astype(np.float32)
    visible = np.array([groups, groups - 100, 200], dtype=np.int32)    # the last row has fewer visible groups than k: -1 padding
    qb, kb, wb, vb = gpu.upload(q_bits), gpu.upload(key_bits), gpu.upload(weights), gpu.upload(visible)
    scores, indices = gpu.buffer(batch * groups * 4), gpu.buffer(batch * k * 4)
    gpu.index_top_k(qb.base(), kb.base(), wb.base(), vb.base(), batch, groups, iheads, idim, 1.0, scores.base(), k, indices.base())
    got_scores = _read(gpu, scores, np.float32, batch * groups).reshape(batch, groups)
    got_indices = _read(gpu, indices, np.int32, batch * k).reshape(batch, k)
    for b in range(batch):
        want = oracle.index_scores(q_vals[b:b + 1], key_vals[b], weights[b:b + 1], visible[b:b + 1], 1.0)
        assert np.array_equal(got_scores[b].view(np.uint32), want[0].view(np.uint32))
        assert np.array_equal(got_indices[b], oracle.top_k(want, k)[0])
    # without a scores buffer the indices are the same
    gpu.index_top_k(qb.base(), kb.base(), wb.base(), vb.base(), batch, groups, iheads, idim, 1.0, None, k, indices.base())
    assert np.array_equal(_read(gpu, indices, np.int32, batch * k).reshape(batch, k), got_indices)
    aq_bits, aq = _bf16_round(oracle, rng.standard_normal((batch, heads, kdim)).astype(np.float32))
    lat_bits, lat = _bf16_round(oracle, rng.standard_normal((batch, groups, kdim)).astype(np.float32))
    ab, lb, out = gpu.upload(aq_bits), gpu.upload(lat_bits), gpu.buffer(batch * heads * vdim * 4)
    scale = float(1.0 / np.sqrt(kdim))
    gpu.latent_attention(ab.base(), lb.base(), indices.base(), batch, groups, k, heads, kdim, vdim, scale, out.base())
    got = _read(gpu, out, np.float32, batch * heads * vdim).reshape(batch, heads, vdim)
    for b in range(batch):
        want = oracle.latent_attention(aq[b:b + 1], None, None, 0, lat_bits[b], got_indices[b:b + 1], None, vdim, scale)
        close_enough(got[b], want[0], f"sequence {b}")
        assert np.abs(got[b] - want[0]).max() < 5e-5
    for b in (qb, kb, wb, vb, scores, indices, ab, lb, out):
        gpu.release(b)


def test_latent_gather_long_chunks(gpu, oracle):
    # enough (sequence, chunk, head part) workgroups for every compute unit: the gather takes its longer chunks of 128 rows; a
    # selection that is no multiple of the chunk, padded with -1 and with rows out of range, and a head count that fills the
    # last head part only half
    rng = np.random.default_rng(77)
    batch, groups, k, heads, kdim, vdim = 16, 2500, 1000, 48, 576, 512
    aq_bits, aq = _bf16_round(oracle, rng.standard_normal((batch, heads, kdim)).astype(np.float32))
    lat_bits, lat = _bf16_round(oracle, rng.standard_normal((batch, groups, kdim)).astype(np.float32))
    selected = np.stack([rng.permutation(groups)[:k] for _ in range(batch)]).astype(np.int32)
    selected[1, 900:] = -1                              # a short list
    selected[2, ::3] = -1                               # holes
    selected[3, 5] = groups + 7                         # out of range: skipped here (the reference would read past its rows)
    selected[4, :] = -1                                 # nothing selected: zeros
    ab, lb, sb, out = gpu.upload(aq_bits), gpu.upload(lat_bits), gpu.upload(selected), gpu.buffer(batch * heads * vdim * 4)
    scale = float(1.0 / np.sqrt(kdim))
    gpu.latent_attention(ab.base(), lb.base(), sb.base(), batch, groups, k, heads, kdim, vdim, scale, out.base())
    got = _read(gpu, out, np.float32, batch * heads * vdim).reshape(batch, heads, vdim)
    for b in range(batch):
        if b == 4:
            continue                                    # (0 / 0 in the reference's arithmetic; zeros here, checked below)
        listed = np.where(selected[b:b + 1] >= groups, -1, selected[b:b + 1]).astype(np.int32)
        want = oracle.latent_attention(aq[b:b + 1], None, None, 0, lat_bits[b], listed, None, vdim, scale)
        close_enough(got[b], want[0], f"sequence {b}")
        assert np.abs(got[b] - want[0]).max() < 5e-5
    assert not got[4].any()
    for b in (ab, lb, sb, out):
        gpu.release(b)


def _dspark_check(label, actual, expected):
    # the reference's own bar (dspark_attention_gpu.rs:41-50): |a - b| / (1 + |b|) <= 2e-5
    error = np.abs(actual.astype(np.float64) - expected) / (1.0 + np.abs(expected))
    assert error.max() <= 2e-5, f"{label}: {error.max():.3e}"


def test_dspark_block_attention(gpu, oracle):
    # crates/straydog-engine/tests/dspark_attention_gpu.rs:52-124: 1..5 slots x histories 0, 37, 128 against the F64 statement, half the
    # heads, an anchor that moves on the device, the refusals, and the observable key set and sink mass
    from test_oracle_attention import _dspark_inputs
    from straydog_amd.backend import StraydogError
    q, ring, block, sinks = _dspark_inputs()
    qb, rb, bb, sb = (gpu.upload(a) for a in (q, ring, block, sinks))
    out = gpu.buffer(q.size * 4)
    for slots in range(1, 6):
        for history, anchor in ((0, 0), (37, 149), (128, 389)):
            gpu.dspark_attention(qb.base(), rb.base(), bb.base(), sb.base(), 64, slots, anchor, None, history, out.base())
            want = oracle.dspark_attention(q, ring, block, sinks, 64, slots, anchor, history)
            _dspark_check(f"B={slots} H={history} anchor={anchor}", _read(gpu, out, np.float32, want.size), want)
    for slots in (1, 4):
        gpu.dspark_attention(qb.base(), rb.base(), bb.base(), sb.base(), 32, slots, 149, None, 37, out.base())
        want = oracle.dspark_attention(q, ring, block, sinks, 32, slots, 149, 37)
        _dspark_check(f"B={slots} 32 heads", _read(gpu, out, np.float32, want.size), want)
    anchor = gpu.upload(np.array([389], dtype=np.int32))
    for at in (389, 200, 128):
        gpu.write_buffer(anchor, 0, np.array([at], dtype=np.int32))
        gpu.dspark_attention(qb.base(), rb.base(), bb.base(), sb.base(), 64, 3, 389, anchor.base(), 128, out.base())
        want = oracle.dspark_attention(q, ring, block, sinks, 64, 3, at, 128)
        _dspark_check(f"B=3 anchor on the device at {at}", _read(gpu, out, np.float32, want.size), want)
    for heads, slots, where, history in ((64, 0, 0, 0), (64, 6, 0, 0), (64, 1, 129, 129), (64, 1, 36, 37), (64, 1, 0xffffffff, 0), (0, 1, 0, 0),
                                         (65, 1, 0, 0)):
        with pytest.raises(StraydogError):
            gpu.dspark_attention(qb.base(), rb.base(), bb.base(), sb.base(), heads, slots, where, None, history, out.base())
    # zero queries, a ring that must never be attended, block keys of constant 1..5
    gpu.write_buffer(qb, 0, np.zeros(q.size, np.float32))
    gpu.write_buffer(rb, 0, np.full(ring.size, 23.0, np.float32))
    keys = np.repeat(np.arange(1, 6, dtype=np.float32), 512)
    gpu.write_buffer(bb, 0, keys)
    gpu.write_buffer(sb, 0, np.zeros(64, np.float32))

    def constant():
        gpu.dspark_attention(qb.base(), rb.base(), bb.base(), sb.base(), 64, 5, 0, None, 0, out.base())
        return _read(gpu, out, np.float32, q.size)
    _dspark_check("five keys and one sink", constant(), np.full(q.size, 2.5))
    keys[4 * 512:] = 11.0
    gpu.write_buffer(bb, 0, keys)
    _dspark_check("the last key changed", constant(), np.full(q.size, 3.5))
    for sink, expected in ((1000.0, 0.0), (-1000.0, 4.2)):
        gpu.write_buffer(sb, 0, np.full(64, sink, np.float32))
        _dspark_check(f"sink={sink}", constant(), np.full(q.size, expected))
    for b in (qb, rb, bb, sb, out, anchor):
        gpu.release(b)


def test_device_normal_values_are_the_xorshift_box_muller_stream(gpu, oracle):
    # the harness fills its workloads on the device with the generator the reference's tests use (xorshift64, two draws a Box-Muller
    # pair): the device reaches every stretch of the one stream by jumping, and the values are the host stream's (the double-precision
    # logarithm and sine of the two libraries may differ in the last place, which a float rarely shows)
    for seed, count in ((0x9e3779b97f4a7c15 ^ 1, 300001), (7, 129), (0, 2)):
        out = gpu.buffer(count * 4)
        gpu.fill_normal(out.base(), count, seed, 0)
        got = _read(gpu, out, np.float32, count)
        want = oracle.fill_normal(seed, count)
        differ = np.flatnonzero(got != want)
        assert len(differ) <= max(2, count // 100000), f"{len(differ)} of {count} values differ"
        assert np.allclose(got, want, rtol=3e-7, atol=1e-9)
        gpu.release(out)
    out = gpu.buffer(5000 * 4)
    gpu.fill_uniform(out.base(), 5000, 11, -0.5, 1.5)
    assert np.array_equal(_read(gpu, out, np.float32, 5000), oracle.fill_uniform(11, 5000, -0.5, 1.5))
    gpu.release(out)



def test_sparse_path_operands_off_16_byte_boundaries(gpu, oracle):
    # queries and keys that start 2 bytes off a 16-byte boundary: the matrix-core kernels read whole 16-byte pieces, so such
    # operands take the general kernels -- the same indices and outputs
    rng = np.random.default_rng(91)
    batch, groups, heads, dim, k = 2, 3000, 64, 128, 256
    q_bits, q_vals = _bf16_round(oracle, rng.standard_normal((batch, heads, dim)).astype(np.float32))
    key_bits, key_vals = _bf16_round(oracle, rng.standard_normal((batch, groups, dim)).astype(np.float32))
    weights = rng.random((batch, heads)).astype(np.float32)
    visible = np.array([groups, groups - 9], dtype=np.int32)
    qb, kb = gpu.buffer(q_bits.size * 2 + 16), gpu.buffer(key_bits.size * 2 + 16)
    gpu.write_buffer(qb, 2, q_bits); gpu.write_buffer(kb, 2, key_bits)
    wb, vb, indices = gpu.upload(weights), gpu.upload(visible), gpu.buffer(batch * k * 4)
    gpu.index_top_k(qb.at(2), kb.at(2), wb.base(), vb.base(), batch, groups, heads, dim, 1.0, None, k, indices.base())
    got = _read(gpu, indices, np.int32, batch * k).reshape(batch, k)
    for b in range(batch):
        want = oracle.index_scores(q_vals[b:b + 1], key_vals[b], weights[b:b + 1], visible[b:b + 1], 1.0)
        assert np.array_equal(got[b], oracle.top_k(want, k)[0])
    kdim, vdim, aheads = 576, 512, 32
    a_bits, a_vals = _bf16_round(oracle, rng.standard_normal((batch, aheads, kdim)).astype(np.float32))
    lat_bits, _ = _bf16_round(oracle, rng.standard_normal((batch, groups, kdim)).astype(np.float32))
    ab, lb, out = gpu.upload(a_bits), gpu.buffer(lat_bits.size * 2 + 16), gpu.buffer(batch * aheads * vdim * 4)
    gpu.write_buffer(lb, 2, lat_bits)
    scale = float(1.0 / np.sqrt(kdim))
    gpu.latent_attention(ab.base(), lb.at(2), indices.base(), batch, groups, k, aheads, kdim, vdim, scale, out.base())
    result = _read(gpu, out, np.float32, batch * aheads * vdim).reshape(batch, aheads, vdim)
    for b in range(batch):
        want = oracle.latent_attention(a_vals[b:b + 1], None, None, 0, lat_bits[b], got[b:b + 1], None, vdim, scale)
        close_enough(result[b], want[0], f"sequence {b}")
    for b in (qb, kb, wb, vb, indices, ab, lb, out):
        gpu.release(b)
