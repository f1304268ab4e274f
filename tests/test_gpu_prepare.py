"""GPU parity of the inputs of a dense attention step, written after the reference's own model-free tests:
crates/straydog-engine/tests/fused_gpu.rs:225-268 (a prepared attention step matches sd_op_split + sd_op_rms_norm +
sd_op_rope_halves + sd_op_scatter bit for bit: positions out of order, large angles) and :304-324 (shapes whose sizes
overflow are refused); each op also against the CPU oracle."""
import numpy as np
import pytest

from gpu_util import backend
from test_oracle_qsa import _prepare_case

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gpu():
    with backend(1 << 30) as handle:
        yield handle


def _read(gpu, buffer, count):
    return gpu.read_buffer(buffer, 0, np.float32, count)


@pytest.mark.parametrize("rows,heads,kv_heads,dim,rope_dims,context", [(3, 8, 1, 256, 64, 16), (5, 24, 2, 256, 64, 40), (2, 4, 4, 128, 128, 8),
                                                                      (1, 2, 1, 1000, 0, 30)])
def test_a_prepared_attention_step_matches_its_ops(gpu, oracle, rows, heads, kv_heads, dim, rope_dims, context):
    case = _prepare_case(np.random.default_rng(rows * 100 + dim), rows, heads, kv_heads, dim, max(rope_dims, 2), context)
    if rows == 5:
        case["positions"][3] = 1000           # a position outside the cache writes no row of it
    kv_width = kv_heads * dim
    q_full, v = gpu.upload(case["q_full"]), gpu.upload(case["v"])
    q_weight, k_weight = gpu.upload(case["q_weight"]), gpu.upload(case["k_weight"])
    frequencies, positions = gpu.upload(case["frequencies"]), gpu.upload(case["positions"])

    def outputs():
        return [gpu.buffer(rows * heads * dim * 4), gpu.buffer(rows * heads * dim * 4), gpu.upload(case["k"]), gpu.upload(case["cache"]),
                gpu.upload(case["cache"])]
    # the ops
    q_1, gate_1, k_1, keys_1, values_1 = outputs()
    gpu.split(q_full.base(), rows * heads, dim, q_1.base(), gate_1.base())
    gpu.rms_norm(q_1.base(), q_weight.base(), rows * heads, dim, 1e-6, q_1.base())
    gpu.rms_norm(k_1.base(), k_weight.base(), rows * kv_heads, dim, 1e-6, k_1.base())
    if rope_dims:
        gpu.rope_halves(q_1.base(), rows, heads, dim, rope_dims, positions.base(), frequencies.base())
        gpu.rope_halves(k_1.base(), rows, kv_heads, dim, rope_dims, positions.base(), frequencies.base())
    gpu.scatter(k_1.base(), positions.base(), rows, kv_width, keys_1.base(), context)
    gpu.scatter(v.base(), positions.base(), rows, kv_width, values_1.base(), context)
    # one launch
    q_2, gate_2, k_2, keys_2, values_2 = outputs()
    gpu.attention_prepare(q_full.base(), k_2.base(), v.base(), rows, heads, kv_heads, dim, q_weight.base(), k_weight.base(), 1e-6, rope_dims,
                          positions.base(), frequencies.base(), q_2.base(), gate_2.base(), keys_2.base(), values_2.base(), context)
    sizes = {"queries": rows * heads * dim, "gates": rows * heads * dim, "keys": rows * kv_width, "key cache": context * kv_width,
             "value cache": context * kv_width}
    got = {}
    for label, first, second in (("queries", q_1, q_2), ("gates", gate_1, gate_2), ("keys", k_1, k_2), ("key cache", keys_1, keys_2),
                                 ("value cache", values_1, values_2)):
        a, b = _read(gpu, first, sizes[label]), _read(gpu, second, sizes[label])
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), label
        got[label] = b
    # and the oracle: the reciprocal square root is the device's own (about an ulp), the rest is the same arithmetic
    keys, values = case["cache"].copy(), case["cache"].copy()
    q, gate, k_after = oracle.attention_prepare(case["q_full"], case["k"], case["v"], case["q_weight"], case["k_weight"], 1e-6, rope_dims,
                                                case["positions"], case["frequencies"], keys, values)
    assert np.array_equal(got["gates"], gate.ravel()) and np.array_equal(got["value cache"], values.ravel())
    for label, want in (("queries", q), ("keys", k_after), ("key cache", keys)):
        assert np.allclose(got[label], want.ravel(), rtol=2e-6, atol=1e-6), label
    for b in (q_full, v, q_weight, k_weight, frequencies, positions, q_1, gate_1, k_1, keys_1, values_1, q_2, gate_2, k_2, keys_2, values_2):
        gpu.release(b)


def test_shapes_that_overflow_are_refused(gpu):
    from straydog_amd.backend import StraydogError
    buffer = gpu.buffer(1 << 20)
    floats = gpu.upload(np.zeros(256, dtype=np.float32))
    huge = 1 << 62
    b, f = buffer.base(), floats.base()
    with pytest.raises(StraydogError):
        gpu.split(b, huge, 8, b, b)
    with pytest.raises(StraydogError):
        gpu.rope_halves(b, huge, 4, 8, 4, f, f)
    with pytest.raises(StraydogError):
        gpu.rms_norm(b, f, huge, 16, 1e-6, b)
    with pytest.raises(StraydogError):
        gpu.scatter(b, f, huge, 16, b, 4)
    # heads beyond a launch's dimensions, a context whose cache size wraps (fused_gpu.rs:316-322)
    with pytest.raises(StraydogError):
        gpu.attention_prepare(b, b, b, 1, 1 << 40, 1, 64, f, f, 1e-6, 0, f, f, b, b, b, b, 16)
    with pytest.raises(StraydogError):
        gpu.attention_prepare(b, b, b, 1, 1, 1 << 40, 64, f, f, 1e-6, 0, f, f, b, b, b, b, 16)
    with pytest.raises(StraydogError):
        gpu.attention_prepare(b, b, b, 1, 1, 1, 64, f, f, 1e-6, 0, f, f, b, b, b, b, huge)
    with pytest.raises(StraydogError, match="outside"):
        gpu.rms_norm(b, f, 1, 257, 1e-6, b)                      # the weight holds 256 values
    gpu.release(buffer); gpu.release(floats)


def test_norm_rope_matches_its_ops_and_scatters(gpu):
    # sd_op_norm_rope == sd_op_rms_norm then sd_op_rope (the last rope_dims values, adjacent pairs), rows stored where out_rows says
    rng = np.random.default_rng(31)
    rows, width, rope_dims, out_count = 6, 576, 64, 9
    x = (rng.standard_normal((rows, width)) * 3).astype(np.float32)
    weight = (rng.standard_normal(width) * 2).astype(np.float32)
    positions = np.array([70001, 3, 0, 123456, 9, 77], dtype=np.int32)
    frequencies = (1.6e5 ** (-(2.0 * np.arange(rope_dims // 2)) / rope_dims)).astype(np.float32)
    out_rows = np.array([4, 0, 8, 2, 11, -1], dtype=np.int32)            # the last two lie outside the output: not stored
    xb, wb, pb, fb, rb = (gpu.upload(a) for a in (x, weight, positions, frequencies, out_rows))
    apart = gpu.buffer(rows * width * 4)
    gpu.rms_norm(xb.base(), wb.base(), rows, width, 1e-6, apart.base())
    gpu.rope(apart.base(), rows, 1, width, rope_dims, pb.base(), fb.base())
    want = _read(gpu, apart, rows * width).reshape(rows, width)
    fused = gpu.buffer(rows * width * 4)
    gpu.norm_rope(xb.base(), wb.base(), rows, width, 1e-6, rope_dims, pb.base(), fb.base(), None, fused.base(), rows)
    assert np.array_equal(_read(gpu, fused, rows * width).view(np.uint32), want.reshape(-1).view(np.uint32))
    canary = np.full((out_count, width), -3.25, dtype=np.float32)
    spread = gpu.upload(canary)
    gpu.norm_rope(xb.base(), wb.base(), rows, width, 1e-6, rope_dims, pb.base(), fb.base(), rb.base(), spread.base(), out_count)
    got = _read(gpu, spread, out_count * width).reshape(out_count, width)
    for r in range(rows):
        if 0 <= out_rows[r] < out_count:
            assert np.array_equal(got[out_rows[r]], want[r])
            canary[out_rows[r]] = want[r]
    assert np.array_equal(got, canary), "rows that no index names are left alone"
    from straydog_amd.backend import StraydogError
    with pytest.raises(StraydogError, match="in place"):
        gpu.norm_rope(xb.base(), wb.base(), rows, width, 1e-6, rope_dims, pb.base(), fb.base(), rb.base(), xb.base(), rows)
    for b in (xb, wb, pb, fb, rb, apart, fused, spread):
        gpu.release(b)


def test_attention_rope_table_serves_the_next_attention_once(gpu):
    # sd_attention_turns_reserve / _arm: the norm of the pass's rows writes the table, the next sd_op_sparse_attention of those rows
    # reads it (the same bits as forming the angles), and only that one
    rng = np.random.default_rng(32)
    rows, heads, dim, window, n, selections, rope_dims = 3, 8, 128, 8, 40, 12, 64
    q = rng.standard_normal((rows, heads, dim)).astype(np.float32)
    raw = rng.standard_normal((window, dim)).astype(np.float32)
    compressed = rng.standard_normal((n, dim)).astype(np.float32)
    positions = np.array([70001, 5, 131], dtype=np.int32)
    elsewhere = np.array([11, 70001, 5], dtype=np.int32)
    selected = np.stack([rng.permutation(n)[:selections] for _ in range(rows)]).astype(np.int32)
    sinks = rng.standard_normal(heads).astype(np.float32)
    frequencies = (1.6e5 ** (-(2.0 * np.arange(rope_dims // 2)) / rope_dims)).astype(np.float32)
    side = rng.standard_normal((rows, dim)).astype(np.float32)           # the rows whose norm fills the table
    qb, rb, cb, pb, eb, sb, kb, fb, nb = (gpu.upload(a) for a in (q, raw, compressed, positions, elsewhere, selected, sinks, frequencies, side))
    weight = gpu.upload(np.ones(dim, dtype=np.float32))
    out, normed = gpu.buffer(q.size * 4), gpu.buffer(side.size * 4)

    def attend():
        gpu.sparse_attention(qb.base(), rb.base(), window, pb.base(), window, cb.base(), n, sb.base(), selections, kb.base(), rows, heads, dim,
                             float(1.0 / np.sqrt(dim)), rope_dims, fb.base(), None, out.base())
        return _read(gpu, out, q.size).copy()
    plain = attend()
    gpu.attention_turns_reserve(rows, rope_dims)
    gpu.attention_turns_arm(rows)
    gpu.norm_rope(nb.base(), weight.base(), rows, dim, 1e-6, rope_dims, pb.base(), fb.base(), None, normed.base(), rows)
    assert np.array_equal(attend().view(np.uint32), plain.view(np.uint32)), "the table's turns are the angles' own"
    # a table filled for other positions shows that it is what the next attention reads, and that the one after does not
    gpu.attention_turns_arm(rows)
    gpu.norm_rope(nb.base(), weight.base(), rows, dim, 1e-6, rope_dims, eb.base(), fb.base(), None, normed.base(), rows)
    assert not np.array_equal(attend(), plain)
    assert np.array_equal(attend().view(np.uint32), plain.view(np.uint32))
    # an arm for another number of rows is spent without a table
    gpu.attention_turns_arm(rows + 1)
    gpu.norm_rope(nb.base(), weight.base(), rows, dim, 1e-6, rope_dims, eb.base(), fb.base(), None, normed.base(), rows)
    assert np.array_equal(attend().view(np.uint32), plain.view(np.uint32))
    from straydog_amd.backend import StraydogError
    with pytest.raises(StraydogError, match="rope"):
        gpu.attention_turns_reserve(rows, 130)
    for b in (qb, rb, cb, pb, eb, sb, kb, fb, nb, weight, out, normed):
        gpu.release(b)
