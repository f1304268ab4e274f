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
