"""Pins the oracle's indexer scores, top-k, candidate blocks and Qwen block selection (CPU only).

Independent checks: the top-k rule by brute force (stable sort by (-key, index)) on the adversarial
generator of crates/straydog-engine/tests/fused_gpu.rs:361-388; the canonical score order against a
scalar numpy float32 fma chain (math.fma is absent in Python 3.10, so exact products are formed in
float64 where they are exact: bf16 x bf16 and small integers) and against float64; candidate blocks
against the rule of fused_gpu.rs:504-517; qsa_select by brute force.
"""
import numpy as np
import pytest

MASK = (1 << 64) - 1


class Random:
    # crates/straydog-engine/tests/fused_gpu.rs:39-53
    def __init__(self, seed):
        self.s = seed

    def next(self):
        self.s ^= (self.s << 13) & MASK
        self.s ^= self.s >> 7
        self.s ^= (self.s << 17) & MASK
        return self.s


def _key(value):
    bits = int(np.float32(0.0 if value == 0.0 else value).view(np.uint32))
    return (~bits) & 0xffffffff if bits & 0x80000000 else bits | 0x80000000


def _brute_top_k(scores, k):
    floor = _key(float("-inf"))
    live = [(g, _key(s)) for g, s in enumerate(scores) if _key(s) > floor]
    live.sort(key=lambda item: (-item[1], item[0]))
    kept = sorted(g for g, _ in live[:k])
    return kept + [-1] * (k - len(kept))


def _adversarial(random, rows, groups):
    # fused_gpu.rs:370-379
    out = np.zeros(rows * groups, dtype=np.float32)
    for i in range(rows * groups):
        draw = random.next()
        if groups == 600 and draw % 8 != 0:
            out[i] = -np.inf
            continue
        m = draw % 97
        if m <= 6:
            out[i] = -np.inf
        elif m == 7:
            out[i] = np.inf
        elif m == 8:
            out[i] = -0.0
        else:
            out[i] = ((draw >> 8) % 17) * 0.25 - 2.0 + (0.125 if i % 1000 == 999 else 0.0)
    return out.reshape(rows, groups)


def test_top_k_key_orders_floats(oracle):
    values = [-np.inf, -3.5, -1e-30, -0.0, 0.0, 1e-30, 2.0, np.inf]
    keys = [oracle.top_k_key(v) for v in values]
    assert keys[3] == keys[4]
    assert keys == sorted(keys)
    assert all(_key(v) == k for v, k in zip(values, keys))


@pytest.mark.parametrize("groups", [511, 512, 513, 600, 4096, 30000])
def test_top_k_rule_on_adversarial_ties(oracle, groups):
    random = Random(0x2f6b91d3c0a54e77 ^ groups)
    k = 512
    scores = _adversarial(random, 2, groups)
    got = oracle.top_k(scores, k)
    for row in range(2):
        assert list(got[row]) == _brute_top_k(scores[row], k), (groups, row)


def test_top_k_small_cases(oracle):
    s = np.array([[1.0, 1.0, 1.0, 2.0, -np.inf, 1.0]], dtype=np.float32)
    assert list(oracle.top_k(s, 3)[0]) == [0, 1, 3]           # ties keep the lowest indices, ascending order
    assert list(oracle.top_k(s, 6)[0]) == [0, 1, 2, 3, 5, -1]  # -inf never kept
    z = np.array([[0.0, -0.0, -1.0]], dtype=np.float32)
    assert list(oracle.top_k(z, 1)[0]) == [0]                  # -0 ties +0


def _chain_scores(q, keys, weights, visible, scale):
    """Canonical order in numpy float32; valid when every product q*k is exact in float64 and the running
    fused sum is reproduced by rounding (acc + exact product) once: float64 holds acc + product exactly
    for the operand ranges used here (bf16-valued inputs), so one rounding to float32 equals fmaf."""
    rows, heads, dim = q.shape
    groups = keys.shape[0]
    out = np.full((rows, groups), -np.inf, dtype=np.float32)
    for r in range(rows):
        limit = min(groups, max(int(visible[r]), 0))
        for g in range(limit):
            total = np.float32(0.0)
            for h in range(heads):
                acc = np.float32(0.0)
                for d in range(dim):
                    acc = np.float32(np.float64(acc) + np.float64(q[r, h, d]) * np.float64(keys[g, d]))
                term = np.float32(max(acc, np.float32(0.0)) * weights[r, h])
                total = np.float32(total + term)
            out[r, g] = np.float32(total * np.float32(scale))
    return out


def test_index_scores_canonical_order(oracle):
    rng = np.random.default_rng(21)
    rows, heads, dim, groups = 2, 5, 32, 37
    # bf16-valued operands with a narrow exponent range: acc + q*k is exact in float64
    q = (oracle.to_bf16(rng.standard_normal((rows, heads, dim)).astype(np.float32)).astype(np.uint32) << 16).view(np.float32)
    keys_bits = oracle.to_bf16(rng.standard_normal((groups, dim)).astype(np.float32))
    keys = (keys_bits.astype(np.uint32) << 16).view(np.float32)
    weights = rng.random((rows, heads)).astype(np.float32)
    visible = np.array([groups, 20], dtype=np.int32)
    scale = np.float32(0.37)
    want = _chain_scores(q, keys, weights, visible, scale)
    got = oracle.index_scores(q, keys, weights, visible, scale)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # the same bits from the BF16 (tagged) keys, and with one thread or many
    assert np.array_equal(oracle.index_scores(q, keys_bits, weights, visible, scale, threads=1).view(np.uint32), want.view(np.uint32))
    wide = oracle.index_scores_f64(q, keys, weights, visible, scale)
    finite = np.isfinite(want)
    assert np.array_equal(np.isfinite(wide), finite)
    assert np.abs(wide[finite] - want[finite]).max() < 1e-4
    # a negative visible count sees nothing (gpu/ops.hpp:1707)
    none = oracle.index_scores(q, keys, weights, np.array([-3, 0], np.int32), scale)
    assert np.all(np.isneginf(none))


def test_index_scores_term_is_rounded_before_the_sum(oracle):
    # one head would hide a fused multiply-add; pick values where fma(relu, w, total) differs from round(relu*w) + total
    q = np.zeros((1, 2, 32), dtype=np.float32); keys = np.zeros((1, 32), dtype=np.float32)
    a = np.float32(1.0 + 2.0 ** -12)
    q[0, 0, 0] = np.float32(2.0 ** -30); q[0, 1, 0] = a
    keys[0, 0] = 1.0
    w = np.array([[1.0, a]], dtype=np.float32)
    got = oracle.index_scores(q, keys, w, np.array([1], np.int32), 1.0)[0, 0]
    # a * a = 1 + 2^-11 + 2^-24 is an exact tie in fp32 and rounds (to even) to 1 + 2^-11; adding 2^-30 then changes nothing
    assert got == np.float32(1.0 + 2.0 ** -11)
    # a fused multiply-add would see 2^-30 + (1 + 2^-11 + 2^-24), above the tie, and round up
    assert np.float32(2.0 ** -30 + (1.0 + 2.0 ** -12) ** 2) == np.float32(1.0 + 2.0 ** -11 + 2.0 ** -23)


def test_index_candidates_rule(oracle):
    # fused_gpu.rs:504-517
    rng = np.random.default_rng(22)
    rows, groups, blocks, block = 3, 1000, 40, 8
    scores = rng.standard_normal((rows, groups)).astype(np.float32)
    seen = np.array([groups, 700, 37], dtype=np.int32)
    for r in range(rows):
        scores[r, seen[r]:] = -np.inf
    got = oracle.index_candidates(scores, seen, blocks, block)
    count = (groups + block - 1) // block
    for r in range(rows):
        newest = (int(seen[r]) - 1) // block
        best = [np.inf if b == newest else max(scores[r, b * block:min((b + 1) * block, groups)], key=_key) for b in range(count)]
        assert list(got[r]) == _brute_top_k(best, blocks)


def test_qsa_select_brute_force(oracle):
    rng = np.random.default_rng(23)
    # few blocks: every causal position
    short = oracle.qsa_select(np.zeros(10, np.float32), 17, keep_blocks=8)
    assert list(short) == [float(i) for i in range(18)]
    for position in (41, 42, 43, 100):
        complete = (position + 1) // 4
        scores = (rng.integers(0, 6, complete) * 0.5).astype(np.float32)      # many ties
        got = oracle.qsa_select(scores, position, keep_blocks=8)
        order = sorted(range(complete), key=lambda b: (-int(scores[b].view(np.uint32)), b))[:8]
        want = [float(b * 4 + t) for b in sorted(order) for t in range(4)] + [float(i) for i in range(complete * 4, position + 1)]
        assert list(got) == want


def test_fill_normal_moments(oracle):
    x = oracle.fill_normal(0x9e3779b97f4a7c15, 200000)
    assert abs(float(x.mean())) < 0.01 and abs(float(x.std()) - 1.0) < 0.01
    assert np.array_equal(x, oracle.fill_normal(0x9e3779b97f4a7c15, 200000))
    u = oracle.fill_uniform(5, 100000)
    assert 0.0 <= u.min() and u.max() < 1.0 and abs(float(u.mean()) - 0.5) < 0.01


def _q8_0_rows(rng, heads, cols):
    """ggml Q8_0 rows as the reference's test draws them (fused_gpu.rs:448-455): an FP16 scale of moderate exponent, 32 int8."""
    blocks = heads * cols // 32
    out = np.zeros((blocks, 34), dtype=np.uint8)
    bits = ((rng.integers(0, 2, blocks) << 15) | ((8 + rng.integers(0, 5, blocks)) << 10) | rng.integers(0, 1024, blocks)).astype(np.uint16)
    out[:, 0] = bits & 0xff
    out[:, 1] = bits >> 8
    out[:, 2:] = rng.integers(0, 256, size=(blocks, 32), dtype=np.uint8)
    return out.reshape(-1), bits.view(np.float16).astype(np.float64), out[:, 2:].view(np.int8).astype(np.float64)


def test_index_projection_is_the_stated_order_and_a_dot_product(oracle):
    rng = np.random.default_rng(31)
    heads, cols = 5, 1024
    x = (rng.random(cols) * 4 - 2).astype(np.float32)
    # BF16 rows: against float64, and against the stated order written out with numpy float32 steps
    w = (rng.standard_normal((heads, cols)) * 0.05).astype(np.float32)
    bits = (w.view(np.uint32) >> 16).astype(np.uint16)
    values = (bits.astype(np.uint32) << 16).view(np.float32)
    got = oracle.index_projection(bits.view(np.uint8).reshape(-1), 30, cols, x, heads)
    assert np.allclose(got, values.astype(np.float64) @ x.astype(np.float64), rtol=0, atol=2e-5)
    import math
    def f32(v):
        return float(np.float32(v))
    def fma(a, b, c):         # exact product and sum in Python floats are not exact; use fractions for the single rounding
        from fractions import Fraction
        return f32(Fraction(float(a)) * Fraction(float(b)) + Fraction(float(c)))
    for h in range(2):
        lanes = []
        for lane in range(64):
            total = 0.0
            for u in range(lane, cols // 8, 64):
                chain = 0.0
                for i in range(8):
                    chain = fma(values[h, u * 8 + i], x[u * 8 + i], chain)
                total = f32(np.float32(total) + np.float32(chain))
            lanes.append(total)
        offset = 32
        while offset:
            lanes = [f32(np.float32(lanes[i]) + np.float32(lanes[i + offset])) for i in range(offset)]
            offset //= 2
        assert np.float32(lanes[0]).view(np.uint32) == got[h].view(np.uint32)
    # Q8_0 rows: against float64 of d * q . x, a tiny case against the definition by hand, and block independence
    raw, d, q = _q8_0_rows(rng, heads, cols)
    got = oracle.index_projection(raw, 8, cols, x, heads)
    want = ((d[:, None] * q).reshape(heads, cols) * x.astype(np.float64)).sum(axis=1)
    assert np.allclose(got, want, rtol=1e-5, atol=1e-3 * np.abs(want).max())
    one = np.zeros(34, dtype=np.uint8)
    one[0:2] = np.frombuffer(np.float16(0.5).tobytes(), dtype=np.uint8)
    one[2:5] = np.array([3, 0xfe, 127], dtype=np.uint8)          # 3, -2, 127
    xs = np.zeros(32, dtype=np.float32); xs[:3] = [2.0, 4.0, 1.0]
    assert oracle.index_projection(one, 8, 32, xs, 1)[0] == np.float32(0.5 * (6 - 8 + 127))
