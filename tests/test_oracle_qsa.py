"""Pins the oracle's Qwen block-indexer inputs and scores (CPU only).

Independent checks, none of which retypes the oracle's code path:
* block scores: every fused multiply-add redone in exact rational arithmetic and rounded once to float32 (pure
  Python, a sample of blocks), which separates a fused chain from multiply-then-add; a float64 closed form on the
  whole row; small-integer inputs where every order of summation gives the same bits;
* normalisation and pooling: float64 closed forms of gpu/sparse_attention.hpp:2-23 and :87-108, plus what the
  rotation fixes: the pairs (c, c + 32) keep their norms, position 0 and columns from 64 on are not turned, and the
  ring of sixteen holds the span's last four rows (:132-139).
"""
from fractions import Fraction

import numpy as np


def _round_f32(exact):
    """The float32 nearest to a Fraction, ties to the even mantissa."""
    if exact == 0:
        return np.float32(0.0)
    near = np.float32(float(exact))
    around = [near, np.nextafter(near, np.float32(np.inf)), np.nextafter(near, np.float32(-np.inf))]
    return min(around, key=lambda v: (abs(Fraction(float(v)) - exact), int(v.view(np.uint32)) & 1))


def _exact_score(queries, blocks, token, block):
    total = None
    for h in range(4):
        dot = np.float32(0.0)
        for c in range(128):
            dot = _round_f32(Fraction(float(blocks[c, block])) * Fraction(float(queries[token, h * 128 + c])) + Fraction(float(dot)))
        part = dot if dot > 0 else np.float32(0.0)
        total = part if total is None else np.float32(total + part)
    return total


def _inputs(oracle, seed, steps, pool, stride=512):
    queries = oracle.fill_normal(seed, steps * stride).reshape(steps, stride)
    blocks = oracle.fill_normal(seed ^ 0x55, 128 * pool).reshape(128, pool)
    return queries, blocks


def test_block_scores_are_fused_chains_rounded_once(oracle):
    base, steps, pool = 2049, 4, 530                       # rows 2 and 3 have 513 complete blocks, rows 0 and 1 have 512
    queries, blocks = _inputs(oracle, 11, steps, pool)
    scores = oracle.qsa_block_scores(queries, blocks, base, scores=np.full((steps, pool), -7.0, np.float32))
    assert np.all(scores[:2] == -7.0), "rows with no more than 512 complete blocks are not scored"
    assert np.all(scores[2:, 513:] == -7.0), "blocks past the row's complete count are left alone"
    separates = 0
    for token, block in [(2, 0), (2, 512), (3, 17), (3, 300), (2, 255), (3, 511), (2, 100), (3, 412)]:
        want = _exact_score(queries, blocks, token, block)
        assert scores[token, block].view(np.uint32) == want.view(np.uint32)
        unfused = sum(np.float32(max(0.0, _unfused(queries[token, h * 128:h * 128 + 128], blocks[:, block]))) for h in range(4))
        separates += np.float32(unfused) != want
    assert separates, "the sample must hold a case where multiply-then-add differs from the fused chain"


def _unfused(q, k):
    dot = np.float32(0.0)
    for c in range(128):
        dot = np.float32(dot + np.float32(k[c] * q[c]))
    return float(dot)


def test_block_scores_float64_and_integers(oracle):
    base, steps, pool = 3000, 6, 900
    queries, blocks = _inputs(oracle, 12, steps, pool, stride=640)
    scores = oracle.qsa_block_scores(queries, blocks, base)
    for token in range(steps):
        complete = (base + token + 1) // 4
        q = queries[token, :512].astype(np.float64).reshape(4, 128)
        want = np.maximum(q @ blocks[:, :complete].astype(np.float64), 0.0).sum(axis=0)
        assert np.allclose(scores[token, :complete], want, rtol=1e-5, atol=1e-4)
        assert np.all(scores[token, complete:] == 0.0)
    # small integers: every partial sum is exact, so any correct order gives these bits
    rng = np.random.default_rng(5)
    queries = rng.integers(-3, 4, (steps, 512)).astype(np.float32)
    blocks = rng.integers(-3, 4, (128, pool)).astype(np.float32)
    scores = oracle.qsa_block_scores(queries, blocks, base)
    complete = (base + 1) // 4
    want = np.maximum(queries[0].astype(np.int64).reshape(4, 128) @ blocks[:, :complete].astype(np.int64), 0).sum(axis=0)
    assert np.array_equal(scores[0, :complete], want.astype(np.float32))


def _rope64(values, position):
    """The turned vectors in float64, and how far each value may move when the float32 angle (position over a
    float32 power, gpu/sparse_attention.hpp:4) lands one float32 step away: at position 70000 a step is 0.008 rad."""
    out, slack = values.copy(), np.zeros_like(values)
    c = np.arange(32)
    angle = (np.float32(position) / np.power(np.float32(1e7), (c / 32.0).astype(np.float32))).astype(np.float32)
    step = np.spacing(angle).astype(np.float64)
    angle = angle.astype(np.float64)
    low, high = values[..., :32], values[..., 32:64]
    out[..., :32] = low * np.cos(angle) - high * np.sin(angle)
    out[..., 32:64] = high * np.cos(angle) + low * np.sin(angle)
    slack[..., :32] = slack[..., 32:64] = 2.0 * step * np.hypot(low, high)
    return out, slack


def _close(got, want, slack, tolerance=2e-5):
    return np.all(np.abs(got - want) <= tolerance + tolerance * np.abs(want) + slack)


def test_normalize_closed_form_and_rotation_invariants(oracle):
    rng = np.random.default_rng(3)
    for width, heads, stride in ((256, 24, 512), (256, 2, 256), (128, 4, 128)):
        rows, position = 3, 70001
        source = rng.standard_normal(rows * heads * stride).astype(np.float32) * 3
        norm = (0.4 + 1.2 * rng.random(width)).astype(np.float32)
        got = oracle.qsa_normalize(source, norm, rows, heads, width, stride, position)
        x = source.reshape(rows * heads, stride)[:, :width].astype(np.float64)
        flat = x * norm / np.sqrt((x * x).mean(axis=1, keepdims=True) + 1e-6)
        for r in range(rows):
            span = slice(r * heads, (r + 1) * heads)
            want, slack = _rope64(flat[span], position + r)
            assert _close(got[span], want, slack)
            assert slack.max() < 0.1 and not _close(got[span], _rope64(flat[span], position + r + 1)[0], slack), "the check tells positions apart"
            # a rotation keeps each pair's norm and leaves columns from 64 on alone
            assert np.allclose(got[span, :32].astype(np.float64) ** 2 + got[span, 32:64].astype(np.float64) ** 2,
                               flat[span, :32] ** 2 + flat[span, 32:64] ** 2, rtol=1e-4, atol=1e-6)
            assert np.allclose(got[span, 64:], flat[span, 64:], rtol=1e-6, atol=1e-7)
        still = oracle.qsa_normalize(source, norm, 1, heads, width, stride, 0)
        assert np.allclose(still, flat[:heads], rtol=1e-6, atol=1e-7), "position 0 turns nothing"


def test_pool_closed_form_and_ring(oracle):
    rng = np.random.default_rng(4)
    pool = 40
    norm = (0.4 + 1.2 * rng.random(128)).astype(np.float32)
    stream = rng.standard_normal((97, 128)).astype(np.float32)            # the index-key input of every position
    blocks = np.zeros((128, pool), np.float32)
    history = np.zeros((16, 128), np.float32)
    base = 0
    for steps in (1, 2, 5, 3, 1, 1, 1, 7, 4, 16, 9, 2, 45):               # spans that start and end inside blocks
        oracle.qsa_pool(stream[base:base + steps], history, norm, pool, base, blocks)
        base += steps
        for p in range(max(0, base - min(steps, 4)), base):
            assert np.array_equal(history[p % 16], stream[p]), "the ring holds the span's last four rows"
    assert base == 97
    for block in range(97 // 4):
        x = stream[block * 4:block * 4 + 4].astype(np.float64).mean(axis=0)
        flat = x * norm / np.sqrt((x * x).mean() + 1e-6)
        want, slack = _rope64(flat[None], block * 4)
        assert _close(blocks[:, block], want[0], slack[0])
    assert np.all(blocks[:, 97 // 4:] == 0.0), "an incomplete block is not pooled"


def _prepare_case(rng, rows=3, heads=8, kv_heads=1, dim=256, rope_dims=64, context=16):
    # the shapes and the out-of-order positions of crates/straydog-engine/tests/fused_gpu.rs:225-268
    case = dict(q_full=(rng.standard_normal((rows, heads, 2 * dim)) * 4).astype(np.float32),
                k=(rng.standard_normal((rows, kv_heads, dim)) * 4).astype(np.float32),
                v=(rng.standard_normal((rows, kv_heads, dim)) * 4).astype(np.float32),
                q_weight=(rng.standard_normal(dim) * 2).astype(np.float32), k_weight=(rng.standard_normal(dim) * 2).astype(np.float32),
                frequencies=np.power(np.float32(1e7), -(2.0 * np.arange(rope_dims // 2, dtype=np.float32)) / np.float32(rope_dims)).astype(np.float32),
                positions=np.array([9, 2, 13][:rows] + list(range(20, 20 + max(0, rows - 3))), dtype=np.int32)[:rows],
                cache=rng.standard_normal((context, kv_heads * dim)).astype(np.float32))
    return case


def test_rms_norm_and_rope_halves_closed_forms(oracle):
    rng = np.random.default_rng(6)
    for width in (64, 256, 1000):
        x = (rng.standard_normal((5, width)) * 3).astype(np.float32)
        weight = (rng.standard_normal(width) * 2).astype(np.float32)
        got = oracle.rms_norm(x, weight, 1e-6)
        x64 = x.astype(np.float64)
        want = x64 / np.sqrt((x64 * x64).mean(axis=1, keepdims=True) + 1e-6) * weight
        assert np.allclose(got, want, rtol=3e-6, atol=1e-7)
    x = rng.standard_normal((3, 4, 96)).astype(np.float32)
    positions = np.array([0, 70001, 5], dtype=np.int32)
    frequencies = np.power(1e7, -np.arange(16) / 16.0).astype(np.float32)
    got = oracle.rope_halves(x, 32, positions, frequencies)
    angle = positions[:, None, None].astype(np.float64) * frequencies.astype(np.float64)
    low, high = x[..., :16].astype(np.float64), x[..., 16:32].astype(np.float64)
    assert np.allclose(got[..., :16], low * np.cos(angle) - high * np.sin(angle), rtol=1e-6, atol=1e-7)
    assert np.allclose(got[..., 16:32], low * np.sin(angle) + high * np.cos(angle), rtol=1e-6, atol=1e-7)
    assert np.array_equal(got[..., 32:], x[..., 32:]) and np.array_equal(got[0], x[0]), "columns past the rope and position 0 are not turned"
    assert np.allclose(got[..., :16].astype(np.float64) ** 2 + got[..., 16:32].astype(np.float64) ** 2, low ** 2 + high ** 2, rtol=1e-5)


def test_prepared_step_equals_its_parts(oracle):
    case = _prepare_case(np.random.default_rng(7))
    keys, values = case["cache"].copy(), case["cache"].copy()
    q, gate, k_after = oracle.attention_prepare(case["q_full"], case["k"], case["v"], case["q_weight"], case["k_weight"], 1e-6, 64,
                                                case["positions"], case["frequencies"], keys, values)
    rows, heads, dim = 3, 8, 256
    assert np.array_equal(gate, case["q_full"][:, :, dim:])
    want_q = oracle.rope_halves(oracle.rms_norm(case["q_full"][:, :, :dim].reshape(-1, dim), case["q_weight"], 1e-6).reshape(rows, heads, dim), 64,
                                case["positions"], case["frequencies"])
    want_k = oracle.rope_halves(oracle.rms_norm(case["k"].reshape(-1, dim), case["k_weight"], 1e-6).reshape(rows, 1, dim), 64, case["positions"],
                                case["frequencies"])
    assert np.array_equal(q, want_q) and np.array_equal(k_after, want_k)
    want_keys, want_values = case["cache"].copy(), case["cache"].copy()
    for r, p in enumerate(case["positions"]):
        want_keys[p], want_values[p] = want_k[r].reshape(-1), case["v"][r].reshape(-1)
    assert np.array_equal(keys, want_keys) and np.array_equal(values, want_values)
