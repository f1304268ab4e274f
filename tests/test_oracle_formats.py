"""Pins the oracle's conversions and K/V row codec (CPU only).

Independent checks: numpy float16 (exhaustive over all 65536 halves and random floats), the BF16
formula and special values of crates/straydog-engine/tests/ds_state_bf16_gpu.rs:26-33,49-67, the Q8_0
row invariants of crates/straydog-engine/src/gpu.rs:4096-4142 (with that file's generator :4083-4091),
an independent numpy restatement of kv_encode, and the six real ggml Q8_0 blocks of the reference
fixture tests/golden/format_blocks.json decoded as tests/formats.rs:84-90 spells it.
"""
import json
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def test_f16_to_f32_every_half(oracle):
    halves = np.arange(65536, dtype=np.uint16)
    want = halves.view(np.float16).astype(np.float32)
    got = np.array([oracle.f16_to_f32(h) for h in halves], dtype=np.float32)
    nan = np.isnan(want)      # a NaN's payload does not survive the trip through a C float return value: NaN-ness only
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_f32_to_f16_matches_numpy_rne(oracle):
    rng = np.random.default_rng(1)
    # every magnitude class: normals, subnormals, ties, overflow edge (65520 rounds to inf)
    xs = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * 10.0 ** rng.integers(-9, 6, 20000),
        np.array([0.0, -0.0, 65504.0, 65519.99, 65520.0, 1e6, -1e6, 5.9604645e-8, 2.9802322e-8, 2.98023224e-8 * 1.0001,
                  6.1035156e-5, 6.097555e-5, 1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, 2.0 ** -25, 2.0 ** -26], dtype=np.float32),
        np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32)[: 0x7c00],
    ]).astype(np.float32)
    with np.errstate(over="ignore"):
        want = xs.astype(np.float16).view(np.uint16)
    got = np.array([oracle.f32_to_f16(x) for x in xs], dtype=np.uint16)
    assert np.array_equal(got, want)


def _bf16_rule(bits):
    # ds_state_bf16_gpu.rs:27-33
    if bits & 0x7fffffff > 0x7f800000:
        return ((bits >> 16) | 0x40) & 0xffff
    return ((bits + 0x7fff + ((bits >> 16) & 1)) >> 16) & 0xffff


def test_bf16_rounding_rule_and_specials(oracle):
    rng = np.random.default_rng(2)
    bits = rng.integers(0, 2 ** 32, 20000, dtype=np.uint64).astype(np.uint32)
    special = np.array([0x00000000, 0x80000000, 0x3f800000, 0x3f808000, 0x3f818000, 0x3f807fff, 0x3f808001, 0x7f7fffff,
                        0x7f800000, 0xff800000, 0x7f800001, 0x7fc00000, 0xffc00001, 0x00000001, 0x00008000, 0x00018000],
                       dtype=np.uint32)
    bits = np.concatenate([bits, special])
    got = oracle.to_bf16(bits.view(np.float32))
    want = np.array([_bf16_rule(int(b)) for b in bits], dtype=np.uint16)
    assert np.array_equal(got, want)
    # ties to even, by hand: 1.0 + 2^-8 (exact tie) stays 1.0; 1.0 + 3*2^-8 rounds up to 1.0 + 2^-6
    assert oracle.f32_to_bf16(1.0 + 2.0 ** -8) == 0x3f80
    assert oracle.f32_to_bf16(1.0 + 3 * 2.0 ** -8) == 0x3f82


def _gpu_rs_row(seed, magnitude):
    # crates/straydog-engine/src/gpu.rs:4083-4091 (xorshift32)
    state = (seed * 2654435761) & 0xffffffff
    state = max(state, 1)
    out = np.zeros(256, dtype=np.float32)
    for i in range(256):
        state ^= (state << 13) & 0xffffffff
        state ^= state >> 17
        state ^= (state << 5) & 0xffffffff
        out[i] = (np.float32(state) / np.float32(0xffffffff) * np.float32(2.0) - np.float32(1.0)) * np.float32(magnitude)
    return out


def _numpy_kv_row(values):
    """kv_encode restated with numpy float16/float32 only."""
    dim = values.shape[0]
    blocks = values.reshape(-1, 32)
    top = np.abs(blocks).max(axis=1)
    with np.errstate(over="ignore"):
        half = (top / np.float32(127.0)).astype(np.float32).astype(np.float16)
    scale = half.astype(np.float32)
    safe = np.where(scale > 0, scale, np.float32(1.0))
    q = np.clip(np.rint((blocks / safe[:, None]).astype(np.float32)), -127, 127)
    q = np.where(scale[:, None] > 0, q, 0).astype(np.int8)
    return np.concatenate([q.reshape(dim).view(np.uint8), half.view(np.uint16).astype("<u2").view(np.uint8)])


def test_q8_row_layout_values_then_scales(oracle):
    # gpu.rs:4096-4113
    values = ((np.arange(256, dtype=np.float32) - 128.0) / 16.0).astype(np.float32)
    packed = oracle.kv_q8_row(values)
    assert packed.shape == (272,)
    for block in range(8):
        part = values[block * 32:(block + 1) * 32]
        top = np.abs(part).max()
        scale = int(packed[256 + 2 * block]) | int(packed[257 + 2 * block]) << 8
        assert scale == int(np.float32(top / np.float32(127.0)).astype(np.float16).view(np.uint16))
        largest = block * 32 + int(np.argmax(np.abs(part)))
        assert abs(int(packed[largest].view(np.int8))) == 127
        assert (packed[largest].view(np.int8) < 0) == (values[largest] < 0)
    assert packed[128].view(np.int8) == 0


def test_q8_rows_round_trip_within_half_a_scale(oracle):
    # gpu.rs:4115-4142
    for seed in range(1, 200):
        magnitude = [1e-3, 0.1, 1.0, 30.0, 600.0][seed % 5]
        values = _gpu_rs_row(seed, magnitude)
        packed = oracle.kv_q8_row(values)
        assert np.array_equal(packed, _numpy_kv_row(values)), seed
        back = oracle.kv_q8_values(packed, 256)
        scales = packed[256:].view("<u2").view(np.float16).astype(np.float32)
        error = np.abs(back - values)
        assert np.all(error <= np.repeat(scales, 32) * 0.5 * 1.001 + np.abs(values) * 1e-3), seed
    zero = oracle.kv_q8_row(np.zeros(256, dtype=np.float32))
    assert not zero.any() and not oracle.kv_q8_values(zero, 256).any()
    values = _gpu_rs_row(7, 1.0)
    before = oracle.kv_q8_row(values)
    values[3] = 500.0
    after = oracle.kv_q8_row(values)
    assert np.array_equal(before[32:256], after[32:256]) and np.array_equal(before[258:272], after[258:272])
    assert after[3].view(np.int8) == 127


def test_q8_row_head_dim_128_is_the_same_rule(oracle):
    rng = np.random.default_rng(3)
    for _ in range(50):
        values = (rng.standard_normal(128) * 10.0 ** rng.integers(-3, 3)).astype(np.float32)
        packed = oracle.kv_q8_row(values)
        assert packed.shape == (136,)
        assert np.array_equal(packed, _numpy_kv_row(values))
        back = oracle.kv_q8_values(packed, 128)
        want = packed[:128].view(np.int8).astype(np.float32) * np.repeat(packed[128:].view("<u2").view(np.float16).astype(np.float32), 32)
        assert np.array_equal(back.view(np.uint32), want.view(np.uint32))


def test_q8_rint_ties_to_even(oracle):
    # scale exactly 1/64: x = 2.5/64 is a tie and must round to 2, 3.5/64 to 4
    values = np.zeros(32, dtype=np.float32)
    values[0] = 127.0 / 64.0
    values[1], values[2], values[3], values[4] = 2.5 / 64, 3.5 / 64, -2.5 / 64, -0.5 / 64
    packed = oracle.kv_q8_row(values)
    assert list(packed[:5].view(np.int8)) == [127, 2, 4, -2, 0]


def test_real_ggml_q8_0_blocks_decode(oracle):
    golden = json.load(open(os.path.join(HERE, "golden", "q8_0_blocks.json")))["blocks"]
    assert len(golden) == 6
    for case in golden:
        data = np.frombuffer(bytes.fromhex(case["data"]), dtype=np.uint8)
        assert data.size == 34
        d = data[:2].view("<u2").view(np.float16).astype(np.float32)[0]
        want = d * data[2:].view(np.int8).astype(np.float32)     # tests/formats.rs:84-90
        got = oracle.ggml_q8_0_dequantize(data)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), case["source"]


def test_ggml_q8_0_quantize_round_trip(oracle):
    rng = np.random.default_rng(4)
    values = rng.standard_normal(32 * 40).astype(np.float32)
    blocks = oracle.ggml_q8_0_quantize(values)
    for b in range(40):
        part = values[b * 32:(b + 1) * 32]
        d = np.float32(np.abs(part).max() / np.float32(127.0))
        block = blocks[b * 34:(b + 1) * 34]
        assert block[:2].view("<u2")[0] == d.astype(np.float16).view(np.uint16)
        inverse = np.float32(1.0) / d
        want = np.where(part * inverse >= 0, np.floor(part * inverse + np.float32(0.5)), np.ceil(part * inverse - np.float32(0.5)))
        assert np.array_equal(block[2:].view(np.int8), want.astype(np.int8))
