"""GPU parity of Qwen's block indexer (sdx_qsa_normalize, sdx_qsa_pool, sdx_qsa_index) against the CPU oracle.

The cases follow the reference's own regression of this stage, gpu/tests/qsa_interval_test.cpp:58-118: gaussian keys and
queries, topic-correlated ones, exact ties at the 512th best score, zero queries, small magnitudes; every row must select
the blocks, in the order and with the ties, of the exact rule, and the block scores must be the same bits.
"""
import numpy as np
import pytest

from gpu_util import backend

pytestmark = pytest.mark.gpu

CANARY = np.float32(-77.5)


@pytest.fixture(scope="module")
def gpu():
    with backend(4 << 30) as handle:
        yield handle


def _read(gpu, buffer, dtype, count):
    return gpu.read_buffer(buffer, 0, dtype, count)


def _case(oracle, mode, base, steps, pool, stride, seed):
    """Pooled keys [128, pool] and index queries [steps, stride] in the manner of qsa_interval_test.cpp:71-93."""
    rng = np.random.default_rng(seed)
    complete_all = (base + steps) // 4
    topics = rng.standard_normal((64, 128)).astype(np.float32)
    strength = {"g": 0.0, "t": 1.0, "d": 2.5, "z": 0.0, "s": 0.0}[mode]
    scale = 1.0e-4 if mode == "s" else 1.0
    weight_k = (0.4 + 1.2 * rng.random(128)).astype(np.float32)
    weight_q = (0.4 + 1.2 * rng.random(128)).astype(np.float32)
    x = rng.standard_normal((complete_all, 128)).astype(np.float32) + strength * 0.6 * topics[(np.arange(complete_all) // 48 * 2654435761 % 64)]
    x = x / np.sqrt((x * x).mean(axis=1, keepdims=True) + 1e-6) * weight_k * scale
    blocks = np.zeros((128, pool), dtype=np.float32)
    blocks[:, :complete_all] = x.T
    blocks[:, complete_all:] = np.nan                      # never read: a block past the last row's complete count
    queries = np.zeros((steps, stride), dtype=np.float32)
    for r in range(steps):
        for h in range(4):
            z = ((base + r) // 700 + h * 5) * 40503 % 64
            v = rng.standard_normal(128).astype(np.float32) + strength * 0.6 * topics[z]
            queries[r, h * 128:(h + 1) * 128] = v / np.sqrt((v * v).mean() + 1e-6) * weight_q * scale
    queries[:, 512:] = 1.0e9                                # the rest of a row's stride belongs to others
    if mode == "z":
        queries[::2, :512] = 0.0
    if mode == "d" and complete_all > 600:
        # blocks around the 512th best of the last row given the same key: exact ties where the cut falls
        scores = oracle.qsa_block_scores(queries[-1:], np.nan_to_num(blocks), base + steps - 1)[0][:complete_all]
        order = sorted(range(complete_all), key=lambda b: (-float(scores[b]), b))
        for k in range(6):
            blocks[:, order[512 + 2 * k + (k & 1)]] = blocks[:, order[505 + 3 * k]]
    return queries, blocks


def _run_index(gpu, queries, blocks, base, selected, dynamic=False):
    steps, stride = queries.shape
    pool = blocks.shape[1]
    qb, kb = gpu.upload(queries), gpu.upload(blocks)
    scores = gpu.upload(np.full(steps * pool, CANARY, dtype=np.float32))
    indices = gpu.upload(np.full(steps * selected + 8, CANARY, dtype=np.float32))
    counts = gpu.upload(np.full(steps, CANARY, dtype=np.float32))
    position = gpu.upload(np.array([base], dtype=np.uint32)) if dynamic else None
    gpu.qsa_index(qb.base(), stride, kb.base(), pool, 0 if dynamic else base, steps, selected, scores.base(), indices.base(), counts.base(),
                  dynamic_base=position.base() if dynamic else None)
    out = (_read(gpu, scores, np.float32, steps * pool).reshape(steps, pool), _read(gpu, indices, np.float32, steps * selected + 8),
           _read(gpu, counts, np.float32, steps))
    for b in (qb, kb, scores, indices, counts) + ((position,) if dynamic else ()):
        gpu.release(b)
    return out


def _check(oracle, queries, blocks, base, selected, got):
    scores, indices, counts = got
    steps, pool = queries.shape[0], blocks.shape[1]
    want_scores = oracle.qsa_block_scores(queries, np.nan_to_num(blocks), base)
    assert np.all(indices[steps * selected:] == CANARY), "nothing is written past the last row's selection"
    for r in range(steps):
        position = base + r
        complete = (position + 1) // 4
        if complete > 512:
            assert np.array_equal(scores[r, :complete].view(np.uint32), want_scores[r, :complete].view(np.uint32)), f"row {r}: score bits"
            want = oracle.qsa_select(want_scores[r], position)
        else:
            want = np.arange(position + 1, dtype=np.float32)
        assert np.all(scores[r, max(complete, 0) if complete > 512 else 0:] == CANARY), f"row {r}: scores outside the row's blocks are not touched"
        assert counts[r] == float(len(want)), f"row {r}: count {counts[r]} != {len(want)}"
        row = indices[r * selected:(r + 1) * selected]
        assert np.array_equal(row[:len(want)], want), f"row {r}: selection"
        assert np.all(row[len(want):] == CANARY), f"row {r}: entries past the count are not touched"


@pytest.mark.parametrize("mode,base,steps,context,stride", [
    ("g", 30000, 1, 32768, 512),        # a decode row
    ("t", 2044, 8, 4096, 512),          # a verification span across the 512-block line: rows that keep everything, rows that select
    ("g", 9000, 5, 16384, 640),         # a verification span (a wider row stride)
    ("t", 9001, 100, 16384, 512),       # a prefill chunk: the tiled form, rows of different complete counts
    ("d", 20000, 37, 32768, 512),       # exact ties where the cut falls
    ("z", 5000, 12, 8192, 512),         # zero queries: every score ties at zero, the earliest 512 blocks win
    ("s", 7000, 3, 8192, 512),          # small magnitudes
    ("g", 262100, 3, 262144, 512),      # the longest context: rows re-read per pass
    ("g", 70000, 2, 131072, 512),       # 16 values a thread
    ("g", 100, 20, 1024, 512),          # a short context: every row keeps every causal position
    ("d", 60000, 4, 65536, 512),        # a few long rows are thinned by many workgroups first: exact ties where the cut falls,
    ("t", 100000, 8, 131072, 512),      # ... clustered scores,
    ("z", 40000, 2, 65536, 512),        # ... and zero queries, whose lists do not fit: the row's workgroup does it all
])
def test_block_scores_and_selection(gpu, oracle, mode, base, steps, context, stride):
    pool = context // 4 + 1
    selected = min(base + steps, 2052)
    queries, blocks = _case(oracle, mode, base, steps, pool, stride, seed=base + steps)
    _check(oracle, queries, blocks, base, selected, _run_index(gpu, queries, blocks, base, selected))


def _run_interval(gpu, queries, blocks, base, selected, state=None):
    """sdx_qsa_index_interval on host arrays; `state` keeps the key buffer, scratch and packed-operand count between calls."""
    steps, stride = queries.shape
    pool = blocks.shape[1]
    qb = gpu.upload(queries)
    if state is None or "keys" not in state:
        held = {"keys": gpu.upload(blocks), "scratch": gpu.buffer(gpu.qsa_index_interval_scratch(steps, pool)), "valid": [0]}
        if state is not None:
            state.update(held)
    else:
        held = state
    scores = gpu.buffer(steps * pool * 4)
    indices = gpu.upload(np.full(steps * selected + 8, CANARY, dtype=np.float32))
    counts = gpu.upload(np.full(steps, CANARY, dtype=np.float32))
    gpu.qsa_index_interval(qb.base(), stride, held["keys"].base(), pool, base, steps, selected, scores.base(), indices.base(), counts.base(),
                           held["scratch"], held["valid"])
    out = (_read(gpu, indices, np.float32, steps * selected + 8), _read(gpu, counts, np.float32, steps),
           gpu.qsa_index_interval_undecided(held["scratch"], steps, pool))
    for b in (qb, scores, indices, counts) + (() if state is not None else (held["keys"], held["scratch"])):
        gpu.release(b)
    return out


def _check_selection(oracle, queries, blocks, base, selected, indices, counts):
    steps = queries.shape[0]
    want_scores = oracle.qsa_block_scores(queries, np.nan_to_num(blocks), base)
    assert np.all(indices[steps * selected:] == CANARY)
    for r in range(steps):
        want = oracle.qsa_select(want_scores[r], base + r)
        assert counts[r] == float(len(want)), f"row {r}: count {counts[r]} != {len(want)}"
        row = indices[r * selected:(r + 1) * selected]
        assert np.array_equal(row[:len(want)], want), f"row {r}: selection"
        assert np.all(row[len(want):] == CANARY), f"row {r}: entries past the count are not touched"


@pytest.mark.parametrize("mode,base,steps,context,decided", [
    ("g", 40000, 37, 65536, True),       # gaussian keys: the intervals decide every row
    ("t", 100000, 130, 131072, True),    # clustered scores, two row groups, rows of different complete counts
    ("d", 60000, 20, 65536, True),       # exact ties where the cut falls: the band's order and ties are the exact kernels'
    ("z", 40000, 6, 65536, False),       # zero queries on every other row: every block ties, the exact kernels take those rows
    ("s", 50000, 9, 65536, None),        # magnitudes around the smallest normal FP16: wide bounds, whoever decides
])
def test_interval_selection_is_the_exact_one(gpu, oracle, mode, base, steps, context, decided):
    # the reference's qsa_interval_test.cpp cases (:71-93 inputs, :95-140 "the selection is qsa_select_rows', block for block")
    pool = context // 4 + 1
    queries, blocks = _case(oracle, mode, base, steps, pool, 512, seed=base + steps)
    indices, counts, undecided = _run_interval(gpu, queries, blocks, base, 2052)
    _check_selection(oracle, queries, blocks, base, 2052, indices, counts)
    if decided is True:
        assert undecided == 0, f"{undecided} rows went to the exact kernels"
    if decided is False:
        assert undecided == (steps + 1) // 2


def test_interval_selection_with_inputs_beyond_fp16_and_kept_operands(gpu, oracle):
    base, steps, pool = 50000, 24, 65536 // 4 + 1
    queries, blocks = _case(oracle, "g", base, 2 * steps, pool, 512, seed=9)
    state = {}
    first = _run_interval(gpu, queries[:steps], blocks, base, 2052, state)
    _check_selection(oracle, queries[:steps], blocks, base, 2052, first[0], first[1])
    assert first[2] == 0 and state["valid"][0] == (base + steps) // 4
    # the next chunk packs only the new blocks' operands
    second = _run_interval(gpu, queries[steps:], blocks, base + steps, 2052, state)
    _check_selection(oracle, queries[steps:], blocks, base + steps, 2052, second[0], second[1])
    assert second[2] == 0 and state["valid"][0] == (base + 2 * steps) // 4
    for b in (state["keys"], state["scratch"]):
        gpu.release(b)
    # a key element beyond FP16 leaves every row that sees its block to the exact kernels; a query row beyond it, that row
    wild = blocks.copy()
    wild[7, 300] = 1.0e6
    got = _run_interval(gpu, queries[:steps], wild, base, 2052)
    _check_selection(oracle, queries[:steps], wild, base, 2052, got[0], got[1])
    assert got[2] == steps
    loud = queries[:steps].copy()
    loud[5, 130] = -7.0e4
    got = _run_interval(gpu, loud, blocks, base, 2052)
    _check_selection(oracle, loud, blocks, base, 2052, got[0], got[1])
    assert got[2] == 1
    # below position 32768 the call is sdx_qsa_index
    queries, blocks = _case(oracle, "g", 9000, 5, 16384 // 4 + 1, 512, seed=10)
    got = _run_interval(gpu, queries, blocks, 9000, 2052)
    _check_selection(oracle, queries, blocks, 9000, 2052, got[0], got[1])


def test_interval_selection_of_a_chunk_at_242k_tokens(gpu):
    # the bench's shape: 256 rows at position 242000 of a 262144-token context, against the exact kernels on the same device data
    steps, base, pool = 256, 242000, 262144 // 4 + 1
    queries, blocks = gpu.buffer(steps * 512 * 4), gpu.buffer(128 * pool * 4)
    gpu.fill_normal(queries.base(), steps * 512, 61, 0)
    gpu.fill_normal(blocks.base(), 128 * pool, 62, 0)
    outs = []
    scores = gpu.buffer(steps * pool * 4)
    scratch = gpu.buffer(gpu.qsa_index_interval_scratch(steps, pool))
    for interval in (False, True):
        indices, counts = gpu.buffer(steps * 2052 * 4), gpu.buffer(steps * 4)
        if interval:
            gpu.qsa_index_interval(queries.base(), 512, blocks.base(), pool, base, steps, 2052, scores.base(), indices.base(), counts.base(), scratch)
        else:
            gpu.qsa_index(queries.base(), 512, blocks.base(), pool, base, steps, 2052, scores.base(), indices.base(), counts.base())
        outs.append((_read(gpu, indices, np.float32, steps * 2052), _read(gpu, counts, np.float32, steps)))
        gpu.release(indices); gpu.release(counts)
    assert np.array_equal(outs[0][1], outs[1][1])
    assert np.array_equal(outs[0][0], outs[1][0])
    assert gpu.qsa_index_interval_undecided(scratch, steps, pool) <= 2
    for b in (queries, blocks, scores, scratch):
        gpu.release(b)


def test_device_resident_position(gpu, oracle):
    # the replayable form: the position is read on the device, the launch shape does not depend on it
    base, steps, context = 12345, 4, 32768
    pool = context // 4 + 1
    queries, blocks = _case(oracle, "g", base, steps, pool, 512, seed=5)
    blocks = np.nan_to_num(blocks)
    _check(oracle, queries, blocks, base, 2052, _run_index(gpu, queries, blocks, base, 2052, dynamic=True))


def _rope_slack(want, position):
    """How far a turned value may move when the float32 angle lands one float32 step away (the power function's last bit)."""
    slack = np.zeros(want.shape, dtype=np.float64)
    c = np.arange(32)
    angle = (np.float32(position) / np.power(np.float32(1e7), (c / 32.0).astype(np.float32))).astype(np.float32)
    slack[..., :32] = slack[..., 32:64] = 2.0 * np.spacing(angle).astype(np.float64) * np.hypot(want[..., :32], want[..., 32:64])
    return slack


def _close(got, want, slack):
    return np.all(np.abs(got.astype(np.float64) - want) <= 2e-5 + 2e-5 * np.abs(want) + slack)


@pytest.mark.parametrize("width,heads,stride", [(256, 24, 512), (256, 2, 256), (128, 4, 128)])
def test_normalize(gpu, oracle, width, heads, stride):
    rng = np.random.default_rng(width + heads)
    rows, position = 5, 123457
    source = (rng.standard_normal(rows * heads * stride) * 3).astype(np.float32)
    norm = (0.4 + 1.2 * rng.random(width)).astype(np.float32)
    want = oracle.qsa_normalize(source, norm, rows, heads, width, stride, position)
    sb, nb = gpu.upload(source), gpu.upload(norm)
    target = sb if stride == width else gpu.buffer(rows * heads * width * 4)       # in place where the rows are dense, as the reference does
    gpu.qsa_normalize(sb.base(), nb.base(), rows, heads, width, stride, position, target.base())
    got = _read(gpu, target, np.float32, rows * heads * width).reshape(rows * heads, width)
    for r in range(rows):
        span = slice(r * heads, (r + 1) * heads)
        assert _close(got[span], want[span].astype(np.float64), _rope_slack(want[span], position + r))
    assert np.array_equal(got[:, 64:], want[:, 64:]), "columns that are not turned: the same bits (tree-ordered sum, exact division)"
    for b in {sb, nb, target}:
        gpu.release(b)


def test_pool_over_spans(gpu, oracle):
    # spans that start and end inside blocks; the ring of sixteen carries the inputs of a block across calls
    rng = np.random.default_rng(8)
    pool, base = 600, 2000
    norm = (0.4 + 1.2 * rng.random(128)).astype(np.float32)
    want_blocks, want_history = np.zeros((128, pool), np.float32), rng.standard_normal((16, 128)).astype(np.float32)
    bb, hb, nb = gpu.upload(want_blocks), gpu.upload(want_history), gpu.upload(norm)
    for steps in (1, 2, 5, 3, 1, 1, 1, 7, 4, 16, 9, 2, 45, 256):
        incoming = rng.standard_normal((steps, 128)).astype(np.float32)
        ib = gpu.upload(incoming)
        gpu.qsa_pool(ib.base(), hb.base(), nb.base(), pool, base, steps, bb.base())
        oracle.qsa_pool(incoming, want_history, norm, pool, base, want_blocks)
        gpu.release(ib)
        base += steps
    assert np.array_equal(_read(gpu, hb, np.float32, 16 * 128).reshape(16, 128), want_history)
    got = _read(gpu, bb, np.float32, 128 * pool).reshape(128, pool)
    for block in range(2000 // 4, base // 4):
        assert _close(got[:, block], want_blocks[:, block].astype(np.float64), _rope_slack(want_blocks[:, block], block * 4)), f"block {block}"
    untouched = np.ones(pool, bool)
    untouched[2000 // 4:base // 4] = False
    assert np.all(got[:, untouched] == 0.0)
    for b in (bb, hb, nb):
        gpu.release(b)


def test_refusals(gpu):
    from straydog_amd.backend import StraydogError as GpuError
    pool, steps = 1025, 2
    q, k = gpu.buffer(steps * 512 * 4), gpu.buffer(128 * pool * 4)
    scores, indices, counts = gpu.buffer(steps * pool * 4), gpu.buffer(steps * 2052 * 4), gpu.buffer(steps * 4)
    args = dict(queries=q.base(), query_stride=512, blocks=k.base(), pool=pool, base=3000, steps=steps, selected=2052, scores=scores.base(),
                indices=indices.base(), counts=counts.base())
    gpu.qsa_index(**args)
    for change, text in ((dict(base=4099), "fit the pool"), (dict(selected=2051), "selected"), (dict(query_stride=511), "stride"),
                         (dict(pool=70000), "65537"), (dict(steps=0), "steps"), (dict(counts=counts.at(4)), "outside")):
        with pytest.raises(GpuError, match=text):
            gpu.qsa_index(**{**args, **change})
    with pytest.raises(GpuError, match="width"):
        gpu.qsa_normalize(q.base(), k.base(), 1, 4, 64, 64, 0, q.base())
    with pytest.raises(GpuError, match="fit the pool"):
        gpu.qsa_pool(q.base(), k.base(), k.base(), 10, 100, 4, k.base())
    for b in (q, k, scores, indices, counts):
        gpu.release(b)


def _qwen_case(oracle, rng, row_bytes, context, base, steps, selected=2052):
    """The Qwen state (planes x context rows) with `base` cached positions, a span's packed input with realistic selection
    lists (sdx_qsa_index's rule on random scores) and one adversarial list; the oracle's outputs and the state afterwards."""
    state = np.zeros(context * 4 * row_bytes, dtype=np.uint8)
    old_k = rng.standard_normal((1, base, 2, 256)).astype(np.float32)
    old_v = rng.standard_normal((1, base, 2, 256)).astype(np.float32)
    oracle.kv_write(state, row_bytes, context, 2, 256, np.zeros((1, 1), np.int32), np.zeros(1, np.int32), old_k, old_v)
    q = rng.standard_normal((steps, 24, 256)).astype(np.float32)
    k = rng.standard_normal((steps, 2, 256)).astype(np.float32)
    v = rng.standard_normal((steps, 2, 256)).astype(np.float32)
    indices = np.full((steps, selected), -1.0, dtype=np.float32)
    counts = np.zeros(steps, dtype=np.float32)
    for s in range(steps):
        if s == steps - 1:
            # entries that do not count: past the row's position, negative, past the context; and a short list
            row = np.concatenate([np.sort(rng.permutation(base + s + 1)[:77]), [base + s + 3, -2.0, context + 1, base + s]]).astype(np.float32)
        else:
            row = oracle.qsa_select(rng.random(context // 4 + 1).astype(np.float32), base + s)
        indices[s, :row.size] = row
        counts[s] = row.size
    packed = np.concatenate([q.ravel(), k.ravel(), v.ravel(), indices.ravel(), counts]).astype(np.float32)
    want = oracle.attention_sequence(state, row_bytes, context, base, steps, selected, packed).reshape(steps, 24, 256)
    return state, q, indices, counts, want


@pytest.mark.parametrize("row_bytes", [272, 512])
@pytest.mark.parametrize("paged", [False, True])
def test_selected_attention(gpu, oracle, row_bytes, paged):
    # the attention of a Qwen decode / verification pass over each row's selection: Q8_0 and FP16 rows, the reference's state
    # layout and a shuffled page table, FP32 and FP16 queries and outputs, the sigmoid gate, a device-resident position
    from gpu_util import close_enough
    rng = np.random.default_rng(row_bytes + paged)
    context, base, steps, selected = 4096, 3000, 5, 2052
    state, q, indices, counts, want = _qwen_case(oracle, rng, row_bytes, context, base, steps, selected)
    planes = state.reshape(4, context, row_bytes)
    if paged:
        page_tokens, pages = 256, context // 256
        order = rng.permutation(pages + 3)[:pages].astype(np.int32)
        host = np.zeros((pages + 3, 4, page_tokens, row_bytes), dtype=np.uint8)
        for p in range(pages):
            host[order[p]] = planes[:, p * page_tokens:(p + 1) * page_tokens]
        pool, buffer = gpu.kv_pool(pages + 3, page_tokens, 2, 256, row_bytes)
        table = gpu.upload(order)
    else:
        host = planes
        pool, buffer = gpu.kv_pool(1, context, 2, 256, row_bytes)
        table = None
    gpu.write_buffer(buffer, 0, np.ascontiguousarray(host).reshape(-1))
    gate = rng.standard_normal((steps, 24, 512)).astype(np.float32) * 2
    ib, cb, gb = gpu.upload(indices), gpu.upload(counts), gpu.upload(gate)
    scratch = gpu.buffer(gpu.selected_attention_scratch(steps, 2, selected))
    position = gpu.upload(np.array([base], dtype=np.uint32))
    for q_f16, out_f16, gated, dynamic in ((False, False, False, False), (True, True, True, False), (False, False, True, True)):
        qb = gpu.upload(q.astype(np.float16) if q_f16 else q)
        out = gpu.buffer(steps * 24 * 256 * (2 if out_f16 else 4))
        gpu.selected_attention(pool, table.base() if paged else None, context, 0 if dynamic else base, ib.base(), selected, cb.base(), qb.base(),
                               q_f16, steps, 24, 0.0625, out.base(), out_f16, scratch, gate=gb.at(256 * 4) if gated else None, gate_stride=512,
                               dynamic_base=position.base() if dynamic else None)
        got = _read(gpu, out, np.float16 if out_f16 else np.float32, steps * 24 * 256).astype(np.float32).reshape(steps, 24, 256)
        expect = want * (1.0 / (1.0 + np.exp(-gate[:, :, 256:].astype(np.float64)))) if gated else want
        close_enough(got, expect, f"selected attention f16={q_f16} gated={gated} dynamic={dynamic}")
        gpu.release(qb); gpu.release(out)
    for b in (ib, cb, gb, scratch, position, buffer) + ((table,) if paged else ()):
        gpu.release(b)


def test_selected_attention_of_a_prompt_chunk(gpu, oracle):
    # what the prompt path does from position 8192 on (gpu/qsa_prompt_attention.hpp:218-234, gpu/sparse_attention_compute.hpp:589-608):
    # a chunk of 256 rows, each with its own selection list, over Q8_0 rows behind a shuffled page table, gated, FP16 in and out
    from gpu_util import close_enough
    rng = np.random.default_rng(256)
    context, base, steps, selected, row_bytes = 12288, 9000, 256, 2052, 272
    state, q, indices, counts, want = _qwen_case(oracle, rng, row_bytes, context, base, steps, selected)
    planes = state.reshape(4, context, row_bytes)
    page_tokens, pages = 256, context // 256
    order = rng.permutation(pages + 2)[:pages].astype(np.int32)
    host = np.zeros((pages + 2, 4, page_tokens, row_bytes), dtype=np.uint8)
    for p in range(pages):
        host[order[p]] = planes[:, p * page_tokens:(p + 1) * page_tokens]
    pool, buffer = gpu.kv_pool(pages + 2, page_tokens, 2, 256, row_bytes)
    table = gpu.upload(order)
    gpu.write_buffer(buffer, 0, host.reshape(-1))
    gate = rng.standard_normal((steps, 24, 512)).astype(np.float32) * 2
    ib, cb, gb, qb = gpu.upload(indices), gpu.upload(counts), gpu.upload(gate), gpu.upload(q.astype(np.float16))
    scratch = gpu.buffer(gpu.selected_attention_scratch(steps, 2, selected))
    out = gpu.buffer(steps * 24 * 256 * 2)
    gpu.selected_attention(pool, table.base(), context, base, ib.base(), selected, cb.base(), qb.base(), True, steps, 24, 0.0625, out.base(), True,
                           scratch, gate=gb.at(256 * 4), gate_stride=512)
    got = _read(gpu, out, np.float16, steps * 24 * 256).astype(np.float32).reshape(steps, 24, 256)
    expect = want * (1.0 / (1.0 + np.exp(-gate[:, :, 256:].astype(np.float64))))
    close_enough(got, expect, "a chunk of 256 rows")
    for b in (ib, cb, gb, qb, scratch, out, buffer, table):
        gpu.release(b)


@pytest.mark.parametrize("row_bytes,paged,steps", [(272, True, 40), (512, False, 23), (272, False, 7)])
def test_selected_attention_as_a_union_walk(gpu, oracle, row_bytes, paged, steps):
    # the rows of a chunk sharing one walk over the union of their selections (the reference's qsa_flash_wmma over qsa_union_blocks,
    # gpu/sparse_attention_compute.hpp:841-1041): the same outputs as the per-row form, against the oracle; lists with entries that do
    # not count, Q8_0 and FP16 rows, the state layout and a shuffled page table, the gate, FP16 in and out
    from gpu_util import close_enough
    rng = np.random.default_rng(1000 + row_bytes + steps)
    context, base, selected = 4096, 2900, 2052
    state, q, indices, counts, want = _qwen_case(oracle, rng, row_bytes, context, base, steps, selected)
    planes = state.reshape(4, context, row_bytes)
    if paged:
        page_tokens, pages = 256, context // 256
        order = rng.permutation(pages + 3)[:pages].astype(np.int32)
        host = np.zeros((pages + 3, 4, page_tokens, row_bytes), dtype=np.uint8)
        for p in range(pages):
            host[order[p]] = planes[:, p * page_tokens:(p + 1) * page_tokens]
        pool, buffer = gpu.kv_pool(pages + 3, page_tokens, 2, 256, row_bytes)
        table = gpu.upload(order)
    else:
        host = planes
        pool, buffer = gpu.kv_pool(1, context, 2, 256, row_bytes)
        table = None
    gpu.write_buffer(buffer, 0, np.ascontiguousarray(host).reshape(-1))
    gate = rng.standard_normal((steps, 24, 512)).astype(np.float32) * 2
    ib, cb, gb = gpu.upload(indices), gpu.upload(counts), gpu.upload(gate)
    scratch = gpu.buffer(gpu.selected_attention_union_scratch(steps, 24, 2, selected, context))
    for q_f16, out_f16, gated in ((False, False, False), (True, True, True)):
        qb = gpu.upload(q.astype(np.float16) if q_f16 else q)
        out = gpu.buffer(steps * 24 * 256 * (2 if out_f16 else 4))
        gpu.selected_attention_union(pool, table.base() if paged else None, context, base, ib.base(), selected, cb.base(), qb.base(), q_f16, steps, 24,
                                     0.0625, out.base(), out_f16, scratch, gate=gb.at(256 * 4) if gated else None, gate_stride=512)
        got = _read(gpu, out, np.float16 if out_f16 else np.float32, steps * 24 * 256).astype(np.float32).reshape(steps, 24, 256)
        expect = want * (1.0 / (1.0 + np.exp(-gate[:, :, 256:].astype(np.float64)))) if gated else want
        close_enough(got, expect, f"union walk f16={q_f16} gated={gated}")
        gpu.release(qb); gpu.release(out)
    for b in (ib, cb, gb, scratch, buffer) + ((table,) if paged else ()):
        gpu.release(b)


def test_index_then_attend_on_the_device(gpu, oracle):
    # the two stages chained on the device, as a decode pass runs them: sdx_qsa_index's lists feed sdx_selected_attention unchanged
    from gpu_util import close_enough
    rng = np.random.default_rng(77)
    context, base, steps, row_bytes = 8192, 6000, 3, 272
    pool_blocks = context // 4 + 1
    queries, blocks = _case(oracle, "t", base, steps, pool_blocks, 512, seed=9)
    blocks = np.nan_to_num(blocks)
    state = np.zeros(context * 4 * row_bytes, dtype=np.uint8)
    k = rng.standard_normal((1, base + steps, 2, 256)).astype(np.float32)
    v = rng.standard_normal((1, base + steps, 2, 256)).astype(np.float32)
    oracle.kv_write(state, row_bytes, context, 2, 256, np.zeros((1, 1), np.int32), np.zeros(1, np.int32), k, v)
    q = rng.standard_normal((steps, 24, 256)).astype(np.float32)
    scores = oracle.qsa_block_scores(queries, blocks, base)
    indices = np.full((steps, 2052), -1.0, dtype=np.float32)
    counts = np.zeros(steps, dtype=np.float32)
    for r in range(steps):
        row = oracle.qsa_select(scores[r], base + r)
        indices[r, :row.size] = row
        counts[r] = row.size
    # the oracle rewrites the span's K/V rows from its packed input: hand it the rows the state already holds (decoded values
    # re-encode to the same bytes)
    held_k = np.stack([oracle.kv_q8_values(state.reshape(4, context, row_bytes)[h, base:base + steps], 256) for h in range(2)], axis=1)
    held_v = np.stack([oracle.kv_q8_values(state.reshape(4, context, row_bytes)[2 + h, base:base + steps], 256) for h in range(2)], axis=1)
    packed = np.concatenate([q.ravel(), held_k.ravel(), held_v.ravel(), indices.ravel(), counts]).astype(np.float32)
    before = state.copy()
    want = oracle.attention_sequence(state, row_bytes, context, base, steps, 2052, packed).reshape(steps, 24, 256)
    assert np.array_equal(before, state)
    pool, buffer = gpu.kv_pool(1, context, 2, 256, row_bytes)
    gpu.write_buffer(buffer, 0, state)
    qb, kb, qq = gpu.upload(queries), gpu.upload(blocks), gpu.upload(q)
    sb, ib, cb = gpu.buffer(steps * pool_blocks * 4), gpu.buffer(steps * 2052 * 4), gpu.buffer(steps * 4)
    out = gpu.buffer(steps * 24 * 256 * 4)
    scratch = gpu.buffer(gpu.selected_attention_scratch(steps, 2, 2052))
    gpu.qsa_index(qb.base(), 512, kb.base(), pool_blocks, base, steps, 2052, sb.base(), ib.base(), cb.base())
    gpu.selected_attention(pool, None, context, base, ib.base(), 2052, cb.base(), qq.base(), False, steps, 24, 0.0625, out.base(), False, scratch)
    got = _read(gpu, out, np.float32, steps * 24 * 256).reshape(steps, 24, 256)
    close_enough(got, want, "index then attend")
    for b in (qb, kb, qq, sb, ib, cb, out, scratch, buffer):
        gpu.release(b)


@pytest.mark.parametrize("row_bytes,paged,steps,first", [(272, False, 1, 2047), (272, True, 5, 2047), (512, False, 8, 3001)])
def test_decode_stage_in_one_call_equals_its_parts(gpu, oracle, row_bytes, paged, steps, first):
    # sdx_qsa_decode_attend (qsa_decode_attend_rows, gpu/qsa_decode.hpp:113-129): "three launches in one, the same values" -- the
    # prepared queries, K/V bytes, pooled blocks and ring equal those of sdx_qsa_normalize + sdx_kv_write + sdx_qsa_pool, and the
    # attended rows equal sdx_qsa_index + sdx_selected_attention on them, bit for bit; the rows cross a block's end and the
    # 512-block line, positions live on the device
    rng = np.random.default_rng(steps * 10 + row_bytes)
    heads, kv_heads, context = 24, 2, 4096
    pool_blocks, stride = context // 4 + 1, 24 * 512 + 2 * 512 + 640 + 11
    projections = (rng.standard_normal((steps, stride)) * 2).astype(np.float32)
    norms = [(0.4 + 1.2 * rng.random(n)).astype(np.float32) for n in (256, 256, 128, 128)]
    blocks = np.zeros((128, pool_blocks), dtype=np.float32)
    blocks[:, :first // 4] = rng.standard_normal((128, first // 4)).astype(np.float32)
    history = rng.standard_normal((16, 128)).astype(np.float32)
    positions = np.arange(first, first + steps, dtype=np.uint32)
    page_tokens = 256 if paged else context
    pages = context // page_tokens
    order = rng.permutation(pages).astype(np.int32)
    if row_bytes == 272:
        filled = rng.integers(0, 256, pages * 4 * page_tokens * row_bytes, dtype=np.uint8)
    else:
        filled = rng.standard_normal(pages * 4 * page_tokens * 256).astype(np.float16).view(np.uint8)
    if row_bytes == 272:                                   # random bytes would make NaN scales: give every row sane FP16 scales
        rows = filled.reshape(-1, 272)
        rows[:, 256:] = np.tile(np.frombuffer(np.float16(0.01).tobytes(), np.uint8), 8)

    def fresh():
        kv, buffer = gpu.kv_pool(pages, page_tokens, kv_heads, 256, row_bytes)
        gpu.write_buffer(buffer, 0, filled)
        return dict(kv=kv, buffer=buffer, table=gpu.upload(order) if paged else None, projections=gpu.upload(projections), blocks=gpu.upload(blocks),
                    history=gpu.upload(history), norms=[gpu.upload(n) for n in norms], positions=gpu.upload(positions),
                    attended=gpu.buffer(steps * heads * 256 * 4))

    def read_state(s):
        return dict(kv=_read(gpu, s["buffer"], np.uint8, filled.size), blocks=_read(gpu, s["blocks"], np.float32, blocks.size),
                    history=_read(gpu, s["history"], np.float32, history.size), projections=_read(gpu, s["projections"], np.float32, projections.size),
                    attended=_read(gpu, s["attended"], np.float32, steps * heads * 256))
    # one call
    one = fresh()
    state = gpu.qsa_state(one["kv"], one["table"].base() if paged else None, context, one["blocks"].base(), one["history"].base(),
                          *[n.base() for n in one["norms"]], heads)
    scratch = gpu.buffer(gpu.qsa_decode_attend_scratch(steps, heads, kv_heads, context))
    gpu.qsa_decode_attend(state, one["projections"].base(), stride, steps, one["positions"].base(), one["positions"].base(), scratch, one["attended"].base())
    got = read_state(one)
    # the parts
    two = fresh()
    base = two["projections"].base()
    queries = gpu.buffer(steps * heads * 256 * 4)
    keys = gpu.buffer(steps * kv_heads * 256 * 4)
    values = gpu.buffer(steps * kv_heads * 256 * 4)
    index_keys = gpu.buffer(steps * 128 * 4)
    for r in range(steps):
        at = base + r * stride * 4
        gpu.qsa_normalize(at, two["norms"][0].base(), 1, heads, 256, 512, first + r, queries.at(r * heads * 256 * 4))
        gpu.qsa_normalize(at + heads * 512 * 4, two["norms"][1].base(), 1, kv_heads, 256, 256, first + r, keys.at(r * kv_heads * 256 * 4))
        gpu.qsa_normalize(at + (heads * 512 + kv_heads * 512) * 4, two["norms"][2].base(), 1, 4, 128, 128, first + r, at + (heads * 512 + kv_heads * 512) * 4)
        gpu.write_buffer(values, r * kv_heads * 256 * 4, projections[r, heads * 512 + kv_heads * 256:heads * 512 + kv_heads * 512])
        gpu.write_buffer(index_keys, r * 128 * 4, projections[r, heads * 512 + kv_heads * 512 + 512:heads * 512 + kv_heads * 512 + 640])
    start = gpu.upload(np.array([first], dtype=np.int32))
    table = two["table"].base() if paged else gpu.upload(np.zeros(1, np.int32)).base()
    gpu.kv_write(two["kv"], table, pages, start.base(), keys.base(), values.base(), False, 1, steps)
    for r in range(steps):           # row by row, as a verification's rows are pooled: every row enters the ring
        gpu.qsa_pool(index_keys.at(r * 128 * 4), two["history"].base(), two["norms"][3].base(), pool_blocks, first + r, 1, two["blocks"].base())
    scores, indices, counts = gpu.buffer(steps * pool_blocks * 4), gpu.buffer(steps * 2052 * 4), gpu.buffer(steps * 4)
    gpu.qsa_index(base + (heads * 512 + kv_heads * 512) * 4, stride, two["blocks"].base(), pool_blocks, first, steps, 2052, scores.base(), indices.base(),
                  counts.base())
    partial = gpu.buffer(gpu.selected_attention_scratch(steps, kv_heads, 2052))
    gpu.selected_attention(two["kv"], two["table"].base() if paged else None, context, first, indices.base(), 2052, counts.base(), queries.base(), False,
                           steps, heads, 0.0625, two["attended"].base(), False, partial, gate=base + 256 * 4, gate_stride=512, gate_row_stride=stride)
    want = read_state(two)
    for what in ("kv", "blocks", "history", "projections", "attended"):
        a, b = got[what], want[what]
        assert np.array_equal(a.view(np.uint8), b.view(np.uint8)), what
    assert np.all(np.isfinite(got["attended"])) and np.abs(got["attended"]).max() > 0


@pytest.mark.parametrize("row_bytes,paged,context,first,spans", [(272, True, 4096, 1990, (100,)), (512, False, 40960, 36001, (64, 37))])
def test_prompt_chunk_stage_in_one_call_equals_its_parts(gpu, oracle, row_bytes, paged, context, first, spans):
    # sdx_qsa_prefill_attend (the stage of qsa_prefill, gpu/sparse_attention.hpp:444-506): normalised rows, K/V bytes, pooled blocks
    # and ring equal those of sdx_qsa_normalize + sdx_kv_write + sdx_qsa_pool over the span, and the attended rows equal
    # sdx_qsa_index_interval + sdx_selected_attention (gated) on them, bit for bit: before the 512-block line and across it with
    # the exact kernels, and past 32768 positions by intervals, the packed keys carried from one chunk to the next
    rng = np.random.default_rng(context + first)
    heads, kv_heads = 24, 2
    pool_blocks, stride = context // 4 + 1, 24 * 512 + 2 * 512 + 640 + 5
    norms = [(0.4 + 1.2 * rng.random(n)).astype(np.float32) for n in (256, 256, 128, 128)]
    blocks = np.zeros((128, pool_blocks), dtype=np.float32)
    blocks[:, :first // 4] = rng.standard_normal((128, first // 4)).astype(np.float32)
    history = rng.standard_normal((16, 128)).astype(np.float32)
    page_tokens = 256 if paged else context
    pages = context // page_tokens
    order = rng.permutation(pages).astype(np.int32)
    if row_bytes == 272:
        filled = rng.integers(0, 256, pages * 4 * page_tokens * row_bytes, dtype=np.uint8)
        rows = filled.reshape(-1, 272)
        rows[:, 256:] = np.tile(np.frombuffer(np.float16(0.01).tobytes(), np.uint8), 8)
    else:
        filled = rng.standard_normal(pages * 4 * page_tokens * 256).astype(np.float16).view(np.uint8)
    most = max(spans)

    def fresh():
        kv, buffer = gpu.kv_pool(pages, page_tokens, kv_heads, 256, row_bytes)
        gpu.write_buffer(buffer, 0, filled)
        return dict(kv=kv, buffer=buffer, table=gpu.upload(order) if paged else None, projections=gpu.buffer(most * stride * 4), blocks=gpu.upload(blocks),
                    history=gpu.upload(history), norms=[gpu.upload(n) for n in norms], attended=gpu.buffer(most * heads * 256 * 4))

    def read_state(s, steps):
        return dict(kv=_read(gpu, s["buffer"], np.uint8, filled.size), blocks=_read(gpu, s["blocks"], np.float32, blocks.size),
                    history=_read(gpu, s["history"], np.float32, history.size), projections=_read(gpu, s["projections"], np.float32, steps * stride),
                    attended=_read(gpu, s["attended"], np.float32, steps * heads * 256))
    one, two = fresh(), fresh()
    state = gpu.qsa_state(one["kv"], one["table"].base() if paged else None, context, one["blocks"].base(), one["history"].base(),
                          *[n.base() for n in one["norms"]], heads)
    scratch = gpu.buffer(gpu.qsa_prefill_attend_scratch(most, heads, kv_heads, context))
    valid_one, valid_two = [0], [0]
    queries, keys, values = gpu.buffer(most * heads * 256 * 4), gpu.buffer(most * kv_heads * 256 * 4), gpu.buffer(most * kv_heads * 256 * 4)
    index_keys = gpu.buffer(most * 128 * 4)
    scores, indices, counts = gpu.buffer(most * pool_blocks * 4), gpu.buffer(most * 2052 * 4), gpu.buffer(most * 4)
    interval = gpu.buffer(gpu.qsa_index_interval_scratch(most, pool_blocks))
    partial = gpu.buffer(gpu.selected_attention_scratch(most, kv_heads, 2052))
    table_two = two["table"].base() if paged else gpu.upload(np.zeros(1, np.int32)).base()
    at = first
    for steps in spans:
        projections = (rng.standard_normal((steps, stride)) * 2).astype(np.float32)
        # one call
        gpu.write_buffer(one["projections"], 0, projections)
        gpu.qsa_prefill_attend(state, one["projections"].base(), stride, steps, at, scratch, one["attended"].base(), valid_one)
        got = read_state(one, steps)
        # the parts
        gpu.write_buffer(two["projections"], 0, projections)
        base = two["projections"].base()
        for r in range(steps):
            row = base + r * stride * 4
            gpu.qsa_normalize(row, two["norms"][0].base(), 1, heads, 256, 512, at + r, queries.at(r * heads * 256 * 4))
            gpu.qsa_normalize(row + heads * 512 * 4, two["norms"][1].base(), 1, kv_heads, 256, 256, at + r, keys.at(r * kv_heads * 256 * 4))
            gpu.qsa_normalize(row + (heads * 512 + kv_heads * 512) * 4, two["norms"][2].base(), 1, 4, 128, 128, at + r, row + (heads * 512 + kv_heads * 512) * 4)
        gpu.write_buffer(values, 0, np.ascontiguousarray(projections[:, heads * 512 + kv_heads * 256:heads * 512 + kv_heads * 512]))
        gpu.write_buffer(index_keys, 0, np.ascontiguousarray(projections[:, heads * 512 + kv_heads * 512 + 512:heads * 512 + kv_heads * 512 + 640]))
        start = gpu.upload(np.array([at], dtype=np.int32))
        gpu.kv_write(two["kv"], table_two, pages, start.base(), keys.base(), values.base(), False, 1, steps)
        gpu.qsa_pool(index_keys.base(), two["history"].base(), two["norms"][3].base(), pool_blocks, at, steps, two["blocks"].base())
        gpu.qsa_index_interval(base + (heads * 512 + kv_heads * 512) * 4, stride, two["blocks"].base(), pool_blocks, at, steps, 2052, scores.base(), indices.base(),
                               counts.base(), interval, valid_two)
        gpu.selected_attention(two["kv"], two["table"].base() if paged else None, context, at, indices.base(), 2052, counts.base(), queries.base(), False,
                               steps, heads, 0.0625, two["attended"].base(), False, partial, gate=base + 256 * 4, gate_stride=512, gate_row_stride=stride)
        want = read_state(two, steps)
        for what in ("kv", "blocks", "history", "projections", "attended"):
            assert np.array_equal(got[what].view(np.uint8), want[what].view(np.uint8)), f"{what} after the chunk at {at}"
        assert valid_one == valid_two and np.all(np.isfinite(got["attended"])) and np.abs(got["attended"]).max() > 0
        gpu.release(start)
        at += steps
    if first >= 32768:
        assert valid_one[0] > 0, "past 32768 positions the packed keys are carried to the next chunk"
    with pytest.raises(RuntimeError, match="scratch too small"):
        gpu.qsa_prefill_attend(state, one["projections"].base(), stride, most, first, gpu.buffer(4096), one["attended"].base())
    with pytest.raises(RuntimeError, match="inside the context"):
        gpu.qsa_prefill_attend(state, one["projections"].base(), stride, most, context - 1, scratch, one["attended"].base())
