"""numpy front end of the CPU oracle (liboracle.so).  TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py may import this package;
the product (straydog_amd) never does.  Each wrapper is a thin typed call into oracle.c, whose
functions cite the reference lines they restate.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")


def build(force=False):
    """Compile liboracle.so with the Makefile beside it."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-C", _HERE, "CC=gcc"], check=True, capture_output=True)


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    return ctypes.CDLL(_LIB_PATH)


_lib = _load()
_sz, _i32p, _vp = ctypes.c_size_t, ctypes.c_void_p, ctypes.c_void_p


def _ptr(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def _sig(name, restype, *argtypes):
    fn = getattr(_lib, name)
    fn.restype = restype
    fn.argtypes = list(argtypes)
    return fn


_f16_to_f32 = _sig("sdo_f16_to_f32", ctypes.c_float, ctypes.c_uint16)
_f32_to_f16 = _sig("sdo_f32_to_f16", ctypes.c_uint16, ctypes.c_float)
_f32_to_bf16 = _sig("sdo_f32_to_bf16", ctypes.c_uint16, ctypes.c_float)
_to_bf16 = _sig("sdo_to_bf16", None, _vp, _sz, _vp)
_kv_q8_row = _sig("sdo_kv_q8_row", None, _vp, _sz, _vp)
_kv_q8_values = _sig("sdo_kv_q8_values", None, _vp, _sz, _vp)
_ggml_q = _sig("sdo_ggml_q8_0_quantize", None, _vp, _sz, _vp)
_ggml_d = _sig("sdo_ggml_q8_0_dequantize", None, _vp, _sz, _vp)
_kv_write = _sig("sdo_kv_write", None, _vp, _sz, _sz, _sz, _sz, _vp, _sz, _vp, _vp, _vp, _sz, _sz)
_paged = _sig("sdo_paged_attention", None, _vp, _sz, _sz, _sz, _sz, _vp, _sz, _vp, _vp, _sz, _sz, _sz,
              ctypes.c_float, _vp, _vp, ctypes.c_int)
_att_seq = _sig("sdo_attention_sequence", None, _vp, _sz, _sz, _sz, _sz, _sz, _vp, _vp)
_op_att = _sig("sdo_op_attention", None, _vp, _vp, _vp, _sz, _vp, _sz, _sz, _sz, _sz, ctypes.c_float, _vp, _vp)
_op_att64 = _sig("sdo_op_attention_f64", None, _vp, _vp, _vp, _sz, _vp, _sz, _sz, _sz, _sz, ctypes.c_float, _vp, _vp, _vp)
_idx = _sig("sdo_index_scores", None, _vp, _vp, ctypes.c_int, _vp, _vp, _sz, _sz, _sz, _sz, ctypes.c_float, _vp, ctypes.c_int)
_idx64 = _sig("sdo_index_scores_f64", None, _vp, _vp, ctypes.c_int, _vp, _vp, _sz, _sz, _sz, _sz, ctypes.c_float, _vp)
_idx_proj = _sig("sdo_index_projection", None, _vp, ctypes.c_int, _sz, _vp, _sz, _vp)
_topk_key = _sig("sdo_top_k_key", ctypes.c_uint32, ctypes.c_float)
_topk = _sig("sdo_top_k", None, _vp, _sz, _sz, _sz, _vp)
_cand = _sig("sdo_index_candidates", None, _vp, _vp, _sz, _sz, _sz, _sz, _vp)
_latent = _sig("sdo_latent_attention", None, _vp, _vp, _sz, _vp, _sz, _vp, ctypes.c_int, _vp, _sz, _vp, _sz, _sz, _sz, _sz,
               ctypes.c_float, _sz, _vp, _vp, _vp, ctypes.c_int)
_compress = _sig("sdo_compress", None, _vp, _vp, _sz, _sz, _sz, _vp)
_qsa_select = _sig("sdo_qsa_select", _sz, _vp, _sz, _sz, _vp)
_dspark = _sig("sdo_dspark_attention", None, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz, _vp)
_rms_norm = _sig("sdo_rms_norm", None, _vp, _vp, _sz, _sz, ctypes.c_float, _vp)
_rope_halves = _sig("sdo_rope_halves", None, _vp, _sz, _sz, _sz, _sz, _vp, _vp)
_attention_prepare = _sig("sdo_attention_prepare", None, _vp, _vp, _vp, _sz, _sz, _sz, _sz, _vp, _vp, ctypes.c_float, _sz, _vp, _vp, _vp, _vp,
                          _vp, _vp, _sz)
_qsa_normalize = _sig("sdo_qsa_normalize", None, _vp, _vp, _sz, _sz, _sz, _sz, _sz, _vp)
_qsa_pool = _sig("sdo_qsa_pool", None, _vp, _vp, _vp, _sz, _sz, _sz, _vp)
_qsa_block_scores = _sig("sdo_qsa_block_scores", None, _vp, _sz, _vp, _sz, _sz, _sz, _vp)
_fill_n = _sig("sdo_fill_normal", None, ctypes.c_uint64, _vp, _sz)
_fill_u = _sig("sdo_fill_uniform", None, ctypes.c_uint64, _vp, _sz, ctypes.c_float, ctypes.c_float)
max_threads = _sig("sdo_max_threads", ctypes.c_int)


def f16_to_f32(h):
    return float(_f16_to_f32(int(h)))


def f32_to_f16(x):
    return int(_f32_to_f16(float(np.float32(x))))


def f32_to_bf16(x):
    return int(_f32_to_bf16(ctypes.c_float(np.float32(x))))


def to_bf16(x):
    x = _f32(x)
    out = np.empty(x.shape, dtype=np.uint16)
    _to_bf16(_ptr(x), x.size, _ptr(out))
    return out


def top_k_key(x):
    return int(_topk_key(ctypes.c_float(np.float32(x))))


def kv_q8_row_bytes(dim):
    return dim + dim // 32 * 2


def kv_q8_row(values):
    values = _f32(values)
    dim = values.shape[-1]
    flat = values.reshape(-1, dim)
    out = np.zeros((flat.shape[0], kv_q8_row_bytes(dim)), dtype=np.uint8)
    for i in range(flat.shape[0]):
        _kv_q8_row(_ptr(flat[i]), dim, _ptr(out[i]))
    return out.reshape(values.shape[:-1] + (kv_q8_row_bytes(dim),))


def kv_q8_values(rows, dim):
    rows = np.ascontiguousarray(rows, dtype=np.uint8)
    flat = rows.reshape(-1, rows.shape[-1])
    out = np.zeros((flat.shape[0], dim), dtype=np.float32)
    for i in range(flat.shape[0]):
        _kv_q8_values(_ptr(flat[i]), dim, _ptr(out[i]))
    return out.reshape(rows.shape[:-1] + (dim,))


def ggml_q8_0_quantize(values):
    values = _f32(values).reshape(-1)
    out = np.zeros(values.size // 32 * 34, dtype=np.uint8)
    _ggml_q(_ptr(values), values.size, _ptr(out))
    return out


def ggml_q8_0_dequantize(blocks):
    blocks = np.ascontiguousarray(blocks, dtype=np.uint8).reshape(-1)
    count = blocks.size // 34 * 32
    out = np.zeros(count, dtype=np.float32)
    _ggml_d(_ptr(blocks), count, _ptr(out))
    return out


def pool_bytes(pages, kv_heads, page_tokens, row_bytes):
    return pages * 2 * kv_heads * page_tokens * row_bytes


def kv_write(pool, row_bytes, page_tokens, kv_heads, dim, page_table, positions, keys, values):
    """keys/values [seqs][span][kv_heads][dim] appended in place into the uint8 pool."""
    keys, values = _f32(keys), _f32(values)
    seqs, span = keys.shape[0], keys.shape[1]
    table = _i32(page_table).reshape(seqs, -1)
    positions = _i32(positions)
    assert pool.dtype == np.uint8 and pool.flags["C_CONTIGUOUS"]
    _kv_write(_ptr(pool), row_bytes, page_tokens, kv_heads, dim, _ptr(table), table.shape[1], _ptr(positions),
              _ptr(keys), _ptr(values), seqs, span)


def paged_attention(pool, row_bytes, page_tokens, kv_heads, dim, page_table, positions, q, scale, wide=False, threads=0):
    """q [seqs][span][heads][dim] fp32 -> out (and the float64 evaluation when wide)."""
    q = _f32(q)
    seqs, span, heads, _ = q.shape
    table = _i32(page_table).reshape(seqs, -1)
    positions = _i32(positions)
    out = np.zeros(q.shape, dtype=np.float32)
    out64 = np.zeros(q.shape, dtype=np.float64) if wide else None
    _paged(_ptr(pool), row_bytes, page_tokens, kv_heads, dim, _ptr(table), table.shape[1], _ptr(positions), _ptr(q),
           seqs, span, heads, ctypes.c_float(scale), _ptr(out), _ptr(out64), threads)
    return (out, out64) if wide else out


def attention_sequence(state, row_bytes, context, base, steps, selected, packed):
    packed = _f32(packed)
    out = np.zeros(steps * 24 * 256, dtype=np.float32)
    _att_seq(_ptr(state), row_bytes, context, base, steps, selected, _ptr(packed), _ptr(out))
    return out


def op_attention(q, keys, values, positions, scale, gate=None):
    q, keys, values = _f32(q), _f32(keys), _f32(values)
    rows, heads, dim = q.shape
    context, kv_heads, _ = keys.shape
    positions = _i32(positions)
    gate = None if gate is None else _f32(gate)
    out = np.zeros(q.shape, dtype=np.float32)
    _op_att(_ptr(q), _ptr(keys), _ptr(values), context, _ptr(positions), rows, heads, kv_heads, dim, ctypes.c_float(scale),
            _ptr(gate), _ptr(out))
    return out


def op_attention_f64(q, keys, values, positions, scale, gate=None):
    q, keys, values = _f32(q), _f32(keys), _f32(values)
    rows, heads, dim = q.shape
    context, kv_heads, _ = keys.shape
    positions = _i32(positions)
    gate = None if gate is None else _f32(gate)
    out = np.zeros(q.shape, dtype=np.float64)
    bound = np.zeros(q.shape, dtype=np.float64)
    _op_att64(_ptr(q), _ptr(keys), _ptr(values), context, _ptr(positions), rows, heads, kv_heads, dim, ctypes.c_float(scale),
              _ptr(gate), _ptr(out), _ptr(bound))
    return out, bound


def _keys_arg(keys):
    if keys.dtype == np.uint16:
        return np.ascontiguousarray(keys), 1
    return _f32(keys), 0


def index_scores(q, keys, weights, visible, scale, threads=0):
    """q [rows][heads][dim] fp32; keys [groups][dim] fp32 or uint16 (BF16 bits)."""
    q, weights, visible = _f32(q), _f32(weights), _i32(visible)
    keys, bf16 = _keys_arg(keys)
    rows, heads, dim = q.shape
    groups = keys.shape[0]
    out = np.zeros((rows, groups), dtype=np.float32)
    _idx(_ptr(q), _ptr(keys), bf16, _ptr(weights), _ptr(visible), rows, groups, heads, dim, ctypes.c_float(scale), _ptr(out), threads)
    return out


def index_scores_f64(q, keys, weights, visible, scale):
    q, weights, visible = _f32(q), _f32(weights), _i32(visible)
    keys, bf16 = _keys_arg(keys)
    rows, heads, dim = q.shape
    groups = keys.shape[0]
    out = np.zeros((rows, groups), dtype=np.float64)
    _idx64(_ptr(q), _ptr(keys), bf16, _ptr(weights), _ptr(visible), rows, groups, heads, dim, ctypes.c_float(scale), _ptr(out))
    return out


def index_projection(matrix, kind, cols, x, heads):
    """matrix: uint8 bytes of heads rows, BF16 (kind 30) or ggml Q8_0 blocks (kind 8); x [cols] fp32."""
    matrix, x = np.ascontiguousarray(matrix, dtype=np.uint8), _f32(x)
    out = np.zeros(heads, dtype=np.float32)
    _idx_proj(_ptr(matrix), kind, cols, _ptr(x), heads, _ptr(out))
    return out


def top_k(scores, k):
    scores = _f32(scores)
    rows, groups = scores.shape
    out = np.zeros((rows, k), dtype=np.int32)
    _topk(_ptr(scores), rows, groups, k, _ptr(out))
    return out


def index_candidates(scores, visible, blocks, block):
    scores, visible = _f32(scores), _i32(visible)
    rows, groups = scores.shape
    out = np.zeros((rows, blocks), dtype=np.int32)
    _cand(_ptr(scores), _ptr(visible), rows, groups, blocks, block, _ptr(out))
    return out


def latent_attention(q, raw, positions, window, compressed, selected, sinks, vdim, scale, rope_dims=0, frequencies=None,
                     wide=False, threads=0):
    """q [rows][heads][kdim]; raw [raw_rows][kdim] or None; compressed [n][kdim] fp32 or uint16; selected [rows][selections]."""
    q = _f32(q)
    rows, heads, kdim = q.shape
    raw = None if raw is None else _f32(raw)
    raw_rows = 0 if raw is None else raw.shape[0]
    positions = None if positions is None else _i32(positions)
    bf16 = 0
    if compressed is not None:
        compressed, bf16 = _keys_arg(compressed)
    selected = None if selected is None else _i32(selected)
    selections = 0 if selected is None else selected.shape[1]
    sinks = None if sinks is None else _f32(sinks)
    frequencies = None if frequencies is None else _f32(frequencies)
    out = np.zeros((rows, heads, vdim), dtype=np.float32)
    out64 = np.zeros((rows, heads, vdim), dtype=np.float64) if wide else None
    _latent(_ptr(q), _ptr(raw), raw_rows, _ptr(positions), window, _ptr(compressed), bf16, _ptr(selected), selections, _ptr(sinks),
            rows, heads, kdim, vdim, ctypes.c_float(scale), rope_dims, _ptr(frequencies), _ptr(out), _ptr(out64), threads)
    return (out, out64) if wide else out


def compress(kv, gate, ratio):
    kv = _f32(kv)
    dim = kv.shape[-1]
    groups = kv.shape[0] // ratio
    gate = None if gate is None else _f32(gate)
    out = np.zeros((groups, dim), dtype=np.float32)
    _compress(_ptr(kv), _ptr(gate), groups, ratio, dim, _ptr(out))
    return out


def qsa_select(scores, position, keep_blocks=512):
    scores = _f32(scores)
    out = np.zeros(keep_blocks * 4 + 4 + max(0, position + 1), dtype=np.float32)
    count = _qsa_select(_ptr(scores), position, keep_blocks, _ptr(out))
    return out[:count].copy()


def dspark_attention(q, ring, block, sinks, heads, slots, anchor, history):
    q, ring, block, sinks = _f32(q), _f32(ring), _f32(block), _f32(sinks)
    out = np.zeros(slots * heads * 512, dtype=np.float64)
    _dspark(_ptr(q), _ptr(ring), _ptr(block), _ptr(sinks), heads, slots, anchor, history, _ptr(out))
    return out


def rms_norm(x, weight, eps):
    x, weight = _f32(x), _f32(weight)
    out = np.zeros_like(x)
    _rms_norm(_ptr(x), _ptr(weight), x.shape[0], x.shape[1], ctypes.c_float(eps), _ptr(out))
    return out


def rope_halves(x, rope_dims, positions, frequencies):
    """x: [rows, vectors, width]; returns the turned copy."""
    out, positions, frequencies = _f32(x).copy(), _i32(positions), _f32(frequencies)
    _rope_halves(_ptr(out), out.shape[0], out.shape[1], out.shape[2], rope_dims, _ptr(positions), _ptr(frequencies))
    return out


def attention_prepare(q_full, k, v, q_weight, k_weight, eps, rope_dims, positions, frequencies, keys, values):
    """q_full [rows, heads, 2*dim], k/v [rows, kv_heads, dim]; keys/values [context, kv_heads*dim] are updated in place.
    Returns (q, gate, k_after)."""
    q_full, k, v = _f32(q_full), _f32(k).copy(), _f32(v)
    rows, heads, dim = q_full.shape[0], q_full.shape[1], q_full.shape[2] // 2
    q_weight, k_weight, positions, frequencies = _f32(q_weight), _f32(k_weight), _i32(positions), _f32(frequencies)
    assert keys.dtype == np.float32 and values.dtype == np.float32 and keys.flags.c_contiguous and values.flags.c_contiguous
    q, gate = np.zeros((rows, heads, dim), np.float32), np.zeros((rows, heads, dim), np.float32)
    _attention_prepare(_ptr(q_full), _ptr(k), _ptr(v), rows, heads, k.shape[1], dim, _ptr(q_weight), _ptr(k_weight), ctypes.c_float(eps),
                       rope_dims, _ptr(positions), _ptr(frequencies), _ptr(q), _ptr(gate), _ptr(keys), _ptr(values), keys.shape[0])
    return q, gate, k


def qsa_normalize(source, norm, rows, heads, width, stride, position):
    """source: flat floats, row r head h at (r * heads + h) * stride; returns [rows * heads, width]."""
    source, norm = _f32(source).reshape(-1), _f32(norm)
    out = np.zeros((rows * heads, width), dtype=np.float32)
    _qsa_normalize(_ptr(source), _ptr(norm), rows, heads, width, stride, position, _ptr(out))
    return out


def qsa_pool(incoming, history, norm, pool, base, blocks):
    """Updates `blocks` ([128, pool]) and `history` ([16, 128]) in place for rows base .. base + len(incoming)."""
    incoming, norm = _f32(incoming), _f32(norm)
    assert history.dtype == np.float32 and blocks.dtype == np.float32 and history.flags.c_contiguous and blocks.flags.c_contiguous
    _qsa_pool(_ptr(incoming), _ptr(history), _ptr(norm), pool, base, incoming.shape[0], _ptr(blocks))


def qsa_block_scores(queries, blocks, base, scores=None):
    """queries: [steps, stride >= 512]; blocks: [128, pool].  Returns [steps, pool] (zeros where the reference writes nothing)."""
    queries, blocks = _f32(queries), _f32(blocks)
    steps, pool = queries.shape[0], blocks.shape[1]
    if scores is None:
        scores = np.zeros((steps, pool), dtype=np.float32)
    _qsa_block_scores(_ptr(queries), queries.shape[1], _ptr(blocks), pool, base, steps, _ptr(scores))
    return scores


def fill_normal(seed, count):
    out = np.zeros(count, dtype=np.float32)
    _fill_n(ctypes.c_uint64(seed), _ptr(out), count)
    return out


def fill_uniform(seed, count, lo=0.0, hi=1.0):
    out = np.zeros(count, dtype=np.float32)
    _fill_u(ctypes.c_uint64(seed), _ptr(out), count, ctypes.c_float(lo), ctypes.c_float(hi))
    return out
