"""Host-side mirror of the reference's safe wrappers over the C ABI for the attention path:
`Backend` / `Buffer` of crates/straydog-engine/src/gpu.rs:735 and ops.rs:846-886, 1139-1245 (same method
names, argument order and meaning; a failed call raises with sd_error()'s text, as `check` does in
crates/straydog-gpu/src/lib.rs:24-43).  Device pointers are plain integers; host data are numpy arrays.
Everything runs in the HIP library; nothing here computes.
"""
import ctypes

import numpy as np

from . import abi


class StraydogError(RuntimeError):
    pass


class Buffer:
    """A zero-filled device allocation (ops.rs Buffer): base address and size."""

    def __init__(self, pointer, size):
        self.pointer, self.size = pointer, size

    def base(self):
        return self.pointer

    def at(self, offset_bytes):
        return self.pointer + offset_bytes


def _host(array):
    return array.ctypes.data_as(ctypes.c_void_p)


def tagged_bf16(pointer):
    """The reference's state_tag: bit 0 marks a BF16 row pointer passed where FP32 is declared (gpu/ops.hpp:1205-1214)."""
    return pointer | 1


class Backend:
    def __init__(self, ordinal=0, budget=1 << 30, library=None):
        self.lib = library or abi.load()
        self.handle = self.lib.sd_create(ordinal, budget)
        if not self.handle:
            raise StraydogError(self.error())

    def error(self):
        text = self.lib.sd_error()
        return text.decode("utf-8", "replace") if text else ""

    def check(self, code):
        if code is None or code < 0:
            raise StraydogError(self.error())
        return code

    def close(self):
        if self.handle:
            self.lib.sd_destroy(self.handle)
            self.handle = None

    def __enter__(self):
        return self

    def __exit__(self, *_):
        self.close()

    # ---- allocations and transfers -------------------------------------------------
    def device_state(self):
        """(free device bytes, total device bytes, the handle's workspace bytes, timing events recorded)."""
        values = (abi.c_u64 * 4)()
        self.check(self.lib.sdx_device_state(self.handle, values))
        return tuple(int(v) for v in values)

    def memory(self):
        used, budget = abi.c_u64(), abi.c_u64()
        self.check(self.lib.sd_memory(self.handle, ctypes.byref(used), ctypes.byref(budget)))
        return used.value, budget.value

    def buffer(self, size):
        pointer = self.lib.sd_buffer(self.handle, size)
        if not pointer:
            raise StraydogError(self.error())
        return Buffer(pointer, size)

    def release(self, buffer):
        self.check(self.lib.sd_release(self.handle, buffer.pointer))

    def write_buffer(self, buffer, offset, values):
        values = np.ascontiguousarray(values)
        self.check(self.lib.sd_buffer_write(self.handle, buffer.pointer, offset, _host(values), values.nbytes))

    def read_buffer(self, buffer, offset, dtype, count):
        out = np.empty(count, dtype=dtype)
        self.check(self.lib.sd_buffer_read(self.handle, buffer.pointer, offset, _host(out), out.nbytes))
        return out

    def upload(self, values):
        """A buffer holding `values` (the tests' upload helper: buffer + write_buffer)."""
        values = np.ascontiguousarray(values)
        buffer = self.buffer(max(values.nbytes, 4))
        if values.nbytes:
            self.write_buffer(buffer, 0, values)
        return buffer

    def synchronize(self):
        self.check(self.lib.sdx_synchronize(self.handle))

    def kv_format(self, row):
        self.check(self.lib.sd_kv_format(self.handle, row))

    # ---- reference ops ---------------------------------------------------------------
    def attention_sequence(self, state, context, base, steps, selected, packed):
        packed = np.ascontiguousarray(packed, dtype=np.float32)
        out = np.empty(steps * 24 * 256, dtype=np.float32)
        self.check(self.lib.sd_attention_sequence(self.handle, state, context, base, steps, selected, _host(packed), packed.size,
                                                  _host(out), out.size))
        return out

    def attention(self, q, keys, values, context, positions, rows, heads, kv_heads, dim, scale, gate, scratch, out):
        self.check(self.lib.sd_op_attention(self.handle, q, keys, values, context, positions, rows, heads, kv_heads, dim, scale,
                                            gate, scratch.pointer if scratch else None, scratch.size if scratch else 0, out))

    def sparse_attention(self, q, raw, raw_rows, positions, window, compressed, compressed_rows, selected, selections, sinks, rows,
                         heads, dim, scale, rope_dims, frequencies, scratch, out):
        self.check(self.lib.sd_op_sparse_attention(self.handle, q, raw, raw_rows, positions, window, compressed, compressed_rows,
                                                   selected, selections, sinks, rows, heads, dim, scale, rope_dims, frequencies,
                                                   scratch.pointer if scratch else None, scratch.size if scratch else 0, out))

    def dspark_attention(self, q, ring, block, sinks, heads, slots, anchor, anchor_at, history, out):
        self.check(self.lib.sd_op_dspark_attention(self.handle, q, ring, block, sinks, heads, slots, anchor, anchor_at, history, out))

    def rope(self, x, rows, vectors, width, rope_dims, positions, frequencies, inverse=False):
        self.check(self.lib.sd_op_rope(self.handle, x, rows, vectors, width, rope_dims, positions, frequencies, int(inverse)))

    def compress(self, kv, gate, groups, ratio, dim, out):
        self.check(self.lib.sd_op_compress(self.handle, kv, gate, groups, ratio, dim, out))

    def index_scores(self, q, keys, weights, visible, rows, groups, heads, dim, scale, scores):
        self.check(self.lib.sd_op_index_scores(self.handle, q, keys, weights, visible, rows, groups, heads, dim, scale, scores))

    def top_k(self, scores, rows, groups, k, out):
        self.check(self.lib.sd_op_top_k(self.handle, scores, rows, groups, k, out))

    def index_candidates(self, scores, visible, rows, groups, blocks, block, out, scratch):
        self.check(self.lib.sd_op_index_candidates(self.handle, scores, visible, rows, groups, blocks, block, out, scratch.pointer,
                                                   scratch.size))

    def index_select(self, q, keys, weights, visible, rows, groups, heads, dim, scale, rope, scores, k, out, within=None):
        rope_dims, positions, frequencies = rope if rope else (0, None, None)
        candidates, blocks, block = within if within else (None, 0, 0)
        self.check(self.lib.sd_op_index_select(self.handle, q, keys, weights, visible, rows, groups, heads, dim, scale, rope_dims,
                                               positions, frequencies, scores, k, out, candidates, blocks, block))

    def index_projection(self, matrix, kind, cols, x, heads, weights):
        self.check(self.lib.sdx_index_projection(self.handle, matrix, kind, cols, x, heads, weights))

    def index_select_proj(self, proj, x, q, keys, weights, visible, groups, heads, dim, scale, rope, scores, k, out, within=None):
        """ops.rs index_select_proj: proj = (matrix, kind, cols); one row."""
        matrix, kind, cols = proj
        rope_dims, positions, frequencies = rope if rope else (0, None, None)
        candidates, blocks, block = within if within else (None, 0, 0)
        self.check(self.lib.sd_op_index_select_proj(self.handle, matrix, kind, cols, x, q, keys, weights, visible, groups, heads, dim, scale,
                                                    rope_dims, positions, frequencies, scores, k, out, candidates, blocks, block))

    def to_bf16(self, x, count, out):
        self.check(self.lib.sd_op_to_bf16(self.handle, x, count, out))

    # ---- paged cache extensions --------------------------------------------------------
    # ---- the inputs of a dense attention step (ops.rs: split, rms_norm, rope_halves, scatter, attention_prepare) ----
    def split(self, x, rows, width, first, second):
        self.check(self.lib.sd_op_split(self.handle, x, rows, width, first, second))

    def rms_norm(self, x, weight, rows, width, eps, out):
        self.check(self.lib.sd_op_rms_norm(self.handle, x, weight, rows, width, eps, out))

    def norm_rope(self, x, weight, rows, width, eps, rope_dims, positions, frequencies, out_rows, out, out_count):
        self.check(self.lib.sd_op_norm_rope(self.handle, x, weight, rows, width, eps, rope_dims, positions, frequencies, out_rows, out, out_count))

    def attention_turns_reserve(self, rows, rope_dims):
        self.check(self.lib.sd_attention_turns_reserve(self.handle, rows, rope_dims))

    def attention_turns_arm(self, rows):
        self.check(self.lib.sd_attention_turns_arm(self.handle, rows))

    def rope_halves(self, x, rows, vectors, width, rope_dims, positions, frequencies):
        self.check(self.lib.sd_op_rope_halves(self.handle, x, rows, vectors, width, rope_dims, positions, frequencies))

    def scatter(self, x, rows, count, width, out, out_rows):
        self.check(self.lib.sd_op_scatter(self.handle, x, rows, count, width, out, out_rows))

    def attention_prepare(self, q_full, k, v, rows, heads, kv_heads, dim, q_weight, k_weight, eps, rope_dims, positions, frequencies, q, gate,
                          keys, values, context):
        self.check(self.lib.sd_op_attention_prepare(self.handle, q_full, k, v, rows, heads, kv_heads, dim, q_weight, k_weight, eps, rope_dims,
                                                    positions, frequencies, q, gate, keys, values, context))

    def kv_pool(self, pages, page_tokens, kv_heads, dim, row_bytes):
        size = pages * 2 * kv_heads * page_tokens * row_bytes
        buffer = self.buffer(size)
        return abi.KvPool(buffer.pointer, pages, page_tokens, kv_heads, dim, row_bytes), buffer

    # ---- the paged K/V cache the library keeps ----
    def kv_cache(self, pages, page_tokens, kv_heads, dim, row_bytes, sequences, max_context):
        """(cache, pool struct, device page table, table stride)."""
        cache = self.lib.sdx_kv_cache_create(self.handle, pages, page_tokens, kv_heads, dim, row_bytes, sequences, max_context)
        if not cache:
            raise StraydogError(self.error())
        pool, table, stride = abi.KvPool(), ctypes.c_void_p(), abi.c_u64()
        self.check(self.lib.sdx_kv_cache_view(self.handle, cache, ctypes.byref(pool), ctypes.byref(table), ctypes.byref(stride)))
        return cache, pool, table.value, stride.value

    def kv_cache_destroy(self, cache):
        self.check(self.lib.sdx_kv_cache_destroy(self.handle, cache))

    def kv_cache_reserve(self, cache, sequence, tokens):
        self.check(self.lib.sdx_kv_cache_reserve(self.handle, cache, sequence, tokens))

    def kv_cache_truncate(self, cache, sequence, tokens):
        self.check(self.lib.sdx_kv_cache_truncate(self.handle, cache, sequence, tokens))

    def kv_cache_fork(self, cache, source, target, tokens):
        self.check(self.lib.sdx_kv_cache_fork(self.handle, cache, source, target, tokens))

    def kv_cache_usage(self, cache, sequence=0):
        held, free = abi.c_u64(), abi.c_u64()
        self.check(self.lib.sdx_kv_cache_usage(self.handle, cache, sequence, ctypes.byref(held), ctypes.byref(free)))
        return held.value, free.value

    def kv_cache_view(self, cache):
        """(pool struct, device page table, table stride) as they are now (a growth moves the pool)."""
        pool, table, stride = abi.KvPool(), ctypes.c_void_p(), abi.c_u64()
        self.check(self.lib.sdx_kv_cache_view(self.handle, cache, ctypes.byref(pool), ctypes.byref(table), ctypes.byref(stride)))
        return pool, table.value, stride.value

    # ---- rows that are not in HBM: the cache's host tier, the VRAM stage, growth ----
    def kv_cache_host(self, cache, host_pages):
        self.check(self.lib.sdx_kv_cache_host(self.handle, cache, host_pages))

    def kv_cache_park(self, cache, sequence):
        self.check(self.lib.sdx_kv_cache_park(self.handle, cache, sequence))

    def kv_cache_resume(self, cache, sequence):
        self.check(self.lib.sdx_kv_cache_resume(self.handle, cache, sequence))

    def kv_cache_stage(self, cache, sequence, tokens):
        """(pool struct, device page table, table stride) of the sequence's first `tokens` positions in the VRAM stage."""
        pool, table, stride = abi.KvPool(), ctypes.c_void_p(), abi.c_u64()
        self.check(self.lib.sdx_kv_cache_stage(self.handle, cache, sequence, tokens, ctypes.byref(pool), ctypes.byref(table), ctypes.byref(stride)))
        return pool, table.value, stride.value

    def kv_cache_gather(self, cache, sequence, context, base, indices, selected, counts, first, rows, renumbered):
        """The union of the selections of rows first .. first + rows - 1 copied into the VRAM stage and the lists renumbered:
        (rows taken, positions gathered, pool struct, device page table, table stride)."""
        taken, gathered = abi.c_u64(), abi.c_u64()
        pool, table, stride = abi.KvPool(), ctypes.c_void_p(), abi.c_u64()
        self.check(self.lib.sdx_kv_cache_gather(self.handle, cache, sequence, context, base, indices, selected, counts, first, rows, renumbered,
                                                ctypes.byref(taken), ctypes.byref(gathered), ctypes.byref(pool), ctypes.byref(table), ctypes.byref(stride)))
        return taken.value, gathered.value, pool, table.value, stride.value

    def kv_cache_unstage(self, cache, sequence, first, count):
        self.check(self.lib.sdx_kv_cache_unstage(self.handle, cache, sequence, first, count))

    def kv_cache_grow(self, cache, pages):
        self.check(self.lib.sdx_kv_cache_grow(self.handle, cache, pages))

    def kv_cache_residency(self, cache, sequence=0):
        """(parked, host pages free, pages of the sequence the stage holds)."""
        parked, free, staged = abi.c_u64(), abi.c_u64(), abi.c_u64()
        self.check(self.lib.sdx_kv_cache_residency(self.handle, cache, sequence, ctypes.byref(parked), ctypes.byref(free), ctypes.byref(staged)))
        return bool(parked.value), free.value, staged.value

    def kv_stage(self, pointer, rows):
        self.check(self.lib.sd_kv_stage(self.handle, pointer, rows))

    def host_state(self, size):
        """A Buffer of `size` bytes in mapped, page-locked host memory (kernels reach it over the bus)."""
        pointer = self.lib.sd_host_state(self.handle, size)
        if not pointer:
            raise StraydogError(self.error())
        return Buffer(pointer, size)

    def kv_write(self, pool, page_table, table_stride, positions, keys, values, input_f16, seqs, span):
        self.check(self.lib.sdx_kv_write(self.handle, ctypes.byref(pool), page_table, table_stride, positions, keys, values,
                                         int(input_f16), seqs, span))

    def paged_attention_scratch(self, seqs, span, heads, dim, max_context):
        return int(self.lib.sdx_paged_attention_scratch(seqs, span, heads, dim, max_context))

    def paged_attention(self, pool, page_table, table_stride, positions, max_context, q, q_f16, seqs, span, heads, scale, out,
                        out_f16, scratch):
        self.check(self.lib.sdx_paged_attention(self.handle, ctypes.byref(pool), page_table, table_stride, positions, max_context,
                                                q, int(q_f16), seqs, span, heads, scale, out, int(out_f16), scratch.pointer,
                                                scratch.size))

    def prefill_tiles_bytes(self, seqs, kv_heads, dim, max_context):
        return int(self.lib.sdx_prefill_tiles_bytes(seqs, kv_heads, dim, max_context))

    def prefill_wave_rows(self, rows):
        """Waves of 64 query rows (the default) or of 32 for the prompt kernel at 128 columns, on this handle from now on."""
        self.check(self.lib.sdx_prefill_wave_rows(self.handle, rows))

    def prefill_chunk(self, pool, page_table, table_stride, positions, max_context, keys, values, kv_f16, q, q_f16, seqs, span, heads, scale,
                      out, out_f16, tiles, valid=None):
        """A prompt chunk in one call: K/V append (keys/values may be None) + causal attention; `tiles` (a Buffer) keeps the cached
        rows' operand tiles between chunks, `valid` the device array of positions whose tiles are still good."""
        self.check(self.lib.sdx_prefill_chunk(self.handle, ctypes.byref(pool), page_table, table_stride, positions, max_context, keys, values,
                                              int(kv_f16), q, int(q_f16), seqs, span, heads, scale, out, int(out_f16), tiles.pointer, tiles.size,
                                              valid))

    def paged_attention_static(self, pool, page_table, table_stride, positions, max_context, q, q_f16, seqs, span, heads, scale, out,
                               out_f16):
        """sdx_paged_attention with the partial results in the library's own area: the call allocates nothing."""
        self.check(self.lib.sdx_paged_attention_static(self.handle, ctypes.byref(pool), page_table, table_stride, positions, max_context,
                                                       q, int(q_f16), seqs, span, heads, scale, out, int(out_f16)))

    def selected_attention_scratch(self, rows, kv_heads, selected):
        return int(self.lib.sdx_selected_attention_scratch(rows, kv_heads, selected))

    def selected_attention(self, pool, page_table, context, base, indices, selected, counts, q, q_f16, rows, heads, scale, out, out_f16,
                           scratch, gate=None, gate_stride=0, gate_row_stride=0, dynamic_base=None):
        self.check(self.lib.sdx_selected_attention(self.handle, ctypes.byref(pool), page_table, context, base, dynamic_base, indices, selected,
                                                   counts, q, int(q_f16), rows, heads, scale, gate, gate_stride, gate_row_stride, out, int(out_f16),
                                                   scratch.pointer, scratch.size))

    def selected_attention_union_scratch(self, rows, heads, kv_heads, selected, context):
        return int(self.lib.sdx_selected_attention_union_scratch(rows, heads, kv_heads, selected, context))

    def selected_attention_union(self, pool, page_table, context, base, indices, selected, counts, q, q_f16, rows, heads, scale, out, out_f16,
                                 scratch, gate=None, gate_stride=0, gate_row_stride=0):
        self.check(self.lib.sdx_selected_attention_union(self.handle, ctypes.byref(pool), page_table, context, base, indices, selected, counts, q,
                                                         int(q_f16), rows, heads, scale, gate, gate_stride, gate_row_stride, out, int(out_f16),
                                                         scratch.pointer, scratch.size))

    def qsa_state(self, pool, page_table, context, blocks, history, q_norm, k_norm, index_q_norm, index_k_norm, heads):
        """An sdx_qsa_state over device pointers (the pool struct is kept alive by the returned object)."""
        state = abi.QsaState(ctypes.pointer(pool), page_table, context, blocks, history, q_norm, k_norm, index_q_norm, index_k_norm, heads)
        state._pool = pool
        return state

    def qsa_decode_attend_scratch(self, steps, heads, kv_heads, context):
        return int(self.lib.sdx_qsa_decode_attend_scratch(steps, heads, kv_heads, context))

    def qsa_decode_attend(self, state, projections, stride, steps, positions, ropes, scratch, attended):
        self.check(self.lib.sdx_qsa_decode_attend(self.handle, ctypes.byref(state), projections, stride, steps, positions, ropes, scratch.pointer,
                                                  scratch.size, attended))

    def qsa_prefill_attend_scratch(self, steps, heads, kv_heads, context):
        return int(self.lib.sdx_qsa_prefill_attend_scratch(steps, heads, kv_heads, context))

    def qsa_prefill_attend(self, state, projections, stride, steps, base, scratch, attended, valid=None):
        """A prompt chunk's attention stage in one call; `valid` is a one-element list (the interval scheme's packed blocks, in and out)."""
        held = abi.c_u64(valid[0] if valid else 0)
        self.check(self.lib.sdx_qsa_prefill_attend(self.handle, ctypes.byref(state), projections, stride, steps, base, scratch.pointer, scratch.size,
                                                   ctypes.byref(held) if valid is not None else None, attended))
        if valid is not None:
            valid[0] = held.value

    def index_top_k(self, q_index, keys, weights, visible, batch, groups, heads, dim, scale, scores, k, indices):
        self.check(self.lib.sdx_index_top_k(self.handle, q_index, keys, weights, visible, batch, groups, heads, dim, scale, scores,
                                            k, indices))

    def index_score_bounds(self, q_index, keys, weights, visible, batch, groups, heads, dim, scale, lower, upper):
        self.check(self.lib.sdx_index_score_bounds(self.handle, q_index, keys, weights, visible, batch, groups, heads, dim, scale, lower,
                                                   upper))

    def qsa_normalize(self, source, norm, rows, heads, width, stride, position, target):
        self.check(self.lib.sdx_qsa_normalize(self.handle, source, norm, rows, heads, width, stride, position, target))

    def qsa_pool(self, incoming, history, norm, pool, base, steps, blocks):
        self.check(self.lib.sdx_qsa_pool(self.handle, incoming, history, norm, pool, base, steps, blocks))

    def qsa_index(self, queries, query_stride, blocks, pool, base, steps, selected, scores, indices, counts, dynamic_base=None):
        self.check(self.lib.sdx_qsa_index(self.handle, queries, query_stride, blocks, pool, base, dynamic_base, steps, selected, scores,
                                          indices, counts))

    def qsa_index_interval_scratch(self, steps, pool):
        return self.lib.sdx_qsa_index_interval_scratch(steps, pool)

    def qsa_index_interval(self, queries, query_stride, blocks, pool, base, steps, selected, scores, indices, counts, scratch, valid=None):
        """The chunk's selection by intervals; `valid` is a one-element list holding the blocks the scratch still has packed (in and out)."""
        held = abi.c_u64(valid[0] if valid else 0)
        self.check(self.lib.sdx_qsa_index_interval(self.handle, queries, query_stride, blocks, pool, base, steps, selected, scores, indices,
                                                   counts, scratch.base(), scratch.size, ctypes.byref(held) if valid is not None else None))
        if valid is not None:
            valid[0] = held.value

    def qsa_index_interval_undecided(self, scratch, steps, pool):
        rows = abi.c_u64()
        self.check(self.lib.sdx_qsa_index_interval_undecided(self.handle, scratch.base(), steps, pool, ctypes.byref(rows)))
        return rows.value

    def latent_attention(self, q, latents, selected, batch, groups, k, heads, kdim, vdim, scale, out):
        self.check(self.lib.sdx_latent_attention(self.handle, q, latents, selected, batch, groups, k, heads, kdim, vdim, scale, out))

    # ---- graphs of ops (gpu.rs graph_begin / graph_end / graph_run) ----
    def graph_begin(self):
        self.check(self.lib.sd_graph_begin(self.handle))

    def graph_end(self, key, keep=True):
        self.check(self.lib.sd_graph_end(self.handle, key, int(keep)))

    def graph_run(self, key):
        """True when a graph is stored under key and was queued."""
        return self.check(self.lib.sd_graph_run(self.handle, key)) == 0

    # ---- conversation checkpoints --------------------------------------------------------
    def checkpoint_buffer(self, size):
        """Page-locked host memory of `size` bytes; returns its address."""
        pointer = self.lib.sd_checkpoint_buffer(self.handle, size)
        if not pointer:
            raise StraydogError(self.error())
        return pointer

    def checkpoint_release(self, pointer):
        self.check(self.lib.sdx_checkpoint_release(self.handle, pointer))

    def checkpoint_copy(self, save, states, buffer):
        """Whole allocations (device pointers) into (save) or out of a checkpoint buffer, packed in order."""
        array = (ctypes.c_void_p * len(states))(*states)
        self.check(self.lib.sd_checkpoint_copy(self.handle, int(save), array, len(states), buffer))

    def checkpoint_clone(self, source, target):
        self.check(self.lib.sd_checkpoint_clone(self.handle, source, target))

    def state_copy(self, state, offset, pitch, width, height, host, first, save):
        """`height` runs of `width` floats, `pitch` apart, from float `offset` of the allocation, to (save) or from the
        C-contiguous float32 array `host` of height x width."""
        assert host.dtype == np.float32 and host.flags["C_CONTIGUOUS"] and host.size == width * height
        self.check(self.lib.sd_state_copy(self.handle, state, offset, pitch, width, height, host.ctypes.data, first, int(save)))

    # ---- harness helpers ----------------------------------------------------------------
    def event(self):
        return self.check(self.lib.sdx_event_record(self.handle))

    def elapsed_ms(self, begin, end):
        ms = abi.c_float()
        self.check(self.lib.sdx_event_elapsed(self.handle, begin, end, ctypes.byref(ms)))
        return ms.value

    def events_clear(self):
        self.check(self.lib.sdx_events_clear(self.handle))

    def profile(self, enable):
        self.check(self.lib.sdx_profile(self.handle, int(enable)))

    def profile_read(self):
        """(summed milliseconds of the ops' dominant kernels, launches) since profiling was enabled."""
        ms, launches = ctypes.c_double(), abi.c_u64()
        self.check(self.lib.sdx_profile_read(self.handle, ctypes.byref(ms), ctypes.byref(launches)))
        return ms.value, launches.value

    def compute_units(self):
        return self.check(self.lib.sdx_device_compute_units(self.handle))

    def fill_normal(self, out, count, seed, kind=0):
        self.check(self.lib.sdx_fill_normal(self.handle, out, count, seed, kind))

    def fill_uniform(self, out, count, seed, lo=0.0, hi=1.0):
        self.check(self.lib.sdx_fill_uniform(self.handle, out, count, seed, lo, hi))

    def mfma_probe(self, trips, live=False):
        """Queues the matrix-core probe (live: operands that change from product to product); returns the floating-point
        operations it performs."""
        flops = ctypes.c_double()
        self.check(self.lib.sdx_mfma_probe(self.handle, trips, int(live), ctypes.byref(flops)))
        return flops.value

    def read_probe(self, source, size, blocks_per_cu=8, unroll=4):
        self.check(self.lib.sdx_read_probe(self.handle, source, size, blocks_per_cu, unroll))

    def paged_stream_probe(self, pool):
        """Queues the loads-only walk of the pool in the decode kernel's order; returns the bytes it reads."""
        size = abi.c_u64()
        self.check(self.lib.sdx_paged_stream_probe(self.handle, ctypes.byref(pool), ctypes.byref(size)))
        return size.value

    def copy(self, target, source, size):
        self.check(self.lib.sdx_copy(self.handle, target, source, size))
