/* The part of Straydog's GPU C ABI that this MI355X (gfx950) attention library implements.
 *
 * Every function keeps the name, argument order, argument meaning and error convention of the
 * reference declaration it replaces (cited per function as gpu/straydog_gpu.h:LINE of the reference
 * checkout, with the reference body it stands in for), so the Rust host's bindings call it unchanged.
 * Conventions (reference gpu/straydog_gpu.h:1-5): a negative int or a null pointer is a failure that
 * sd_error() then describes for the calling thread; other int results are 0 or a query's answer;
 * handles are opaque; no exception crosses this boundary.  Ops are queued on the device's one compute
 * stream and return at once; only reads (sd_buffer_read, sd_download) wait for the stream.  Every
 * pointer an op takes must lie inside one allocation of the same device (reference gpu/ops.hpp:4-26).
 *
 * The attention *stages* that the reference reaches only through whole-layer span calls, and the
 * synthetic paged/batched configurations, are in straydog_gpu_ext.h (sdx_*).
 */
#ifndef STRAYDOG_GPU_H
#define STRAYDOG_GPU_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- Errors and devices ---- */
/* reference straydog_gpu.h:17 (gpu/core.hpp:172): the calling thread's last failure text, valid until its next call. */
const char* sd_error(void);
/* reference straydog_gpu.h:18 */
int sd_device_count(void);
/* reference straydog_gpu.h:21: name (NUL-terminated, cut to capacity), free and total bytes of device `ordinal`. */
int sd_device_info(int ordinal, char* name, size_t capacity, uint64_t* free_bytes, uint64_t* total_bytes);
/* reference straydog_gpu.h:35-36 (gpu/kernels.cpp:3511-3614): a device handle with a VRAM budget in bytes that every
 * allocation is charged against; one compute stream. */
void* sd_create(int ordinal, uint64_t budget);
void sd_destroy(void* handle);
/* reference straydog_gpu.h:37: bytes allocated so far and the budget. */
int sd_memory(void* handle, uint64_t* used, uint64_t* budget);

/* ---- Allocations and transfers ---- */
/* reference straydog_gpu.h:44 (gpu/host_io.hpp:81-109): a new allocation holding a copy of `data`; the caller's
 * memory is free on return, the bytes land in stream order. */
void* sd_upload(void* handle, const void* data, uint64_t bytes);
/* reference straydog_gpu.h:49: an allocation whose bytes arrive later (only its 64-byte tail is zeroed). */
void* sd_allocate(void* handle, uint64_t bytes);
/* reference straydog_gpu.h:58: stage caller memory into all of an allocation. */
int sd_write(void* handle, void* pointer, const void* data, uint64_t bytes);
/* reference straydog_gpu.h:64-68 */
int sd_release(void* handle, void* pointer);
int sd_allocation_bytes(void* handle, const void* pointer, uint64_t* bytes);
int sd_zero(void* handle, void* pointer);
/* reference straydog_gpu.h:69 (gpu/host_io.hpp:113-140): copy out and wait for the stream. */
int sd_download(void* handle, void* pointer, void* output, uint64_t bytes);
/* reference straydog_gpu.h:152-156 (gpu/kernels.cpp:4555-4592): a zero-filled buffer (synchronised before return),
 * writes staged in stream order, reads that wait for the stream. */
void* sd_buffer(void* handle, uint64_t bytes);
int sd_buffer_write(void* handle, void* buffer, uint64_t offset, const void* data, uint64_t bytes);
int sd_buffer_read(void* handle, const void* buffer, uint64_t offset, void* output, uint64_t bytes);

/* ---- Graphs of ops ---- */
/* reference straydog_gpu.h:177-183 (gpu/kernels.cpp:4765-4813): between sd_graph_begin and sd_graph_end (keep: store it under key,
 * replacing any; else drop it) the ops queued on the device's stream are recorded rather than run; only ops with no host data
 * (no buffer writes) that allocate nothing may be recorded.  sd_graph_run queues a recorded graph: 0, or 1 when none is stored
 * under key. */
int sd_graph_begin(void* handle);
int sd_graph_end(void* handle, uint64_t key, int keep);
int sd_graph_run(void* handle, uint64_t key);

/* ---- conversation checkpoints ---- */
/* reference straydog_gpu.h:115 (gpu/kernels.cpp:3905-3915): page-locked host memory of `bytes` for copies of sequence state;
 * it lives until the handle is destroyed (or sdx_checkpoint_release, straydog_gpu_ext.h). */
void* sd_checkpoint_buffer(void* handle, uint64_t bytes);
/* reference straydog_gpu.h:116 (gpu/kernels.cpp:3962-3990): `count` (1..4096) whole device allocations copied into (save != 0)
 * or out of a checkpoint buffer, packed in the order given, the stream waited for once; refuses a buffer that is not a
 * checkpoint buffer, a state that is not an allocation, and states that do not fit the buffer. */
int sd_checkpoint_copy(void* handle, int save, void* const* states, uint64_t count, void* buffer);
/* reference straydog_gpu.h:118 (gpu/kernels.cpp:3951-3961): checkpoint buffer `to` receives what `from` holds (equal sizes),
 * after the stream -- and the copies into `from` it still had -- is done. */
int sd_checkpoint_clone(void* handle, void* from, void* to);
/* reference straydog_gpu.h:120-121 (gpu/kernels.cpp:3996-4041): part of a state to (save != 0) or from host memory: `height`
 * runs of `width` floats, `pitch` floats apart, from float `offset` of the allocation (a K/V plane's positions are one run, a
 * block indexer's pooled blocks one run per column); host rows are packed.  `first` is where the reference truncates the VRAM
 * mirrors of a host-resident K/V; this library keeps K/V in HBM only and ignores it. */
int sd_state_copy(void* handle, void* state, uint64_t offset, uint64_t pitch, uint64_t width, uint64_t height, float* host, uint64_t first,
                  int save);

/* ---- K/V format ---- */
/* reference straydog_gpu.h:113 (gpu/kernels.cpp:4266-4274): the bytes of a K/V row of the Qwen state, 512 (FP16) or
 * 272 (Q8_0: 256 int8 then eight FP16 block scales, gpu/core.hpp:397-403).  Default 272. */
int sd_kv_format(void* handle, uint32_t row);
/* reference straydog_gpu.h:114 (gpu/kernels.cpp:4277-4290): registers an allocation of this device, exactly rows x 4096 bytes
 * (rows <= 2^22, not a host state), as the VRAM stage that rows held in host memory are copied into to be attended from;
 * "invalid Straydog K/V stage" otherwise.  What a former stage held is forgotten and recorded graphs are dropped.  The paged
 * cache's `stage` / `unstage` (straydog_gpu_ext.h) are what fills and drains it. */
int sd_kv_stage(void* handle, void* pointer, uint64_t rows);
/* reference straydog_gpu.h:98 (gpu/kernels.cpp:3876-3903): `bytes` of zeroed, mapped, page-locked host memory that kernels read
 * and write over the bus; owned like a device allocation (ops take pointers into it, sd_release frees it) but outside the VRAM
 * budget.  Null on failure. */
void* sd_host_state(void* handle, uint64_t bytes);
/* reference straydog_gpu.h:99 (gpu/kernels.cpp:3824-3847): page-locks and zeroes host states of these sizes on a thread of its
 * own; sd_host_state then takes one of the right size (in any order) once the thread is done.  One prefetch at a time. */
int sd_host_states_prefetch(void* handle, const uint64_t* sizes, uint64_t count);
/* reference straydog_gpu.h:112 (gpu/kernels.cpp:4292-4300): 1, host-resident state is supported. */
int sd_host_state_supported(void* handle);

/* ---- Attention ops ---- */
/* reference straydog_gpu.h:528 (gpu/kernels.cpp:4387-4419, kernels :79-165): selection-list attention of `steps` rows at
 * positions base.. over the Qwen state (4 planes of `context` rows: K head 0, K head 1, V head 0, V head 1).  Host
 * pointers: input = [steps*24*256 q | steps*2*256 k | steps*2*256 v | steps*selected indices as floats | steps counts],
 * output = steps*24*256 floats.  The rows' K/V are written first; scale 1/16; an index is attended when
 * 0 <= index <= base+step and index < context. */
int sd_attention_sequence(void* handle, void* state, uint64_t context, uint64_t base, uint64_t steps, uint64_t selected,
                          const float* input, uint64_t input_count, float* output, uint64_t output_count);
/* reference straydog_gpu.h:451 (gpu/token_mixing.hpp:652-693, kernels :356-520): causal grouped-query attention of
 * q (rows x heads x dim) at `positions` over FP32 caches keys/values (context x kv_heads x dim), each row up to its
 * position (clipped to the cache), times sigmoid(gate) when given.  scratch: rows x heads x splits x (dim + 2) floats,
 * splits = min(64, max(1, 256 / (rows x heads))). */
int sd_op_attention(void* handle, const float* q, const float* keys, const float* values, uint64_t context, const int32_t* positions,
                    uint64_t rows, uint64_t heads, uint64_t kv_heads, uint64_t dim, float scale, const float* gate, float* scratch,
                    uint64_t scratch_bytes, float* out);
/* reference straydog_gpu.h:385 (gpu/kernels.cpp:5311-5476, kernels gpu/ops.hpp:1240-1677): latent attention.  Each query
 * attends the window rows of `raw` ending at its position (position p in row p % raw_rows) and the compressed rows
 * `selected` lists (-1: none), keys = values, with a per-head sink in the max and the denominator.  `compressed` may
 * carry bit 0 (BF16 rows, gpu/ops.hpp:1205-1214).  rope_dims rotates q's last values by positions * frequencies on the
 * way in and the output back.  scratch is optional and unused by this implementation. */
int sd_op_sparse_attention(void* handle, const float* q, const float* raw, uint64_t raw_rows, const int32_t* positions, uint64_t window,
                           const float* compressed, uint64_t compressed_rows, const int32_t* selected, uint64_t selections,
                           const float* sinks, uint64_t rows, uint64_t heads, uint64_t dim, float scale, uint64_t rope_dims,
                           const float* frequencies, float* scratch, uint64_t scratch_bytes, float* out);
/* reference straydog_gpu.h:399-406 (gpu/dspark_attention.hpp:1-101): DSpark's noncausal block attention.  q/out [slots][heads][512]
 * (1..64 heads, 1..5 slots), K = V ring [128][512], block keys [slots][512], sinks [heads]; rope already applied.  Every query sees
 * the history positions [anchor - history, anchor) (row p % 128 of the ring) and all the block's keys; scale 1/sqrt(512); the sink
 * enters the maximum and the denominator only.  anchor_at, when not null, is a device-resident anchor that replaces `anchor`. */
int sd_op_dspark_attention(void* handle, const float* q, const float* ring, const float* block, const float* sinks, uint64_t heads, uint64_t slots,
                           uint32_t anchor, const int32_t* anchor_at, uint64_t history, float* out);
/* reference straydog_gpu.h:271 (gpu/kernels.cpp:4942-4956, kernel gpu/ops.hpp:107-120): the last rope_dims values of each of
 * a row's `vectors` vectors of `width` rotated in adjacent pairs by positions[row] * frequencies[pair] (sine and cosine in
 * double); inverse: by the angle times -1. */
int sd_op_rope(void* handle, float* x, uint64_t rows, uint64_t vectors, uint64_t width, uint64_t rope_dims, const int32_t* positions,
               const float* frequencies, int inverse);
/* reference straydog_gpu.h:407 (gpu/kernels.cpp:5478-5485, kernel gpu/ops.hpp:1681-1694): per-channel softmax pooling. */
int sd_op_compress(void* handle, const float* kv, const float* gate, uint64_t groups, uint64_t ratio, uint64_t dim, float* out);
/* reference straydog_gpu.h:408 (gpu/kernels.cpp:5487-5499, kernel gpu/ops.hpp:1700-1739): scores[row][g] =
 * scale * sum_h relu(q[row][h] . keys[g]) * weights[row][h] for g < visible[row], -inf beyond, in the canonical
 * order (fmaf over the columns in order, each head's term rounded, heads added in order).  keys may be BF16-tagged. */
int sd_op_index_scores(void* handle, const float* q, const float* keys, const float* weights, const int32_t* visible, uint64_t rows,
                       uint64_t groups, uint64_t heads, uint64_t dim, float scale, float* scores);
/* reference straydog_gpu.h:409 (gpu/kernels.cpp:5669-5676, gpu/ops.hpp:1766-1941): each row's k highest scores' indices in
 * ascending index order; ties keep the lower index; -inf never kept; -1 fills empty slots. */
int sd_op_top_k(void* handle, const float* scores, uint64_t rows, uint64_t groups, uint64_t k, int32_t* out);
/* reference straydog_gpu.h:414 (gpu/kernels.cpp:5524-5540, gpu/ops.hpp:1942-1975): a row's candidate blocks. */
int sd_op_index_candidates(void* handle, const float* scores, const int32_t* visible, uint64_t rows, uint64_t groups, uint64_t blocks,
                           uint64_t block, int32_t* out, float* scratch, uint64_t scratch_bytes);
/* reference straydog_gpu.h:419 (gpu/kernels.cpp:5561-5618, gpu/ops.hpp:1993-2230): rope of q (q itself unchanged),
 * sd_op_index_scores and sd_op_top_k in one call: the same scores and indices, bit for bit. */
int sd_op_index_select(void* handle, const float* q, const float* keys, const float* weights, const int32_t* visible, uint64_t rows,
                       uint64_t groups, uint64_t heads, uint64_t dim, float scale, uint64_t rope_dims, const int32_t* positions,
                       const float* frequencies, float* scores, uint64_t k, int32_t* out, const int32_t* candidates, uint64_t blocks,
                       uint64_t block);
/* reference straydog_gpu.h:422 (gpu/kernels.cpp:5620-5667, gpu/ops.hpp:2267-2300): sd_op_index_select of one decode row with the
 * projection of x into the heads' weights ahead of it: weights[h] = row h of the heads x proj_cols matrix proj_weights . x, the
 * rows BF16 (proj_kind 30) or ggml Q8_0 blocks (proj_kind 8); other kinds are refused.  `weights` receives them.  The same
 * weights, scores and indices, bit for bit, as sdx_index_projection (straydog_gpu_ext.h) followed by sd_op_index_select. */
int sd_op_index_select_proj(void* handle, const void* proj_weights, int proj_kind, uint64_t proj_cols, const float* x, const float* q,
                            const float* keys, float* weights, const int32_t* visible, uint64_t groups, uint64_t heads, uint64_t dim, float scale,
                            uint64_t rope_dims, const int32_t* positions, const float* frequencies, float* scores, uint64_t k, int32_t* out,
                            const int32_t* candidates, uint64_t blocks, uint64_t block);
/* ---- The inputs of a dense attention step (its neighbours in a span) ---- */
/* reference straydog_gpu.h:446 (gpu/token_mixing.hpp:246-252, :628-637): rows of [first | second], `width` each, apart. */
int sd_op_split(void* handle, const float* x, uint64_t rows, uint64_t width, float* first, float* second);
/* reference straydog_gpu.h:251 (gpu/kernels.cpp:4901-4913, gpu/ops.hpp:28-59): output = input * rsqrt(mean(input^2) + eps) * weight
 * per row; the sum of squares in the order of the reference's 256-thread halving tree.  May run in place. */
int sd_op_rms_norm(void* handle, const float* input, const float* weight, uint64_t rows, uint64_t width, float eps, float* output);
/* reference straydog_gpu.h:252-254 (gpu/kernels.cpp:4915-4940, gpu/ops.hpp:60-106): sd_op_rms_norm, then the last rope_dims values
 * of each row turned in adjacent pairs by positions[row] * frequencies[pair] (as sd_op_rope), the row stored at row out_rows[row]
 * of `out` (out_count rows; the row itself when out_rows is null).  Fills an armed attention rope table of exactly `rows` rows. */
int sd_op_norm_rope(void* handle, const float* input, const float* weight, uint64_t rows, uint64_t width, float eps, uint64_t rope_dims,
                    const int32_t* positions, const float* frequencies, const int32_t* out_rows, float* out, uint64_t out_count);
/* reference straydog_gpu.h:382-389 (gpu/kernels.cpp:558-616, :5288-5303): the attention rope table of a pass, rows x rope_dims/2 pairs
 * of (cosine, sine) forward and inverse.  Reserve allocates it (outside a recorded graph; a larger request replaces it); arm makes
 * the next sd_op_norm_rope of exactly `rows` rows (0 clears) write it, and the next sd_op_sparse_attention of those rows then reads
 * it instead of forming the angles again: the same bits. */
int sd_attention_turns_reserve(void* handle, uint64_t rows, uint64_t rope_dims);
int sd_attention_turns_arm(void* handle, uint64_t rows);
/* reference straydog_gpu.h:452 (gpu/token_mixing.hpp:254-274, :639-650): the leading rope_dims values of each of a row's
 * `vectors` vectors of `width` turned in pairs (i, i + rope_dims/2) by positions[row] * frequencies[i], angles in double. */
int sd_op_rope_halves(void* handle, float* x, uint64_t rows, uint64_t vectors, uint64_t width, uint64_t rope_dims, const int32_t* positions,
                      const float* frequencies);
/* reference straydog_gpu.h:307 (gpu/kernels.cpp:5244-5252, gpu/ops.hpp:1171-1175): out[rows[i]] = x[i], `width` values a row.
 * An index outside 0 .. out_rows - 1 writes nothing here (the reference leaves it undefined). */
int sd_op_scatter(void* handle, const float* x, const int32_t* rows, uint64_t count, uint64_t width, float* out, uint64_t out_rows);
/* reference straydog_gpu.h:447-451 (gpu/token_mixing.hpp:276-338, :601-626): an attention step's inputs in one launch:
 * sd_op_split of q_full (rows x heads x [query | gate], each dim) into q and gate, sd_op_rms_norm of the queries (q_weight) and
 * of k's heads (k_weight, in place), sd_op_rope_halves of both (rope_dims), and sd_op_scatter of k and v (rows x kv_heads x dim)
 * to rows `positions` of keys and values (context rows each); the same bits as the separate ops.  A position outside the
 * cache writes no row of it. */
int sd_op_attention_prepare(void* handle, const float* q_full, float* k, const float* v, uint64_t rows, uint64_t heads, uint64_t kv_heads,
                            uint64_t dim, const float* q_weight, const float* k_weight, float eps, uint64_t rope_dims, const int32_t* positions,
                            const float* frequencies, float* q, float* gate, float* keys, float* values, uint64_t context);
/* reference straydog_gpu.h:459 (gpu/token_mixing.hpp:728-744): out = x as BF16, nearest even, a NaN stays a NaN. */
int sd_op_to_bf16(void* handle, const float* x, uint64_t count, void* out);

#ifdef __cplusplus
}
#endif
#endif
