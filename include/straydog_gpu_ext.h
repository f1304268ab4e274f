/* Extension entry points of the MI355X attention library (sdx_*).
 *
 * The reference reaches its decode / verify / prefill attention only inside whole-layer span calls
 * (sd_decode_span, sd_verify_span, sd_prefill_span: gpu/straydog_gpu.h:526,536,571 of the reference), which also
 * run GEMVs, hyper-connections and MoE.  These entry points expose the attention *stage* of those spans on its
 * own, generalised to a paged, batched K/V cache, with the same conventions as straydog_gpu.h: device-resident
 * arguments (positions are read on the device so a recorded graph replays without new host arguments, as
 * gpu/qsa_decode.hpp:1-4 does), ops queued on the handle's stream, negative result = failure described by
 * sd_error().  Each one cites the reference code whose arithmetic it stands in for.
 */
#ifndef STRAYDOG_GPU_EXT_H
#define STRAYDOG_GPU_EXT_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* A paged K/V cache.  Page p holds, for page_tokens consecutive positions, 2*kv_heads planes: the keys of K/V head
 * h in plane h, its values in plane kv_heads + h (the reference's plane order, gpu/core.hpp:397-403, inside a page).
 * A plane is page_tokens rows of row_bytes: Q8_0 (row_bytes = dim + dim/16: dim int8 then dim/32 FP16 block scales,
 * the reference's kv_row_q8 rule, 272 bytes at dim 256 and 136 at dim 128) or FP16 (row_bytes = 2*dim).
 * Byte offset of (page, plane, token) = ((page * 2*kv_heads + plane) * page_tokens + token) * row_bytes.
 * page_tokens is a multiple of 32; dim is 128 or 256. */
typedef struct sdx_kv_pool {
    void* pages;
    uint64_t page_count;
    uint32_t page_tokens;
    uint32_t kv_heads;
    uint32_t dim;
    uint32_t row_bytes;
} sdx_kv_pool;

/* Append K/V rows (reference write_attention_kv + kv_encode, gpu/kernels.cpp:58-98): row r of sequence s goes to
 * position positions[s] + r through page_table[s * table_stride + position / page_tokens].  keys/values are
 * [seqs][span][kv_heads][dim], FP32 (input_f16 = 0) or FP16 (1).  Q8_0 encoding is bit-exact kv_encode. */
int sdx_kv_write(void* handle, const sdx_kv_pool* pool, const int32_t* page_table, uint64_t table_stride, const int32_t* positions,
                 const void* keys, const void* values, int input_f16, uint64_t seqs, uint64_t span);

/* A paged K/V cache kept by the library: the pool and the sequences' page tables, both in device memory, in the layout the
 * entry points above and below take.  It stands where the reference has its K/V residency code (gpu/kv_stage.hpp:1-184: the mirror
 * ring, the prefix stage, kv_layout / kv_prefetch) and sd_kv_grow (gpu/straydog_gpu.h:105-109): with the rows resident in HBM
 * what is left of that is which pages a sequence owns.  Table changes are uploaded in stream order; no call waits for the device.
 *   create    a pool of `pages` pages and a table for `sequences` sequences of up to max_context tokens (null on failure)
 *   view      the pool struct, the device table and its stride, for sdx_kv_write / sdx_paged_attention / sdx_selected_attention
 *   reserve   the sequence holds pages for `tokens` positions afterwards (growth without copies; "out of pages" changes nothing)
 *   truncate  pages past `tokens` positions are given back (a rejected speculation, a rewind; 0 releases the sequence)
 *   fork      sequence `to` (empty) starts as the first `tokens` positions of `from`: whole pages are shared by reference count,
 *             the last, partial page is copied, so either sequence may append from position `tokens` on
 *   usage     pages the sequence holds, pages free
 * Destroy a cache before its device. */
void* sdx_kv_cache_create(void* handle, uint64_t pages, uint32_t page_tokens, uint32_t kv_heads, uint32_t dim, uint32_t row_bytes,
                          uint64_t sequences, uint64_t max_context);
int sdx_kv_cache_destroy(void* handle, void* cache);
int sdx_kv_cache_view(void* handle, void* cache, sdx_kv_pool* pool, const int32_t** page_table, uint64_t* table_stride);
int sdx_kv_cache_reserve(void* handle, void* cache, uint64_t sequence, uint64_t tokens);
int sdx_kv_cache_truncate(void* handle, void* cache, uint64_t sequence, uint64_t tokens);
int sdx_kv_cache_fork(void* handle, void* cache, uint64_t from, uint64_t to, uint64_t tokens);
int sdx_kv_cache_usage(void* handle, void* cache, uint64_t sequence, uint64_t* pages_held, uint64_t* pages_free);

/* Rows that are not in HBM (the reference's host-resident K/V: gpu/kv_stage.hpp:4-184, sd_kv_stage gpu/kernels.cpp:4277-4290,
 * sd_kv_grow :4048-4140), on the paged cache.  Pages move on a stream of their own behind the compute stream's queued work; the
 * compute stream waits for them at its next call that touches K/V pages, not before (the prefetch between two layers).
 *   host      gives the cache a tier of `host_pages` pages in page-locked host memory the library allocates (once)
 *   park      the sequence's pages are copied to host pages and its HBM pages freed at once; it keeps its rows but can only be
 *             staged, truncated or resumed
 *   resume    a parked sequence takes HBM pages again and its rows are copied back ("out of pages" changes nothing)
 *   stage     the first `tokens` positions of a parked sequence in the VRAM stage registered with sd_kv_stage: only the pages
 *             the stage does not hold of it yet are copied; pool / page_table / table_stride are the view to attend through
 *             (one sequence: row 0 of the table)
 *   unstage   rows [first, first + count) that were written through the staged view go back to the sequence's host pages
 *             (taking host pages as it grows)
 *   grow      the pool becomes `pages` pages: a new allocation, the old pages copied on the device, the old one released (VRAM
 *             for both during the copy); a view taken before is stale, recorded graphs are dropped.  A device without room
 *             answers "not enough VRAM for the K/V of this sequence" and changes nothing
 *   residency whether the sequence is parked, host pages free, pages of the sequence the stage holds */
int sdx_kv_cache_host(void* handle, void* cache, uint64_t host_pages);
int sdx_kv_cache_park(void* handle, void* cache, uint64_t sequence);
int sdx_kv_cache_resume(void* handle, void* cache, uint64_t sequence);
int sdx_kv_cache_stage(void* handle, void* cache, uint64_t sequence, uint64_t tokens, sdx_kv_pool* pool, const int32_t** page_table,
                       uint64_t* table_stride);
int sdx_kv_cache_unstage(void* handle, void* cache, uint64_t sequence, uint64_t first, uint64_t count);
int sdx_kv_cache_grow(void* handle, void* cache, uint64_t pages);
int sdx_kv_cache_residency(void* handle, void* cache, uint64_t sequence, uint64_t* parked, uint64_t* host_pages_free, uint64_t* staged_pages);
/* The union gather for a sparse (selection-list) pass over a sequence whose rows are not in HBM -- the reference's qsa_mark_selection,
 * qsa_place_union, qsa_gather_union and qsa_renumber_selection as qsa_attention_gathered drives them (gpu/sparse_attention_compute.hpp:
 * 677-733, gpu/prefill_batch.hpp:224-254, kv_union_count gpu/kv_stage.hpp:166-172).  The blocks of four positions that the selections
 * of query rows first .. first + rows - 1 name (entries that count by sdx_selected_attention's rule, row r at position base + r) are
 * copied once, in block order, from the sequence's pages -- the host tier of a parked sequence, read over the bus, or the pool -- into
 * the VRAM stage registered with sd_kv_stage, and the lists are renumbered to the places there (renumbered: [.][selected] floats at
 * the same rows; an entry that does not count becomes -1): a row then attends the same keys and values in the same order, the same
 * bits, through pool / page_table / table_stride (the stage in the pool's page layout) with the same context, positions and counts:
 *     sdx_selected_attention(handle, pool, page_table, context, base + first, NULL, renumbered + first * selected, selected,
 *                            counts + first, q of row first, ..., *taken rows, ...)
 * *taken: how many of the rows the stage holds the union of -- the rows are halved until their union fits (0: the stage is too small
 * for a single row's selection; nothing was gathered); the caller attends those and calls again from first + *taken.  *union_rows
 * (may be null): the positions gathered.  The union's size is read back from the device at each attempt (the call waits for the
 * stream, as the reference's does), so it cannot be recorded into a graph; what the stage held before is forgotten. */
int sdx_kv_cache_gather(void* handle, void* cache, uint64_t sequence, uint64_t context, uint64_t base, const float* indices, uint64_t selected,
                        const float* counts, uint64_t first, uint64_t rows, float* renumbered, uint64_t* taken, uint64_t* union_rows, sdx_kv_pool* pool,
                        const int32_t** page_table, uint64_t* table_stride);

/* Causal grouped-query attention over the paged cache: the attention step of a decode (span 1), a speculative
 * verify (span <= 8) or a prefill chunk (any span), i.e. qsa_decode_parts/qsa_decode_merge, qsa_flash and
 * qsa_prompt_attention of the reference (gpu/sparse_attention_compute.hpp:41-170, :176-279,
 * gpu/qsa_prompt_attention.hpp:47-213) with the dense selection 0..position.  Row r of sequence s attends
 * positions t <= positions[s] + r.  q/out are [seqs][span][heads][dim], FP32 or FP16 each; softmax and sums in
 * FP32; K/V and probabilities enter the matrix cores as FP16.  max_context bounds positions[s] + span (it sizes the
 * launch; positions themselves stay on the device).  scratch holds the split partial results:
 * sdx_paged_attention_scratch bytes. */
uint64_t sdx_paged_attention_scratch(uint64_t seqs, uint64_t span, uint64_t heads, uint64_t dim, uint64_t max_context);
int sdx_paged_attention(void* handle, const sdx_kv_pool* pool, const int32_t* page_table, uint64_t table_stride,
                        const int32_t* positions, uint64_t max_context, const void* q, int q_f16, uint64_t seqs, uint64_t span,
                        uint64_t heads, float scale, void* out, int out_f16, void* scratch, uint64_t scratch_bytes);

/* A prompt chunk in one call: the chunk's K/V rows appended to the cache and its queries attended -- the K/V write and the
 * attention stage of the reference's prompt passes (write_attention_kv gpu/kernels.cpp:79-98, then qsa_prompt_attention
 * gpu/qsa_prompt_attention.hpp:47-213, 220-234, inside sd_prefill_span) with the dense selection 0..position.  The bits of
 * sdx_kv_write followed by sdx_paged_attention on the same arguments (cache bytes and outputs; 128 columns, Q8_0 or FP16 rows),
 * in two launches where those take three, and without unpacking the prompt's earlier rows again at every chunk: the FP16 operand
 * tiles of the cached rows, which sdx_paged_attention rebuilds in the handle's workspace on every call, live in `tiles`, device
 * memory of sdx_prefill_tiles_bytes(seqs, kv_heads, 128, max_context) bytes that the caller keeps between the chunks of a prompt.
 *   keys/values  [seqs][span][kv_heads][dim] FP32 (kv_f16 = 0) or FP16 (1), rows for positions[s] .. positions[s] + span - 1; both
 *                null when the rows are in the cache already (the call then only attends)
 *   valid        device, int32 [seqs], or null: the leading positions of each sequence whose tiles `tiles` still holds from earlier
 *                calls on the same cache rows (in a chunked prefill: positions itself -- everything before this chunk); null or 0
 *                rebuilds every tile.  A position above positions[s] counts as positions[s].
 * Rows at positions >= max_context are neither stored nor attended. */
uint64_t sdx_prefill_tiles_bytes(uint64_t seqs, uint64_t kv_heads, uint64_t dim, uint64_t max_context);
/* Which of the two prompt kernels takes spans at 128 columns on this handle from now on: waves of 64 query rows, one a SIMD, the
 * queries and output accumulators in the accumulation registers (the default), or waves of 32 rows, two a SIMD.  Same rows a
 * workgroup, same tiles, same grid; only agreement to rounding is promised, though the bits have been the same in every case tried
 * (the 32 rows that raise their reference maxima together are the same in both).  No counterpart in the reference: a tuning switch, kept so that either kernel can be measured
 * and tested beside the other.  Anything but 32 or 64 is refused. */
int sdx_prefill_wave_rows(void* handle, uint64_t rows);
int sdx_prefill_chunk(void* handle, const sdx_kv_pool* pool, const int32_t* page_table, uint64_t table_stride, const int32_t* positions,
                      uint64_t max_context, const void* keys, const void* values, int kv_f16, const void* q, int q_f16, uint64_t seqs,
                      uint64_t span, uint64_t heads, float scale, void* out, int out_f16, void* tiles, uint64_t tiles_bytes,
                      const int32_t* valid);

/* The same attention for callers that cannot allocate device memory or pass a scratch buffer: code under graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.  The split partial results live in
 * an area of sdx_paged_attention_static_bytes() bytes (16 MiB) that the library itself holds on every GPU it runs on until the
 * process ends; a batch that would need more (sdx_paged_attention_scratch says how much a shape can need at most; the call
 * computes the exact figure) and spans with more query rows per K/V head than the decode kernel takes (64 at 128 columns, 32 at
 * 256) are refused with an error.  The call allocates nothing.  All calls on one GPU share that area: calls that overlap in
 * time on one GPU (two handles, two streams) race; calls queued on one handle's stream do not.  Same results, bit for bit, as
 * sdx_paged_attention. */
uint64_t sdx_paged_attention_static_bytes(void);
int sdx_paged_attention_static(void* handle, const sdx_kv_pool* pool, const int32_t* page_table, uint64_t table_stride,
                               const int32_t* positions, uint64_t max_context, const void* q, int q_f16, uint64_t seqs, uint64_t span,
                               uint64_t heads, float scale, void* out, int out_f16);

/* Qwen's block indexer (the reference runs it inside sd_qsa_sequence / sd_decode_span / sd_prefill_span; here its stages are
 * callable on their own).  All buffers are device memory of the handle.
 *
 * sdx_qsa_normalize = qsa_normalize (gpu/sparse_attention.hpp:8-23, rope :2-6): rows x heads vectors of `width` (128 or 256)
 * floats, `stride` floats apart, RMS-normalised with the weight `norm` and turned for position + row; target [rows*heads][width]
 * (may be the source when stride == width). */
int sdx_qsa_normalize(void* handle, const float* source, const float* norm, uint64_t rows, uint64_t heads, uint64_t width, uint64_t stride,
                      uint64_t position, float* target);
/* sdx_qsa_pool = qsa_pool + qsa_save_history (gpu/sparse_attention.hpp:87-108, 132-139; call site :497-501): the blocks of four
 * positions completed by rows base .. base + steps are pooled from `incoming` [steps][128] and the ring `history` [16][128] into
 * blocks[column * pool + block]; the ring then takes the span's last four rows. */
int sdx_qsa_pool(void* handle, const float* incoming, float* history, const float* norm, uint64_t pool, uint64_t base, uint64_t steps,
                 float* blocks);
/* sdx_qsa_index = qsa_index_exact (gpu/sparse_attention.hpp:403-414: qsa_block_scores :141-155 / qsa_block_scores_tiled
 * :247-298, then qsa_select :172-241 / qsa_select_rows :314-400) for rows at positions base .. base + steps - 1.
 * queries: [steps][query_stride], the 4 x 128 normalised index queries at each row's start; blocks: [128][pool] pooled keys;
 * scores: steps x pool floats of scratch (holds the scores of rows with more than 512 complete blocks afterwards);
 * indices: [steps][selected] positions as floats, counts: [steps] as floats -- the two tails of the reference's packed
 * buffer (gpu/sparse_attention.hpp:177-178, 240).  dynamic_base, if not null, is a device-resident position that replaces
 * `base` (the decode and verification passes' replayable form, gpu/qsa_decode.hpp:36-38, 125-127; up to 8 rows).
 * The same bits as the reference's kernels: scores by fused chains in column order, ties to the earliest blocks. */
int sdx_qsa_index(void* handle, const float* queries, uint64_t query_stride, const float* blocks, uint64_t pool, uint64_t base,
                  const uint32_t* dynamic_base, uint64_t steps, uint64_t selected, float* scores, float* indices, float* counts);

/* sdx_qsa_index_interval = the reference's selection by intervals for prompt chunks (gpu/qsa_interval.hpp:1-36 the bound, :601-626
 * qsa_iv_chunk): the same indices and counts as sdx_qsa_index, block for block, from FP16 matrix products with a proven error
 * bound; only the blocks whose bound straddles the 512th best score are scored exactly.  A row the scheme cannot decide (its
 * guessed threshold too high, too many blocks near the 512th, an input beyond FP16 or not a number) is decided by sdx_qsa_index's
 * kernels in the same call: more time, never a different result.  Spans below position 32768 go to sdx_qsa_index as they are.
 * scores: steps x pool floats of scratch (afterwards: matrix-unit scores at the kept blocks, exact ones for undecided rows).
 * scratch: sdx_qsa_index_interval_scratch(steps, pool) bytes.  valid (host, may be null): in, the number of blocks whose packed
 * operands `scratch` still holds from the previous call on the same keys (0 when the keys' earlier blocks changed or the scratch
 * was used otherwise); out, this call's.  No device-resident position: the scheme serves chunks, not recorded decode steps. */
uint64_t sdx_qsa_index_interval_scratch(uint64_t steps, uint64_t pool);
int sdx_qsa_index_interval(void* handle, const float* queries, uint64_t query_stride, const float* blocks, uint64_t pool, uint64_t base, uint64_t steps,
                           uint64_t selected, float* scores, float* indices, float* counts, void* scratch, uint64_t scratch_bytes, uint64_t* valid);
/* For harnesses: how many rows the last sdx_qsa_index_interval on this scratch (same steps and pool) left to the exact kernels
 * (waits for the device). */
int sdx_qsa_index_interval_undecided(void* handle, const void* scratch, uint64_t steps, uint64_t pool, uint64_t* rows);

/* The attention stage of a Qwen decode or verification pass in one call: the reference's qsa_decode_attend / qsa_decode_attend_rows
 * (gpu/qsa_decode.hpp:28-44, 113-129; kernel qsa_normalize_rows :86-111).  For rows r < steps (1..8) at the consecutive positions
 * positions[r] with rope positions ropes[r], both device-resident (a recorded pass replays at the next position):
 *   projections + r * stride holds the row's [heads x (query 256 | gate 256) | kv_heads x key 256 | kv_heads x value 256 |
 *   4 x index query 128 | index key 128];
 *   1. one launch: queries, keys and index queries RMS-normalised and turned (sdx_qsa_normalize's arithmetic; index queries in
 *      place), the keys and values appended to the K/V rows at the positions (sdx_kv_write's bytes), the index keys pooled into
 *      blocks / history row by row (sdx_qsa_pool's arithmetic);
 *   2. sdx_qsa_index on the normalised index queries;  3. sdx_selected_attention over each row's selection with the gate.
 * attended: [steps][heads][256] FP32.  scratch: sdx_qsa_decode_attend_scratch bytes (normalised queries, scores, selections,
 * attention partials). */
typedef struct sdx_qsa_state {
    const sdx_kv_pool* kv;          /* rows of 256 columns, Q8_0 or FP16 */
    const int32_t* page_table;      /* the sequence's pages, or null when one page holds the context (the reference's state layout) */
    uint64_t context;
    float* blocks;                  /* [128][context / 4 + 1] pooled index keys */
    float* history;                 /* [16][128] the index keys' ring */
    const float* q_norm;            /* 256 */
    const float* k_norm;            /* 256 */
    const float* index_q_norm;      /* 128 */
    const float* index_k_norm;      /* 128 */
    uint64_t heads;                 /* query heads, a multiple of the K/V heads, at most 16 each */
} sdx_qsa_state;
uint64_t sdx_qsa_decode_attend_scratch(uint64_t steps, uint64_t heads, uint64_t kv_heads, uint64_t context);
int sdx_qsa_decode_attend(void* handle, const sdx_qsa_state* state, float* projections, uint64_t stride, uint64_t steps, const uint32_t* positions,
                          const uint32_t* ropes, void* scratch, uint64_t scratch_bytes, float* attended);

/* The attention stage of a prompt chunk in one call: the stage of the reference's qsa_prefill for a span of rows at the consecutive
 * positions base .. base + steps - 1 (gpu/sparse_attention.hpp:444-506: qsa_normalize, the K/V write, qsa_pool + qsa_save_history
 * :497-501, the selection -- qsa_iv_chunk gpu/qsa_interval.hpp:601-626 past 32768 positions, qsa_index_exact before --, the
 * attention over each row's selection gpu/qsa_prompt_attention.hpp:220-234 and qsa_gate).  projections as for sdx_qsa_decode_attend
 * (index queries normalised in place); rope positions are the positions.  The values of the separate entry points, bit for bit:
 * sdx_qsa_normalize on queries, keys and index queries, sdx_kv_write, sdx_qsa_pool over the span, sdx_qsa_index_interval,
 * sdx_selected_attention with the gate.  attended: [steps][heads][256] FP32.  scratch: sdx_qsa_prefill_attend_scratch bytes on a
 * 256-byte boundary; its tail holds the interval scheme's packed keys, which are carried from chunk to chunk when the caller passes
 * the same scratch and the `valid` its last call left (host, in and out, may be null; 0 after the pooled keys' earlier blocks
 * changed), as for sdx_qsa_index_interval. */
uint64_t sdx_qsa_prefill_attend_scratch(uint64_t steps, uint64_t heads, uint64_t kv_heads, uint64_t context);
int sdx_qsa_prefill_attend(void* handle, const sdx_qsa_state* state, float* projections, uint64_t stride, uint64_t steps, uint64_t base, void* scratch,
                           uint64_t scratch_bytes, uint64_t* valid, float* attended);

/* Selection-list attention over K/V rows of 256 columns (Q8_0 or FP16): the reference's qsa_attention / qsa_attention_rows
 * (gpu/sparse_attention_compute.hpp:609-647: qsa_decode_parts :41-135 + qsa_decode_merge :139-170) followed by qsa_gate
 * (gpu/sparse_attention.hpp:439-442).  Row r, at position base + r (or *dynamic_base + r, a device-resident position),
 * attends the positions its list names: indices [rows][selected] and counts [rows], both floats, as sdx_qsa_index and the
 * reference's packed buffer hold them; an entry counts iff 0 <= raw <= position and raw < context (gpu/kernels.cpp:100-165).
 * The rows come from `pool` through page_table ([ceil(context / page_tokens)] pages of the one sequence) or, with a null
 * page_table, from a pool whose single page holds the context (which is the reference's state layout, planes x context).
 * q and out are [rows][heads][256], FP32 or FP16 each; gate (optional) is read at gate[r * gate_row_stride + h * gate_stride + c]
 * (gate_row_stride 0: heads * gate_stride) and out *= sigmoid(gate).  heads / kv_heads <= 16.  scratch: sdx_selected_attention_scratch(rows, kv_heads, selected) bytes. */
uint64_t sdx_selected_attention_scratch(uint64_t rows, uint64_t kv_heads, uint64_t selected);
int sdx_selected_attention(void* handle, const sdx_kv_pool* pool, const int32_t* page_table, uint64_t context, uint64_t base,
                           const uint32_t* dynamic_base, const float* indices, uint64_t selected, const float* counts, const void* q, int q_f16,
                           uint64_t rows, uint64_t heads, float scale, const float* gate, uint64_t gate_stride, uint64_t gate_row_stride, void* out, int out_f16,
                           void* scratch, uint64_t scratch_bytes);
/* The same attention for the rows of a prompt chunk as a union walk (the reference's qsa_flash_wmma over qsa_mark_blocks /
 * qsa_union_blocks, gpu/sparse_attention_compute.hpp:744-755, 841-896, 906-1041): the tokens whose query rows share a tile of 64
 * rows walk the union of their selections once, a K/V row converted once for all of them, a bit per (entry, token) masking what a
 * token did not select (2 to 16 heads a K/V head).  It pays when consecutive tokens select mostly the same positions, as the rows of a real prompt do; on
 * selections that do not overlap it gains nothing over sdx_selected_attention.  Same arguments (no device-resident position),
 * same rule for entries that count; an entry a row names twice counts once; a row with no entry that counts gives zeros.
 * scratch: sdx_selected_attention_union_scratch(rows, heads, kv_heads, selected, context) bytes (a word per position and tile). */
uint64_t sdx_selected_attention_union_scratch(uint64_t rows, uint64_t heads, uint64_t kv_heads, uint64_t selected, uint64_t context);
int sdx_selected_attention_union(void* handle, const sdx_kv_pool* pool, const int32_t* page_table, uint64_t context, uint64_t base,
                                 const float* indices, uint64_t selected, const float* counts, const void* q, int q_f16, uint64_t rows, uint64_t heads,
                                 float scale, const float* gate, uint64_t gate_stride, uint64_t gate_row_stride, void* out, int out_f16, void* scratch,
                                 uint64_t scratch_bytes);

/* Top-k indexed sparse attention over BF16 latent K/V for a batch of sequences (one decode row each):
 * stage 1+2 = sd_op_index_scores + sd_op_top_k per sequence (gpu/ops.hpp:1700-1739, 1766-1941) with each sequence's own
 * keys [batch][groups][dim] BF16; q_index [batch][heads][dim] BF16; weights [batch][heads] FP32; visible [batch].
 * scores (optional, [batch][groups] FP32) receives the canonical scores; indices [batch][k] int32, ascending,
 * ties to the lowest index, -1 padding: bit-exact. */
int sdx_index_top_k(void* handle, const void* q_index, const void* keys, const float* weights, const int32_t* visible, uint64_t batch,
                    uint64_t groups, uint64_t heads, uint64_t dim, float scale, float* scores, uint64_t k, int32_t* indices);
/* The projection inside sd_op_index_select_proj on its own (the reference forms it with sd_op_linear, its GEMV stack, whose
 * summation order follows a per-device lane count: gpu/gemv_common.hpp:785-812): weights[h] = row h of proj_weights . x for
 * heads <= 64 rows of proj_cols <= 8192 columns, BF16 (kind 30, 16-byte aligned rows, cols a multiple of 8) or ggml Q8_0 (kind 8,
 * cols a multiple of 32).  The order of the sums is fixed: a unit (8 BF16 columns or a Q8_0 block) is one chain of fused
 * multiply-adds over its columns from zero (Q8_0: over float(q) * x, then times the block's scale); unit u belongs to lane
 * u % 64, which adds its units in order; the 64 lane sums are added pairwise at distances 32, 16, 8, 4, 2, 1. */
int sdx_index_projection(void* handle, const void* proj_weights, int proj_kind, uint64_t proj_cols, const float* x, uint64_t heads, float* weights);
/* The bracket the matrix cores put around every canonical score of stage 1 (dim 128, heads a multiple of 16 up to 64):
 * lower[b][g] <= score <= upper[b][g], -inf for groups that are not visible.  sdx_index_top_k without a scores buffer
 * scores canonically only the groups whose upper bound reaches the k-th highest lower bound (the approach of the
 * reference's interval indexer, gpu/qsa_interval.hpp:152-419); this entry exposes the brackets for inspection. */
int sdx_index_score_bounds(void* handle, const void* q_index, const void* keys, const float* weights, const int32_t* visible, uint64_t batch,
                           uint64_t groups, uint64_t heads, uint64_t dim, float scale, float* lower, float* upper);
/* stage 3 = op_sparse_attention_kernel's arithmetic (gpu/ops.hpp:1240-1297) without window or sink, keys = the
 * selected rows' kdim columns, values = their first vdim columns: q [batch][heads][kdim] BF16, latents
 * [batch][groups][kdim] BF16, selected [batch][k] (-1 skipped), out [batch][heads][vdim] FP32. */
int sdx_latent_attention(void* handle, const void* q, const void* latents, const int32_t* selected, uint64_t batch, uint64_t groups,
                         uint64_t k, uint64_t heads, uint64_t kdim, uint64_t vdim, float scale, float* out);

/* Harness helpers: wait for the handle's stream; events on that stream (ids >= 2) and the time between two;
 * counter-based N(0,1) / U[lo,hi) fills for synthetic benchmark inputs; a plain copy kernel for measuring the
 * HBM ceiling and calibrating byte counters. */
int sdx_synchronize(void* handle);
int64_t sdx_event_record(void* handle);
int sdx_event_elapsed(void* handle, int64_t begin, int64_t end, float* milliseconds);
int sdx_events_clear(void* handle);
int sdx_device_compute_units(void* handle);
/* For harnesses that check what a call allocates: values[0..3] = the device's free and total memory as the driver reports them
 * (hipMemGetInfo), the bytes of the handle's workspace, and the number of timing events sdx_profile has recorded. */
int sdx_device_state(void* handle, uint64_t* values);
/* Kernel timing for benchmarks: while enabled, each op launches its dominant kernel through the extended launch, whose two
 * events take the kernel's own start and end on the handle's stream; sdx_profile_read waits for the stream and returns the
 * summed kernel time and the launch count.  sdx_profile(handle, 0|1) clears what was recorded.  Launches recorded into a graph
 * (sd_graph_begin .. sd_graph_end) are not timed. */
int sdx_profile(void* handle, int enable);
int sdx_profile_read(void* handle, double* milliseconds, uint64_t* launches);
/* Seeded N(0,1) values from the generator family of the reference's tests (crates/straydog-engine/tests/fused_gpu.rs:39-53,
 * gpu/tests/qsa_interval_test.cpp:12-18): one xorshift64 stream from `seed` (0: 0x9e3779b97f4a7c15), two draws a Box-Muller
 * pair in double precision, uniforms ((x >> 11) + 0.5) / 2^53, cosine and sine both kept, value i of the stream at out[i].  The
 * same family, not those tests' values: their seeding and their uniforms differ, so no fixture of the reference is reproduced.
 * The threads reach their stretches of the stream by jumping (the generator is linear). */
int sdx_fill_normal(void* handle, void* out, uint64_t count, uint64_t seed, int out_kind /* 0 f32, 1 f16, 2 bf16 */);
int sdx_fill_uniform(void* handle, float* out, uint64_t count, uint64_t seed, float lo, float hi);
int sdx_copy(void* handle, void* target, const void* source, uint64_t bytes);
/* Frees a buffer of sd_checkpoint_buffer before the handle is destroyed (the reference keeps them for the handle's life). */
int sdx_checkpoint_release(void* handle, void* buffer);
/* Read-only streaming probe (16-byte loads, `unroll` per lane per trip, `blocks_per_cu` workgroups per compute unit). */
int sdx_read_probe(void* handle, const void* source, uint64_t bytes, uint32_t blocks_per_cu, uint32_t unroll);
/* The decode kernel's way through a pool with the arithmetic left out (no counterpart in the reference: a harness probe): every
 * K and V plane of every page read once in the decode kernel's order -- a workgroup of four waves per K/V head of a run of pages,
 * the waves taking alternate 32-token steps, a step's two slabs by 1 KiB global->LDS loads.  *bytes receives what the launch reads;
 * time it with the events above: what the pool's layout and that order of asking give by themselves. */
int sdx_paged_stream_probe(void* handle, const sdx_kv_pool* pool, uint64_t* bytes);
/* Matrix-core probe: eight waves per compute unit, each `trips` x 32 independent v_mfma_f32_16x16x32_f16; *flops receives the
 * floating-point operations the launch performs (time it with the events above).  live = 0: tame constant operands, the
 * rate at the clock the box holds for them; live = 1: pseudo-random operands that change from product to product, as real
 * data does -- the matrix cores then draw more and the clock (and the rate) settles lower. */
int sdx_mfma_probe(void* handle, uint32_t trips, int live, double* flops);

#ifdef __cplusplus
}
#endif
#endif
