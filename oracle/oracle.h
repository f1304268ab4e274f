/* CPU oracle for the Straydog attention path.  TEST INFRASTRUCTURE ONLY.
 *
 * This is a from-scratch CPU restatement of the reference's attention arithmetic, used as the
 * checker by tests/, by __graft_entry__.smoke() and by the cpu_baseline leg of bench.py.  The
 * product (straydog_amd/ and its HIP library) never links, imports or calls anything in here.
 *
 * Every function names the reference file:line whose arithmetic it restates (paths are relative
 * to the reference checkout).  What pins each function independently of this file (golden
 * vectors held by the reference's own tests, numpy/float64 closed forms, brute force) is listed
 * in tests/test_oracle_*.py; a function without such a pin is marked PARITY UNPINNED here.
 *
 * Pinned: sdo_f32_to_f16 / sdo_f16_to_f32 (numpy float16, exhaustive), sdo_f32_to_bf16 (formula of
 * ds_state_bf16_gpu.rs:27-33 + its special values), sdo_kv_q8_row / sdo_kv_q8_values (invariants of
 * gpu.rs:4096-4142 + independent numpy restatement), sdo_ggml_q8_0_* (six real GGUF blocks of
 * tests/golden/format_blocks.json), sdo_q8_paged_attention / sdo_attention_sequence /
 * sdo_op_attention (float64 numpy softmax + the derived bound of attention_gpu.rs:28-31),
 * sdo_index_scores (float64 closed form + scalar-vs-vector bit equality), sdo_top_k (brute-force
 * stable sort + the adversarial generator of fused_gpu.rs:370-379), sdo_latent_attention (float64
 * closed form + special cases), sdo_compress (float64 closed form), sdo_qsa_select (brute force),
 * sdo_qsa_block_scores (exact rational arithmetic rounded once per fused step, in pure Python, + float64 closed form),
 * sdo_qsa_normalize / sdo_qsa_pool (float64 closed form; rotation invariants: pair norms kept, position 0 and columns
 * from 64 on unturned; the ring's contents), sdo_rms_norm / sdo_rope_halves / sdo_attention_prepare (float64 closed forms; a
 * rotation keeps pair norms; the fused step equals its parts), sdo_dspark_attention (the known answers of the reference's test,
 * dspark_attention_gpu.rs:101-124, + float64 numpy).
 * PARITY UNPINNED: none of the above; bit-level agreement with the reference's device summation
 * order inside its flash kernels is not claimed anywhere (tolerance-based, see the tests).
 */
#ifndef STRAYDOG_ORACLE_H
#define STRAYDOG_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- scalar conversions: crates/straydog-engine/src/formats.rs:59-102, gpu/token_mixing.hpp:728-735 ---- */
float sdo_f16_to_f32(uint16_t half);
uint16_t sdo_f32_to_f16(float value);            /* round to nearest even; >= 65520 -> inf; subnormals kept */
uint16_t sdo_f32_to_bf16(float value);           /* round to nearest even; a NaN stays a (quiet) NaN */
float sdo_bf16_to_f32(uint16_t half);
void sdo_to_bf16(const float* x, size_t count, uint16_t* out);

/* ---- Q8_0 K/V row: gpu/kernels.cpp:58-74 (kv_encode, kv_put), :38-44 (kv_load);
 *      crates/straydog-engine/src/gpu.rs:536-561 (kv_q8_row, kv_q8_values).
 * A row is one head's `dim` values of one position: dim int8, then dim/32 FP16 scales (LE).  dim % 32 == 0. */
size_t sdo_kv_q8_row_bytes(size_t dim);
void sdo_kv_q8_row(const float* values, size_t dim, uint8_t* row);
void sdo_kv_q8_values(const uint8_t* row, size_t dim, float* values);
/* The FP16 row (kv_row_f16): dim halves. */
void sdo_kv_f16_row(const float* values, size_t dim, uint8_t* row);
void sdo_kv_f16_values(const uint8_t* row, size_t dim, float* values);

/* ---- ggml block_q8_0 {f16 d; int8 qs[32]}: crates/straydog-engine/src/formats.rs:104-116, 232-236 ---- */
void sdo_ggml_q8_0_quantize(const float* values, size_t count, uint8_t* blocks);
void sdo_ggml_q8_0_dequantize(const uint8_t* blocks, size_t count, float* out);

/* ---- Append K/V rows to a paged pool: gpu/kernels.cpp:79-98 (write_attention_kv) generalised to pages.
 * Pool layout: byte offset of (page p, plane pi, token i) = ((p * 2*kv_heads + pi) * page_tokens + i) * row_bytes;
 * plane pi = kv head h for keys, kv_heads + h for values (the reference's "each K/V head's keys, then each one's
 * values", gpu/core.hpp:397-403, with `context` = page_tokens inside a page).  row_bytes selects Q8_0
 * (dim + dim/16) or FP16 (2*dim).
 * keys/values: [seqs][span][kv_heads][dim] fp32; row r of sequence s lands at position positions[s] + r. */
void sdo_kv_write(uint8_t* pool, size_t row_bytes, size_t page_tokens, size_t kv_heads, size_t dim,
                  const int32_t* page_table, size_t table_stride, const int32_t* positions,
                  const float* keys, const float* values, size_t seqs, size_t span);

/* ---- Dense causal GQA over the paged Q8_0/FP16 cache (BASELINE configs 0-3).
 * The arithmetic is gpu/kernels.cpp:100-165 (attention_scores + attention_reduce) with the selection
 * list 0..position: s_t = scale * sum_d K[t][d]*q[d]; two-pass softmax; o = sum_t (p_t / L) V[t].
 * Row r of sequence s attends positions t <= positions[s] + r (causal inside the span, all of the context).
 * q/out: [seqs][span][heads][dim].  out64 (optional): the same in double over the same operands. */
void sdo_paged_attention(const uint8_t* pool, size_t row_bytes, size_t page_tokens, size_t kv_heads, size_t dim,
                         const int32_t* page_table, size_t table_stride, const int32_t* positions,
                         const float* q, size_t seqs, size_t span, size_t heads, float scale,
                         float* out, double* out64, int threads);

/* ---- Selection-list attention over the Qwen state: gpu/kernels.cpp:100-165, :4387-4419.
 * state: planes [2*2][context] rows of row_bytes (272 Q8_0 / 512 FP16); input is the packed float row
 * [steps*24*256 q | steps*2*256 k | steps*2*256 v | steps*selected indices (as floats) | steps counts];
 * the new K/V rows are written at base+step first (write_attention_kv), then 24 heads attend. */
void sdo_attention_sequence(uint8_t* state, size_t row_bytes, size_t context, size_t base, size_t steps,
                            size_t selected, const float* input, float* output);

/* ---- Dense causal GQA over FP32 caches: gpu/token_mixing.hpp:356-520, 652-693 (sd_op_attention);
 *      F64 twin + derived bound: crates/straydog-engine/tests/attention_gpu.rs:50-87.
 * keys/values [context][kv_heads][dim]; length_r = min(positions[r]+1, context); optional sigmoid gate. */
void sdo_op_attention(const float* q, const float* keys, const float* values, size_t context, const int32_t* positions,
                      size_t rows, size_t heads, size_t kv_heads, size_t dim, float scale, const float* gate, float* out);
void sdo_op_attention_f64(const float* q, const float* keys, const float* values, size_t context, const int32_t* positions,
                          size_t rows, size_t heads, size_t kv_heads, size_t dim, float scale, const float* gate,
                          double* out, double* bound);

/* ---- Indexer scores in the canonical order: gpu/ops.hpp:1700-1739 (and :2171-2189).
 * keys_bf16 != 0: keys are uint16 BF16 bits (the reference's tagged pointer), widened exactly. */
void sdo_index_scores(const float* q, const void* keys, int keys_bf16, const float* weights, const int32_t* visible,
                      size_t rows, size_t groups, size_t heads, size_t dim, float scale, float* scores, int threads);
/* The same sum in double without the canonical rounding (crates/straydog-engine/examples/ds41_reference.rs:487-494). */
void sdo_index_scores_f64(const float* q, const void* keys, int keys_bf16, const float* weights, const int32_t* visible,
                          size_t rows, size_t groups, size_t heads, size_t dim, float scale, double* scores);

/* ---- The indexer's projection (sd_op_index_select_proj, gpu/kernels.cpp:5620-5667): weights[h] = matrix row h . x, rows BF16
 *      (kind 30) or ggml Q8_0 blocks (kind 8: FP16 scale then 32 int8, crates/straydog-engine/src/formats.rs:104-116, 232-236).
 *      The reference's GEMV fixes no summation order across devices (gpu/gemv_common.hpp:785-812: `lanes` is tuned per device);
 *      this is the library's stated order for 64 lanes: unit chains from zero, lane u % 64 adds its units in order, lane sums
 *      added pairwise at distances 32 .. 1.  Pinned by a float64 dot product and by the order's own definition on small cases. */
void sdo_index_projection(const uint8_t* matrix, int kind, size_t cols, const float* x, size_t heads, float* weights);

/* ---- Top-k: gpu/ops.hpp:1766-1874 (top_k_key, top_k_row); rule crates/straydog-engine/tests/fused_gpu.rs:326-358. */
uint32_t sdo_top_k_key(float value);
void sdo_top_k(const float* scores, size_t rows, size_t groups, size_t k, int32_t* out);

/* ---- Candidate blocks: gpu/ops.hpp:1942-1975, rule crates/straydog-engine/tests/fused_gpu.rs:504-517. */
void sdo_index_candidates(const float* scores, const int32_t* visible, size_t rows, size_t groups, size_t blocks,
                          size_t block, int32_t* out);

/* ---- Latent sparse attention: gpu/ops.hpp:1240-1297 (op_sparse_attention_kernel), rope :1318-1328,
 *      CPU twin crates/straydog-engine/examples/ds41_reference.rs:385-411, rotate :185-195.
 * Keys: window rows max(0,p-window+1)..p of `raw` (row t % raw_rows; kdim wide), then compressed rows
 * selected[row][*] (-1 skipped).  Values are the first vdim columns of the same rows.  sinks may be NULL
 * (no sink term); window may be 0 (BASELINE config 4: kdim 576, vdim 512).  With rope_dims, q's last
 * rope_dims values are rotated (adjacent pairs, double sincos) on the way in and the output's last
 * rope_dims back (only meaningful when kdim == vdim).  compressed_bf16 != 0: uint16 BF16 rows. */
void sdo_latent_attention(const float* q, const float* raw, size_t raw_rows, const int32_t* positions, size_t window,
                          const void* compressed, int compressed_bf16, const int32_t* selected, size_t selections,
                          const float* sinks, size_t rows, size_t heads, size_t kdim, size_t vdim, float scale,
                          size_t rope_dims, const float* frequencies, float* out, double* out64, int threads);

/* ---- Compression pooling: gpu/ops.hpp:1681-1694; twin ds41_reference.rs:440-452. */
void sdo_compress(const float* kv, const float* gate, size_t groups, size_t ratio, size_t dim, float* out);

/* ---- Qwen block selection: gpu/sparse_attention.hpp:172-241 (qsa_select).
 * scores: [pool] non-negative block scores of one token at `position`; writes up to `selected` (2052) indices
 * as floats and returns the count. */
size_t sdo_qsa_select(const float* scores, size_t position, size_t keep_blocks, float* indices);

/* ---- Qwen block indexer inputs and scores: gpu/sparse_attention.hpp:2-23 (qsa_rope, qsa_normalize), :87-108 + :132-139
 * (qsa_pool, qsa_save_history), :141-155 (qsa_block_scores).  blocks: [128][pool] column-major pooled keys; history: the ring
 * of the last sixteen index-key inputs [16][128], updated by sdo_qsa_pool; scores: [steps][pool], written for rows with more
 * than 512 complete blocks, blocks below the row's complete count. */
void sdo_qsa_normalize(const float* source, const float* norm, size_t rows, size_t heads, size_t width, size_t stride,
                       size_t position, float* target);
void sdo_qsa_pool(const float* incoming, float* history, const float* norm, size_t pool, size_t base, size_t steps, float* blocks);
void sdo_qsa_block_scores(const float* queries, size_t query_stride, const float* blocks, size_t pool, size_t base, size_t steps,
                          float* scores);

/* ---- The inputs of a dense attention step: gpu/ops.hpp:28-59 (rms norm, halving-tree sum of squares), gpu/token_mixing.hpp:254-274
 * (rope of halves, double angles), :276-338 (the fused step: split, norm, rope, scatter into the caches). */
void sdo_rms_norm(const float* input, const float* weight, size_t rows, size_t width, float eps, float* output);
void sdo_rope_halves(float* x, size_t rows, size_t vectors, size_t width, size_t rope_dims, const int32_t* positions,
                     const float* frequencies);
void sdo_attention_prepare(const float* q_full, float* k, const float* v, size_t rows, size_t heads, size_t kv_heads, size_t dim,
                           const float* q_weight, const float* k_weight, float eps, size_t rope_dims, const int32_t* positions,
                           const float* frequencies, float* q, float* gate, float* keys, float* values, size_t context);

/* ---- DSpark's noncausal block attention in double: gpu/dspark_attention.hpp:1-101; the statement of
 * crates/straydog-engine/tests/dspark_attention_gpu.rs:26-40.  q/out [slots][heads][512], ring [128][512], block [slots][512]. */
void sdo_dspark_attention(const float* q, const float* ring, const float* block, const float* sinks, size_t heads, size_t slots,
                          size_t anchor, size_t history, double* out);

/* ---- Seeded inputs: xorshift64 (crates/straydog-engine/tests/fused_gpu.rs:39-53) -> Box-Muller
 *      (gpu/tests/qsa_interval_test.cpp:12-18). */
void sdo_fill_normal(uint64_t seed, float* out, size_t count);
void sdo_fill_uniform(uint64_t seed, float* out, size_t count, float lo, float hi);

int sdo_max_threads(void);

#ifdef __cplusplus
}
#endif
#endif
