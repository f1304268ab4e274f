/* CPU oracle for the Straydog attention path: TEST INFRASTRUCTURE ONLY (see oracle.h).
 * Plain C11, fp32 arithmetic exactly as written (build with -ffp-contract=off; fused multiply-adds
 * appear only where the reference spells fmaf).  OpenMP is used only to spread independent rows. */
#include "oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

static inline uint32_t bits_of(float v) { uint32_t b; memcpy(&b, &v, 4); return b; }
static inline float float_of(uint32_t b) { float v; memcpy(&v, &b, 4); return v; }

int sdo_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ------------------------------------------------------------------ conversions */

/* formats.rs:59-79 */
float sdo_f16_to_f32(uint16_t half) {
    const uint32_t sign = (uint32_t)(half >> 15) << 31;
    uint32_t exponent = (half >> 10) & 0x1f, mantissa = half & 0x3ff;
    if (exponent == 0) {
        if (mantissa == 0) return float_of(sign);
        exponent = 127 - 15 + 1;
        while (!(mantissa & 0x400)) { mantissa <<= 1; --exponent; }
        return float_of(sign | (exponent << 23) | ((mantissa & 0x3ff) << 13));
    }
    if (exponent == 0x1f) return float_of(sign | 0x7f800000u | (mantissa << 13));
    return float_of(sign | ((exponent + 127 - 15) << 23) | (mantissa << 13));
}

/* formats.rs:81-102: nearest even; overflow to infinity; below half the smallest subnormal to zero. */
uint16_t sdo_f32_to_f16(float value) {
    const uint32_t bits = bits_of(value);
    const uint16_t sign = (uint16_t)((bits >> 16) & 0x8000);
    const int exponent = (int)((bits >> 23) & 0xff) - 127 + 15;
    const uint32_t mantissa = bits & 0x7fffff;
    if (exponent >= 0x1f) return sign | 0x7c00;
    if (exponent <= 0) {
        if (exponent < -10) return sign;
        const uint32_t full = mantissa | 0x800000;
        const uint32_t shift = (uint32_t)(14 - exponent);
        const uint32_t kept = full >> shift, rest = full & ((1u << shift) - 1), half = 1u << (shift - 1);
        return sign | (uint16_t)(kept + (rest > half || (rest == half && (kept & 1))));
    }
    const uint32_t kept = mantissa >> 13, rest = mantissa & 0x1fff;
    const uint32_t rounded = (((uint32_t)exponent << 10) | kept) + (rest > 0x1000 || (rest == 0x1000 && (kept & 1)));
    return sign | (uint16_t)rounded;
}

/* token_mixing.hpp:728-735, ds_state_bf16_gpu.rs:27-33 */
uint16_t sdo_f32_to_bf16(float value) {
    const uint32_t bits = bits_of(value);
    if ((bits & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((bits >> 16) | 0x40u);
    return (uint16_t)((bits + 0x7fffu + ((bits >> 16) & 1u)) >> 16);
}
float sdo_bf16_to_f32(uint16_t half) { return float_of((uint32_t)half << 16); }
void sdo_to_bf16(const float* x, size_t count, uint16_t* out) {
    for (size_t i = 0; i < count; ++i) out[i] = sdo_f32_to_bf16(x[i]);
}

/* ------------------------------------------------------------------ K/V rows */

size_t sdo_kv_q8_row_bytes(size_t dim) { return dim + dim / 32 * 2; }

/* kernels.cpp:58-74 / gpu.rs:536-551: scale = f16(max|x| / 127); q = clamp(rint(x / f32(scale)), -127, 127). */
void sdo_kv_q8_row(const float* values, size_t dim, uint8_t* row) {
    for (size_t block = 0; block < dim / 32; ++block) {
        const float* part = values + block * 32;
        float top = 0.0f;
        for (int i = 0; i < 32; ++i) top = fmaxf(top, fabsf(part[i]));
        const uint16_t half = sdo_f32_to_f16(top / 127.0f);
        const float scale = sdo_f16_to_f32(half);
        for (int i = 0; i < 32; ++i) {
            int q = 0;
            if (scale > 0.0f) {
                const float r = nearbyintf(part[i] / scale);   /* default rounding mode: ties to even */
                q = r > 127.0f ? 127 : r < -127.0f ? -127 : (int)r;
            }
            row[block * 32 + i] = (uint8_t)(int8_t)q;
        }
        row[dim + 2 * block] = (uint8_t)(half & 0xff);
        row[dim + 2 * block + 1] = (uint8_t)(half >> 8);
    }
}

/* kernels.cpp:38-44 / gpu.rs:553-561 */
void sdo_kv_q8_values(const uint8_t* row, size_t dim, float* values) {
    for (size_t c = 0; c < dim; ++c) {
        const size_t block = c / 32;
        const float scale = sdo_f16_to_f32((uint16_t)(row[dim + 2 * block] | (row[dim + 2 * block + 1] << 8)));
        values[c] = (float)(int8_t)row[c] * scale;
    }
}

void sdo_kv_f16_row(const float* values, size_t dim, uint8_t* row) {
    for (size_t c = 0; c < dim; ++c) {
        const uint16_t h = sdo_f32_to_f16(values[c]);
        row[2 * c] = (uint8_t)(h & 0xff); row[2 * c + 1] = (uint8_t)(h >> 8);
    }
}
void sdo_kv_f16_values(const uint8_t* row, size_t dim, float* values) {
    for (size_t c = 0; c < dim; ++c) values[c] = sdo_f16_to_f32((uint16_t)(row[2 * c] | (row[2 * c + 1] << 8)));
}

static void row_values(const uint8_t* row, size_t row_bytes, size_t dim, float* values) {
    if (row_bytes == 2 * dim) sdo_kv_f16_values(row, dim, values); else sdo_kv_q8_values(row, dim, values);
}
static void row_store(const float* values, size_t row_bytes, size_t dim, uint8_t* row) {
    if (row_bytes == 2 * dim) sdo_kv_f16_row(values, dim, row); else sdo_kv_q8_row(values, dim, row);
}

/* formats.rs:104-116: d = max|x|/127 kept in fp32 for the division, q = round-half-away(x * (1/d)). */
void sdo_ggml_q8_0_quantize(const float* values, size_t count, uint8_t* blocks) {
    for (size_t b = 0; b < count / 32; ++b) {
        const float* group = values + b * 32;
        float top = 0.0f;
        for (int i = 0; i < 32; ++i) top = fmaxf(top, fabsf(group[i]));
        const float d = top / 127.0f, inverse = d != 0.0f ? 1.0f / d : 0.0f;
        const uint16_t h = sdo_f32_to_f16(d);
        uint8_t* out = blocks + b * 34;
        out[0] = (uint8_t)(h & 0xff); out[1] = (uint8_t)(h >> 8);
        for (int i = 0; i < 32; ++i) out[2 + i] = (uint8_t)(int8_t)roundf(group[i] * inverse);
    }
}
/* formats.rs:232-236 */
void sdo_ggml_q8_0_dequantize(const uint8_t* blocks, size_t count, float* out) {
    for (size_t b = 0; b < count / 32; ++b) {
        const uint8_t* in = blocks + b * 34;
        const float d = sdo_f16_to_f32((uint16_t)(in[0] | (in[1] << 8)));
        for (int i = 0; i < 32; ++i) out[b * 32 + i] = d * (float)(int8_t)in[2 + i];
    }
}

/* ------------------------------------------------------------------ paged cache */

static inline const uint8_t* pool_row(const uint8_t* pool, size_t row_bytes, size_t page_tokens, size_t kv_heads,
                                      const int32_t* table, size_t plane, size_t position) {
    const size_t page = (size_t)table[position / page_tokens], at = position % page_tokens;
    return pool + ((page * 2 * kv_heads + plane) * page_tokens + at) * row_bytes;
}

void sdo_kv_write(uint8_t* pool, size_t row_bytes, size_t page_tokens, size_t kv_heads, size_t dim,
                  const int32_t* page_table, size_t table_stride, const int32_t* positions,
                  const float* keys, const float* values, size_t seqs, size_t span) {
    for (size_t s = 0; s < seqs; ++s)
        for (size_t r = 0; r < span; ++r)
            for (size_t h = 0; h < kv_heads; ++h) {
                const size_t position = (size_t)positions[s] + r;
                const size_t at = ((s * span + r) * kv_heads + h) * dim;
                row_store(keys + at, row_bytes, dim,
                          (uint8_t*)pool_row(pool, row_bytes, page_tokens, kv_heads, page_table + s * table_stride, h, position));
                row_store(values + at, row_bytes, dim,
                          (uint8_t*)pool_row(pool, row_bytes, page_tokens, kv_heads, page_table + s * table_stride, kv_heads + h, position));
            }
}

/* One (sequence, kv head): all grouped query heads of all span rows over the positions they may see.
 * Scores as kernels.cpp:100-121 (sum over columns in order, then the scale), the softmax and the weighted
 * values as kernels.cpp:123-165 (max; p = expf(s - max); L = sum p; p /= L; o = sum p * v). */
static void attend_group(const uint8_t* pool, size_t row_bytes, size_t page_tokens, size_t kv_heads, size_t dim,
                         const int32_t* table, size_t first_position, const float* q, size_t span, size_t heads,
                         size_t kvh, float scale, float* out, double* out64) {
    const size_t group = heads / kv_heads, total = first_position + span;   /* positions 0 .. total-1 exist */
    float* k = (float*)malloc(total * dim * sizeof(float));
    float* v = (float*)malloc(total * dim * sizeof(float));
    float* p = (float*)malloc(total * sizeof(float));
    double* p64 = out64 ? (double*)malloc(total * sizeof(double)) : NULL;
    for (size_t t = 0; t < total; ++t) {
        row_values(pool_row(pool, row_bytes, page_tokens, kv_heads, table, kvh, t), row_bytes, dim, k + t * dim);
        row_values(pool_row(pool, row_bytes, page_tokens, kv_heads, table, kv_heads + kvh, t), row_bytes, dim, v + t * dim);
    }
    for (size_t r = 0; r < span; ++r) {
        const size_t length = first_position + r + 1;
        for (size_t g = 0; g < group; ++g) {
            const size_t head = kvh * group + g;
            const float* query = q + (r * heads + head) * dim;
            float top = -INFINITY;
            for (size_t t = 0; t < length; ++t) {
                float sum = 0.0f;
                const float* key = k + t * dim;
                for (size_t d = 0; d < dim; ++d) sum += key[d] * query[d];
                p[t] = sum * scale;
                top = fmaxf(top, p[t]);
                if (p64) {
                    double wide = 0.0;
                    for (size_t d = 0; d < dim; ++d) wide += (double)key[d] * (double)query[d];
                    p64[t] = wide * (double)scale;
                }
            }
            float denominator = 0.0f;
            for (size_t t = 0; t < length; ++t) { p[t] = expf(p[t] - top); denominator += p[t]; }
            for (size_t t = 0; t < length; ++t) p[t] /= denominator;
            float* o = out + (r * heads + head) * dim;
            for (size_t d = 0; d < dim; ++d) o[d] = 0.0f;
            for (size_t t = 0; t < length; ++t) {
                const float w = p[t];
                const float* value = v + t * dim;
                for (size_t d = 0; d < dim; ++d) o[d] += w * value[d];
            }
            if (out64) {
                double top64 = -INFINITY, total64 = 0.0;
                for (size_t t = 0; t < length; ++t) top64 = fmax(top64, p64[t]);
                for (size_t t = 0; t < length; ++t) { p64[t] = exp(p64[t] - top64); total64 += p64[t]; }
                double* o64 = out64 + (r * heads + head) * dim;
                for (size_t d = 0; d < dim; ++d) o64[d] = 0.0;
                for (size_t t = 0; t < length; ++t) {
                    const double w = p64[t] / total64;
                    const float* value = v + t * dim;
                    for (size_t d = 0; d < dim; ++d) o64[d] += w * (double)value[d];
                }
            }
        }
    }
    free(k); free(v); free(p); free(p64);
}

void sdo_paged_attention(const uint8_t* pool, size_t row_bytes, size_t page_tokens, size_t kv_heads, size_t dim,
                         const int32_t* page_table, size_t table_stride, const int32_t* positions,
                         const float* q, size_t seqs, size_t span, size_t heads, float scale,
                         float* out, double* out64, int threads) {
    const long items = (long)(seqs * kv_heads);
    if (threads <= 0) threads = sdo_max_threads();
    #pragma omp parallel for schedule(dynamic, 1) num_threads(threads)
    for (long item = 0; item < items; ++item) {
        const size_t s = (size_t)item / kv_heads, kvh = (size_t)item % kv_heads;
        const size_t at = s * span * heads * dim;
        attend_group(pool, row_bytes, page_tokens, kv_heads, dim, page_table + s * table_stride, (size_t)positions[s],
                     q + at, span, heads, kvh, scale, out + at, out64 ? out64 + at : NULL);
    }
}

/* kernels.cpp:4387-4419 with :79-98, :100-165.  Qwen shape: 24 query heads, 2 K/V heads, 256 columns, scale 1/16. */
void sdo_attention_sequence(uint8_t* state, size_t row_bytes, size_t context, size_t base, size_t steps,
                            size_t selected, const float* input, float* output) {
    enum { HEADS = 24, KV = 2, DIM = 256 };
    const size_t keys_start = steps * HEADS * DIM, values_start = keys_start + steps * KV * DIM;
    const size_t index_start = steps * (HEADS * DIM + 2 * KV * DIM), count_start = index_start + steps * selected;
    for (size_t step = 0; step < steps; ++step)
        for (size_t h = 0; h < KV; ++h) {
            row_store(input + keys_start + (step * KV + h) * DIM, row_bytes, DIM, state + (h * context + base + step) * row_bytes);
            row_store(input + values_start + (step * KV + h) * DIM, row_bytes, DIM, state + ((KV + h) * context + base + step) * row_bytes);
        }
    float* scores = (float*)malloc(selected * sizeof(float));
    float key[DIM], value[DIM];
    for (size_t step = 0; step < steps; ++step) {
        const size_t count = (size_t)input[count_start + step];
        const float* list = input + index_start + step * selected;
        for (size_t head = 0; head < HEADS; ++head) {
            const size_t kvh = head / (HEADS / KV);
            const float* query = input + (step * HEADS + head) * DIM;
            float top = -INFINITY;
            for (size_t slot = 0; slot < selected; ++slot) {
                float result = -INFINITY;
                if (slot < count) {
                    const float raw = list[slot];
                    if (raw >= 0 && raw <= (float)(base + step) && raw < (float)context) {
                        row_values(state + (kvh * context + (size_t)raw) * row_bytes, row_bytes, DIM, key);
                        result = 0.0f;
                        for (size_t c = 0; c < DIM; ++c) result += key[c] * query[c];
                        result *= 0.0625f;
                    }
                }
                scores[slot] = result;
                top = fmaxf(top, result);
            }
            float denominator = 0.0f;
            for (size_t slot = 0; slot < selected; ++slot) { scores[slot] = expf(scores[slot] - top); denominator += scores[slot]; }
            for (size_t slot = 0; slot < selected; ++slot) scores[slot] /= denominator;
            float* o = output + (step * HEADS + head) * DIM;
            for (size_t c = 0; c < DIM; ++c) o[c] = 0.0f;
            for (size_t slot = 0; slot < count && slot < selected; ++slot) {
                const float raw = list[slot];
                if (raw >= 0 && raw <= (float)(base + step) && raw < (float)context) {
                    row_values(state + ((KV + kvh) * context + (size_t)raw) * row_bytes, row_bytes, DIM, value);
                    for (size_t c = 0; c < DIM; ++c) o[c] += scores[slot] * value[c];
                }
            }
        }
    }
    free(scores);
}

/* ------------------------------------------------------------------ dense causal GQA over fp32 caches */

static inline float sigmoidf_(float x) { return 1.0f / (1.0f + expf(-x)); }

/* token_mixing.hpp:356-520 (the arithmetic both kernels share), attention_gpu.rs:50-87 (the statement). */
void sdo_op_attention(const float* q, const float* keys, const float* values, size_t context, const int32_t* positions,
                      size_t rows, size_t heads, size_t kv_heads, size_t dim, float scale, const float* gate, float* out) {
    float* p = (float*)malloc(context * sizeof(float));
    for (size_t row = 0; row < rows; ++row) {
        size_t length = (size_t)positions[row] + 1;
        if (length > context) length = context;
        for (size_t head = 0; head < heads; ++head) {
            const size_t kh = head / (heads / kv_heads);
            const float* query = q + (row * heads + head) * dim;
            float top = -INFINITY;
            for (size_t t = 0; t < length; ++t) {
                const float* key = keys + (t * kv_heads + kh) * dim;
                float sum = 0.0f;
                for (size_t d = 0; d < dim; ++d) sum += query[d] * key[d];
                p[t] = sum * scale;
                top = fmaxf(top, p[t]);
            }
            float total = 0.0f;
            for (size_t t = 0; t < length; ++t) { p[t] = expf(p[t] - top); total += p[t]; }
            float* o = out + (row * heads + head) * dim;
            for (size_t d = 0; d < dim; ++d) {
                float sum = 0.0f;
                for (size_t t = 0; t < length; ++t) sum += p[t] * values[(t * kv_heads + kh) * dim + d];
                sum /= total;
                if (gate) sum *= sigmoidf_(gate[(row * heads + head) * dim + d]);
                o[d] = sum;
            }
        }
    }
    free(p);
}

static double gamma_(size_t operations) {
    const double nu = (double)operations * ldexp(1.0, -24);
    return nu / (1.0 - nu);
}

/* attention_gpu.rs:50-87, :28-31: the F64 evaluation over exactly the fp32 operands and the derived bound
 * max|v| * (expm1(2 * gamma(2 dim + 1) * sum|q k| * |scale|) + gamma(8 L + 32) + 16 * 2^-24). */
void sdo_op_attention_f64(const float* q, const float* keys, const float* values, size_t context, const int32_t* positions,
                          size_t rows, size_t heads, size_t kv_heads, size_t dim, float scale, const float* gate,
                          double* out, double* bound) {
    double* w = (double*)malloc(context * sizeof(double));
    for (size_t row = 0; row < rows; ++row) {
        size_t length = (size_t)positions[row] + 1;
        if (length > context) length = context;
        for (size_t head = 0; head < heads; ++head) {
            const size_t kh = head / (heads / kv_heads);
            const float* query = q + (row * heads + head) * dim;
            double error = 0.0, top = -INFINITY;
            for (size_t t = 0; t < length; ++t) {
                const float* key = keys + (t * kv_heads + kh) * dim;
                double sum = 0.0, absolute = 0.0;
                for (size_t d = 0; d < dim; ++d) {
                    const double product = (double)query[d] * (double)key[d];
                    sum += product; absolute += fabs(product);
                }
                error = fmax(error, gamma_(2 * dim + 1) * absolute * fabs((double)scale));
                w[t] = sum * (double)scale;
                top = fmax(top, w[t]);
            }
            double total = 0.0;
            for (size_t t = 0; t < length; ++t) { w[t] = exp(w[t] - top); total += w[t]; }
            for (size_t d = 0; d < dim; ++d) {
                double sum = 0.0, largest = 0.0;
                for (size_t t = 0; t < length; ++t) {
                    const double value = (double)values[(t * kv_heads + kh) * dim + d];
                    sum += w[t] * value;
                    largest = fmax(largest, fabs(value));
                }
                const size_t at = (row * heads + head) * dim + d;
                const double gating = gate ? 1.0 / (1.0 + exp(-(double)gate[at])) : 1.0;
                out[at] = sum / total * gating;
                if (bound) bound[at] = largest * (expm1(2.0 * error) + gamma_(8 * length + 32) + 16.0 * ldexp(1.0, -24));
            }
        }
    }
    free(w);
}

/* ------------------------------------------------------------------ indexer scores */

/* ops.hpp:1700-1739: each dot a chain of fmaf over the columns in order; each head's term
 * max(dot, 0) * weight rounded on its own; the terms added in head order; the scale last.
 * Eight keys are carried side by side so the compiler can vectorise across keys; every chain keeps its order. */
void sdo_index_scores(const float* q, const void* keys, int keys_bf16, const float* weights, const int32_t* visible,
                      size_t rows, size_t groups, size_t heads, size_t dim, float scale, float* scores, int threads) {
    enum { LANES = 8 };
    if (threads <= 0) threads = sdo_max_threads();
    const long tiles = (long)((groups + LANES - 1) / LANES);
    for (size_t row = 0; row < rows; ++row) {
        const int32_t seen = visible[row] > 0 ? visible[row] : 0;
        const size_t limit = groups < (size_t)seen ? groups : (size_t)seen;
        const float* row_q = q + row * heads * dim;
        const float* row_w = weights + row * heads;
        #pragma omp parallel for schedule(static) num_threads(threads)
        for (long tile = 0; tile < tiles; ++tile) {
            const size_t g0 = (size_t)tile * LANES;
            float kt[1024][LANES];
            float* wide = NULL;
            float (*k)[LANES] = kt;
            if (dim > 1024) { wide = (float*)malloc(dim * LANES * sizeof(float)); k = (float (*)[LANES])wide; }
            for (size_t j = 0; j < LANES; ++j) {
                const size_t g = g0 + j;
                for (size_t d = 0; d < dim; ++d) {
                    float value = 0.0f;
                    if (g < limit) value = keys_bf16 ? sdo_bf16_to_f32(((const uint16_t*)keys)[g * dim + d]) : ((const float*)keys)[g * dim + d];
                    k[d][j] = value;
                }
            }
            float total[LANES] = {0};
            for (size_t h = 0; h < heads; ++h) {
                float acc[LANES] = {0};
                const float* query = row_q + h * dim;
                for (size_t d = 0; d < dim; ++d) {
                    const float x = query[d];
                    for (int j = 0; j < LANES; ++j) acc[j] = fmaf(x, k[d][j], acc[j]);
                }
                const float w = row_w[h];
                for (int j = 0; j < LANES; ++j) {
                    const float term = fmaxf(acc[j], 0.0f) * w;
                    total[j] = total[j] + term;
                }
            }
            for (size_t j = 0; j < LANES && g0 + j < groups; ++j)
                scores[row * groups + g0 + j] = g0 + j < limit ? total[j] * scale : -INFINITY;
            free(wide);
        }
    }
}

/* The indexer's projection in the library's stated order for 64 lanes (see oracle.h). */
void sdo_index_projection(const uint8_t* matrix, int kind, size_t cols, const float* x, size_t heads, float* weights) {
    const size_t unit = kind == 30 ? 8 : 32, units = cols / unit, row_bytes = kind == 30 ? cols * 2 : cols / 32 * 34;
    for (size_t head = 0; head < heads; ++head) {
        const uint8_t* row = matrix + head * row_bytes;
        float lanes[64];
        for (size_t lane = 0; lane < 64; ++lane) {
            float sum = 0.0f;
            for (size_t u = lane; u < units; u += 64) {
                float chain = 0.0f;
                if (kind == 30) {
                    for (size_t i = 0; i < 8; ++i) {
                        const uint8_t* at = row + (u * 8 + i) * 2;
                        chain = fmaf(sdo_bf16_to_f32((uint16_t)(at[0] | (at[1] << 8))), x[u * 8 + i], chain);
                    }
                } else {
                    const uint8_t* block = row + u * 34;
                    for (size_t i = 0; i < 32; ++i) chain = fmaf((float)(int8_t)block[2 + i], x[u * 32 + i], chain);
                    chain *= sdo_f16_to_f32((uint16_t)(block[0] | (block[1] << 8)));
                }
                sum = sum + chain;
            }
            lanes[lane] = sum;
        }
        for (size_t offset = 32; offset; offset /= 2)
            for (size_t lane = 0; lane < offset; ++lane) lanes[lane] = lanes[lane] + lanes[lane + offset];
        weights[head] = lanes[0];
    }
}

void sdo_index_scores_f64(const float* q, const void* keys, int keys_bf16, const float* weights, const int32_t* visible,
                          size_t rows, size_t groups, size_t heads, size_t dim, float scale, double* scores) {
    for (size_t row = 0; row < rows; ++row) {
        const int32_t seen = visible[row] > 0 ? visible[row] : 0;
        const size_t limit = groups < (size_t)seen ? groups : (size_t)seen;
        for (size_t g = 0; g < groups; ++g) {
            double total = 0.0;
            for (size_t h = 0; h < heads && g < limit; ++h) {
                double dot = 0.0;
                for (size_t d = 0; d < dim; ++d) {
                    const float key = keys_bf16 ? sdo_bf16_to_f32(((const uint16_t*)keys)[g * dim + d]) : ((const float*)keys)[g * dim + d];
                    dot += (double)q[(row * heads + h) * dim + d] * (double)key;
                }
                total += fmax(dot, 0.0) * (double)weights[row * heads + h];
            }
            scores[row * groups + g] = g < limit ? total * (double)scale : -INFINITY;
        }
    }
}

/* ------------------------------------------------------------------ top-k */

/* ops.hpp:1766-1769 / fused_gpu.rs:327-330 */
uint32_t sdo_top_k_key(float value) {
    const uint32_t bits = bits_of(value == 0.0f ? 0.0f : value);
    return (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u);
}

static int descending_u32(const void* a, const void* b) {
    const uint32_t x = *(const uint32_t*)a, y = *(const uint32_t*)b;
    return x < y ? 1 : x > y ? -1 : 0;
}

/* fused_gpu.rs:334-358 */
void sdo_top_k(const float* scores, size_t rows, size_t groups, size_t k, int32_t* out) {
    const uint32_t floor = sdo_top_k_key(-INFINITY);
    uint32_t* keys = (uint32_t*)malloc((groups ? groups : 1) * sizeof(uint32_t));
    uint32_t* sorted = (uint32_t*)malloc((groups ? groups : 1) * sizeof(uint32_t));
    for (size_t row = 0; row < rows; ++row) {
        const float* s = scores + row * groups;
        int32_t* o = out + row * k;
        size_t live = 0;
        for (size_t g = 0; g < groups; ++g) {
            keys[g] = sdo_top_k_key(s[g]);
            if (keys[g] > floor) sorted[live++] = keys[g];
        }
        size_t kept = 0;
        if (live <= k) {
            for (size_t g = 0; g < groups; ++g) if (keys[g] > floor) o[kept++] = (int32_t)g;
        } else {
            qsort(sorted, live, sizeof(uint32_t), descending_u32);
            const uint32_t threshold = sorted[k - 1];
            size_t above = 0;
            for (size_t g = 0; g < groups; ++g) above += keys[g] > floor && keys[g] > threshold;
            size_t need = k - above;
            for (size_t g = 0; g < groups; ++g) {
                if (keys[g] <= floor) continue;
                if (keys[g] > threshold) o[kept++] = (int32_t)g;
                else if (keys[g] == threshold && need > 0) { o[kept++] = (int32_t)g; --need; }
            }
        }
        for (; kept < k; ++kept) o[kept] = -1;
    }
    free(keys); free(sorted);
}

/* ops.hpp:1956-1965 then op_top_k_kernel over the blocks' tops; fused_gpu.rs:504-517. */
void sdo_index_candidates(const float* scores, const int32_t* visible, size_t rows, size_t groups, size_t blocks,
                          size_t block, int32_t* out) {
    const size_t count = (groups + block - 1) / block;
    float* tops = (float*)malloc(count * sizeof(float));
    for (size_t row = 0; row < rows; ++row) {
        const float* s = scores + row * groups;
        const size_t seen_raw = visible[row] > 0 ? (size_t)visible[row] : 0;
        const size_t seen = groups < seen_raw ? groups : seen_raw;
        for (size_t b = 0; b < count; ++b) {
            float top = seen && b == (seen - 1) / block ? INFINITY : -INFINITY;
            const size_t end = groups < (b + 1) * block ? groups : (b + 1) * block;
            for (size_t g = b * block; g < end; ++g) top = fmaxf(top, s[g]);
            tops[b] = top;
        }
        sdo_top_k(tops, 1, count, blocks, out + row * blocks);
    }
    free(tops);
}

/* ------------------------------------------------------------------ latent sparse attention */

/* ops.hpp:1318-1328 + ds41_reference.rs:185-195: adjacent pairs of the last rope_dims values, angle in double. */
static void rotate_tail(float* x, size_t width, size_t rope_dims, const float* frequencies, int64_t position, int inverse) {
    const size_t start = width - rope_dims;
    for (size_t i = 0; i < rope_dims / 2; ++i) {
        const double angle = (double)position * (double)frequencies[i] * (inverse ? -1.0 : 1.0);
        const double s = sin(angle), c = cos(angle);
        const double a = (double)x[start + 2 * i], b = (double)x[start + 2 * i + 1];
        x[start + 2 * i] = (float)(a * c - b * s);
        x[start + 2 * i + 1] = (float)(a * s + b * c);
    }
}

static inline float latent_value(const void* base, int bf16, size_t row, size_t width, size_t col) {
    return bf16 ? sdo_bf16_to_f32(((const uint16_t*)base)[row * width + col]) : ((const float*)base)[row * width + col];
}

/* ops.hpp:1240-1297 */
void sdo_latent_attention(const float* q, const float* raw, size_t raw_rows, const int32_t* positions, size_t window,
                          const void* compressed, int compressed_bf16, const int32_t* selected, size_t selections,
                          const float* sinks, size_t rows, size_t heads, size_t kdim, size_t vdim, float scale,
                          size_t rope_dims, const float* frequencies, float* out, double* out64, int threads) {
    if (threads <= 0) threads = sdo_max_threads();
    const long items = (long)(rows * heads);
    #pragma omp parallel for schedule(dynamic, 1) num_threads(threads)
    for (long item = 0; item < items; ++item) {
        const size_t row = (size_t)item / heads, head = (size_t)item % heads;
        const int64_t p = positions ? positions[row] : 0;
        int64_t first = p - (int64_t)window + 1;
        if (first < 0) first = 0;
        const size_t raw_count = window ? (size_t)(p - first + 1) : 0, total = raw_count + selections;
        float* query = (float*)malloc(kdim * sizeof(float));
        memcpy(query, q + (row * heads + head) * kdim, kdim * sizeof(float));
        if (rope_dims) rotate_tail(query, kdim, rope_dims, frequencies, p, 0);
        float* w = (float*)malloc((total ? total : 1) * sizeof(float));
        double* w64 = out64 ? (double*)malloc((total ? total : 1) * sizeof(double)) : NULL;
        const float sink = sinks ? sinks[head] : -INFINITY;
        float top = sink;
        double top64 = sink;
        for (size_t index = 0; index < total; ++index) {
            const void* base; int bf16; size_t at; int present = 1;
            if (index < raw_count) { base = raw; bf16 = 0; at = (size_t)(first + (int64_t)index) % raw_rows; }
            else {
                const int32_t chosen = selected[row * selections + (index - raw_count)];
                present = chosen >= 0; base = compressed; bf16 = compressed_bf16; at = present ? (size_t)chosen : 0;
            }
            if (!present) { w[index] = -INFINITY; if (w64) w64[index] = -INFINITY; continue; }
            float dot = 0.0f; double dot64 = 0.0;
            for (size_t i = 0; i < kdim; ++i) {
                const float value = latent_value(base, bf16, at, kdim, i);
                dot += query[i] * value;
                dot64 += (double)query[i] * (double)value;
            }
            w[index] = dot * scale;
            top = fmaxf(top, w[index]);
            if (w64) { w64[index] = dot64 * (double)scale; top64 = fmax(top64, w64[index]); }
        }
        float sum = 0.0f; double sum64 = 0.0;
        for (size_t index = 0; index < total; ++index) {
            w[index] = w[index] == -INFINITY ? 0.0f : expf(w[index] - top);
            sum += w[index];
            if (w64) { w64[index] = w64[index] == -INFINITY ? 0.0 : exp(w64[index] - top64); sum64 += w64[index]; }
        }
        const float denominator = sum + (sinks ? expf(sink - top) : 0.0f);
        const double denominator64 = sum64 + (sinks ? exp((double)sink - top64) : 0.0);
        float* o = out + (row * heads + head) * vdim;
        double* o64 = out64 ? out64 + (row * heads + head) * vdim : NULL;
        for (size_t i = 0; i < vdim; ++i) {
            float acc = 0.0f; double acc64 = 0.0;
            for (size_t index = 0; index < total; ++index) {
                if (w[index] == 0.0f && !(w64 && w64[index] != 0.0)) continue;
                const void* base; int bf16; size_t at;
                if (index < raw_count) { base = raw; bf16 = 0; at = (size_t)(first + (int64_t)index) % raw_rows; }
                else { base = compressed; bf16 = compressed_bf16; at = (size_t)selected[row * selections + (index - raw_count)]; }
                const float value = latent_value(base, bf16, at, kdim, i);
                if (w[index] != 0.0f) acc += w[index] * value;
                if (w64) acc64 += w64[index] * (double)value;
            }
            o[i] = acc / denominator;
            if (o64) o64[i] = acc64 / denominator64;
        }
        if (rope_dims) {
            rotate_tail(o, vdim, rope_dims, frequencies, p, 1);
            if (o64) {
                const size_t start = vdim - rope_dims;
                for (size_t i = 0; i < rope_dims / 2; ++i) {
                    const double angle = (double)p * (double)frequencies[i] * -1.0;
                    const double s = sin(angle), c = cos(angle), a = o64[start + 2 * i], b = o64[start + 2 * i + 1];
                    o64[start + 2 * i] = a * c - b * s; o64[start + 2 * i + 1] = a * s + b * c;
                }
            }
        }
        free(query); free(w); free(w64);
    }
}

/* ops.hpp:1681-1694 */
void sdo_compress(const float* kv, const float* gate, size_t groups, size_t ratio, size_t dim, float* out) {
    for (size_t group = 0; group < groups; ++group)
        for (size_t col = 0; col < dim; ++col) {
            if (!gate) { out[group * dim + col] = kv[group * dim + col]; continue; }
            float top = -INFINITY;
            for (size_t r = 0; r < ratio; ++r) top = fmaxf(top, gate[(group * ratio + r) * dim + col]);
            float sum = 0.0f, acc = 0.0f;
            for (size_t r = 0; r < ratio; ++r) {
                const float w = expf(gate[(group * ratio + r) * dim + col] - top);
                sum += w; acc += w * kv[(group * ratio + r) * dim + col];
            }
            out[group * dim + col] = acc / sum;
        }
}

/* ------------------------------------------------------------------ Qwen block selection */

/* sparse_attention.hpp:172-241: the best `keep_blocks` (512) complete 4-token blocks by raw bits of their
 * non-negative scores, ties to the earliest blocks, in block order, four positions each; then the
 * positions of the incomplete block; every causal position when there are no more than keep_blocks blocks. */
size_t sdo_qsa_select(const float* scores, size_t position, size_t keep_blocks, float* indices) {
    const size_t complete = (position + 1) / 4;
    if (complete <= keep_blocks) {
        for (size_t i = 0; i <= position; ++i) indices[i] = (float)i;
        return position + 1;
    }
    uint32_t* sorted = (uint32_t*)malloc(complete * sizeof(uint32_t));
    for (size_t b = 0; b < complete; ++b) sorted[b] = bits_of(scores[b]);
    qsort(sorted, complete, sizeof(uint32_t), descending_u32);
    const uint32_t threshold = sorted[keep_blocks - 1];
    free(sorted);
    size_t above = 0;
    for (size_t b = 0; b < complete; ++b) above += bits_of(scores[b]) > threshold;
    size_t need = keep_blocks - above, out = 0;
    for (size_t b = 0; b < complete; ++b) {
        const uint32_t value = bits_of(scores[b]);
        int take = value > threshold;
        if (value == threshold && need > 0) { take = 1; --need; }
        if (take) for (size_t tap = 0; tap < 4; ++tap) indices[out++] = (float)(b * 4 + tap);
    }
    for (size_t i = complete * 4; i <= position; ++i) indices[out++] = (float)i;
    return out;
}

/* ------------------------------------------------------------------ Qwen block indexer: norm, rope, pool, scores */

/* sparse_attention.hpp:2-6: the first 64 columns turn in pairs (c, c + 32) by position / 1e7^(c % 32 / 32). */
static float qsa_rope(float own, float partner, size_t column, size_t position) {
    if (column >= 64) return own;
    const float angle = (float)position / powf(1e7f, (float)(column % 32) / 32.0f);
    return own * cosf(angle) + (column < 32 ? -partner : partner) * sinf(angle);
}

/* The sum of squares as the kernels' halving tree forms it (sparse_attention.hpp:14-17, 101-104): sums[c] += sums[c + offset]. */
static float qsa_tree_sum(float* sums, size_t width) {
    for (size_t offset = width / 2; offset; offset /= 2)
        for (size_t c = 0; c < offset; ++c) sums[c] += sums[c + offset];
    return sums[0];
}

/* sparse_attention.hpp:8-23 (qsa_normalize): rows x heads vectors of `width` (128 or 256) at `stride` floats apart, RMS-normalised
 * with the weight `norm`, the first 64 columns turned for position + row. */
void sdo_qsa_normalize(const float* source, const float* norm, size_t rows, size_t heads, size_t width, size_t stride,
                       size_t position, float* target) {
    float values[256], sums[256];
    for (size_t head = 0; head < rows * heads; ++head) {
        const size_t token = head / heads;
        for (size_t c = 0; c < width; ++c) { const float x = source[head * stride + c]; values[c] = x * norm[c]; sums[c] = x * x; }
        const float denominator = sqrtf(qsa_tree_sum(sums, width) / (float)width + 1e-6f);
        for (size_t c = 0; c < width; ++c) {
            const float own = values[c] / denominator;
            const float partner = c < 64 ? values[(c + 32) % 64] / denominator : 0.0f;
            target[head * width + c] = qsa_rope(own, partner, c, position + token);
        }
    }
}

/* sparse_attention.hpp:87-108 (qsa_pool) then :132-139 (qsa_save_history): every block of four positions completed by rows
 * base .. base + steps is the mean of its four index-key inputs (earlier ones from the ring of sixteen), normalised and turned
 * for the block's first position, stored column-major blocks[c * pool + block]; the ring then takes the span's last four rows. */
void sdo_qsa_pool(const float* incoming, float* history, const float* norm, size_t pool, size_t base, size_t steps, float* blocks) {
    float values[128], sums[128];
    for (size_t block = base / 4; block < (base + steps) / 4; ++block) {
        const size_t begin = block * 4;
        for (size_t c = 0; c < 128; ++c) {
            float x = 0.0f;
            for (size_t tap = 0; tap < 4; ++tap) {
                const size_t pos = begin + tap;
                x += pos < base ? history[(pos % 16) * 128 + c] : incoming[(pos - base) * 128 + c];
            }
            x /= 4.0f;
            values[c] = x * norm[c]; sums[c] = x * x;
        }
        const float denominator = sqrtf(qsa_tree_sum(sums, 128) / 128.0f + 1e-6f);
        for (size_t c = 0; c < 128; ++c) {
            const float own = values[c] / denominator;
            const float partner = c < 64 ? values[(c + 32) % 64] / denominator : 0.0f;
            blocks[c * pool + block] = qsa_rope(own, partner, c, begin);
        }
    }
    const size_t kept = steps < 4 ? steps : 4;
    for (size_t i = 0; i < kept * 128; ++i) {
        const size_t token = steps - kept + i / 128;
        history[((base + token) % 16) * 128 + i % 128] = incoming[token * 128 + i % 128];
    }
}

/* sparse_attention.hpp:141-155 (qsa_block_scores; the same bits as the tiled form, :243-246): for every row with more than
 * 512 complete blocks, score(block) = sum over the four heads, in order, of the positive part of the head's dot product, each
 * dot product a chain of fused multiply-adds over the 128 columns in order.  Other entries of `scores` are left alone. */
void sdo_qsa_block_scores(const float* queries, size_t query_stride, const float* blocks, size_t pool, size_t base, size_t steps,
                          float* scores) {
    #pragma omp parallel for schedule(dynamic, 1)
    for (size_t token = 0; token < steps; ++token) {
        const size_t complete = (base + token + 1) / 4;
        if (complete <= 512) continue;
        for (size_t block = 0; block < complete; ++block) {
            float dot[4] = {0.0f, 0.0f, 0.0f, 0.0f};
            for (size_t c = 0; c < 128; ++c) {
                const float key = blocks[c * pool + block];
                for (size_t h = 0; h < 4; ++h) dot[h] = fmaf(key, queries[token * query_stride + h * 128 + c], dot[h]);
            }
            float total = fmaxf(dot[0], 0.0f) + fmaxf(dot[1], 0.0f);
            total += fmaxf(dot[2], 0.0f);
            total += fmaxf(dot[3], 0.0f);
            scores[token * pool + block] = total;
        }
    }
}

/* ------------------------------------------------------------------ the inputs of a dense attention step */

/* ops.hpp:28-55 (op_rms_norm_row with tree256_first_wave): thread t of 256 sums the squares of columns t, t + 256, ... (a fused
 * multiply-add each, as the device compiler contracts it), the 256 partial sums are added in halving-tree order, and
 * out = (x * rsqrt(mean + eps)) * weight. */
void sdo_rms_norm(const float* input, const float* weight, size_t rows, size_t width, float eps, float* output) {
    for (size_t r = 0; r < rows; ++r) {
        const float* x = input + r * width;
        float sums[256];
        for (size_t t = 0; t < 256; ++t) {
            float sum = 0.0f;
            for (size_t c = t; c < width; c += 256) sum = fmaf(x[c], x[c], sum);
            sums[t] = sum;
        }
        const float scale = 1.0f / sqrtf(qsa_tree_sum(sums, 256) / (float)width + eps);
        for (size_t c = 0; c < width; ++c) output[r * width + c] = x[c] * scale * weight[c];
    }
}

/* token_mixing.hpp:254-274: pair (i, i + pairs) of each vector's leading values turned by position * frequency, in double. */
void sdo_rope_halves(float* x, size_t rows, size_t vectors, size_t width, size_t rope_dims, const int32_t* positions,
                     const float* frequencies) {
    const size_t pairs = rope_dims / 2;
    for (size_t r = 0; r < rows; ++r)
        for (size_t v = 0; v < vectors; ++v)
            for (size_t i = 0; i < pairs; ++i) {
                float* first = x + (r * vectors + v) * width + i;
                float* second = first + pairs;
                const double angle = (double)positions[r] * (double)frequencies[i];
                const double s = sin(angle), c = cos(angle), a = *first, b = *second;
                *first = (float)(a * c - b * s);
                *second = (float)(a * s + b * c);
            }
}

/* token_mixing.hpp:276-338 (tm_attention_prepare_kernel): q_full rows x heads x [query | gate] split, queries and keys normed
 * and turned, keys (also back into k) and values written to row positions[row] of the caches when it lies inside them. */
void sdo_attention_prepare(const float* q_full, float* k, const float* v, size_t rows, size_t heads, size_t kv_heads, size_t dim,
                           const float* q_weight, const float* k_weight, float eps, size_t rope_dims, const int32_t* positions,
                           const float* frequencies, float* q, float* gate, float* keys, float* values, size_t context) {
    const size_t kv_width = kv_heads * dim;
    for (size_t r = 0; r < rows; ++r) {
        for (size_t h = 0; h < heads; ++h) {
            const float* x = q_full + (r * heads + h) * 2 * dim;
            memcpy(gate + (r * heads + h) * dim, x + dim, dim * sizeof(float));
            sdo_rms_norm(x, q_weight, 1, dim, eps, q + (r * heads + h) * dim);
        }
        sdo_rms_norm(k + r * kv_width, k_weight, kv_heads, dim, eps, k + r * kv_width);
    }
    if (rope_dims) {
        sdo_rope_halves(q, rows, heads, dim, rope_dims, positions, frequencies);
        sdo_rope_halves(k, rows, kv_heads, dim, rope_dims, positions, frequencies);
    }
    for (size_t r = 0; r < rows; ++r) {
        if (positions[r] < 0 || (size_t)positions[r] >= context) continue;
        memcpy(keys + (size_t)positions[r] * kv_width, k + r * kv_width, kv_width * sizeof(float));
        memcpy(values + (size_t)positions[r] * kv_width, v + r * kv_width, kv_width * sizeof(float));
    }
}

/* ------------------------------------------------------------------ DSpark block attention */

/* dspark_attention.hpp:1-101, in double as the reference's own test states it (crates/straydog-engine/tests/dspark_attention_gpu.rs:
 * 26-40): the keys are the ring rows of positions [anchor - history, anchor) (row p % 128) and all the block's keys; the head's sink
 * enters the maximum and the denominator only. */
void sdo_dspark_attention(const float* q, const float* ring, const float* block, const float* sinks, size_t heads, size_t slots,
                          size_t anchor, size_t history, double* out) {
    const size_t dim = 512, total = history + slots;
    double scores[128 + 5];
    for (size_t row = 0; row < slots * heads; ++row) {
        const float* query = q + row * dim;
        const double sink = sinks[row % heads];
        double top = sink;
        for (size_t i = 0; i < total; ++i) {
            const float* key = i < history ? ring + ((anchor - history + i) % 128) * dim : block + (i - history) * dim;
            double dot = 0.0;
            for (size_t d = 0; d < dim; ++d) dot += (double)query[d] * (double)key[d];
            scores[i] = dot / sqrt((double)dim);
            if (scores[i] > top) top = scores[i];
        }
        double denominator = exp(sink - top);
        for (size_t i = 0; i < total; ++i) { scores[i] = exp(scores[i] - top); denominator += scores[i]; }
        for (size_t d = 0; d < dim; ++d) {
            double sum = 0.0;
            for (size_t i = 0; i < total; ++i) {
                const float* key = i < history ? ring + ((anchor - history + i) % 128) * dim : block + (i - history) * dim;
                sum += scores[i] * (double)key[d];
            }
            out[row * dim + d] = sum / denominator;
        }
    }
}

/* ------------------------------------------------------------------ seeded inputs */

static inline uint64_t xorshift64(uint64_t* s) { *s ^= *s << 13; *s ^= *s >> 7; *s ^= *s << 17; return *s; }

void sdo_fill_uniform(uint64_t seed, float* out, size_t count, float lo, float hi) {
    uint64_t s = seed ? seed : 0x9e3779b97f4a7c15ull;
    for (size_t i = 0; i < count; ++i) out[i] = lo + (hi - lo) * (float)((double)(xorshift64(&s) >> 40) / 16777216.0);
}

void sdo_fill_normal(uint64_t seed, float* out, size_t count) {
    uint64_t s = seed ? seed : 0x9e3779b97f4a7c15ull;
    for (size_t i = 0; i < count; i += 2) {
        const double u = ((double)(xorshift64(&s) >> 11) + 0.5) / 9007199254740992.0;
        const double v = ((double)(xorshift64(&s) >> 11) + 0.5) / 9007199254740992.0;
        const double r = sqrt(-2.0 * log(u));
        out[i] = (float)(r * cos(6.283185307179586 * v));
        if (i + 1 < count) out[i + 1] = (float)(r * sin(6.283185307179586 * v));
    }
}
