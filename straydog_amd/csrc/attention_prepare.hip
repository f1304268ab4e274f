// The inputs of a dense attention step over FP32 caches, as the reference prepares them for sd_op_attention:
//   sd_op_split             [query | gate] rows apart                       gpu/token_mixing.hpp:246-252, :628-637
//   sd_op_rms_norm          x / sqrt(mean(x^2) + eps) * weight per row      gpu/ops.hpp:28-59, gpu/kernels.cpp:4901-4913
//   sd_op_rope_halves       pairs (i, i + pairs) turned, angles in double   gpu/token_mixing.hpp:254-274, :639-650
//   sd_op_scatter           rows to the rows an index list names            gpu/ops.hpp:1171-1175, gpu/kernels.cpp:5244-5252
//   sd_op_attention_prepare all of it for one step in one launch            gpu/token_mixing.hpp:276-338, :601-626
//   sd_op_norm_rope         rms norm, then the last values turned in adjacent pairs, rows scattered; fills the attention rope
//                           table when one is armed                          gpu/ops.hpp:60-106, gpu/kernels.cpp:4915-4940
//   sd_attention_turns_reserve / _arm   that table                          gpu/kernels.cpp:558-616, :5288-5303
// The fused entry gives the bits of the separate ones (the reference's own test of it, tests/fused_gpu.rs:225-268): the sum of
// squares is formed per thread over the columns c = t, t + 256, ... by fused multiply-adds and then over the 256 threads in
// halving-tree order, the scale is rsqrt of the mean plus eps, a value is (x * scale) * weight, and a pair is turned by
// sincos of double(position) * double(frequency) with the products and sums in double.
// One workgroup of 256 threads (four waves) per vector; nothing here is hot: a step has a few dozen vectors.
#include "device.hpp"
#include "tree_sum.hpp"
#include "../../include/straydog_gpu.h"

using namespace sd;

namespace {

constexpr unsigned THREADS = 256, MAX_DIM = 1024;

__device__ __forceinline__ void turn_pair(float* first, float* second, int32_t position, float frequency) {
    const double angle = double(position) * double(frequency);
    double s, c;
    sincos(angle, &s, &c);
    const double a = *first, b = *second;
    *first = float(a * c - b * s);
    *second = float(a * s + b * c);
}

// The workgroup's row scaled: out[c] = x[c] * rsqrt(mean(x^2) + eps) * weight[c].  out may be x, or LDS.
__device__ __forceinline__ void norm_row(const float* x, const float* weight, size_t width, float eps, float* out, float* sums) {
    float sum = 0.0f;
    for (size_t col = threadIdx.x; col < width; col += THREADS) sum = fmaf(x[col], x[col], sum);
    const float scale = rsqrtf(tree_sum(sum, sums, THREADS) / float(width) + eps);
    for (size_t col = threadIdx.x; col < width; col += THREADS) out[col] = x[col] * scale * weight[col];
}

__global__ void __launch_bounds__(THREADS) split_kernel(const float* x, size_t count, size_t width, float* first, float* second) {
    const size_t index = size_t(blockIdx.x) * THREADS + threadIdx.x;
    if (index >= count) return;
    const size_t row = index / width, col = index % width;
    first[index] = x[row * 2 * width + col];
    second[index] = x[row * 2 * width + width + col];
}

__global__ void __launch_bounds__(THREADS) rms_norm_kernel(const float* input, const float* weight, size_t width, float eps, float* output) {
    __shared__ float sums[THREADS];
    norm_row(input + size_t(blockIdx.x) * width, weight, width, eps, output + size_t(blockIdx.x) * width, sums);
}

__global__ void __launch_bounds__(THREADS) rope_halves_kernel(float* x, size_t count, size_t vectors, size_t width, size_t pairs,
                                                              const int32_t* positions, const float* frequencies) {
    const size_t index = size_t(blockIdx.x) * THREADS + threadIdx.x;
    if (index >= count) return;
    const size_t row = index / (vectors * pairs), rest = index % (vectors * pairs), vector = rest / pairs, pair = rest % pairs;
    float* v = x + (row * vectors + vector) * width;
    turn_pair(v + pair, v + pair + pairs, positions[row], frequencies[pair]);
}

// A row index outside the output is skipped (the reference's kernel would write there).
__global__ void __launch_bounds__(THREADS) scatter_kernel(const float* x, const int32_t* rows, size_t count, size_t width, float* out, size_t out_rows) {
    const size_t index = size_t(blockIdx.x) * THREADS + threadIdx.x;
    if (index >= count * width) return;
    const int32_t row = rows[index / width];
    if (row >= 0 && size_t(row) < out_rows) out[size_t(row) * width + index % width] = x[index];
}

// blockIdx.y = row; blockIdx.x = a query head, then the key heads, then the value heads.
__global__ void __launch_bounds__(THREADS) prepare_kernel(const float* q_full, float* k, const float* v, size_t heads, size_t kv_heads, size_t dim,
                                                          const float* q_weight, const float* k_weight, float eps, size_t pairs,
                                                          const int32_t* positions, const float* frequencies, float* q, float* gate, float* keys,
                                                          float* values, size_t context) {
    __shared__ float sums[THREADS];
    __shared__ float normed[MAX_DIM];
    const size_t row = blockIdx.y, vector = blockIdx.x, kv_width = kv_heads * dim;
    const unsigned t = threadIdx.x;
    const int32_t at = positions[row];
    const bool cached = at >= 0 && size_t(at) < context;      // a position outside the cache writes no row of it
    if (vector >= heads + kv_heads) {
        if (!cached) return;
        const size_t head = vector - heads - kv_heads;
        const float* source = v + (row * kv_heads + head) * dim;
        float* target = values + size_t(at) * kv_width + head * dim;
        for (size_t col = t; col < dim; col += THREADS) target[col] = source[col];
        return;
    }
    const bool query = vector < heads;
    const float* x = query ? q_full + (row * heads + vector) * 2 * dim : k + (row * kv_heads + (vector - heads)) * dim;
    if (query) {
        float* g = gate + (row * heads + vector) * dim;
        for (size_t col = t; col < dim; col += THREADS) g[col] = x[dim + col];
    }
    norm_row(x, query ? q_weight : k_weight, dim, eps, normed, sums);
    __syncthreads();
    for (size_t pair = t; pair < pairs; pair += THREADS) turn_pair(normed + pair, normed + pair + pairs, at, frequencies[pair]);
    __syncthreads();
    if (query) {
        float* target = q + (row * heads + vector) * dim;
        for (size_t col = t; col < dim; col += THREADS) target[col] = normed[col];
    } else {
        const size_t head = vector - heads;
        float* own = k + (row * kv_heads + head) * dim;
        float* cache_row = keys + (cached ? size_t(at) : 0) * kv_width + head * dim;
        for (size_t col = t; col < dim; col += THREADS) {
            own[col] = normed[col];
            if (cached) cache_row[col] = normed[col];
        }
    }
}

// rms norm of row blockIdx.x, its last 2 * pairs values turned in adjacent pairs, stored at row rows[blockIdx.x] of the output
// (the row itself without `rows`).  With a table the turns go there too: forward, and the inverse from the angle times -1.
__global__ void __launch_bounds__(THREADS) norm_rope_kernel(const float* input, const float* weight, size_t width, float eps, size_t pairs,
                                                            const int32_t* positions, const float* frequencies, const int32_t* rows, float* output,
                                                            size_t out_count, double2* forward, double2* inverse) {
    __shared__ float sums[THREADS];
    const size_t index = blockIdx.x;
    const float* row = input + index * width;
    const int64_t target = rows ? int64_t(rows[index]) : int64_t(index);
    const bool stored = target >= 0 && size_t(target) < out_count;      // a row outside the output is not stored (its table entry is)
    float* out = output + (stored ? size_t(target) : 0) * width;
    float sum = 0.0f;
    for (size_t col = threadIdx.x; col < width; col += THREADS) sum = fmaf(row[col], row[col], sum);
    const float scale = rsqrtf(tree_sum(sum, sums, THREADS) / float(width) + eps);
    const size_t plain = width - 2 * pairs;
    if (stored)
        for (size_t col = threadIdx.x; col < plain; col += THREADS) out[col] = row[col] * scale * weight[col];
    for (size_t pair = threadIdx.x; pair < pairs; pair += THREADS) {
        const size_t col = plain + 2 * pair;
        const double angle = double(positions[index]) * double(frequencies[pair]);
        double s, c;
        sincos(angle, &s, &c);
        const double a = row[col] * scale * weight[col], b = row[col + 1] * scale * weight[col + 1];
        if (stored) {
            out[col] = float(a * c - b * s);
            out[col + 1] = float(a * s + b * c);
        }
        if (forward) {
            forward[index * pairs + pair] = make_double2(c, s);
            sincos(angle * -1.0, &s, &c);
            inverse[index * pairs + pair] = make_double2(c, s);
        }
    }
}

unsigned launch_dim(uint64_t count, uint64_t most) {
    if (!count || count > most) throw std::runtime_error("Straydog op: a launch is out of range");
    return unsigned(count);
}

}  // namespace

extern "C" {

int sd_op_split(void* handle, const float* x, uint64_t rows, uint64_t width, float* first, float* second) {
    SD_OP_BEGIN
    if (!rows || !width) throw std::runtime_error("invalid Straydog split shape");
    op_span(value, x, checked_floats({rows, 2, width}), "a split input");
    op_span(value, first, checked_floats({rows, width}), "a split output");
    op_span(value, second, checked_floats({rows, width}), "a split output");
    const size_t count = checked_product({rows, width});
    split_kernel<<<checked_blocks(count), THREADS, 0, value.stream>>>(x, count, size_t(width), first, second);
    SD_OP_END
}

int sd_op_rms_norm(void* handle, const float* input, const float* weight, uint64_t rows, uint64_t width, float eps, float* output) {
    SD_OP_BEGIN
    if (!rows || !width) throw std::runtime_error("invalid Straydog norm shape");
    op_span(value, input, checked_floats({rows, width}), "a norm input");
    op_span(value, weight, checked_floats({width}), "a norm weight");
    op_span(value, output, checked_floats({rows, width}), "a norm output");
    rms_norm_kernel<<<launch_dim(rows, 0x7fffffffu), THREADS, 0, value.stream>>>(input, weight, size_t(width), eps, output);
    SD_OP_END
}

int sd_op_norm_rope(void* handle, const float* input, const float* weight, uint64_t rows, uint64_t width, float eps, uint64_t rope_dims,
                    const int32_t* positions, const float* frequencies, const int32_t* out_rows, float* out, uint64_t out_count) {
    SD_OP_BEGIN
    if (!rows || !width || rope_dims % 2 || rope_dims > width || (!out_rows && out_count < rows)) throw std::runtime_error("invalid Straydog norm shape");
    op_span(value, input, checked_floats({rows, width}), "a norm input");
    op_span(value, weight, checked_floats({width}), "a norm weight");
    if (rope_dims) {
        op_span(value, positions, checked_floats({rows}), "rope positions");
        op_span(value, frequencies, checked_floats({rope_dims / 2}), "rope frequencies");
    }
    op_span(value, out, checked_floats({out_count, width}), "a norm output");
    if (out_rows) {
        op_span(value, out_rows, checked_floats({rows}), "output rows");
        if (out == input) throw std::runtime_error("a scattered norm cannot run in place");
    }
    // an armed table of exactly these rows and pairs is filled by this launch (the arm is spent either way)
    const size_t pairs = size_t(rope_dims / 2), armed = value.turns_armed;
    value.turns_armed = 0;
    const bool publish = armed && armed == rows && pairs && pairs == value.turns_pairs && value.turns && value.turns_rows >= rows;
    norm_rope_kernel<<<launch_dim(rows, 0x7fffffffu), THREADS, 0, value.stream>>>(input, weight, size_t(width), eps, pairs, positions, frequencies,
                                                                                 out_rows, out, size_t(out_count), publish ? value.turns : nullptr,
                                                                                 publish ? value.turns + value.turns_rows * value.turns_pairs : nullptr);
    if (publish) { value.turns_ready = true; value.turns_ready_rows = size_t(rows); value.turns_ready_pairs = pairs; }
    SD_OP_END
}

int sd_attention_turns_reserve(void* handle, uint64_t rows, uint64_t rope_dims) {
    SD_OP_BEGIN
    if (rope_dims > 128 || rope_dims % 2) throw std::runtime_error("invalid Straydog attention rope");
    const size_t pairs = size_t(rope_dims / 2);
    if (rows && pairs && !(value.turns && value.turns_pairs == pairs && value.turns_rows >= rows)) {
        if (value.recording) throw std::runtime_error("an attention rope table cannot be allocated while a graph is recorded");
        if (value.turns && !value.graphs.empty()) throw std::runtime_error("an attention rope table cannot grow after a graph was recorded");
        if (value.turns) {
            SD_CHECK(hipStreamSynchronize(value.stream));
            release(value, value.turns);
            value.turns = nullptr;
        }
        value.turns = static_cast<double2*>(allocate(value, checked_product({rows, uint64_t(pairs), sizeof(double2), 2}), false));
        value.turns_rows = size_t(rows); value.turns_pairs = pairs; value.turns_armed = 0; value.turns_ready = false;
    }
    SD_OP_END
}

int sd_attention_turns_arm(void* handle, uint64_t rows) {
    SD_OP_BEGIN
    value.turns_armed = size_t(rows);
    value.turns_ready = false;
    SD_OP_END
}

int sd_op_rope_halves(void* handle, float* x, uint64_t rows, uint64_t vectors, uint64_t width, uint64_t rope_dims, const int32_t* positions,
                      const float* frequencies) {
    SD_OP_BEGIN
    if (!rows || !vectors || !rope_dims || rope_dims % 2 || rope_dims > width) throw std::runtime_error("invalid Straydog rope shape");
    op_span(value, x, checked_floats({rows, vectors, width}), "a rotated buffer");
    op_span(value, positions, checked_floats({rows}), "rope positions");
    op_span(value, frequencies, checked_floats({rope_dims / 2}), "rope frequencies");
    const size_t count = checked_product({rows, vectors, rope_dims / 2});
    rope_halves_kernel<<<checked_blocks(count), THREADS, 0, value.stream>>>(x, count, size_t(vectors), size_t(width), size_t(rope_dims / 2), positions,
                                                                           frequencies);
    SD_OP_END
}

int sd_op_scatter(void* handle, const float* x, const int32_t* rows, uint64_t count, uint64_t width, float* out, uint64_t out_rows) {
    SD_OP_BEGIN
    if (!count || !width || !out_rows) throw std::runtime_error("invalid Straydog scatter shape");
    op_span(value, x, checked_floats({count, width}), "written rows");
    op_span(value, rows, checked_floats({count}), "row indices");
    op_span(value, out, checked_floats({out_rows, width}), "a scatter output");
    scatter_kernel<<<checked_blocks(checked_product({count, width})), THREADS, 0, value.stream>>>(x, rows, size_t(count), size_t(width), out, size_t(out_rows));
    SD_OP_END
}

int sd_op_attention_prepare(void* handle, const float* q_full, float* k, const float* v, uint64_t rows, uint64_t heads, uint64_t kv_heads,
                            uint64_t dim, const float* q_weight, const float* k_weight, float eps, uint64_t rope_dims, const int32_t* positions,
                            const float* frequencies, float* q, float* gate, float* keys, float* values, uint64_t context) {
    SD_OP_BEGIN
    if (!rows || rows > 65535 || !heads || heads > 1024 || !kv_heads || kv_heads > 1024 || !dim || dim > MAX_DIM || rope_dims % 2 || rope_dims > dim ||
        !context)
        throw std::runtime_error("invalid Straydog attention prepare shape");
    const size_t kv_width = checked_product({kv_heads, dim});
    op_span(value, q_full, checked_floats({rows, heads, 2 * dim}), "an attention query projection");
    op_span(value, k, checked_floats({rows, kv_width}), "attention keys");
    op_span(value, v, checked_floats({rows, kv_width}), "attention values");
    op_span(value, q_weight, checked_floats({dim}), "a query norm weight");
    op_span(value, k_weight, checked_floats({dim}), "a key norm weight");
    op_span(value, positions, checked_floats({rows}), "rope positions");
    if (rope_dims) op_span(value, frequencies, checked_floats({rope_dims / 2}), "rope frequencies");
    op_span(value, q, checked_floats({rows, heads, dim}), "attention queries");
    op_span(value, gate, checked_floats({rows, heads, dim}), "attention gates");
    op_span(value, keys, checked_floats({context, kv_width}), "a key cache");
    op_span(value, values, checked_floats({context, kv_width}), "a value cache");
    const dim3 grid(launch_dim(heads + 2 * kv_heads, 0x7fffffffu), launch_dim(rows, 65535));
    prepare_kernel<<<grid, THREADS, 0, value.stream>>>(q_full, k, v, size_t(heads), size_t(kv_heads), size_t(dim), q_weight, k_weight, eps,
                                                      size_t(rope_dims / 2), positions, frequencies, q, gate, keys, values, size_t(context));
    SD_OP_END
}

}  // extern "C"
