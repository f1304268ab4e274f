// The inputs of a dense attention step over FP32 caches, as the reference prepares them for sd_op_attention:
//   sd_op_split             [query | gate] rows apart                       gpu/token_mixing.hpp:246-252, :628-637
//   sd_op_rms_norm          x / sqrt(mean(x^2) + eps) * weight per row      gpu/ops.hpp:28-59, gpu/kernels.cpp:4901-4913
//   sd_op_rope_halves       pairs (i, i + pairs) turned, angles in double   gpu/token_mixing.hpp:254-274, :639-650
//   sd_op_scatter           rows to the rows an index list names            gpu/ops.hpp:1171-1175, gpu/kernels.cpp:5244-5252
//   sd_op_attention_prepare all of it for one step in one launch            gpu/token_mixing.hpp:276-338, :601-626
//   sd_op_norm_rope         rms norm, then the last values turned in adjacent pairs, rows scattered; fills the attention rope
//                           table when one is armed                          gpu/ops.hpp:60-106, gpu/kernels.cpp:4915-4940
//   sd_attention_turns_reserve / _arm   that table                          gpu/kernels.cpp:558-616, :5288-5303
//
// What the results' bits depend on, and all that is taken from the reference: a row's sum of squares is 256 partial sums --
// partial t over the columns t, t + 256, ... by fused multiply-adds -- added in halving-tree order; the scale is rsqrt of the
// mean plus eps; a value is (x * scale) * weight; a pair is turned by sincos of double(position) * double(frequency) with the
// products in double.  The fused entry gives the bits of the separate ones (the reference's test, tests/fused_gpu.rs:225-268).
//
// Shape of the work on gfx950: ONE WAVE PER VECTOR, no LDS and no barriers.  Lane L of a wave64 holds the four partial sums
// L, L + 64, L + 128, L + 192 of its vector, so the halving tree's first two levels are two adds inside the lane and the other
// six are lane shifts; the scale is then in every lane and each lane scales and turns the columns it read.  A workgroup is four
// independent waves (four vectors).  An angle depends on (row, pair) only, so the rope entry forms each sincos once and turns
// that pair in every vector of the row.
#include "device.hpp"
#include "../../include/straydog_gpu.h"

using namespace sd;

namespace {

constexpr unsigned LANES = 64, WAVES = 4, THREADS = LANES * WAVES;
constexpr unsigned PARTIALS = 256;            // the sums' shape: column c belongs to partial sum c % 256
constexpr uint64_t MAX_DIM = 1024;

struct Turn { double cosine, sine; };
__device__ __forceinline__ Turn turn_of(int32_t position, float frequency) {
    Turn t;
    sincos(double(position) * double(frequency), &t.sine, &t.cosine);
    return t;
}
// (a, b) turned; every entry point goes through this one expression, so fused and separate results are the same bits
__device__ __forceinline__ float2 turned(float first, float second, const Turn& t) {
    const double a = first, b = second;
    return make_float2(float(a * t.cosine - b * t.sine), float(a * t.sine + b * t.cosine));
}

// rsqrt(mean(x^2) + eps) of a vector, the same value in every lane of the wave that calls it.
__device__ __forceinline__ float wave_scale(const float* x, size_t width, float eps, unsigned lane) {
    float partial[PARTIALS / LANES] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (size_t first = 0; first < width; first += PARTIALS)
        #pragma unroll
        for (unsigned j = 0; j < PARTIALS / LANES; ++j) {
            const size_t col = first + j * LANES + lane;
            if (col < width) partial[j] = fmaf(x[col], x[col], partial[j]);
        }
    // tree levels 128 and 64 pair partial t with t + 128, then t with t + 64: both partners sit in this lane
    float sum = (partial[0] + partial[2]) + (partial[1] + partial[3]);
    #pragma unroll
    for (unsigned offset = LANES / 2; offset; offset /= 2) sum += __shfl_down(sum, offset);
    sum = __shfl(sum, 0);
    return rsqrtf(sum / float(width) + eps);
}

__device__ __forceinline__ unsigned wave_in_grid() { return blockIdx.x * WAVES + threadIdx.x / LANES; }

// first | second halves of every row pulled apart; a thread moves four floats when the width allows it.
template<typename Piece>
__global__ void __launch_bounds__(THREADS) split_kernel(const Piece* x, size_t pieces, size_t width, Piece* first, Piece* second) {
    const size_t at = size_t(blockIdx.x) * THREADS + threadIdx.x;
    if (at >= pieces) return;
    const Piece* from = x + at + at / width * width;       // row r of the input starts 2 * r * width pieces in
    first[at] = from[0];
    second[at] = from[width];
}

__global__ void __launch_bounds__(THREADS) rms_norm_kernel(const float* input, const float* weight, size_t rows, size_t width, float eps, float* output) {
    const size_t row = wave_in_grid();
    if (row >= rows) return;
    const unsigned lane = threadIdx.x % LANES;
    const float* x = input + row * width;
    float* out = output + row * width;
    const float scale = wave_scale(x, width, eps, lane);
    for (size_t col = lane; col < width; col += LANES) out[col] = x[col] * scale * weight[col];
}

// A thread per (row, pair): one sincos, then that pair of every vector of the row.
__global__ void __launch_bounds__(THREADS) rope_halves_kernel(float* x, size_t count, size_t vectors, size_t width, size_t pairs,
                                                              const int32_t* positions, const float* frequencies) {
    const size_t at = size_t(blockIdx.x) * THREADS + threadIdx.x;
    if (at >= count) return;
    const size_t row = at / pairs, pair = at % pairs;
    const Turn t = turn_of(positions[row], frequencies[pair]);
    float* v = x + row * vectors * width + pair;
    for (size_t vector = 0; vector < vectors; ++vector, v += width) {
        const float2 pair_out = turned(v[0], v[pairs], t);
        v[0] = pair_out.x;
        v[pairs] = pair_out.y;
    }
}

// A wave per written row.  A row index outside the output is skipped (the reference's kernel would write there).
__global__ void __launch_bounds__(THREADS) scatter_kernel(const float* x, const int32_t* rows, size_t count, size_t width, float* out, size_t out_rows) {
    const size_t source = wave_in_grid();
    if (source >= count) return;
    const int64_t target = rows[source];
    if (target < 0 || size_t(target) >= out_rows) return;
    const float* from = x + source * width;
    float* to = out + size_t(target) * width;
    for (size_t col = threadIdx.x % LANES; col < width; col += LANES) to[col] = from[col];
}

// One step's inputs in one launch.  Wave w of the grid takes vector w % per_row of row w / per_row, per_row = heads + 2 *
// kv_heads: the query heads (split off their gates, normed, turned), the key heads (normed, turned, written back and into the
// cache row of the position), the value heads (copied into the cache row).
struct PrepareArgs {
    const float* q_full; float* k; const float* v;
    size_t rows, heads, kv_heads, dim, pairs, context;
    const float *q_weight, *k_weight;
    float eps;
    const int32_t* positions; const float* frequencies;
    float *q, *gate, *keys, *values;
};
__global__ void __launch_bounds__(THREADS) prepare_kernel(PrepareArgs a) {
    const size_t per_row = a.heads + 2 * a.kv_heads, wave = wave_in_grid();
    if (wave >= a.rows * per_row) return;
    const size_t row = wave / per_row, vector = wave % per_row;
    const unsigned lane = threadIdx.x % LANES;
    const int32_t position = a.positions[row];
    const bool cached = position >= 0 && size_t(position) < a.context;      // a position outside the cache writes no row of it
    const size_t cache_at = (cached ? size_t(position) : 0) * a.kv_heads * a.dim;
    if (vector >= a.heads + a.kv_heads) {
        if (!cached) return;
        const size_t head = vector - a.heads - a.kv_heads;
        const float* from = a.v + (row * a.kv_heads + head) * a.dim;
        float* to = a.values + cache_at + head * a.dim;
        for (size_t col = lane; col < a.dim; col += LANES) to[col] = from[col];
        return;
    }
    const bool is_query = vector < a.heads;
    const size_t head = is_query ? vector : vector - a.heads;
    const float* x = is_query ? a.q_full + (row * a.heads + head) * 2 * a.dim : a.k + (row * a.kv_heads + head) * a.dim;
    const float* weight = is_query ? a.q_weight : a.k_weight;
    float* out = is_query ? a.q + (row * a.heads + head) * a.dim : a.k + (row * a.kv_heads + head) * a.dim;   // keys in place
    float* cache_row = !is_query && cached ? a.keys + cache_at + head * a.dim : nullptr;
    if (is_query) {
        float* g = a.gate + (row * a.heads + head) * a.dim;
        for (size_t col = lane; col < a.dim; col += LANES) g[col] = x[a.dim + col];
    }
    // every lane has read all it needs of x before any lane has the scale, so the keys may be overwritten below
    const float scale = wave_scale(x, a.dim, a.eps, lane);
    const auto store = [&](size_t col, float value) {
        out[col] = value;
        if (cache_row) cache_row[col] = value;
    };
    for (size_t pair = lane; pair < a.pairs; pair += LANES) {
        const size_t partner = pair + a.pairs;
        const float2 pair_out = turned(x[pair] * scale * weight[pair], x[partner] * scale * weight[partner], turn_of(position, a.frequencies[pair]));
        store(pair, pair_out.x);
        store(partner, pair_out.y);
    }
    for (size_t col = 2 * a.pairs + lane; col < a.dim; col += LANES) store(col, x[col] * scale * weight[col]);
}

// A wave per row: rms norm, the last 2 * pairs values turned in adjacent pairs, stored at row rows[index] of the output (the
// row itself without `rows`).  With a table the turns go there too: forward, and the inverse from the angle times -1.
__global__ void __launch_bounds__(THREADS) norm_rope_kernel(const float* input, const float* weight, size_t count, size_t width, float eps, size_t pairs,
                                                            const int32_t* positions, const float* frequencies, const int32_t* rows, float* output,
                                                            size_t out_count, double2* forward, double2* inverse) {
    const size_t index = wave_in_grid();
    if (index >= count) return;
    const unsigned lane = threadIdx.x % LANES;
    const float* x = input + index * width;
    const int64_t target = rows ? int64_t(rows[index]) : int64_t(index);
    const bool stored = target >= 0 && size_t(target) < out_count;      // a row outside the output is not stored (its table entry is)
    float* out = output + (stored ? size_t(target) : 0) * width;
    const float scale = wave_scale(x, width, eps, lane);
    const size_t plain = width - 2 * pairs;
    for (size_t pair = lane; pair < pairs; pair += LANES) {
        const size_t col = plain + 2 * pair;
        const double angle = double(positions[index]) * double(frequencies[pair]);
        Turn t;
        sincos(angle, &t.sine, &t.cosine);
        const float2 pair_out = turned(x[col] * scale * weight[col], x[col + 1] * scale * weight[col + 1], t);
        if (forward) {
            forward[index * pairs + pair] = make_double2(t.cosine, t.sine);
            Turn back;
            sincos(angle * -1.0, &back.sine, &back.cosine);
            inverse[index * pairs + pair] = make_double2(back.cosine, back.sine);
        }
        if (stored) { out[col] = pair_out.x; out[col + 1] = pair_out.y; }
    }
    if (stored)
        for (size_t col = lane; col < plain; col += LANES) out[col] = x[col] * scale * weight[col];
}

// Workgroups of four waves for `waves` waves.
unsigned wave_grid(uint64_t waves) {
    const uint64_t groups = (waves + WAVES - 1) / WAVES;
    if (!groups || groups > 0x7fffffffu) throw std::runtime_error("Straydog op: a launch is out of range");
    return unsigned(groups);
}

void require(bool shape_ok, const char* op) {
    if (!shape_ok) throw std::runtime_error(std::string("invalid Straydog ") + op + " shape");
}

// What the rope operands of an op must cover.
void rope_operands(Device& d, const int32_t* positions, const float* frequencies, uint64_t rows, uint64_t pairs) {
    op_span(d, positions, checked_floats({rows}), "rope positions");
    op_span(d, frequencies, checked_floats({pairs}), "rope frequencies");
}

}  // namespace

extern "C" {

int sd_op_split(void* handle, const float* x, uint64_t rows, uint64_t width, float* first, float* second) {
    SD_OP_BEGIN
    require(rows && width, "split");
    const size_t half = checked_floats({rows, width});
    op_span(value, x, checked_product({half, 2}), "a split input");
    op_span(value, first, half, "a split output");
    op_span(value, second, half, "a split output");
    const auto aligned = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
    if (width % 4 == 0 && aligned(x) && aligned(first) && aligned(second))
        split_kernel<float4><<<checked_blocks(half / 16), THREADS, 0, value.stream>>>(reinterpret_cast<const float4*>(x), half / 16, size_t(width / 4),
                                                                                     reinterpret_cast<float4*>(first), reinterpret_cast<float4*>(second));
    else
        split_kernel<float><<<checked_blocks(half / 4), THREADS, 0, value.stream>>>(x, half / 4, size_t(width), first, second);
    SD_OP_END
}

int sd_op_rms_norm(void* handle, const float* input, const float* weight, uint64_t rows, uint64_t width, float eps, float* output) {
    SD_OP_BEGIN
    require(rows && width, "norm");
    const size_t bytes = checked_floats({rows, width});
    op_span(value, input, bytes, "a norm input");
    op_span(value, weight, checked_floats({width}), "a norm weight");
    op_span(value, output, bytes, "a norm output");
    rms_norm_kernel<<<wave_grid(rows), THREADS, 0, value.stream>>>(input, weight, size_t(rows), size_t(width), eps, output);
    SD_OP_END
}

int sd_op_norm_rope(void* handle, const float* input, const float* weight, uint64_t rows, uint64_t width, float eps, uint64_t rope_dims,
                    const int32_t* positions, const float* frequencies, const int32_t* out_rows, float* out, uint64_t out_count) {
    SD_OP_BEGIN
    const uint64_t pairs = rope_dims / 2;
    require(rows && width && rope_dims % 2 == 0 && rope_dims <= width && (out_rows || out_count >= rows), "norm");
    op_span(value, input, checked_floats({rows, width}), "a norm input");
    op_span(value, weight, checked_floats({width}), "a norm weight");
    if (pairs) rope_operands(value, positions, frequencies, rows, pairs);
    op_span(value, out, checked_floats({out_count, width}), "a norm output");
    if (out_rows) {
        op_span(value, out_rows, checked_floats({rows}), "output rows");
        if (out == input) throw std::runtime_error("a scattered norm cannot run in place");
    }
    // The pass's rope table: an arm is spent by the next call whatever its shape; the call fills the table only if it has
    // exactly the armed rows and the table's pairs.
    const size_t armed = value.turns_armed;
    value.turns_armed = 0;
    const bool fills = armed && armed == rows && pairs && pairs == value.turns_pairs && value.turns && value.turns_rows >= rows;
    double2* const forward = fills ? value.turns : nullptr;
    norm_rope_kernel<<<wave_grid(rows), THREADS, 0, value.stream>>>(input, weight, size_t(rows), size_t(width), eps, size_t(pairs), positions, frequencies,
                                                                   out_rows, out, size_t(out_count), forward,
                                                                   fills ? forward + value.turns_rows * value.turns_pairs : nullptr);
    if (fills) { value.turns_ready = true; value.turns_ready_rows = size_t(rows); value.turns_ready_pairs = size_t(pairs); }
    SD_OP_END
}

int sd_attention_turns_reserve(void* handle, uint64_t rows, uint64_t rope_dims) {
    SD_OP_BEGIN
    if (rope_dims > 128 || rope_dims % 2) throw std::runtime_error("invalid Straydog attention rope");
    const size_t pairs = size_t(rope_dims / 2);
    const bool enough = value.turns && value.turns_pairs == pairs && value.turns_rows >= rows;
    if (rows && pairs && !enough) {
        // a recorded graph holds the table's address: it is neither made nor moved once one exists or is being made
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
    const uint64_t pairs = rope_dims / 2;
    require(rows && vectors && pairs && rope_dims % 2 == 0 && rope_dims <= width, "rope");
    op_span(value, x, checked_floats({rows, vectors, width}), "a rotated buffer");
    rope_operands(value, positions, frequencies, rows, pairs);
    const size_t count = checked_product({rows, pairs});
    rope_halves_kernel<<<checked_blocks(count), THREADS, 0, value.stream>>>(x, count, size_t(vectors), size_t(width), size_t(pairs), positions, frequencies);
    SD_OP_END
}

int sd_op_scatter(void* handle, const float* x, const int32_t* rows, uint64_t count, uint64_t width, float* out, uint64_t out_rows) {
    SD_OP_BEGIN
    require(count && width && out_rows, "scatter");
    op_span(value, x, checked_floats({count, width}), "written rows");
    op_span(value, rows, checked_floats({count}), "row indices");
    op_span(value, out, checked_floats({out_rows, width}), "a scatter output");
    scatter_kernel<<<wave_grid(count), THREADS, 0, value.stream>>>(x, rows, size_t(count), size_t(width), out, size_t(out_rows));
    SD_OP_END
}

int sd_op_attention_prepare(void* handle, const float* q_full, float* k, const float* v, uint64_t rows, uint64_t heads, uint64_t kv_heads,
                            uint64_t dim, const float* q_weight, const float* k_weight, float eps, uint64_t rope_dims, const int32_t* positions,
                            const float* frequencies, float* q, float* gate, float* keys, float* values, uint64_t context) {
    SD_OP_BEGIN
    const auto counted = [](uint64_t n, uint64_t most) { return n && n <= most; };
    require(counted(rows, 65535) && counted(heads, 1024) && counted(kv_heads, 1024) && counted(dim, MAX_DIM) && rope_dims % 2 == 0 && rope_dims <= dim && context,
            "attention prepare");
    PrepareArgs args{q_full, k, v, size_t(rows), size_t(heads), size_t(kv_heads), size_t(dim), size_t(rope_dims / 2), size_t(context),
                     q_weight, k_weight, eps, positions, frequencies, q, gate, keys, values};
    const size_t per_query = checked_floats({rows, heads, dim}), per_kv = checked_floats({rows, kv_heads, dim}), cache = checked_floats({context, kv_heads, dim});
    op_span(value, q_full, checked_product({per_query, 2}), "an attention query projection");
    op_span(value, k, per_kv, "attention keys");
    op_span(value, v, per_kv, "attention values");
    op_span(value, q_weight, checked_floats({dim}), "a query norm weight");
    op_span(value, k_weight, checked_floats({dim}), "a key norm weight");
    op_span(value, positions, checked_floats({rows}), "rope positions");
    if (args.pairs) op_span(value, frequencies, checked_floats({args.pairs}), "rope frequencies");
    op_span(value, q, per_query, "attention queries");
    op_span(value, gate, per_query, "attention gates");
    op_span(value, keys, cache, "a key cache");
    op_span(value, values, cache, "a value cache");
    prepare_kernel<<<wave_grid(checked_product({rows, heads + 2 * kv_heads})), THREADS, 0, value.stream>>>(args);
    SD_OP_END
}

}  // extern "C"
