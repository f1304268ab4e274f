// FP32 attention ops of the reference ABI, every product and sum in FP32:
//   sd_op_attention        causal GQA over FP32 caches (reference gpu/token_mixing.hpp:356-520, entry :652-693)
//   sd_attention_sequence  selection-list attention over the Qwen Q8_0/FP16 state (gpu/kernels.cpp:79-165, :4387-4419)
// One kernel serves both: a workgroup owns (row, K/V head, split of the keys) and all query heads of that K/V head,
// so each key and value is read once for the whole group.  Keys go through LDS 32 columns at a time (a thread per
// key sums its columns in order), the online softmax runs a wave per head with lane = key, values are summed a
// thread per column.  The splits' (max, sum, unnormalised output) are merged by a second kernel that also applies
// the optional sigmoid gate.
#include "device.hpp"
#include "kv_codec.hpp"
#include "../../include/straydog_gpu.h"

using namespace sd;

namespace {

constexpr int TILE = 64, SLICE = 32, THREADS = 256, MAX_GROUP = 16, MAX_COLS = 4;

// Keys and values of the FP32 caches [context][kv_heads][dim]; row r sees keys 0 .. min(positions[r] + 1, context) - 1.
struct DenseSource {
    const float* keys; const float* values; const int32_t* positions;
    size_t context, kv_heads, dim;
    __device__ size_t count(size_t row) const {
        const int64_t p = positions[row];
        const size_t length = p < 0 ? 0 : size_t(p) + 1;
        return length < context ? length : context;
    }
    __device__ bool valid(size_t, size_t) const { return true; }
    __device__ float key(size_t, size_t kvh, size_t i, size_t c) const { return keys[(i * kv_heads + kvh) * dim + c]; }
    __device__ float value(size_t, size_t kvh, size_t i, size_t c) const { return values[(i * kv_heads + kvh) * dim + c]; }
};

// The Qwen state: planes [2 * kv_heads][context] of K/V rows; row `step` attends the tokens its selection list names
// (floats; valid when 0 <= raw <= base + step and raw < context), `count` of them.
struct SelectedSource {
    const uint8_t* state; const float* indices; const float* counts;
    size_t context, base, selected, kv_heads, dim;
    unsigned row_bytes;
    __device__ size_t count(size_t row) const {
        const size_t n = size_t(counts[row]);
        return n < selected ? n : selected;
    }
    __device__ bool valid(size_t row, size_t i) const {
        const float raw = indices[row * selected + i];
        return raw >= 0 && raw <= float(base + row) && raw < float(context);
    }
    __device__ const uint8_t* at(size_t row, size_t plane, size_t i) const {
        return state + (plane * context + size_t(indices[row * selected + i])) * row_bytes;
    }
    __device__ float key(size_t row, size_t kvh, size_t i, size_t c) const { return kv_value(at(row, kvh, i), unsigned(c), unsigned(dim), row_bytes != 2 * dim); }
    __device__ float value(size_t row, size_t kvh, size_t i, size_t c) const { return kv_value(at(row, kv_heads + kvh, i), unsigned(c), unsigned(dim), row_bytes != 2 * dim); }
};

template<class Source>
__global__ void __launch_bounds__(THREADS) fp32_attention_kernel(Source source, const float* q, size_t heads, size_t kv_heads, size_t dim,
                                                                 float scale, float* partial) {
    const size_t item = blockIdx.x, split = blockIdx.y, splits = gridDim.y;
    const size_t row = item / kv_heads, kvh = item % kv_heads, group = heads / kv_heads;
    const unsigned t = threadIdx.x, lane = t % 64, wave = t / 64;
    extern __shared__ float lds[];
    float* qs = lds;                                  // [group][dim]
    float* ks = qs + group * dim;                     // [TILE][SLICE + 1]
    float* ps = ks + TILE * (SLICE + 1);              // [group][TILE]
    float* top = ps + group * TILE;                   // [group] running maximum
    float* total = top + group;                       // [group] running sum
    float* rescale = total + group;                   // [group] this tile's correction
    for (size_t i = t; i < group * dim; i += THREADS) qs[i] = q[(row * heads + kvh * group) * dim + i];
    for (size_t i = t; i < group; i += THREADS) { top[i] = -INFINITY; total[i] = 0.0f; }
    const size_t length = source.count(row), share = (length + splits - 1) / splits;
    const size_t begin = min(length, split * share), end = min(length, begin + share);
    float out[MAX_GROUP][MAX_COLS];
    #pragma unroll
    for (int h = 0; h < MAX_GROUP; ++h)
        #pragma unroll
        for (int a = 0; a < MAX_COLS; ++a) out[h][a] = 0.0f;
    __syncthreads();
    for (size_t start = begin; start < end; start += TILE) {
        const size_t count = min(size_t(TILE), end - start);
        // scores: thread (key = lane, heads wave, wave + 4, ...) sums its key's columns in order
        const bool present = lane < count && source.valid(row, start + lane);
        float acc[MAX_GROUP / 4];
        #pragma unroll
        for (int j = 0; j < MAX_GROUP / 4; ++j) acc[j] = 0.0f;
        for (size_t d0 = 0; d0 < dim; d0 += SLICE) {
            __syncthreads();
            for (unsigned e = t; e < TILE * SLICE; e += THREADS) {
                const unsigned key = e / SLICE, c = e % SLICE;
                float value = 0.0f;
                if (key < count && d0 + c < dim && source.valid(row, start + key)) value = source.key(row, kvh, start + key, d0 + c);
                ks[key * (SLICE + 1) + c] = value;
            }
            __syncthreads();
            const size_t width = min(size_t(SLICE), dim - d0);
            #pragma unroll
            for (int j = 0; j < MAX_GROUP / 4; ++j) {
                const size_t h = wave + 4 * j;
                if (h < group) {
                    float sum = acc[j];
                    for (size_t c = 0; c < width; ++c) sum += qs[h * dim + d0 + c] * ks[lane * (SLICE + 1) + c];
                    acc[j] = sum;
                }
            }
        }
        #pragma unroll
        for (int j = 0; j < MAX_GROUP / 4; ++j) {
            const size_t h = wave + 4 * j;
            if (h < group) ps[h * TILE + lane] = present ? acc[j] * scale : -INFINITY;
        }
        __syncthreads();
        // online softmax: a wave per head, lane = key
        for (size_t h = wave; h < group; h += 4) {
            const float s = ps[h * TILE + lane];
            float tile_top = s;
            for (unsigned offset = 32; offset; offset /= 2) tile_top = fmaxf(tile_top, __shfl_xor(tile_top, offset));
            const float before = top[h], now = fmaxf(before, tile_top);
            const float w = s == -INFINITY ? 0.0f : expf(s - now);
            float sum = w;
            for (unsigned offset = 32; offset; offset /= 2) sum += __shfl_xor(sum, offset);
            const float correction = before == -INFINITY ? 0.0f : expf(before - now);
            ps[h * TILE + lane] = w;
            if (!lane) { top[h] = now; total[h] = total[h] * correction + sum; rescale[h] = correction; }
        }
        __syncthreads();
        // values: a thread per column
        #pragma unroll
        for (int a = 0; a < MAX_COLS; ++a) {
            const size_t d = t + size_t(a) * THREADS;
            if (d >= dim) break;
            #pragma unroll
            for (int h = 0; h < MAX_GROUP; ++h) if (size_t(h) < group) out[h][a] *= rescale[h];
            for (size_t i = 0; i < count; ++i) {
                if (!source.valid(row, start + i)) continue;
                const float v = source.value(row, kvh, start + i, d);
                #pragma unroll
                for (int h = 0; h < MAX_GROUP; ++h) if (size_t(h) < group) out[h][a] += ps[h * TILE + i] * v;
            }
        }
        __syncthreads();
    }
    #pragma unroll
    for (int h = 0; h < MAX_GROUP; ++h) {
        if (size_t(h) >= group) break;
        float* mine = partial + ((row * heads + kvh * group + h) * splits + split) * (dim + 2);
        #pragma unroll
        for (int a = 0; a < MAX_COLS; ++a) {
            const size_t d = t + size_t(a) * THREADS;
            if (d < dim) mine[d] = out[h][a];
        }
        if (!t) { mine[dim] = top[h]; mine[dim + 1] = total[h]; }
    }
}

// (row, head): the splits merged, normalised, gated.  A split that saw nothing has maximum -inf and weighs 0.
__global__ void __launch_bounds__(THREADS) fp32_attention_merge_kernel(const float* partial, size_t splits, size_t dim, const float* gate, float* out) {
    const size_t pair = blockIdx.x;
    const float* first = partial + pair * splits * (dim + 2);
    float top = -INFINITY;
    for (size_t s = 0; s < splits; ++s) top = fmaxf(top, first[s * (dim + 2) + dim]);
    float total = 0.0f;
    for (size_t s = 0; s < splits; ++s) {
        const float m = first[s * (dim + 2) + dim];
        total += m == -INFINITY ? 0.0f : first[s * (dim + 2) + dim + 1] * expf(m - top);
    }
    for (size_t d = threadIdx.x; d < dim; d += THREADS) {
        float sum = 0.0f;
        for (size_t s = 0; s < splits; ++s) {
            const float m = first[s * (dim + 2) + dim];
            if (m != -INFINITY) sum += first[s * (dim + 2) + d] * expf(m - top);
        }
        float value = sum / total;
        if (gate) value *= 1.0f / (1.0f + expf(-gate[pair * dim + d]));
        out[pair * dim + d] = value;
    }
}

// The new rows of sd_attention_sequence into the state's planes (reference write_attention_kv, gpu/kernels.cpp:79-98).
__global__ void __launch_bounds__(THREADS) state_write_kernel(uint8_t* state, unsigned row_bytes, size_t context, size_t base, size_t steps,
                                                              size_t heads, size_t kv_heads, unsigned dim, const float* input) {
    const size_t index = size_t(blockIdx.x) * blockDim.x + threadIdx.x, quads = dim / 4, per_kind = steps * kv_heads * quads;
    const bool live = index < 2 * per_kind;
    const size_t at = live ? index % per_kind : 0;
    const bool is_value = live && index >= per_kind;
    const size_t quad = at % quads, head = at / quads % kv_heads, step = at / quads / kv_heads;
    const float* from = input + steps * heads * dim + (is_value ? steps * kv_heads * dim : 0) + (step * kv_heads + head) * dim + quad * 4;
    const float x[4] = {from[0], from[1], from[2], from[3]};
    uint8_t* row = state + (((is_value ? kv_heads : 0) + head) * context + base + step) * row_bytes;
    kv_store_quad(row, unsigned(quad), dim, row_bytes != 2 * dim, x, live);
}

size_t attention_lds(size_t group, size_t dim) { return (group * dim + TILE * (SLICE + 1) + group * TILE + 3 * group) * 4; }

template<class Source>
void launch(Device& d, const Source& source, const float* q, size_t rows, size_t heads, size_t kv_heads, size_t dim, float scale,
            size_t splits, float* partial, const float* gate, float* out) {
    const size_t shared = attention_lds(heads / kv_heads, dim);
    raise_shared_limit(d, reinterpret_cast<const void*>(&fp32_attention_kernel<Source>), 160 * 1024 - 64);
    fp32_attention_kernel<Source><<<dim3(unsigned(rows * kv_heads), unsigned(splits)), THREADS, shared, d.stream>>>(source, q, heads, kv_heads, dim, scale, partial);
    SD_CHECK(hipGetLastError());
    fp32_attention_merge_kernel<<<unsigned(rows * heads), THREADS, 0, d.stream>>>(partial, splits, dim, gate, out);
}

}  // namespace

extern "C" {

int sd_op_attention(void* handle, const float* q, const float* keys, const float* values, uint64_t context, const int32_t* positions,
                    uint64_t rows, uint64_t heads, uint64_t kv_heads, uint64_t dim, float scale, const float* gate, float* scratch,
                    uint64_t scratch_bytes, float* out) {
    SD_OP_BEGIN
    if (!rows || !heads || !kv_heads || heads % kv_heads || heads / kv_heads > MAX_GROUP || !dim || dim > 1024 || !context ||
        checked_product({rows, heads}) > 65535 * 64)
        throw std::runtime_error("invalid Straydog attention shape");
    op_span(value, q, checked_floats({rows, heads, dim}), "attention queries");
    op_span(value, keys, checked_floats({context, kv_heads, dim}), "attention keys");
    op_span(value, values, checked_floats({context, kv_heads, dim}), "attention values");
    op_span(value, positions, checked_floats({rows}), "attention positions");
    if (gate) op_span(value, gate, checked_floats({rows, heads, dim}), "an attention gate");
    op_span(value, out, checked_floats({rows, heads, dim}), "an attention output");
    // the reference's split count and scratch contract (gpu/token_mixing.hpp:677-681)
    const size_t pairs = size_t(rows * heads);
    const size_t splits = std::min<size_t>(64, std::max<size_t>(1, 256 / pairs));
    const size_t partial_bytes = checked_floats({pairs, splits, dim + 2});
    if (!scratch || scratch_bytes < partial_bytes) throw std::runtime_error("Straydog attention scratch too small");
    op_span(value, scratch, partial_bytes, "attention scratch");
    if (attention_lds(size_t(heads / kv_heads), size_t(dim)) > 160 * 1024 - 64) throw std::runtime_error("invalid Straydog attention shape");
    const DenseSource source{keys, values, positions, size_t(context), size_t(kv_heads), size_t(dim)};
    launch(value, source, q, size_t(rows), size_t(heads), size_t(kv_heads), size_t(dim), scale, splits, scratch, gate, out);
    SD_OP_END
}

int sd_attention_sequence(void* handle, void* state, uint64_t context, uint64_t base, uint64_t steps, uint64_t selected,
                          const float* input, uint64_t input_count, float* output, uint64_t output_count) {
    try {
        Device& value = device(handle);
        constexpr size_t HEADS = 24, KV = 2, DIM = 256, MAX_BATCH = 256;
        if (!input || !output || !context || context > 262144 || !steps || steps > MAX_BATCH || base > context || steps > context - base ||
            !selected || selected > 2052)
            throw std::runtime_error("invalid Straydog attention dimensions");
        {
            std::lock_guard<std::mutex> lock(value.mutex);
            const auto found = value.allocations.find(static_cast<const uint8_t*>(state));
            if (found == value.allocations.end() || found->second != context * 4 * value.kv_row)
                throw std::runtime_error("Straydog attention state size mismatch");
        }
        if (input_count != steps * (HEADS * DIM + 2 * KV * DIM + selected + 1) || output_count != steps * HEADS * DIM)
            throw std::runtime_error("Straydog attention workspace mismatch");
        // Counts are host-readable metadata; validate before any kernel reads them.
        const size_t count_offset = size_t(steps * (HEADS * DIM + 2 * KV * DIM + selected));
        for (size_t step = 0; step < steps; ++step) {
            const float count = input[count_offset + step];
            if (!(count >= 1 && count <= float(selected)) || count != float(size_t(count)))
                throw std::runtime_error("invalid Straydog attention selection count");
        }
        const size_t input_bytes = size_t(input_count) * 4, output_bytes = size_t(output_count) * 4;
        const size_t partial_bytes = size_t(steps) * HEADS * (DIM + 2) * 4;
        uint8_t* space = static_cast<uint8_t*>(workspace(value, input_bytes + output_bytes + partial_bytes + 512));
        float* device_input = reinterpret_cast<float*>(space);
        float* device_output = reinterpret_cast<float*>(space + ((input_bytes + 255) & ~size_t(255)));
        float* partial = reinterpret_cast<float*>(space + ((input_bytes + 255) & ~size_t(255)) + ((output_bytes + 255) & ~size_t(255)));
        upload(value, device_input, input, input_bytes);
        const size_t quads = 2 * size_t(steps) * KV * (DIM / 4);
        state_write_kernel<<<checked_blocks(quads), THREADS, 0, value.stream>>>(static_cast<uint8_t*>(state), value.kv_row, size_t(context),
            size_t(base), size_t(steps), HEADS, KV, unsigned(DIM), device_input);
        SD_CHECK(hipGetLastError());
        const size_t index_start = size_t(steps) * (HEADS * DIM + 2 * KV * DIM);
        const SelectedSource source{static_cast<const uint8_t*>(state), device_input + index_start, device_input + index_start + steps * selected,
                                    size_t(context), size_t(base), size_t(selected), KV, DIM, value.kv_row};
        launch(value, source, device_input, size_t(steps), HEADS, KV, DIM, 0.0625f, 1, partial, nullptr, device_output);
        SD_CHECK(hipGetLastError());
        download(value, output, device_output, output_bytes);
        return 0;
    } catch (const std::exception& e) { last_error = e.what(); return -1; }
}

}  // extern "C"
