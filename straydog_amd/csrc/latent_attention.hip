// Latent sparse attention: each query attends a sliding window of raw rows and the compressed rows its selection
// lists, the same row serving as key and value, with an optional per-head sink that enters the maximum and the
// denominator only (reference gpu/ops.hpp:1240-1297, rope :1318-1328, entry gpu/kernels.cpp:5311-5476; CPU twin
// crates/straydog-engine/examples/ds41_reference.rs:385-411).  The batched entry of the sparse top-k path uses the
// same kernel without window or sink, keys kdim wide and values their first vdim columns.
//
// A workgroup owns one row and 8 of its heads, so a gathered row is read once for 8 heads: scores with 8 adjacent
// lanes (the heads) sharing a key row, a wave per head for the softmax, then a thread per output column.
#include "device.hpp"
#include "../../include/straydog_gpu.h"
#include "../../include/straydog_gpu_ext.h"

using namespace sd;

namespace sd {
bool latent_gather_supported(uint64_t kdim, uint64_t vdim);
uint64_t latent_gather_scratch(uint64_t batch, uint64_t k, uint64_t heads, uint64_t vdim);
void latent_gather(Device& d, const void* q, const void* latents, const int32_t* selected, uint64_t batch, uint64_t groups, uint64_t k,
                   uint64_t heads, float scale, float* out, float* partial);
}

namespace {

constexpr int HB = 8, THREADS = 256, PAD = 4, MAX_COLS = 4;

struct LatentArgs {
    const float* q;                 // [rows][heads][kdim]
    const uint16_t* q_bf16;         // or BF16 queries (the batched entry)
    const float* raw; size_t raw_rows;
    const int32_t* positions; size_t window;
    const void* compressed; size_t compressed_batch_stride;   // values per row of the batch (0: one table for every row)
    const int32_t* selected; size_t selections;
    const float* sinks;
    size_t heads, kdim, vdim;
    float scale;
    size_t pairs; const float* frequencies;
    const double2* forward; const double2* inverse;   // the pass's rope table (cosine, sine per row and pair), or null: angles formed here
    float* out;
};

template<bool BF16>
__device__ __forceinline__ float latent_value(const void* row, size_t col) {
    if (BF16) return __uint_as_float(uint32_t(static_cast<const uint16_t*>(row)[col]) << 16);
    return static_cast<const float*>(row)[col];
}

template<bool BF16>
__global__ void __launch_bounds__(THREADS) latent_attention_kernel(LatentArgs a) {
    const size_t row = blockIdx.y, head0 = size_t(blockIdx.x) * HB;
    const unsigned t = threadIdx.x, lane = t % 64, wave = t / 64;
    const size_t heads_here = min(size_t(HB), a.heads - head0);
    const int64_t p = a.positions ? a.positions[row] : 0;
    const int64_t first = a.window ? (p - int64_t(a.window) + 1 < 0 ? 0 : p - int64_t(a.window) + 1) : 0;
    const size_t raw_count = a.window ? size_t(p - first + 1) : 0, total = raw_count + a.selections;
    const size_t stride = a.kdim + PAD;
    extern __shared__ float lds[];
    float* qs = lds;                         // [HB][kdim + PAD]; reused for the output rows at the end
    float* w = qs + HB * stride;             // [HB][total]
    float* denominators = w + HB * total;    // [HB]
    // queries, their last 2 * pairs values rotated (angle, sine and cosine in double)
    const size_t rotated = a.kdim - 2 * a.pairs;
    for (size_t i = t; i < heads_here * a.kdim; i += THREADS) {
        const size_t h = i / a.kdim, c = i % a.kdim, at = (row * a.heads + head0 + h) * a.kdim;
        const auto load = [&](size_t col) { return a.q_bf16 ? __uint_as_float(uint32_t(a.q_bf16[at + col]) << 16) : a.q[at + col]; };
        float value = load(c);
        if (c >= rotated) {
            const size_t pair = (c - rotated) / 2;
            double s, co;
            if (a.forward) { const double2 turn = a.forward[row * a.pairs + pair]; co = turn.x; s = turn.y; }
            else sincos(double(p) * double(a.frequencies[pair]), &s, &co);
            const double x = load(rotated + 2 * pair), y = load(rotated + 2 * pair + 1);
            value = (c - rotated) & 1 ? float(x * s + y * co) : float(x * co - y * s);
        }
        qs[h * stride + c] = value;
    }
    __syncthreads();
    const auto key_row = [&](size_t index, bool& bf16) -> const void* {
        if (index < raw_count) { bf16 = false; return a.raw + size_t(first + int64_t(index)) % a.raw_rows * a.kdim; }
        const int32_t at = a.selected[row * a.selections + (index - raw_count)];
        bf16 = BF16;
        if (at < 0) return nullptr;
        const size_t offset = row * a.compressed_batch_stride + size_t(at) * a.kdim;
        return BF16 ? static_cast<const void*>(static_cast<const uint16_t*>(a.compressed) + offset)
                    : static_cast<const void*>(static_cast<const float*>(a.compressed) + offset);
    };
    // scores: 32 keys a pass, the 8 heads of a key in adjacent lanes
    {
        const size_t h = t % HB;
        for (size_t index = t / HB; index < total; index += THREADS / HB) {
            bool bf16;
            const void* key = key_row(index, bf16);
            float dot = 0.0f;
            if (key && h < heads_here) {
                const float* query = qs + h * stride;
                if (bf16) for (size_t c = 0; c < a.kdim; ++c) dot += query[c] * latent_value<true>(key, c);
                else for (size_t c = 0; c < a.kdim; ++c) dot += query[c] * latent_value<false>(key, c);
            }
            if (h < heads_here) w[h * total + index] = key ? dot * a.scale : -INFINITY;
        }
    }
    __syncthreads();
    // softmax weights: a wave per head
    for (size_t h = wave; h < heads_here; h += THREADS / 64) {
        const float sink = a.sinks ? a.sinks[head0 + h] : -INFINITY;
        float top = sink;
        for (size_t i = lane; i < total; i += 64) top = fmaxf(top, w[h * total + i]);
        for (unsigned offset = 32; offset; offset /= 2) top = fmaxf(top, __shfl_xor(top, offset));
        float sum = 0.0f;
        for (size_t i = lane; i < total; i += 64) {
            const float s = w[h * total + i];
            const float weight = s == -INFINITY ? 0.0f : expf(s - top);
            w[h * total + i] = weight;
            sum += weight;
        }
        for (unsigned offset = 32; offset; offset /= 2) sum += __shfl_xor(sum, offset);
        if (!lane) denominators[h] = sum + (a.sinks ? expf(sink - top) : 0.0f);
    }
    __syncthreads();
    // weighted rows: a thread per output column, every head of the workgroup at once
    float acc[HB][MAX_COLS];
    #pragma unroll
    for (int h = 0; h < HB; ++h)
        #pragma unroll
        for (int c = 0; c < MAX_COLS; ++c) acc[h][c] = 0.0f;
    for (size_t index = 0; index < total; ++index) {
        bool bf16;
        const void* key = key_row(index, bf16);
        if (!key) continue;
        #pragma unroll
        for (int c = 0; c < MAX_COLS; ++c) {
            const size_t col = t + size_t(c) * THREADS;
            if (col >= a.vdim) break;
            const float v = bf16 ? latent_value<true>(key, col) : latent_value<false>(key, col);
            #pragma unroll
            for (int h = 0; h < HB; ++h) acc[h][c] += w[size_t(h) * total + index] * v;
        }
    }
    // (w rows of absent heads are never written: their products are discarded below)
    float* rows_out = qs;   // [HB][vdim]
    #pragma unroll
    for (int h = 0; h < HB; ++h)
        #pragma unroll
        for (int c = 0; c < MAX_COLS; ++c) {
            const size_t col = t + size_t(c) * THREADS;
            if (size_t(h) < heads_here && col < a.vdim) rows_out[size_t(h) * a.vdim + col] = acc[h][c] / denominators[h];
        }
    __syncthreads();
    const size_t back = a.vdim - 2 * a.pairs;
    for (size_t i = t; i < heads_here * a.vdim; i += THREADS) {
        const size_t h = i / a.vdim, c = i % a.vdim;
        float value = rows_out[i];
        if (c >= back) {
            const size_t pair = (c - back) / 2;
            double s, co;
            if (a.inverse) { const double2 turn = a.inverse[row * a.pairs + pair]; co = turn.x; s = turn.y; }
            else sincos(double(p) * double(a.frequencies[pair]) * -1.0, &s, &co);
            const double x = rows_out[h * a.vdim + back + 2 * pair], y = rows_out[h * a.vdim + back + 2 * pair + 1];
            value = (c - back) & 1 ? float(x * s + y * co) : float(x * co - y * s);
        }
        a.out[(row * a.heads + head0 + h) * a.vdim + c] = value;
    }
}

void launch(Device& d, const LatentArgs& args, size_t rows, size_t total_keys, bool bf16) {
    const size_t shared = (HB * (args.kdim + PAD) + HB * total_keys + HB) * 4;
    if (shared > 160 * 1024 - 256) throw std::runtime_error("invalid Straydog attention shape");
    raise_shared_limit(d, reinterpret_cast<const void*>(&latent_attention_kernel<true>), 160 * 1024 - 256);
    raise_shared_limit(d, reinterpret_cast<const void*>(&latent_attention_kernel<false>), 160 * 1024 - 256);
    const dim3 grid(unsigned((args.heads + HB - 1) / HB), unsigned(rows));
    if (bf16) latent_attention_kernel<true><<<grid, THREADS, shared, d.stream>>>(args);
    else latent_attention_kernel<false><<<grid, THREADS, shared, d.stream>>>(args);
}

}  // namespace

namespace {

// DSpark's noncausal block attention (reference gpu/dspark_attention.hpp:1-101): every query of the block sees the history
// positions [anchor - history, anchor) of the K = V ring of 128 rows and all the block's keys, 512 columns, scale 1/sqrt(512),
// the head's sink in the maximum and the denominator only.
//
// The keys are the same for every head and every slot of the block, so a workgroup serves ONE HEAD AND ALL ITS SLOTS (up to
// five queries) and every key row it loads is used by all of them: a wave takes every fourth key, lanes across the 512 columns
// (two 16-byte loads a lane), and forms the slots' dot products together, each a wave-wide sum; wave s then turns slot s's
// scores into weights (lanes over the keys, maxima and sums by lane exchanges); the outputs are two columns a thread, one
// value load feeding all the slots' sums.
constexpr int DSPARK_DIM = 512, DSPARK_RING = 128, DSPARK_SLOTS = 5, DSPARK_KEYS = DSPARK_RING + DSPARK_SLOTS, DSPARK_WAVES = 4;
struct DsparkArgs {
    const float *q, *ring, *block, *sinks;
    int heads, slots, history;
    uint32_t anchor;
    const int32_t* anchor_at;      // device-resident anchor, or null
    float scale;
    float* out;
};
__global__ void __launch_bounds__(DSPARK_WAVES * 64) dspark_attention_kernel(DsparkArgs a) {
    __shared__ float weights[DSPARK_SLOTS][DSPARK_KEYS];
    __shared__ float denominators[DSPARK_SLOTS];
    const int head = blockIdx.x, t = threadIdx.x, lane = t % 64, wave = t / 64;
    // ring keys: positions last - count + 1 .. last, last = anchor - 1, at most `history` of them and none below position 0
    const long long last = (long long)(a.anchor_at ? a.anchor_at[0] : int32_t(a.anchor)) - 1;
    const int ring_keys = int(min((long long)a.history, last + 1)), keys = ring_keys + a.slots;
    const long long oldest = last - ring_keys + 1;
    const auto row_of = [&](int key) -> const float* {
        return key < ring_keys ? a.ring + size_t((oldest + key) % DSPARK_RING) * DSPARK_DIM : a.block + size_t(key - ring_keys) * DSPARK_DIM;
    };
    // the slots' queries of this head: a lane keeps its eight columns of each
    float4 query[DSPARK_SLOTS][2];
    #pragma unroll
    for (int s = 0; s < DSPARK_SLOTS; ++s) {
        const float* from = a.q + (size_t(min(s, a.slots - 1)) * a.heads + head) * DSPARK_DIM + 8 * lane;
        query[s][0] = *reinterpret_cast<const float4*>(from);
        query[s][1] = *reinterpret_cast<const float4*>(from + 4);
    }
    for (int key = wave; key < keys; key += DSPARK_WAVES) {
        const float* k = row_of(key) + 8 * lane;
        const float4 k0 = *reinterpret_cast<const float4*>(k), k1 = *reinterpret_cast<const float4*>(k + 4);
        #pragma unroll
        for (int s = 0; s < DSPARK_SLOTS; ++s) {
            float dot = query[s][0].x * k0.x;
            dot = fmaf(query[s][0].y, k0.y, dot); dot = fmaf(query[s][0].z, k0.z, dot); dot = fmaf(query[s][0].w, k0.w, dot);
            dot = fmaf(query[s][1].x, k1.x, dot); dot = fmaf(query[s][1].y, k1.y, dot); dot = fmaf(query[s][1].z, k1.z, dot); dot = fmaf(query[s][1].w, k1.w, dot);
            #pragma unroll
            for (int offset = 32; offset; offset /= 2) dot += __shfl_xor(dot, offset);
            if (lane == 0) weights[s][key] = dot * a.scale;
        }
    }
    __syncthreads();
    // scores -> weights: wave s (and wave 0 again for a fifth slot) owns slot s; a lane holds keys lane, lane + 64, lane + 128
    for (int s = wave; s < a.slots; s += DSPARK_WAVES) {
        const float sink = a.sinks[head];
        float score[3], top = sink;
        #pragma unroll
        for (int i = 0; i < 3; ++i) {
            const int key = lane + 64 * i;
            score[i] = key < keys ? weights[s][key] : -INFINITY;
            top = fmaxf(top, score[i]);
        }
        #pragma unroll
        for (int offset = 32; offset; offset /= 2) top = fmaxf(top, __shfl_xor(top, offset));
        float sum = 0.0f;
        #pragma unroll
        for (int i = 0; i < 3; ++i) {
            const int key = lane + 64 * i;
            const float w = score[i] == -INFINITY ? 0.0f : expf(score[i] - top);
            if (key < keys) weights[s][key] = w;
            sum += w;
        }
        #pragma unroll
        for (int offset = 32; offset; offset /= 2) sum += __shfl_xor(sum, offset);
        if (lane == 0) denominators[s] = sum + expf(sink - top);
    }
    __syncthreads();
    // outputs: columns 2t, 2t + 1 of every slot; a key whose weight is 0 in a slot adds nothing there
    float2 sums[DSPARK_SLOTS];
    #pragma unroll
    for (int s = 0; s < DSPARK_SLOTS; ++s) sums[s] = make_float2(0.0f, 0.0f);
    #pragma unroll 4
    for (int key = 0; key < keys; ++key) {
        const float2 v = *reinterpret_cast<const float2*>(row_of(key) + 2 * t);
        #pragma unroll
        for (int s = 0; s < DSPARK_SLOTS; ++s) {
            const float w = weights[s][key];       // (slots past the block's last hold what the scores of its last slot left: unused)
            sums[s].x = w == 0.0f ? sums[s].x : fmaf(w, v.x, sums[s].x);
            sums[s].y = w == 0.0f ? sums[s].y : fmaf(w, v.y, sums[s].y);
        }
    }
    #pragma unroll
    for (int s = 0; s < DSPARK_SLOTS; ++s)
        if (s < a.slots) {
            const float denominator = denominators[s];
            *reinterpret_cast<float2*>(a.out + (size_t(s) * a.heads + head) * DSPARK_DIM + 2 * t) = make_float2(sums[s].x / denominator, sums[s].y / denominator);
        }
}

}  // namespace

extern "C" {

int sd_op_dspark_attention(void* handle, const float* q, const float* ring, const float* block, const float* sinks, uint64_t heads, uint64_t slots,
                           uint32_t anchor, const int32_t* anchor_at, uint64_t history, float* out) {
    SD_OP_BEGIN
    if (!heads || heads > 64 || !slots || slots > uint64_t(DSPARK_SLOTS) || history > uint64_t(DSPARK_RING) || anchor > uint32_t(INT32_MAX) || history > anchor)
        throw std::runtime_error("invalid DSpark attention block or history range");
    op_span(value, q, checked_floats({slots, heads, uint64_t(DSPARK_DIM)}), "DSpark rotated queries");
    op_span(value, ring, size_t(DSPARK_RING) * DSPARK_DIM * 4, "DSpark history K ring");
    op_span(value, block, checked_floats({slots, uint64_t(DSPARK_DIM)}), "DSpark rotated block keys");
    op_span(value, sinks, checked_floats({heads}), "DSpark attention sinks");
    op_span(value, out, checked_floats({slots, heads, uint64_t(DSPARK_DIM)}), "DSpark attention output");
    if (anchor_at) op_span(value, anchor_at, 4, "DSpark anchor position");
    // anchor = history = 0 gives no ring keys: the block's own keys are always seen
    const DsparkArgs args{q, ring, block, sinks, int(heads), int(slots), int(history), anchor, anchor_at, 1.0f / sqrtf(float(DSPARK_DIM)), out};
    dspark_attention_kernel<<<unsigned(heads), DSPARK_WAVES * 64, 0, value.stream>>>(args);
    SD_OP_END
}

int sd_op_sparse_attention(void* handle, const float* q, const float* raw, uint64_t raw_rows, const int32_t* positions, uint64_t window,
                           const float* compressed, uint64_t compressed_rows, const int32_t* selected, uint64_t selections,
                           const float* sinks, uint64_t rows, uint64_t heads, uint64_t dim, float scale, uint64_t rope_dims,
                           const float* frequencies, float* scratch, uint64_t scratch_bytes, float* out) {
    SD_OP_BEGIN
    (void)scratch; (void)scratch_bytes;
    if (!rows || rows > 65535 || !heads || !dim || dim > 1024 || !window || !raw_rows || rope_dims % 2 || rope_dims > dim || rope_dims > 128)
        throw std::runtime_error("invalid Straydog attention shape");
    if (rope_dims) op_span(value, frequencies, checked_floats({rope_dims / 2}), "rope frequencies");
    op_span(value, q, checked_floats({rows, heads, dim}), "attention queries");
    op_span(value, raw, checked_floats({raw_rows, dim}), "window rows");
    op_span(value, positions, checked_floats({rows}), "query positions");
    if (selections) {
        op_state_span(value, compressed, checked_product({compressed_rows, dim}), "compressed rows");
        op_span(value, selected, checked_floats({rows, selections}), "selected rows");
    }
    op_span(value, sinks, checked_floats({heads}), "attention sinks");
    op_span(value, out, checked_floats({rows, heads, dim}), "an attention output");
    LatentArgs args{};
    args.q = q; args.raw = raw; args.raw_rows = size_t(raw_rows); args.positions = positions; args.window = size_t(window);
    args.compressed = state_base(compressed); args.selected = selected; args.selections = size_t(selections); args.sinks = sinks;
    args.heads = size_t(heads); args.kdim = args.vdim = size_t(dim); args.scale = scale; args.pairs = size_t(rope_dims / 2);
    args.frequencies = frequencies; args.out = out;
    // a table that sd_op_norm_rope filled for exactly these rows stands in for the angles (gpu/kernels.cpp:5349-5361); it serves once
    if (args.pairs && value.turns_ready && value.turns_ready_rows == size_t(rows) && value.turns_ready_pairs == args.pairs) {
        args.forward = value.turns;
        args.inverse = value.turns + value.turns_rows * value.turns_pairs;
    }
    value.turns_ready = false;
    launch(value, args, size_t(rows), size_t(window + selections), state_bf16(compressed));
    SD_OP_END
}

int sdx_latent_attention(void* handle, const void* q, const void* latents, const int32_t* selected, uint64_t batch, uint64_t groups,
                         uint64_t k, uint64_t heads, uint64_t kdim, uint64_t vdim, float scale, float* out) {
    SD_OP_BEGIN
    if (!batch || batch > 65535 || !groups || !k || !heads || !kdim || !vdim || vdim > kdim || kdim > 1024)
        throw std::runtime_error("invalid Straydog attention shape");
    op_span(value, q, checked_product({batch, heads, kdim, 2}), "attention queries");
    op_span(value, latents, checked_product({batch, groups, kdim, 2}), "latent rows");
    op_span(value, selected, checked_floats({batch, k}), "selected rows");
    op_span(value, out, checked_floats({batch, heads, vdim}), "an attention output");
    const bool whole_pieces = (uintptr_t(q) | uintptr_t(latents) | uintptr_t(out)) % 16 == 0;       // the matrix-core kernels move 16 bytes at a time
    if (latent_gather_supported(kdim, vdim) && whole_pieces && groups * kdim * 2 < (uint64_t(1) << 32) && k < (uint64_t(1) << 31)) {      // (a sequence's rows within 32-bit offsets)
        // the matrix-core path; its chunk partials live in the device's workspace (grown outside graph capture)
        float* partial = static_cast<float*>(workspace(value, latent_gather_scratch(batch, k, heads, vdim)));
        latent_gather(value, q, latents, selected, batch, groups, k, heads, scale, out, partial);
        SD_CHECK(hipGetLastError());
        return 0;
    }
    LatentArgs args{};
    args.q_bf16 = static_cast<const uint16_t*>(q); args.compressed = latents; args.compressed_batch_stride = size_t(groups * kdim);
    args.selected = selected; args.selections = size_t(k); args.heads = size_t(heads); args.kdim = size_t(kdim); args.vdim = size_t(vdim);
    args.scale = scale; args.out = out;
    launch(value, args, size_t(batch), size_t(k), true);
    SD_OP_END
}

}  // extern "C"
