// Causal grouped-query attention over the paged Q8_0 / FP16 K/V cache for few query rows per sequence:
// single-token decode and speculative verify spans.  Stands in for the reference's split-K decode pair
// qsa_decode_parts + qsa_decode_merge (gpu/sparse_attention_compute.hpp:41-170) with the dense selection
// 0..position and the reference's FP16-operand convention (Q8_0 -> exact integer in FP16, one rounding by the
// block scale, FP32 sums: gpu/qsa_prompt_attention.hpp:15-33, :144-150).
//
// Shape of the work on gfx950 (wave64, v_mfma_f32_16x16x32_f16):
//   * a workgroup (4 waves) owns one (sequence, K/V head, chunk of the context); its waves take alternate
//     32-token steps, each with its own online softmax, and merge through LDS at the end;
//   * per step a wave forms S^T = K . Q^T (tokens x query rows) with K rows straight from HBM as A operands
//     (lane = token, 8 consecutive columns per lane group), so the C layout (lane = query row, 4 tokens per lane
//     group) is already the B-operand layout of O^T += V^T . P^T: probabilities never move between lanes;
//   * V^T operands are built in registers from 8-byte row pieces of 8 tokens by byte selection;
//   * the next step's rows are requested before the current step is computed (register double buffering).
#include "device.hpp"
#include "../../include/straydog_gpu_ext.h"

#include <hip/hip_fp16.h>

#include <cstdlib>

namespace sd { void validate_pool(Device& d, const sdx_kv_pool* pool); }
using namespace sd;

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(1))) const void* global_ptr;
typedef __attribute__((address_space(3))) void* lds_ptr;

constexpr int WAVES = 4, STEP = 32;
constexpr float NEG_BIG = -1.0e30f;   // a finite "nothing seen yet" maximum: exp2(NEG_BIG - m) is 0, no inf - inf anywhere

struct PagedArgs {
    const uint8_t* pages;
    unsigned page_tokens, kv_heads, heads, group, span;
    const int32_t* page_table;
    size_t table_stride;
    const int32_t* positions;
    const void* q;
    int q_f16;
    float scale_log2;      // softmax scale * log2(e): scores live in the base-2 domain
    float* partial;        // [seq][kv head][chunk][row][dim + 2]
    unsigned chunk_tokens, chunks, rows;   // rows = span * group (query rows per K/V head)
    int max_context;       // positions[s] + span is clipped to this (the launch and the page table are sized for it)
};

__device__ __forceinline__ half2v as_half2(uint32_t bits) { return __builtin_bit_cast(half2v, bits); }

// v_perm_b32: byte i of the result is byte sel[i] of the 8 bytes {high, low} (0-3 = low's bytes, 4-7 = high's, 0x0c = 0x00).
__device__ __forceinline__ uint32_t byte_perm(uint32_t high, uint32_t low, uint32_t sel) { return __builtin_amdgcn_perm(high, low, sel); }

// Two bytes u (an int8 xor 0x80) sitting in FP16 patterns 0x64uu: 0x6400 | u is the FP16 1024 + u exactly; minus 1152 leaves the
// signed byte; one rounding by the block scale (the reference's qsa_q8_half16, gpu/qsa_prompt_attention.hpp:15-33).
__device__ __forceinline__ half2v magic_to_half2(uint32_t pattern, half2v scale) {
    const half2v bias = {(_Float16)1152.0f, (_Float16)1152.0f};
    return (as_half2(pattern) - bias) * scale;
}

// Per-lane byte offsets of the rows a step reads, from the step's first row of the K (or V) plane.  They are the same for
// every full step, so they are formed once; a last, partial step clamps its tokens to the last valid one.
template<int DIM, bool Q8> struct LaneOffsets {
    static constexpr int ROW = Q8 ? DIM + DIM / 16 : 2 * DIM, W = DIM / 16;
    uint32_t k[2], ks[2], v[8], vs[8];
    __device__ __forceinline__ void set(int valid, int li, int g) {
        #pragma unroll
        for (int t = 0; t < 2; ++t) {
            const uint32_t row = uint32_t(min(16 * t + li, valid - 1)) * ROW;
            k[t] = row + (Q8 ? 8 * g : 16 * g);
            ks[t] = row + DIM;
        }
        #pragma unroll
        for (int e = 0; e < 8; ++e) {
            const uint32_t row = uint32_t(min(e < 4 ? 4 * g + e : 16 + 4 * g + (e - 4), valid - 1)) * ROW;
            v[e] = row + (Q8 ? W * li : 2 * W * li);
            vs[e] = row + DIM + 2 * ((W * li) / 32);
        }
    }
};

template<int DIM, bool Q8> struct RowLoad;

// What one step needs from HBM, as raw words.  Q8_0: K tile t (16 tokens, lane li = token) gives each lane 8 columns of
// every 32-column block and the row's scales; V gives lane (li, g) the columns [W*li, W*li + W) (W = DIM/16) of its 8
// tokens {4g..4g+3, 16+4g..16+4g+3} and those columns' block scale.
template<int DIM> struct RowLoad<DIM, true> {
    static constexpr int BLOCKS = DIM / 32, W = DIM / 16;
    uint2 k[2][BLOCKS];
    uint32_t kscale[2][BLOCKS / 2];
    uint32_t v[8][W / 4];
    uint16_t vscale[8];
};
template<int DIM>
__device__ __forceinline__ void load_step(RowLoad<DIM, true>& r, const uint8_t* kplane, const uint8_t* vplane, const LaneOffsets<DIM, true>& o) {
    constexpr int BLOCKS = DIM / 32, W = DIM / 16;
    #pragma unroll
    for (int t = 0; t < 2; ++t) {
        #pragma unroll
        for (int b = 0; b < BLOCKS; ++b) r.k[t][b] = *reinterpret_cast<const uint2*>(kplane + o.k[t] + 32 * b);
        #pragma unroll
        for (int b = 0; b < BLOCKS / 2; ++b) r.kscale[t][b] = *reinterpret_cast<const uint32_t*>(kplane + o.ks[t] + 4 * b);
    }
    #pragma unroll
    for (int e = 0; e < 8; ++e) {
        #pragma unroll
        for (int w = 0; w < W / 4; ++w) r.v[e][w] = *reinterpret_cast<const uint32_t*>(vplane + o.v[e] + 4 * w);
        r.vscale[e] = *reinterpret_cast<const uint16_t*>(vplane + o.vs[e]);
    }
}

// FP16 rows: the same pieces, two bytes a value.
template<int DIM> struct RowLoad<DIM, false> {
    static constexpr int BLOCKS = DIM / 32, W = DIM / 16;
    half8 k[2][BLOCKS];
    uint32_t v[8][W / 2];
};
template<int DIM>
__device__ __forceinline__ void load_step(RowLoad<DIM, false>& r, const uint8_t* kplane, const uint8_t* vplane, const LaneOffsets<DIM, false>& o) {
    constexpr int BLOCKS = DIM / 32, W = DIM / 16;
    #pragma unroll
    for (int t = 0; t < 2; ++t)
        #pragma unroll
        for (int b = 0; b < BLOCKS; ++b) r.k[t][b] = *reinterpret_cast<const half8*>(kplane + o.k[t] + 64 * b);
    #pragma unroll
    for (int e = 0; e < 8; ++e)
        #pragma unroll
        for (int w = 0; w < W / 2; ++w) r.v[e][w] = *reinterpret_cast<const uint32_t*>(vplane + o.v[e] + 4 * w);
}

// The A operand of S^T = K . Q^T for tile t, block b.
template<int DIM>
__device__ __forceinline__ half8 key_operand(const RowLoad<DIM, true>& r, int t, int b) {
    const uint32_t pairs = r.kscale[t][b / 2];
    const half2v scale = as_half2((b & 1) ? byte_perm(pairs, pairs, 0x03020302u) : byte_perm(pairs, pairs, 0x01000100u));
    const uint32_t magic = 0x64646464u;
    const uint32_t lo = r.k[t][b].x ^ 0x80808080u, hi = r.k[t][b].y ^ 0x80808080u;
    const half2v a0 = magic_to_half2(byte_perm(magic, lo, 0x04010400u), scale);
    const half2v a1 = magic_to_half2(byte_perm(magic, lo, 0x04030402u), scale);
    const half2v a2 = magic_to_half2(byte_perm(magic, hi, 0x04010400u), scale);
    const half2v a3 = magic_to_half2(byte_perm(magic, hi, 0x04030402u), scale);
    return half8{a0.x, a0.y, a1.x, a1.y, a2.x, a2.y, a3.x, a3.y};
}
template<int DIM>
__device__ __forceinline__ half8 key_operand(const RowLoad<DIM, false>& r, int t, int b) { return r.k[t][b]; }

// The scales of the lane's 8 tokens as 4 FP16 pairs (tokens e, e+1), formed once a step.
template<int DIM> struct ValueScales { half2v pair[4]; };
template<int DIM>
__device__ __forceinline__ void value_scales(const RowLoad<DIM, true>& r, ValueScales<DIM>& s) {
    #pragma unroll
    for (int e = 0; e < 8; e += 2) s.pair[e / 2] = as_half2(uint32_t(r.vscale[e]) | (uint32_t(r.vscale[e + 1]) << 16));
}
template<int DIM>
__device__ __forceinline__ void value_scales(const RowLoad<DIM, false>&, ValueScales<DIM>&) {}

// The A operand of O^T += V^T . P^T for output tile jj: column W*li + jj of the lane's 8 tokens.
template<int DIM>
__device__ __forceinline__ half8 value_operand(const RowLoad<DIM, true>& r, const ValueScales<DIM>& s, int jj) {
    half2v out[4];
    const int word = jj / 4;
    // bytes (jj % 4) of tokens e (low half) and e + 1 (high half), zero bytes between; the xor turns them into 0x64uu patterns
    const uint32_t sel = 0x0c000c00u | uint32_t(jj % 4) | (uint32_t(4 + jj % 4) << 16);
    #pragma unroll
    for (int e = 0; e < 8; e += 2)
        out[e / 2] = magic_to_half2(byte_perm(r.v[e + 1][word], r.v[e][word], sel) ^ 0x64806480u, s.pair[e / 2]);
    return half8{out[0].x, out[0].y, out[1].x, out[1].y, out[2].x, out[2].y, out[3].x, out[3].y};
}
template<int DIM>
__device__ __forceinline__ half8 value_operand(const RowLoad<DIM, false>& r, const ValueScales<DIM>&, int jj) {
    half2v out[4];
    const int word = jj / 2;
    const uint32_t sel = (jj & 1) ? 0x07060302u : 0x05040100u;
    #pragma unroll
    for (int e = 0; e < 8; e += 2) out[e / 2] = as_half2(byte_perm(r.v[e + 1][word], r.v[e][word], sel));
    return half8{out[0].x, out[0].y, out[1].x, out[1].y, out[2].x, out[2].y, out[3].x, out[3].y};
}

// MODE: 0 = rows straight from HBM into operand registers, 1 = the same with the next step's rows requested before this
// step is computed, 2 = a step's K and V slabs (32 contiguous rows each) copied by fully coalesced 16-byte global->LDS loads
// into the wave's own LDS stage, operands then read from LDS in MFMA layout while the next step's copy is in flight.
template<int DIM, int QT, bool Q8, int MODE, int OCC>
__global__ void __launch_bounds__(WAVES * 64) __attribute__((amdgpu_waves_per_eu(OCC, OCC))) paged_attention_kernel(PagedArgs args) {
    constexpr int ROW = Q8 ? DIM + DIM / 16 : 2 * DIM, BLOCKS = DIM / 32, W = DIM / 16, TILES = DIM / 16;
    const int chunk = blockIdx.x, kvh = blockIdx.y, seq = blockIdx.z;
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), li = lane & 15, g = lane >> 4;
    const int position = args.positions[seq], total = min(position + int(args.span), args.max_context);
    const int chunk_begin = chunk * int(args.chunk_tokens);
    if (chunk_begin >= total) return;
    const int chunk_end = min(total, chunk_begin + int(args.chunk_tokens));
    const int32_t* table = args.page_table + size_t(seq) * args.table_stride;
    const size_t plane_bytes = size_t(args.page_tokens) * ROW;

    // Query rows of this K/V head: row = span_row * group + head_in_group; a lane holds row qt*16 + li as B operands.
    // A row past the last real one holds zeros (its scores are never stored).
    half8 qf[QT][BLOCKS];
    int limit[QT];
    #pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
        const int row = qt * 16 + li;
        const bool real = row < int(args.rows);
        const int span_row = real ? row / int(args.group) : 0, head = kvh * int(args.group) + (real ? row % int(args.group) : 0);
        limit[qt] = real ? position + span_row : 0x7fffffff;
        const size_t at = ((size_t(seq) * args.span + span_row) * args.heads + head) * DIM;
        #pragma unroll
        for (int b = 0; b < BLOCKS; ++b) {
            half8 value = {};
            if (real) {
                if (args.q_f16) value = *reinterpret_cast<const half8*>(static_cast<const _Float16*>(args.q) + at + 32 * b + 8 * g);
                else {
                    const float* from = static_cast<const float*>(args.q) + at + 32 * b + 8 * g;
                    #pragma unroll
                    for (int i = 0; i < 8; ++i) value[i] = (_Float16)from[i];
                }
            }
            qf[qt][b] = value;
        }
    }

    floatx4 acc[QT][TILES];
    float m[QT], l[QT];
    #pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
        m[qt] = NEG_BIG; l[qt] = 0.0f;
        #pragma unroll
        for (int jj = 0; jj < TILES; ++jj) acc[qt][jj] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
    }

    LaneOffsets<DIM, Q8> full;
    full.set(STEP, li, g);
    extern __shared__ float lds[];
    constexpr int SLAB = STEP * ROW;                       // one step's rows of one plane: contiguous in the page
    uint8_t* stage = reinterpret_cast<uint8_t*>(lds) + wave * (2 * SLAB);
    // The (wave-uniform) first row of a step in its K and V planes.
    const auto planes = [&](int token0, const uint8_t*& kplane, const uint8_t*& vplane) {
        const int page = __builtin_amdgcn_readfirstlane(table[token0 / int(args.page_tokens)]);
        const uint8_t* base = args.pages + (size_t(page) * 2 * args.kv_heads) * plane_bytes + size_t(token0 % int(args.page_tokens)) * ROW;
        kplane = base + size_t(kvh) * plane_bytes;
        vplane = base + size_t(args.kv_heads + kvh) * plane_bytes;
    };
    // A step's rows into operand registers, from HBM (MODE 0/1) or from the wave's LDS stage (MODE 2).
    const auto request = [&](RowLoad<DIM, Q8>& rows, int token0) {
        const uint8_t *kplane, *vplane;
        if (MODE >= 2) { kplane = stage; vplane = stage + SLAB; }
        else planes(token0, kplane, vplane);
        const int valid = total - token0;
        if (valid >= STEP) load_step<DIM>(rows, kplane, vplane, full);
        else { LaneOffsets<DIM, Q8> last; last.set(valid, li, g); load_step<DIM>(rows, kplane, vplane, last); }
    };
    // MODE 2: the step's two slabs copied into the stage, 1 KiB per instruction, lanes past a slab's end switched off.
    const auto copy_in = [&](int token0) {
        const uint8_t *kplane, *vplane;
        planes(token0, kplane, vplane);
        #pragma unroll
        for (int part = 0; part < 2; ++part) {
            const uint8_t* from = (part ? vplane : kplane) + 16 * lane;
            #pragma unroll
            for (int j = 0; j < (SLAB + 1023) / 1024; ++j)
                if (1024 * j + 1024 <= SLAB || 16 * lane + 1024 * j < SLAB)
                    __builtin_amdgcn_global_load_lds((global_ptr)(from + 1024 * j), (lds_ptr)(stage + part * SLAB + 1024 * j), 16, 0, 2 /* nt: streamed once */);
        }
    };

    int token0 = chunk_begin + STEP * wave;
    RowLoad<DIM, Q8> current, next;
    if (MODE == 1 && token0 < chunk_end) request(current, token0);
    if (MODE >= 2 && token0 < chunk_end) copy_in(token0);
    for (; token0 < chunk_end; token0 += STEP * WAVES) {
        if (MODE == 1) { if (token0 + STEP * WAVES < chunk_end) request(next, token0 + STEP * WAVES); }
        else if (MODE == 0) request(current, token0);
        else {
            __builtin_amdgcn_s_waitcnt(0x0f70);          // vmcnt(0): the stage holds this step
            request(current, token0);
            __builtin_amdgcn_s_waitcnt(0xc07f);          // lgkmcnt(0): operands are in registers, the stage is free again
            __builtin_amdgcn_sched_barrier(0);
            if (token0 + STEP * WAVES < chunk_end) copy_in(token0 + STEP * WAVES);
            __builtin_amdgcn_sched_barrier(0);
        }
        // S^T tiles: tokens (rows, 4 per lane group) x query rows (lane li)
        floatx4 s[QT][2];
        #pragma unroll
        for (int t = 0; t < 2; ++t) {
            #pragma unroll
            for (int qt = 0; qt < QT; ++qt) s[qt][t] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
            #pragma unroll
            for (int b = 0; b < BLOCKS; ++b) {
                const half8 ka = key_operand<DIM>(current, t, b);
                #pragma unroll
                for (int qt = 0; qt < QT; ++qt) s[qt][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka, qf[qt][b], s[qt][t], 0, 0, 0);
            }
        }
        const bool edge = token0 + STEP - 1 > position;    // wave-uniform: some token of the step is past the first row's position
        half8 pb[QT];
        #pragma unroll
        for (int qt = 0; qt < QT; ++qt) {
            float top = NEG_BIG;
            #pragma unroll
            for (int t = 0; t < 2; ++t)
                #pragma unroll
                for (int r = 0; r < 4; ++r) {
                    float value = s[qt][t][r] * args.scale_log2;
                    if (edge && token0 + 16 * t + 4 * g + r > limit[qt]) value = -INFINITY;
                    s[qt][t][r] = value;
                    top = fmaxf(top, value);
                }
            top = fmaxf(top, __shfl_xor(top, 16));
            top = fmaxf(top, __shfl_xor(top, 32));
            // the running maximum rarely grows after the first steps: rescale only when some row's did
            if (__any(top > m[qt])) {
                const float m_new = fmaxf(m[qt], top);
                const float alpha = __builtin_amdgcn_exp2f(m[qt] - m_new);
                m[qt] = m_new;
                l[qt] *= alpha;
                #pragma unroll
                for (int jj = 0; jj < TILES; ++jj) acc[qt][jj] *= alpha;
            }
            float sum = 0.0f;
            half8 p;
            #pragma unroll
            for (int t = 0; t < 2; ++t)
                #pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float w = __builtin_amdgcn_exp2f(s[qt][t][r] - m[qt]);
                    sum += w;
                    p[4 * t + r] = (_Float16)w;
                }
            pb[qt] = p;
            l[qt] += sum;
        }
        // O^T tiles: columns (rows of the tile, W*row + jj) x query rows
        ValueScales<DIM> vs;
        value_scales<DIM>(current, vs);
        #pragma unroll
        for (int jj = 0; jj < TILES; ++jj) {
            const half8 va = value_operand<DIM>(current, vs, jj);
            #pragma unroll
            for (int qt = 0; qt < QT; ++qt) acc[qt][jj] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va, pb[qt], acc[qt][jj], 0, 0, 0);
        }
        if (MODE == 1) current = next;
    }

    // Merge the waves through LDS: per wave and query row the maximum, the sum and the unnormalised output.
    if (MODE >= 2) __syncthreads();    // the merge area overlays the stages
    constexpr int STRIDE = DIM + 2, QROWS = QT * 16;
    #pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
        float sum = l[qt];
        sum += __shfl_xor(sum, 16);
        sum += __shfl_xor(sum, 32);
        float* row = lds + (size_t(wave) * QROWS + qt * 16 + li) * STRIDE;
        if (g == 0) { row[DIM] = m[qt]; row[DIM + 1] = sum; }
        #pragma unroll
        for (int jj = 0; jj < TILES; ++jj)
            #pragma unroll
            for (int r = 0; r < 4; ++r) row[W * (4 * g + r) + jj] = acc[qt][jj][r];
    }
    __syncthreads();
    float* out = args.partial + ((size_t(seq) * args.kv_heads + kvh) * args.chunks + chunk) * args.rows * STRIDE;
    for (unsigned i = threadIdx.x; i < args.rows * STRIDE; i += WAVES * 64) {
        const unsigned row = i / STRIDE, col = i % STRIDE;
        float top = NEG_BIG;
        #pragma unroll
        for (int w = 0; w < WAVES; ++w) top = fmaxf(top, lds[(size_t(w) * QROWS + row) * STRIDE + DIM]);
        float value;
        if (col == DIM) value = top;
        else {
            value = 0.0f;
            #pragma unroll
            for (int w = 0; w < WAVES; ++w) {
                const float* other = lds + (size_t(w) * QROWS + row) * STRIDE;
                value += other[col] * __builtin_amdgcn_exp2f(other[DIM] - top);
            }
        }
        out[i] = value;
    }
}

// One block per (sequence, span row, head): the chunks' partial results merged and normalised
// (the algebra of the reference's qsa_decode_merge, gpu/sparse_attention_compute.hpp:139-170).
template<int DIM, bool F16_OUT>
__global__ void __launch_bounds__(DIM) paged_merge_kernel(PagedArgs args, void* out) {
    constexpr int STRIDE = DIM + 2;
    const unsigned item = blockIdx.x, head = item % args.heads, span_row = item / args.heads % args.span, seq = item / args.heads / args.span;
    const unsigned kvh = head / args.group, row = span_row * args.group + head % args.group, col = threadIdx.x;
    const int total = min(args.positions[seq] + int(args.span), args.max_context);
    const unsigned used = unsigned((total + int(args.chunk_tokens) - 1) / int(args.chunk_tokens));
    const float* base = args.partial + ((size_t(seq) * args.kv_heads + kvh) * args.chunks) * args.rows * STRIDE + size_t(row) * STRIDE;
    const size_t step = size_t(args.rows) * STRIDE;
    float top = NEG_BIG;
    for (unsigned c = 0; c < used; ++c) top = fmaxf(top, base[c * step + DIM]);
    float sum = 0.0f, value = 0.0f;
    for (unsigned c = 0; c < used; ++c) {
        const float w = __builtin_amdgcn_exp2f(base[c * step + DIM] - top);
        sum += base[c * step + DIM + 1] * w;
        value += base[c * step + col] * w;
    }
    value /= sum;
    const size_t at = size_t(item) * DIM + col;
    if (F16_OUT) static_cast<__half*>(out)[at] = __float2half_rn(value);
    else static_cast<float*>(out)[at] = value;
}

// Tuning switches read once from the environment, as the reference reads its hot-path switches (STRAYDOG_QSA_MMA,
// gpu/sparse_attention_compute.hpp:594): STRAYDOG_DECODE_CHUNK = tokens per workgroup (0: chosen from the shape),
// STRAYDOG_DECODE_MODE = 0|1|2 picks how rows reach the operand registers (see the kernel), STRAYDOG_DECODE_OCCUPANCY the
// waves per SIMD the decode variant is compiled for.
struct Tuning { unsigned chunk = 0; unsigned mode = 2; unsigned occupancy = 4; };
const Tuning& tuning() {
    static const Tuning value = [] {
        Tuning t;
        if (const char* text = std::getenv("STRAYDOG_DECODE_CHUNK")) t.chunk = unsigned(std::strtoul(text, nullptr, 10));
        if (const char* text = std::getenv("STRAYDOG_DECODE_OCCUPANCY")) t.occupancy = unsigned(std::strtoul(text, nullptr, 10));
        if (const char* text = std::getenv("STRAYDOG_DECODE_MODE")) t.mode = unsigned(std::strtoul(text, nullptr, 10));
        return t;
    }();
    return value;
}

unsigned pick_chunk(uint64_t seqs, uint64_t kv_heads, uint64_t max_context, unsigned page_tokens, unsigned compute_units) {
    // one resident round of workgroups when every sequence is at max_context; a chunk is whole 128-token
    // rounds of the four waves and never smaller than 256 tokens
    const uint64_t want = uint64_t(compute_units) * 4;     // four workgroups (16 waves) are resident per compute unit
    uint64_t chunk = (max_context * seqs * kv_heads + want - 1) / want;
    if (tuning().chunk) chunk = tuning().chunk;
    chunk = (chunk + 127) / 128 * 128;
    if (chunk < 256) chunk = 256;
    if (chunk > 4096) chunk = 4096;
    (void)page_tokens;
    return unsigned(chunk);
}

template<int DIM, bool Q8, int PF, int OCC>
void launch(Device& d, const PagedArgs& args, unsigned query_tiles, dim3 grid) {
    size_t shared = size_t(WAVES) * query_tiles * 16 * (DIM + 2) * 4;
    if (PF >= 2) shared = std::max(shared, size_t(WAVES) * 2 * STEP * (Q8 ? DIM + DIM / 16 : 2 * DIM));
    if (shared > 160 * 1024) throw std::runtime_error("Straydog paged attention: too many query rows per K/V head for the decode kernel");
#define SD_CASE(QT) case QT: { \
        static bool raised = false; \
        if (!raised && shared > 64 * 1024) { SD_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&paged_attention_kernel<DIM, QT, Q8, PF, OCC>), hipFuncAttributeMaxDynamicSharedMemorySize, int(shared))); raised = true; } \
        paged_attention_kernel<DIM, QT, Q8, PF, OCC><<<grid, WAVES * 64, shared, d.stream>>>(args); break; }
    switch (query_tiles) {
        SD_CASE(1) SD_CASE(2) SD_CASE(3) SD_CASE(4)
        default: throw std::runtime_error("Straydog paged attention: too many query rows per K/V head for the decode kernel");
    }
#undef SD_CASE
}

}  // namespace

extern "C" {

uint64_t sdx_paged_attention_scratch(uint64_t seqs, uint64_t span, uint64_t heads, uint64_t dim, uint64_t max_context) {
    // the smallest chunk the launch may pick is 256 tokens
    const uint64_t chunks = (max_context + 255) / 256;
    return seqs * span * heads * chunks * (dim + 2) * 4;
}

int sdx_paged_attention(void* handle, const sdx_kv_pool* pool, const int32_t* page_table, uint64_t table_stride,
                        const int32_t* positions, uint64_t max_context, const void* q, int q_f16, uint64_t seqs, uint64_t span,
                        uint64_t heads, float scale, void* out, int out_f16, void* scratch, uint64_t scratch_bytes) {
    SD_OP_BEGIN
    validate_pool(value, pool);
    if (!seqs || seqs > 65535 || !span || !heads || heads % pool->kv_heads || !max_context || max_context > (uint64_t(1) << 30) ||
        !table_stride || max_context > table_stride * pool->page_tokens)
        throw std::runtime_error("invalid Straydog paged attention shape");
    const uint64_t group = heads / pool->kv_heads, rows = span * group;
    const unsigned query_tiles = unsigned((rows + 15) / 16);
    if (query_tiles > 4) throw std::runtime_error("Straydog paged attention: too many query rows per K/V head for the decode kernel");
    op_span(value, page_table, checked_floats({seqs, table_stride}), "a page table");
    op_span(value, positions, checked_floats({seqs}), "query positions");
    op_span(value, q, checked_product({seqs, span, heads, pool->dim, q_f16 ? 2u : 4u}), "attention queries");
    op_span(value, out, checked_product({seqs, span, heads, pool->dim, out_f16 ? 2u : 4u}), "an attention output");
    PagedArgs args{};
    args.pages = static_cast<const uint8_t*>(pool->pages);
    args.page_tokens = pool->page_tokens; args.kv_heads = pool->kv_heads; args.heads = unsigned(heads); args.group = unsigned(group);
    args.span = unsigned(span); args.page_table = page_table; args.table_stride = size_t(table_stride); args.positions = positions;
    args.q = q; args.q_f16 = q_f16; args.scale_log2 = scale * 1.44269504088896341f;
    args.chunk_tokens = pick_chunk(seqs, pool->kv_heads, max_context, pool->page_tokens, value.compute_units);
    args.chunks = unsigned((max_context + args.chunk_tokens - 1) / args.chunk_tokens);
    args.rows = unsigned(rows);
    args.max_context = int(max_context);
    const size_t need = checked_floats({seqs, pool->kv_heads, args.chunks, rows, uint64_t(pool->dim) + 2});
    if (!scratch || scratch_bytes < need) throw std::runtime_error("Straydog paged attention scratch too small");
    op_span(value, scratch, need, "attention scratch");
    args.partial = static_cast<float*>(scratch);
    const dim3 grid(args.chunks, pool->kv_heads, unsigned(seqs));
    const bool q8 = pool->row_bytes != 2 * pool->dim;
    {
    KernelTimer timer(value);
    const unsigned mode = tuning().mode, occupancy = tuning().occupancy;
    if (pool->dim == 128) {
        if (q8 && query_tiles == 1) {
            // the decode shape: the variants differ in how rows reach the operand registers and in waves per SIMD
            if (mode == 2) { if (occupancy >= 4) launch<128, true, 2, 4>(value, args, query_tiles, grid); else if (occupancy == 3) launch<128, true, 2, 3>(value, args, query_tiles, grid); else launch<128, true, 2, 2>(value, args, query_tiles, grid); }
            else if (mode == 1) launch<128, true, 1, 2>(value, args, query_tiles, grid);
            else launch<128, true, 0, 3>(value, args, query_tiles, grid);
        }
        else if (q8) launch<128, true, 2, 1>(value, args, query_tiles, grid);
        else launch<128, false, 2, 1>(value, args, query_tiles, grid);
    } else {
        if (q8) launch<256, true, 2, 1>(value, args, query_tiles, grid); else launch<256, false, 2, 1>(value, args, query_tiles, grid);
    }
    }
    SD_CHECK(hipGetLastError());
    const unsigned items = unsigned(checked_product({seqs, span, heads}));
    if (pool->dim == 128) {
        if (out_f16) paged_merge_kernel<128, true><<<items, 128, 0, value.stream>>>(args, out);
        else paged_merge_kernel<128, false><<<items, 128, 0, value.stream>>>(args, out);
    } else {
        if (out_f16) paged_merge_kernel<256, true><<<items, 256, 0, value.stream>>>(args, out);
        else paged_merge_kernel<256, false><<<items, 256, 0, value.stream>>>(args, out);
    }
    SD_OP_END
}

}  // extern "C"
