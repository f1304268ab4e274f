// The sparse path's indexer: BF16 rounding, compression pooling, rope, indexer scores in the canonical order,
// radix top-k, candidate blocks, and their fused entry points.
//   reference: gpu/token_mixing.hpp:728-744 (to_bf16), gpu/ops.hpp:107-120 (rope), :1681-1694 (compress),
//   :1700-1739 (index scores), :1766-1941 (top-k), :1942-1975 (candidates), gpu/kernels.cpp:5478-5676 (entries).
// Bit-exactness rules kept here: a score is, per head, a chain of fmaf over the columns in order; the head's term
// max(dot, 0) * weight is rounded on its own (no contraction with the sum); the terms are added in head order; the
// scale is applied last.  Top-k compares order-preserving integer keys, keeps the lowest indices among ties and
// emits ascending indices.
#include "device.hpp"
#include <hip/hip_fp16.h>
#include "../../include/straydog_gpu.h"
#include "../../include/straydog_gpu_ext.h"

using namespace sd;

namespace {

__device__ __forceinline__ float bf16_value(uint16_t bits) { return __uint_as_float(uint32_t(bits) << 16); }

// sum + round(a * b): the product is rounded on its own, never contracted with the add into a fused multiply-add
// (the rule of the reference's canonical score order, gpu/ops.hpp:2171-2187).
__device__ __forceinline__ float add_rounded_product(float sum, float a, float b) {
    #pragma clang fp contract(off)
    const float product = a * b;
    return sum + product;
}
__device__ __forceinline__ float rounded_product(float a, float b) {
    #pragma clang fp contract(off)
    return a * b;
}
__device__ __forceinline__ float rounded_sum(float a, float b) {
    #pragma clang fp contract(off)
    return a + b;
}

__global__ void to_bf16_kernel(const float* x, size_t count, uint16_t* out) {
    for (size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x; i < count; i += size_t(gridDim.x) * blockDim.x) {
        const uint32_t bits = __float_as_uint(x[i]);
        out[i] = (bits & 0x7fffffffu) > 0x7f800000u ? uint16_t((bits >> 16) | 0x40u) : uint16_t((bits + 0x7fffu + ((bits >> 16) & 1u)) >> 16);
    }
}

// Per-channel softmax pooling of `ratio` rows into one (reference op_compress_kernel, gpu/ops.hpp:1681-1694): out = sum_r
// softmax_r(gate[r]) * kv[r] for each column on its own.  A thread takes V adjacent columns of a group (one 16-byte load of
// the gates and one of the rows per pooled row when V = 4) and reads each of them ONCE: the maximum runs along with the sums,
// which are scaled down whenever it grows (the usual online form; the quotient does not depend on it).
template<int V> struct Lanes { float v[V]; };
template<int V>
__global__ void __launch_bounds__(256) compress_kernel(const float* kv, const float* gate, size_t pieces, size_t ratio, size_t dim, float* out) {
    const size_t piece = size_t(blockIdx.x) * 256 + threadIdx.x;       // V columns of one group
    if (piece >= pieces) return;
    const size_t per_row = dim / V, group = piece / per_row, at = piece % per_row * V;
    typedef Lanes<V> __attribute__((aligned(4 * V))) Piece;
    if (!gate) {       // nothing to pool: row `group` as it is
        *reinterpret_cast<Piece*>(out + group * dim + at) = *reinterpret_cast<const Piece*>(kv + group * dim + at);
        return;
    }
    float top[V], sum[V], acc[V];
    #pragma unroll
    for (int i = 0; i < V; ++i) { top[i] = -INFINITY; sum[i] = 0.0f; acc[i] = 0.0f; }
    for (size_t r = 0; r < ratio; ++r) {
        const size_t from = (group * ratio + r) * dim + at;
        const Piece g = *reinterpret_cast<const Piece*>(gate + from), x = *reinterpret_cast<const Piece*>(kv + from);
        #pragma unroll
        for (int i = 0; i < V; ++i) {
            const float higher = fmaxf(top[i], g.v[i]);
            // (the first row, and a gate of -inf before any finite one, would give exp(-inf - -inf): nothing is kept then)
            const float keep = top[i] == -INFINITY ? 0.0f : expf(top[i] - higher), w = higher == -INFINITY ? 0.0f : expf(g.v[i] - higher);
            sum[i] = sum[i] * keep + w;
            acc[i] = acc[i] * keep + w * x.v[i];
            top[i] = higher;
        }
    }
    Piece pooled;
    #pragma unroll
    for (int i = 0; i < V; ++i) pooled.v[i] = acc[i] / sum[i];
    *reinterpret_cast<Piece*>(out + group * dim + at) = pooled;
}

// The last 2 * pairs values of each vector rotated in adjacent pairs by positions[row] * frequencies[pair]
// (angle, sine and cosine in double).  `from` may differ from `to` (the fused entry leaves q as it was).
__global__ void rope_kernel(const float* from, float* to, size_t count, size_t vectors, size_t width, size_t pairs, const int32_t* positions,
                            const float* frequencies, int inverse, int copy_rest) {
    const size_t index = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (copy_rest) {   // one thread per value: plain copy of the unrotated part
        const size_t values = count;   // here count = rows * vectors * width
        if (index >= values) return;
        const size_t col = index % width;
        if (col < width - 2 * pairs) { to[index] = from[index]; return; }
        if ((col - (width - 2 * pairs)) & 1) return;
        const size_t row = index / (vectors * width), pair = (col - (width - 2 * pairs)) / 2;
        const double angle = double(positions[row]) * double(frequencies[pair]) * (inverse ? -1.0 : 1.0);
        double s, c;
        sincos(angle, &s, &c);
        const double a = from[index], b = from[index + 1];
        to[index] = float(a * c - b * s);
        to[index + 1] = float(a * s + b * c);
        return;
    }
    if (index >= count) return;
    const size_t row = index / (vectors * pairs), rest = index % (vectors * pairs), vector = rest / pairs, pair = rest % pairs;
    const size_t at = (row * vectors + vector) * width + (width - 2 * pairs) + 2 * pair;
    const double angle = double(positions[row]) * double(frequencies[pair]) * (inverse ? -1.0 : 1.0);
    double s, c;
    sincos(angle, &s, &c);
    const double a = from[at], b = from[at + 1];
    to[at] = float(a * c - b * s);
    to[at + 1] = float(a * s + b * c);
}

// The two-level indexer's numbering (reference gpu/ops.hpp:1942-1951): a row's candidate list names blocks of `block` groups,
// in index order, -1 past the last; place p of the row's scores stands for group list[p / block] * block + p % block, and for
// no group at all (the value `groups`) in an unused slot.
struct CandidateMap {
    const int32_t* list;
    size_t block, groups;
    __device__ __forceinline__ size_t group_at(size_t place) const {
        const size_t slot = place / block;
        const int32_t named = list[slot];
        return named < 0 ? groups : size_t(named) * block + (place - slot * block);
    }
};

// Indexer scores, a thread per scored group.  q is uniform over the workgroup, so its values arrive through
// scalar loads and every fmaf is (scalar q, vector key, vector sum).  H = 32 or 64 heads are carried at once,
// the key's columns 32 at a time; each chain still adds its columns in order.
template<int H, bool BF16>
__global__ void __launch_bounds__(256) index_scores_kernel(const float* __restrict__ q, const void* __restrict__ keys, size_t key_batch_stride,
                                                           const float* __restrict__ weights, const int32_t* __restrict__ visible,
                                                           size_t groups, size_t heads, size_t dim, float scale, float* __restrict__ scores,
                                                           size_t score_stride, const int32_t* __restrict__ candidates, size_t blocks,
                                                           size_t block) {
    const size_t row = blockIdx.y, place = size_t(blockIdx.x) * 256 + threadIdx.x;
    const size_t scored = candidates ? blocks * block : groups;
    const int32_t* row_candidates = candidates ? candidates + row * blocks : nullptr;
    const size_t g = !row_candidates ? place : place < scored ? CandidateMap{row_candidates, block, groups}.group_at(place) : groups;
    const int32_t seen = visible[row];
    const size_t limit = min(groups, size_t(seen > 0 ? seen : 0));
    const size_t key_row = min(g, groups - 1);
    const float* row_q = q + row * heads * dim;
    float acc[H];
    #pragma unroll
    for (int h = 0; h < H; ++h) acc[h] = 0.0f;
    for (size_t d0 = 0; d0 < dim; d0 += 32) {
        float k[32];
        if (BF16) {
            const uint16_t* from = static_cast<const uint16_t*>(keys) + row * key_batch_stride + key_row * dim + d0;
            if (d0 + 32 <= dim && (reinterpret_cast<uintptr_t>(from) & 15) == 0) {
                #pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const uint4 raw = reinterpret_cast<const uint4*>(from)[v];
                    const uint32_t words[4] = {raw.x, raw.y, raw.z, raw.w};
                    #pragma unroll
                    for (int i = 0; i < 4; ++i) { k[8 * v + 2 * i] = __uint_as_float(words[i] << 16); k[8 * v + 2 * i + 1] = __uint_as_float(words[i] & 0xffff0000u); }
                }
            } else {
                #pragma unroll
                for (int c = 0; c < 32; ++c) k[c] = d0 + c < dim ? bf16_value(from[c]) : 0.0f;
            }
        } else {
            const float* from = static_cast<const float*>(keys) + row * key_batch_stride + key_row * dim + d0;
            #pragma unroll
            for (int c = 0; c < 32; ++c) k[c] = d0 + c < dim ? from[c] : 0.0f;
        }
        const int width = int(min(size_t(32), dim - d0));
        #pragma unroll
        for (int h = 0; h < H; ++h) {
            if (size_t(h) < heads) {
                const float* query = row_q + size_t(h) * dim + d0;
                if (width == 32) {
                    #pragma unroll
                    for (int c = 0; c < 32; ++c) acc[h] = __builtin_fmaf(query[c], k[c], acc[h]);
                } else {
                    for (int c = 0; c < width; ++c) acc[h] = __builtin_fmaf(query[c], k[c], acc[h]);
                }
            }
        }
    }
    if (place >= scored) return;
    float total = 0.0f;
    #pragma unroll
    for (int h = 0; h < H; ++h) {
        if (size_t(h) < heads) {
            // the term is rounded before it joins the sum: keep the multiply and the add apart
            total = add_rounded_product(total, fmaxf(acc[h], 0.0f), weights[row * heads + h]);
        }
    }
    scores[row * score_stride + place] = g < limit ? rounded_product(total, scale) : -INFINITY;
}

// ---- top-k -------------------------------------------------------------------------------------------------

// A score as an unsigned key of the same order (the rule of reference gpu/ops.hpp:1766-1769): both zeros are one key, a
// negative value has all its bits turned over, any other its sign bit set.  Integer work only: one mask from the sign.
__device__ __forceinline__ uint32_t top_k_key(float value) {
    uint32_t bits = __float_as_uint(value);
    if (!(bits << 1)) bits = 0;
    const uint32_t negative = uint32_t(int32_t(bits) >> 31);          // all ones below zero
    return bits ^ (negative | 0x80000000u);
}

constexpr int TOPK_THREADS = 1024, TOPK_WAVES = TOPK_THREADS / 64, TOPK_RUN = 8;

// Exclusive prefix of `value` over the workgroup in thread order, and the workgroup's sum.
__device__ __forceinline__ uint32_t block_scan(uint32_t value, uint32_t* wave_sums, uint32_t& total) {
    const unsigned lane = threadIdx.x % 64, wave = threadIdx.x / 64;
    uint32_t inclusive = value;
    #pragma unroll
    for (unsigned offset = 1; offset < 64; offset *= 2) {
        const uint32_t other = __shfl_up(inclusive, offset);
        if (lane >= offset) inclusive += other;
    }
    __syncthreads();
    if (lane == 63) wave_sums[wave] = inclusive;
    __syncthreads();
    uint32_t before = 0, sum = 0;
    #pragma unroll
    for (int w = 0; w < TOPK_WAVES; ++w) {
        const uint32_t c = wave_sums[w];
        before += unsigned(w) < wave ? c : 0u;
        sum += c;
    }
    total = sum;
    return before + inclusive - value;
}

// The same for two values at once (the exclusive prefix of the first is returned): one pair of barriers for both.
__device__ __forceinline__ uint32_t block_scan_pair(uint32_t first, uint32_t second, uint2* wave_sums, uint32_t& total_first, uint32_t& total_second) {
    const unsigned lane = threadIdx.x % 64, wave = threadIdx.x / 64;
    uint32_t inclusive = first, other_inclusive = second;
    #pragma unroll
    for (unsigned offset = 1; offset < 64; offset *= 2) {
        const uint32_t a = __shfl_up(inclusive, offset), b = __shfl_up(other_inclusive, offset);
        if (lane >= offset) { inclusive += a; other_inclusive += b; }
    }
    __syncthreads();
    if (lane == 63) wave_sums[wave] = uint2{inclusive, other_inclusive};
    __syncthreads();
    uint32_t before = 0, sum = 0, other_sum = 0;
    #pragma unroll
    for (int w = 0; w < TOPK_WAVES; ++w) {
        const uint2 c = wave_sums[w];
        before += unsigned(w) < wave ? c.x : 0u;
        sum += c.x; other_sum += c.y;
    }
    total_first = sum; total_second = other_sum;
    return before + inclusive - first;
}

// One workgroup per row.  The k-th highest key by four 8-bit radix passes (MSB first, a 256-bin histogram per pass
// in LDS), then one ordered pass: thread t owns runs of TOPK_RUN consecutive places so a workgroup scan of the kept
// counts gives every kept place its slot in ascending index order.  score(place) and index(place) let the same code
// serve plain rows and candidate-ordered rows.
template<class Score, class Index>
__device__ void top_k_row(Score score, Index index, size_t places, size_t k, int32_t* out) {
    __shared__ uint32_t bins[256];
    __shared__ uint32_t wave_sums[TOPK_WAVES];
    __shared__ uint32_t picked_bin, picked_rank, picked_count, live_total;
    const unsigned t = threadIdx.x;
    const uint32_t floor = top_k_key(-INFINITY);
    uint32_t prefix = 0, rank = uint32_t(k), equal_count = 0;
    bool all = false;
    for (int byte = 3; byte >= 0 && !all; --byte) {
        const int shift = 8 * byte;
        if (t < 256) bins[t] = 0;
        __syncthreads();
        for (size_t place = t; place < places; place += TOPK_THREADS) {
            const uint32_t key = top_k_key(score(place));
            if (key > floor && (byte == 3 || (key >> (shift + 8)) == (prefix >> (shift + 8)))) atomicAdd(&bins[(key >> shift) & 255u], 1u);
        }
        __syncthreads();
        // thread i < 256 holds bin 255 - i: the scan counts keys in higher bins
        const uint32_t count = t < 256 ? bins[255 - t] : 0u;
        uint32_t every;
        const uint32_t above = block_scan(count, wave_sums, every);
        if (t < 256 && above < rank && above + count >= rank) { picked_bin = 255 - t; picked_rank = rank - above; picked_count = count; }
        if (t == 0) live_total = every;
        __syncthreads();
        if (byte == 3 && live_total <= k) { all = true; break; }
        prefix |= picked_bin << shift;
        rank = picked_rank;
        equal_count = picked_count;
        __syncthreads();
    }
    // keys above `prefix` are kept; of the equal_count keys equal to it the first `rank` (lowest indices)
    const uint32_t threshold = prefix, need = all ? 0u : rank;
    (void)equal_count;
    uint32_t slot = 0, ties_seen = 0;
    const size_t tile = size_t(TOPK_THREADS) * TOPK_RUN;
    for (size_t base = 0; base < places; base += tile) {
        const size_t first = base + size_t(t) * TOPK_RUN;
        uint32_t keys[TOPK_RUN];
        uint32_t greater = 0, ties = 0;
        #pragma unroll
        for (int i = 0; i < TOPK_RUN; ++i) {
            keys[i] = first + i < places ? top_k_key(score(first + i)) : floor;
            const bool live = keys[i] > floor;
            greater += live && (all || keys[i] > threshold);
            ties += live && !all && keys[i] == threshold;
        }
        uint32_t tile_greater, tile_ties;
        const uint32_t greater_before = block_scan(greater, wave_sums, tile_greater);
        uint32_t tie_before = ties_seen + block_scan(ties, wave_sums, tile_ties);
        // slot of this thread's first kept place: kept before it = greater before + ties before that were still needed
        uint32_t at = slot + greater_before + (min(tie_before, need) - min(ties_seen, need));
        #pragma unroll
        for (int i = 0; i < TOPK_RUN; ++i) {
            const bool live = keys[i] > floor;
            bool keep = live && (all || keys[i] > threshold);
            if (live && !all && keys[i] == threshold) { keep = tie_before < need; ++tie_before; }
            if (keep) out[at++] = index(first + i);
        }
        slot += tile_greater + (min(ties_seen + tile_ties, need) - min(ties_seen, need));
        ties_seen += tile_ties;
    }
    for (size_t i = slot + t; i < k; i += TOPK_THREADS) out[i] = -1;
}

__global__ void __launch_bounds__(TOPK_THREADS) top_k_kernel(const float* scores, size_t groups, size_t score_stride, size_t k, int32_t* out) {
    const float* s = scores + size_t(blockIdx.x) * score_stride;
    top_k_row([s](size_t g) { return s[g]; }, [](size_t g) { return int32_t(g); }, groups, k, out + size_t(blockIdx.x) * k);
}

// Top-k over a row's candidate groups: scores are stored in candidate order (sd_op_index_select with candidates).
__global__ void __launch_bounds__(TOPK_THREADS) top_k_candidates_kernel(const float* scores, size_t score_stride, size_t groups, const int32_t* candidates,
                                                                        size_t blocks, size_t block, size_t k, int32_t* out) {
    const float* s = scores + size_t(blockIdx.x) * score_stride;
    const CandidateMap map{candidates + size_t(blockIdx.x) * blocks, block, groups};
    top_k_row([=](size_t place) { return map.group_at(place) < groups ? s[place] : -INFINITY; },
              [=](size_t place) { return int32_t(map.group_at(place)); }, blocks * block, k, out + size_t(blockIdx.x) * k);
}

// What the candidate pick ranks blocks by (reference gpu/ops.hpp:1952-1965): a block's highest score, and +inf for the block
// that holds the row's last visible group (the newest, partly filled block is always kept).  A wave per block: its lanes read
// the block's scores side by side and the maximum is five lane exchanges; four blocks a workgroup.
__global__ void __launch_bounds__(256) block_tops_kernel(const float* scores, const int32_t* visible, size_t groups, size_t block, size_t count,
                                                         float* tops) {
    const size_t row = blockIdx.y, b = size_t(blockIdx.x) * 4 + threadIdx.x / 64;
    if (b >= count) return;
    const unsigned lane = threadIdx.x % 64;
    const size_t begin = b * block, end = min(groups, begin + block);
    float top = -INFINITY;
    for (size_t g = begin + lane; g < end; g += 64) top = fmaxf(top, scores[row * groups + g]);
    #pragma unroll
    for (int offset = 32; offset; offset /= 2) top = fmaxf(top, __shfl_xor(top, offset));
    const int64_t newest = min(int64_t(groups), int64_t(visible[row])) - 1;     // the row's last visible group, if it sees any
    if (lane == 0) tops[row * count + b] = newest >= 0 && size_t(newest) / block == b ? INFINITY : top;
}

// ---- the sparse path's indexer on matrix cores --------------------------------------------------------------
//
// The canonical score (one fmaf chain per head, heads added in order) fixes every bit, and a matrix-core sum does not
// follow that order.  So the matrix cores only bracket each score: s~ from BF16 MFMAs with FP32 sums, and a margin e that
// bounds |s~ - s| for the canonical s (the reference takes the same road for its long contexts: approximate scores, a
// threshold, exact work near it only -- gpu/qsa_interval.hpp:152-419).  With L the k-th highest lower bound s~ - e, at least
// k groups score L or more, so a group whose upper bound s~ + e is below L cannot be among the top k, ties included.  The
// others (k and a few) are listed in index order, scored canonically, and the exact top-k runs over that list: the
// result is the canonical one, bit for bit.
//
// Margin: each head's MFMA dot and its canonical chain both differ from the real dot by at most 128 roundings of
// sum|q_d k_d| <= |q_h| |k|; the 1-Lipschitz max(.,0), the weights and the 64-term head sum add at most 130 roundings of
// sum_h |w_h| |dot_h|.  With unit roundoff 2^-23 (safe for truncating accumulators too) that is below 2^-14 |scale| |k| W,
// W = sum_h |w_h| |q_h| (3.8e-5 against 6.1e-5); the norms' own rounding is covered by a further percent.

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int RADIX_BINS = 2048, RADIX_LEVELS = 2, INTERVAL_KEYS = 1024;   // digits of 11 and 11 bits (the cut is the k-th highest lower bound's leading 22 bits: the
                                                                           // last 10 would spare a candidate in a thousand and cost a pass over the bounds); groups per workgroup
constexpr int BRACKET_WAVES = 8, BRACKET_KEYS = 4096, BRACKET_RING = 4;     // the bracket kernel: waves, groups per workgroup, stages per wave
__device__ __forceinline__ uint32_t radix_digit(uint32_t key, int level) { return level == 0 ? key >> 21 : level == 1 ? (key >> 10) & 2047u : key & 1023u; }

// The sum over the four lanes li, li + 16, li + 32, li + 48 in all of them (see paged_rows.hpp for the instructions).
__device__ __forceinline__ float quad_sum(float x) {
    float a = x, b = x;
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b));
    a += b; b = a;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
    return a + b;
}

// One global->LDS load: every lane's 16 bytes from its own address to LDS at to + 16 * lane (to is the wave's), marked as
// read once.  Written as instructions so that the compiler does not know of it: it would guard every later LDS read against
// all such loads in flight, and the ring of stages below is there to keep several in flight; the waits are explicit.
__device__ __forceinline__ void load_to_lds(const void* from, const void* to) {
    typedef __attribute__((address_space(3))) const uint8_t* lds_bytes;
    const uint32_t base = __builtin_amdgcn_readfirstlane(uint32_t(uintptr_t((lds_bytes)to)));
    uint32_t keep;      // M0 names the LDS address; it is put back for whatever else the compiler keeps there
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off nt\n\ts_mov_b32 m0, %0" : "=&s"(keep) : "v"(from), "s"(base) : "memory");
}

// The same from a base address that the whole wave shares (in scalar registers) and a lane's 32-bit offset from it: a loop that
// walks through memory then moves the base with scalar arithmetic and spends no vector instruction on addresses.
__device__ __forceinline__ void load_to_lds(const void* shared_base, uint32_t offset, const void* to) {
    typedef __attribute__((address_space(3))) const uint8_t* lds_bytes;
    const uint32_t base = __builtin_amdgcn_readfirstlane(uint32_t(uintptr_t((lds_bytes)to)));
    const uint64_t from = uint64_t(uintptr_t(shared_base));
    const uint64_t uniform = uint64_t(uint32_t(__builtin_amdgcn_readfirstlane(int(uint32_t(from))))) |
                             uint64_t(uint32_t(__builtin_amdgcn_readfirstlane(int(uint32_t(from >> 32))))) << 32;      // (the builtin gives a signed int)
    uint32_t keep;
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %3 nt\n\ts_mov_b32 m0, %0" : "=&s"(keep) : "v"(offset), "s"(base), "s"(uniform) : "memory");
}

// max(x, 0) as one instruction, an integer maximum of the bits: a negative number, a negative zero or a NaN with the sign set
// gives 0; a NaN without it stays (fmaxf would give 0, and cost an instruction more, which first quiets x).  For brackets
// only: a NaN or an infinity among the inputs reaches the bracket's margin as well, which is then no number either way.
__device__ __forceinline__ float positive_part(float x) { return __int_as_float(max(__float_as_int(x), 0)); }

// A square root good to a few units in the last place (the hardware's, with the scaling that keeps tiny arguments out of the
// flushed range): for bounds that carry a margin of their own.
__device__ __forceinline__ float rough_sqrt(float x) {
    const bool tiny = x < 0x1p-96f;
    const float root = __builtin_amdgcn_sqrtf(tiny ? x * 0x1p+32f : x);
    return tiny ? root * 0x1p-16f : root;
}

// Bounds of the scores of INTERVAL_KEYS groups per workgroup, 16 groups per MFMA tile and wave, and the first radix
// histogram of the lower bounds.  S = Q . K^T with Q (heads x dim) as A operands from registers and K rows as B operands;
// K . K^T from the same registers gives |k|^2 on its diagonal.  A tile's 16 rows are 4 KiB in one piece: they come HBM -> LDS
// by four coalesced 1 KiB global->LDS loads into the wave's ring of stages, three tiles ahead of the one being computed
// (two waves per SIMD leave room for that much in flight).  The loads place piece c of row r at position c ^ r of the row, so that the 16 lanes of an operand read (one
// row each, the same piece) touch 16 different banks.
// The histograms' place: [level][row][bin], and behind them the rows' largest margins (bits of a non-negative float, so that an
// integer atomic maximum orders them).  `rows` = the rows the buffer was made for.
__device__ __forceinline__ uint32_t* radix_bins(uint32_t* histogram, size_t rows, int level, size_t row) {
    return histogram + (size_t(level) * rows + row) * RADIX_BINS;
}
__device__ __forceinline__ uint32_t* widest_margin(uint32_t* histogram, size_t rows, size_t row) { return histogram + size_t(RADIX_LEVELS) * rows * RADIX_BINS + row; }

template<int HEADS>
__global__ void __launch_bounds__(BRACKET_WAVES * 64) index_interval_kernel(const uint16_t* __restrict__ q, const uint16_t* __restrict__ keys, const float* __restrict__ weights,
                                                             const int32_t* __restrict__ visible, size_t groups, float scale,
                                                             float* __restrict__ lower, float* __restrict__ upper, uint32_t* __restrict__ histogram, size_t histogram_rows) {
    constexpr int DIM = 128, HT = HEADS / 16, KS = DIM / 32;
    const size_t row = blockIdx.y;
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), li = lane & 15, g = lane >> 4;
    __shared__ uint32_t bins[RADIX_BINS];
    __shared__ __attribute__((aligned(16))) uint8_t stages[BRACKET_WAVES][BRACKET_RING][4096];
    for (int i = threadIdx.x; i < RADIX_BINS; i += BRACKET_WAVES * 64) bins[i] = 0;
    float widest = 0.0f;            // the largest margin this lane has given a live group
    bf16x8 qa[HT][KS];
    float w[HT][4], own[HT];
    #pragma unroll
    for (int t = 0; t < HT; ++t) {
        #pragma unroll
        for (int b = 0; b < KS; ++b)
            qa[t][b] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(q + (row * HEADS + 16 * t + li) * DIM + 32 * b + 8 * g));
        #pragma unroll
        for (int r = 0; r < 4; ++r) w[t][r] = weights[row * HEADS + 16 * t + 4 * g + r];
        own[t] = weights[row * HEADS + 16 * t + li];
    }
    const int32_t seen = visible[row];
    const size_t limit = min(groups, size_t(seen > 0 ? seen : 0));
    const uint16_t* row_keys = keys + row * groups * DIM;
    const size_t first = size_t(blockIdx.x) * BRACKET_KEYS, end = min(first + BRACKET_KEYS, groups);
    uint32_t place[4];                  // where in a tile's 4 KiB this lane's four pieces lie
    #pragma unroll
    for (int j = 0; j < 4; ++j) { const int r = 4 * j + g; place[j] = uint32_t(r * 256 + (li ^ r) * 16); }
    const auto copy_in = [&](int buffer, size_t tile) {
        if (tile + 16 <= groups) {
            #pragma unroll
            for (int j = 0; j < 4; ++j) load_to_lds(row_keys + tile * DIM, place[j], stages[wave][buffer] + 1024 * j);
        } else {
            // the row's last tile: the rows past the end read the last one again
            #pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int r = 4 * j + g, c = li ^ r;
                const uint16_t* from = row_keys + min(tile + r, groups - 1) * DIM + 8 * c;
                load_to_lds(from, stages[wave][buffer] + 1024 * j);
            }
        }
    };
    constexpr size_t stride = 16 * BRACKET_WAVES;
    // the wave's tiles, `count` of them, one every `stride` groups
    const size_t mine = first + 16 * wave;
    const int count = mine < end ? int((end - mine + stride - 1) / stride) : 0;
    const auto tile_at = [&](int turn) { return mine + size_t(turn) * stride; };
    // the first tiles are asked for before anything waits for the queries: they travel while the margin is worked out
    #pragma unroll
    for (int ahead = 0; ahead < BRACKET_RING; ++ahead)
        if (ahead < count) copy_in(ahead, tile_at(ahead));
    // W of the margin, sum_h |w_h| |q_h|, by every wave for itself: a lane's 32 values of head 16t + li squared and summed, the
    // four lane groups' parts added, the root times |w_h| added over the tile's 16 heads (lanes) and the tiles
    float reach = 0.0f;
    #pragma unroll
    for (int t = 0; t < HT; ++t) {
        float square = 0.0f;
        #pragma unroll
        for (int b = 0; b < KS; ++b) {
            const uint4 bits = __builtin_bit_cast(uint4, qa[t][b]);
            const uint32_t words[4] = {bits.x, bits.y, bits.z, bits.w};
            #pragma unroll
            for (int i = 0; i < 4; ++i) { const float lo = __uint_as_float(words[i] << 16), hi = __uint_as_float(words[i] & 0xffff0000u); square += lo * lo + hi * hi; }
        }
        reach += fabsf(own[t]) * sqrtf(quad_sum(square));
    }
    #pragma unroll
    for (int d = 8; d; d >>= 1) reach += __shfl_xor(reach, d);
    const float bound = reach * fabsf(scale) * (1.0f / 16384.0f) * 1.01f;      // 2^-14 |scale| W, rounded up a little
    __syncthreads();                         // the histogram's bins are zero
    // (the wait for the queries above was a wait for every load so far, the first tiles' among them: none of the compiler's
    // own loads is outstanding, and the loop's waits count the tiles' loads alone)
    __builtin_amdgcn_s_waitcnt(0x0f70);
    // Two tiles a turn, so that one's matrix products run under the other's arithmetic: the pair's operands are read from their
    // stages, the stages take the copies of the pair two turns on, and both tiles are worked out side by side.
    // A tile's 16 groups are finished by 16 lanes (lane group g = li / 4 holds group li's squared norm on the diagonal of
    // K . K^T); the pair's second tile goes to the lanes 32 further on, so one pass of this arithmetic, and one pair of
    // stores, serves both tiles.
    const auto finish = [&](size_t tile0, size_t tile1, bool second, float total0, float total1, const floatx4& norms0, const floatx4& norms1) {
        total0 = quad_sum(total0) * scale;
        total1 = quad_sum(total1) * scale;
        // the diagonal of K . K^T: row 4g + r = column li
        const int r = li & 3;
        const float square0 = r == 0 ? norms0[0] : r == 1 ? norms0[1] : r == 2 ? norms0[2] : norms0[3];
        const float square1 = r == 0 ? norms1[0] : r == 1 ? norms1[1] : r == 2 ? norms1[2] : norms1[3];
        float low_half = square1, high_half = square1;        // after the swap: the lower lanes' value in both halves / the upper lanes'
        asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(low_half), "+v"(high_half));
        const float across = lane < 32 ? high_half : low_half;      // square1 of the lane 32 away
        const bool own = g == (li >> 2), other = g == ((li >> 2) ^ 2);
        const size_t group = (own ? tile0 : tile1) + li;
        if ((own || (other && second)) && group < groups) {
            const float total = own ? total0 : total1;
            const float e = bound * rough_sqrt(own ? square0 : across);
            const bool live = group < limit;
            const float low = live ? total - e : -INFINITY, high = live ? total + e : -INFINITY;
            lower[row * groups + group] = low;
            upper[row * groups + group] = high;
            const uint32_t key = top_k_key(low);
            if (histogram && key > top_k_key(-INFINITY)) atomicAdd(&bins[radix_digit(key, 0)], 1u);
            if (live) widest = fmaxf(widest, e);
        }
    };
    for (int turn = 0, buffer = 0; turn < count; turn += 2, buffer ^= 2) {
        // The pair has landed when only what was issued after its second copy is outstanding: the bounds of the two pairs before
        // (two stores a pair, issued between the copies; memory operations finish in the order issued) and the copies of the
        // pair after this one, four loads a tile.  (The first two pairs had landed before the loop.)
        const int after = count - 1 - turn;                        // tiles after the pair's first
        const bool second = after >= 1;
        if (after >= 3) __builtin_amdgcn_s_waitcnt(0x0f7c); else if (after == 2) __builtin_amdgcn_s_waitcnt(0x0f78);       // 12, 8
        else __builtin_amdgcn_s_waitcnt(0x0f74);                                                                           // 4
        bf16x8 kb[2][KS];
        #pragma unroll
        for (int u = 0; u < 2; ++u) {
            #pragma unroll
            for (int b = 0; b < KS; ++b) kb[u][b] = *reinterpret_cast<const bf16x8*>(stages[wave][buffer + u] + li * 256 + 16 * ((4 * b + g) ^ li));
        }
        __builtin_amdgcn_s_waitcnt(0xc07f);          // the operands are in registers: the stages are free for the next copies
        if (turn + 4 < count) copy_in(buffer, tile_at(turn + 4));
        if (turn + 5 < count) copy_in(buffer + 1, tile_at(turn + 5));
        floatx4 norms[2];
        float total[2];
        #pragma unroll
        for (int u = 0; u < 2; ++u) {          // (the second of a lone tile's pair works on whatever its stage holds, and is dropped)
            norms[u] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
            #pragma unroll
            for (int b = 0; b < KS; ++b) norms[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kb[u][b], kb[u][b], norms[u], 0, 0, 0);
            total[u] = 0.0f;
            #pragma unroll
            for (int t = 0; t < HT; ++t) {
                floatx4 dots = {0.0f, 0.0f, 0.0f, 0.0f};
                #pragma unroll
                for (int b = 0; b < KS; ++b) dots = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qa[t][b], kb[u][b], dots, 0, 0, 0);
                #pragma unroll
                for (int r = 0; r < 4; ++r) total[u] = fmaf(positive_part(dots[r]), w[t][r], total[u]);
            }
        }
        finish(tile_at(turn), tile_at(turn + 1), second, total[0], total[1], norms[0], norms[1]);
    }
    if (!histogram) return;
    #pragma unroll
    for (int d = 32; d; d >>= 1) widest = fmaxf(widest, __shfl_xor(widest, d));
    __shared__ uint32_t widest_of_all;
    if (threadIdx.x == 0) widest_of_all = 0u;
    __syncthreads();
    if (lane == 0 && widest > 0.0f) atomicMax(&widest_of_all, __float_as_uint(widest));
    __syncthreads();
    // (one atomic per workgroup and row: hundreds of waves on one address would queue up at the end of the kernel)
    if (threadIdx.x == 0 && widest_of_all) atomicMax(widest_margin(histogram, histogram_rows, row), widest_of_all);
    uint32_t* to = radix_bins(histogram, histogram_rows, 0, row);
    for (int i = threadIdx.x; i < RADIX_BINS; i += BRACKET_WAVES * 64)
        if (bins[i]) atomicAdd(&to[i], bins[i]);
}

// Where the rank-th highest key lies, one digit at a time, from the levels' histograms (256 threads, every workgroup
// that needs it finds it anew).  After `levels` digits: the key's leading digits and the rank among the keys that share
// them; `everything` when fewer than rank keys are live at all.
struct RadixPick { uint32_t prefix, rank; bool everything; };
__device__ RadixPick radix_pick(uint32_t* histogram, size_t rows, size_t row, int levels, uint32_t k) {
    __shared__ uint32_t wave_sums[4], found[2];
    RadixPick pick{0u, k, false};
    const unsigned t = threadIdx.x, lane = t & 63, wave = t >> 6;
    // thread t owns the 8 bins below 2048 - 8t of every level, highest first; all levels are asked for at once (a level's histogram
    // is one array whatever the digits before it turn out to be), so the levels cost one trip to memory, not one each
    uint4 loaded[RADIX_LEVELS][2];
    #pragma unroll
    for (int level = 0; level < RADIX_LEVELS; ++level)
        if (level < levels) {
            const uint32_t* bins = radix_bins(histogram, rows, level, row);
            loaded[level][0] = *reinterpret_cast<const uint4*>(bins + RADIX_BINS - 8 - 8 * t);
            loaded[level][1] = *reinterpret_cast<const uint4*>(bins + RADIX_BINS - 4 - 8 * t);
        }
    #pragma unroll
    for (int level = 0; level < RADIX_LEVELS; ++level) {
        if (level >= levels) break;
        // a scan in thread order counts the keys in higher bins
        uint32_t mine[8], sum = 0;
        const uint4 a = loaded[level][0], b = loaded[level][1];
        mine[0] = b.w; mine[1] = b.z; mine[2] = b.y; mine[3] = b.x; mine[4] = a.w; mine[5] = a.z; mine[6] = a.y; mine[7] = a.x;
        #pragma unroll
        for (int i = 0; i < 8; ++i) sum += mine[i];
        uint32_t inclusive = sum;
        #pragma unroll
        for (unsigned offset = 1; offset < 64; offset *= 2) { const uint32_t other = __shfl_up(inclusive, offset); if (lane >= offset) inclusive += other; }
        __syncthreads();                              // the shared words of the level before are read
        if (lane == 63) wave_sums[wave] = inclusive;
        __syncthreads();
        uint32_t above = inclusive - sum, every = 0;
        #pragma unroll
        for (unsigned v = 0; v < 4; ++v) { const uint32_t c = wave_sums[v]; above += v < wave ? c : 0u; every += c; }
        if (level == 0 && every < pick.rank) { pick.everything = true; return pick; }
        if (above < pick.rank && above + sum >= pick.rank) {
            uint32_t before = above;
            #pragma unroll
            for (int i = 0; i < 8; ++i) {
                if (before < pick.rank && before + mine[i] >= pick.rank) { found[0] = RADIX_BINS - 1 - (8 * t + i); found[1] = pick.rank - before; }
                before += mine[i];
            }
        }
        __syncthreads();
        pick.prefix = level == 0 ? found[0] << 21 : level == 1 ? pick.prefix | (found[0] << 10) : pick.prefix | found[0];
        pick.rank = found[1];
    }
    return pick;
}

// The second digit's histogram of the lower bounds, over the keys that share the first digit of the k-th highest.
__global__ void __launch_bounds__(256) radix_histogram_kernel(const float* lower, size_t groups, size_t rows, uint32_t k, uint32_t* histogram) {
    const size_t row = blockIdx.y;
    __shared__ uint32_t bins[RADIX_BINS];
    for (int i = threadIdx.x; i < RADIX_BINS; i += 256) bins[i] = 0;
    // (the groups' values are asked for before the pick's own trip to memory ends)
    const size_t first = size_t(blockIdx.x) * INTERVAL_KEYS;
    float values[INTERVAL_KEYS / 256];
    #pragma unroll
    for (int j = 0; j < INTERVAL_KEYS / 256; ++j) { const size_t group = first + threadIdx.x + 256 * j; values[j] = group < groups ? lower[row * groups + group] : -INFINITY; }
    const RadixPick pick = radix_pick(histogram, rows, row, 1, k);
    __syncthreads();
    if (pick.everything) return;
    #pragma unroll
    for (int j = 0; j < INTERVAL_KEYS / 256; ++j) {
        const uint32_t key = top_k_key(values[j]);
        if ((key & 0xffe00000u) == pick.prefix && key > top_k_key(-INFINITY)) atomicAdd(&bins[radix_digit(key, 1)], 1u);
    }
    __syncthreads();
    uint32_t* to = radix_bins(histogram, rows, 1, row);
    for (int i = threadIdx.x; i < RADIX_BINS; i += 256)
        if (bins[i]) atomicAdd(&to[i], bins[i]);
}

// Which groups can still matter, a workgroup per INTERVAL_KEYS groups of a row (a segment), listed in index order in the
// segment's own stretch of `list` (no counting pass over the row first: a reader adds up the segments' counts).
//   candidate   upper bound >= the k-th highest lower bound (its leading 22 bits): nobody else can be among the best k;
//   certain     lower bound above L + 2 E, L the k-th highest lower bound (the next 22-bit step above it) and E the row's widest
//               margin: no upper bound is more than 2 E above its lower bound, so the k-th highest upper bound is at most
//               L + 2 E, fewer than k groups can score as high as this one, and it is among the best k whatever its exact
//               score -- it is listed with the CERTAIN bit and needs no canonical score;
//   the rest of the candidates are the band around the cut: only they are scored canonically.
// With fewer than k live groups everything live is a certain candidate.
//
// The band members of the segment get their canonical score here as well, a wave a member (the workgroup's four waves take the
// members in turn): a lane per head; a wave that has a member reads its head's 128 query values itself, two to a word (a lane
// its own 256 bytes: a load spreads over 64 lines -- staged through LDS by coalesced loads in every workgroup, the same 16 KB a
// row made a thousand workgroups ask for the same lines at the same moment and cost 13 us); a key row is 64 words, lane i
// fetches word i (one coalesced load, the next member's row on its way while this one is used) and the words go round by
// v_readlane, so a member costs a wave 64 broadcasts and 128 multiply-adds in the canonical column order.  Then the member's
// terms are added in head order, a broadcast and an addition a head.  A score lands at its group's place in the list.
constexpr uint32_t CERTAIN = 0x80000000u;
template<int HEADS>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4, 4)))
candidate_segments_kernel(const float* lower, const float* upper, size_t groups, size_t rows, uint32_t k, uint32_t* histogram, int32_t* list, uint32_t* counts,
                          const uint16_t* __restrict__ q, const uint16_t* __restrict__ keys, const float* __restrict__ weights, float scale, float* __restrict__ scores) {
    constexpr int DIM = 128;
    const size_t row = blockIdx.y;
    const size_t first = size_t(blockIdx.x) * INTERVAL_KEYS + 4 * threadIdx.x;        // thread t owns 4 consecutive groups
    // (the groups' bounds are asked for before the pick's own trip to memory ends)
    float low[4], high[4];
    if (first + 3 < groups && (row * groups) % 4 == 0) {
        const float4 l4 = *reinterpret_cast<const float4*>(lower + row * groups + first), h4 = *reinterpret_cast<const float4*>(upper + row * groups + first);
        low[0] = l4.x; low[1] = l4.y; low[2] = l4.z; low[3] = l4.w; high[0] = h4.x; high[1] = h4.y; high[2] = h4.z; high[3] = h4.w;
    } else {
        #pragma unroll
        for (int i = 0; i < 4; ++i) { const bool in = first + i < groups; low[i] = in ? lower[row * groups + first + i] : -INFINITY; high[i] = in ? upper[row * groups + first + i] : -INFINITY; }
    }
    const float widest = __uint_as_float(*widest_margin(histogram, rows, row));
    const RadixPick pick = radix_pick(histogram, rows, row, RADIX_LEVELS, k);
    const uint32_t floor = top_k_key(-INFINITY);
    // L's 22-bit step taken upwards as a value, 2 E added and the sum pushed up a little: a bound on the k-th highest upper bound
    float certain_above = INFINITY;
    if (!pick.everything && pick.prefix <= 0xffffffffu - 1024u) {
        const uint32_t key = pick.prefix + 1024u, bits = key & 0x80000000u ? key ^ 0x80000000u : ~key;
        const float sum = __uint_as_float(bits) + 2.0f * widest;
        certain_above = sum + fabsf(sum) * 1.0e-6f;
        if (!(certain_above == certain_above)) certain_above = INFINITY;      // a NaN in the bounds: nothing is certain
    }
    __shared__ uint32_t wave_sums[4];
    __shared__ uint32_t band_members[INTERVAL_KEYS];              // place in the segment's list << 10 | group within the segment
    uint32_t entry[4], mine = 0, band = 0;
    #pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t high_key = top_k_key(high[i]);
        const bool keep = first + i < groups && (pick.everything ? high_key > floor : high_key >= pick.prefix);
        const bool certain = pick.everything || low[i] > certain_above;
        entry[i] = keep ? uint32_t(first + i) | (certain ? CERTAIN : 0u) : 0xffffffffu;
        mine += keep;
        band += keep && !certain;
    }
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    uint32_t packed = mine | (band << 16), inclusive = packed;        // both counts scanned at once (at most 1024 each)
    #pragma unroll
    for (int offset = 1; offset < 64; offset *= 2) { const uint32_t other = __shfl_up(inclusive, offset); if (lane >= offset) inclusive += other; }
    if (lane == 63) wave_sums[wave] = inclusive;
    __syncthreads();
    uint32_t before = 0, all = 0;
    for (int v = 0; v < 4; ++v) { before += v < wave ? wave_sums[v] : 0u; all += wave_sums[v]; }
    uint32_t at = (before + inclusive - packed) & 0xffffu, band_at = (before + inclusive - packed) >> 16;
    int32_t* out = list + row * groups + size_t(blockIdx.x) * INTERVAL_KEYS;
    #pragma unroll
    for (int i = 0; i < 4; ++i)
        if (entry[i] != 0xffffffffu) {
            if (!(entry[i] & CERTAIN)) band_members[band_at++] = (at << 10) | (4 * threadIdx.x + i);
            out[at++] = int32_t(entry[i]);
        }
    if (threadIdx.x == 0) counts[row * gridDim.x + blockIdx.x] = all;        // candidates | band members << 16
    const int members = int(all >> 16);
    if (!members) return;
    __syncthreads();
    if (wave >= members) return;
    const int head = min(lane, HEADS - 1);
    const float weight = weights[row * HEADS + head];
    // the head's query values, two to a word (a lane reads its own head's 256 bytes: every load spreads over 64 lines, and
    // the many waves that read the same row at the same time do not crowd on one of them)
    uint4 query[DIM / 8];
    #pragma unroll
    for (int j = 0; j < DIM / 8; ++j) query[j] = reinterpret_cast<const uint4*>(q + (row * HEADS + head) * DIM)[j];
    const uint32_t* segment_keys = reinterpret_cast<const uint32_t*>(keys + (row * groups + size_t(blockIdx.x) * INTERVAL_KEYS) * DIM);
    uint32_t member = band_members[wave];
    uint32_t words = segment_keys[size_t(member & 1023u) * (DIM / 2) + lane];
    for (int m = wave; m < members; m += 4) {
        const uint32_t current = words, place = member >> 10;
        if (m + 4 < members) {
            member = band_members[m + 4];
            words = segment_keys[size_t(member & 1023u) * (DIM / 2) + lane];
        }
        // (the queries are widened again for every member -- 128 widened values held across the loop would cost a wave of
        // occupancy -- which the shift and the mask being unknown to the compiler sees to)
        uint32_t up = 16u, high_half = 0xffff0000u;
        asm volatile("" : "+s"(up), "+s"(high_half));
        float dot = 0.0f;
        #pragma unroll
        for (int d = 0; d < DIM; d += 8) {
            const uint32_t pairs[4] = {query[d / 8].x, query[d / 8].y, query[d / 8].z, query[d / 8].w};
            #pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint32_t pair = __builtin_amdgcn_readlane(current, d / 2 + i);
                dot = __builtin_fmaf(__uint_as_float(pairs[i] << up), __uint_as_float(pair << 16), dot);
                dot = __builtin_fmaf(__uint_as_float(pairs[i] & high_half), __uint_as_float(pair & 0xffff0000u), dot);
            }
        }
        // the heads' terms added in head order: lane h holds head h's, every lane adds them all (a broadcast and an addition a
        // head, nothing through LDS)
        const float term = rounded_product(fmaxf(dot, 0.0f), weight);
        float sum = 0.0f;
        #pragma unroll
        for (int h = 0; h < HEADS; ++h) sum = rounded_sum(sum, __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(term), h)));
        if (lane == 0) scores[row * groups + size_t(blockIdx.x) * INTERVAL_KEYS + place] = rounded_product(sum, scale);
    }
}

// The row's best k from its candidates, one workgroup per row: every certain candidate, and of the band the best by canonical
// score (ties to the lowest index) for the places that are left; ascending indices, -1 past the last.  The segments' lists are
// first laid end to end -- in LDS when they fit, else in `flat` (global) -- with one synthetic score each: +inf for a certain
// candidate (above every band member, as it is known to be), the canonical score for a band member; the exact top-k over that
// row is then the result.  A band of at most a thousand is ranked directly (every member counts who beats it, one to eight
// threads a member); anything larger takes the general radix select.
__global__ void __launch_bounds__(TOPK_THREADS) index_finish_kernel(const float* scores, const int32_t* list, const uint32_t* counts, size_t segments, size_t groups,
                                                                    size_t k, float* flat_scores, int32_t* flat_list, int32_t* out, uint32_t* histogram,
                                                                    size_t histogram_rows) {
    const size_t row = blockIdx.x;
    const unsigned t = threadIdx.x;
    // The histograms' last reader ran before this kernel: the row's are zeroed (and its widest margin) for the next call.
    for (int level = 0; level < RADIX_LEVELS; ++level) {
        uint32_t* bins = radix_bins(histogram, histogram_rows, level, row);
        for (unsigned i = t; i < unsigned(RADIX_BINS); i += TOPK_THREADS) bins[i] = 0u;
    }
    if (t == 0) *widest_margin(histogram, histogram_rows, row) = 0u;
    constexpr uint32_t HELD = 6144, RANKED = 1024;
    __shared__ float held_scores[HELD];
    __shared__ int32_t held_list[HELD];
    __shared__ uint32_t segment_base[TOPK_THREADS];
    __shared__ __attribute__((aligned(16))) uint64_t band_order[RANKED + 2];     // a member's key above its place turned over: a higher value beats a lower one
    __shared__ uint32_t wave_sums[TOPK_WAVES], band_filled;
    // the candidates and band members of the row, and where each segment's candidates go in the flat list
    __shared__ uint2 wave_pairs[TOPK_WAVES];
    uint32_t candidates = 0, band = 0;
    for (size_t first = 0; first < segments; first += TOPK_THREADS) {
        const uint32_t count = first + t < segments ? counts[row * segments + first + t] : 0u;
        uint32_t all, all_band;
        const uint32_t before = block_scan_pair(count & 0xffffu, count >> 16, wave_pairs, all, all_band);
        if (first == 0) segment_base[t] = before;
        candidates += all; band += all_band;
        __syncthreads();
    }
    const bool held = candidates <= HELD && segments <= TOPK_THREADS;
    float* const row_scores = held ? held_scores : flat_scores + row * groups;
    int32_t* const row_list = held ? held_list : flat_list + row * groups;
    if (t == 0) band_filled = 0;
    if (held) {
        // a thread per place of the flat list: the segment that holds it by bisection, then one trip to memory for all of them
        __syncthreads();
        for (uint32_t place = t; place < candidates; place += TOPK_THREADS) {
            uint32_t segment = 0;
            for (uint32_t step = TOPK_THREADS / 2; step; step /= 2)
                if (segment + step < segments && segment_base[segment + step] <= place) segment += step;
            // (segments without candidates share their base with the next one: move on to the one that really holds the place)
            const size_t at = row * groups + size_t(segment) * INTERVAL_KEYS + (place - segment_base[segment]);
            const uint32_t entry = uint32_t(list[at]);
            const float scored = scores[at];               // (asked for beside the entry, whether it will count or not: one trip, not two)
            const bool certain = entry & CERTAIN;
            const float score = certain ? INFINITY : scored;
            held_scores[place] = score;
            held_list[place] = int32_t(entry & ~CERTAIN);
            if (!certain && band <= RANKED) {
                const uint32_t slot = atomicAdd(&band_filled, 1u);
                band_order[slot] = (uint64_t(top_k_key(score)) << 32) | (0xffffffffu - place);
            }
        }
        __syncthreads();
    } else {
        // the general way: one segment after the other through global memory, by the whole workgroup
        uint32_t base = 0;
        for (size_t segment = 0; segment < segments; ++segment) {
            const uint32_t count = counts[row * segments + segment] & 0xffffu;
            for (uint32_t i = t; i < count; i += TOPK_THREADS) {
                const uint32_t entry = uint32_t(list[row * groups + segment * INTERVAL_KEYS + i]);
                row_scores[base + i] = entry & CERTAIN ? INFINITY : scores[row * groups + segment * INTERVAL_KEYS + i];
                row_list[base + i] = int32_t(entry & ~CERTAIN);
            }
            base += count;
        }
        __threadfence_block();
        __syncthreads();
    }
    int32_t* const row_out = out + row * k;
    const uint32_t certain = candidates - band;
    if (held && band <= RANKED && certain <= k) {
        // direct ranking: member i is kept when fewer than `room` members beat it (a higher key, or the same key earlier in the list)
        const uint32_t room = uint32_t(min(size_t(band), k - certain)), floor = top_k_key(-INFINITY);
        if (band & 1u) { if (t == 0) band_order[band] = 0; __syncthreads(); }        // (pairs are read: an odd band gets a member that beats nobody)
        // (a short band is shared out over more threads: 2, 4 or 8 of them count a member's betters, each its share of the pairs)
        const uint32_t parts = band <= 128 ? 8u : band <= 256 ? 4u : band <= 512 ? 2u : 1u;
        const uint32_t member = t / parts, part = t % parts;
        uint64_t mine = 0;
        uint32_t beaten_by = 0;
        if (member < band) {
            mine = band_order[member];
            const ulonglong2* pairs = reinterpret_cast<const ulonglong2*>(band_order);
            #pragma unroll 4
            for (uint32_t j = part; j < (band + 1) / 2; j += parts) { const ulonglong2 two = pairs[j]; beaten_by += (two.x > mine) + (two.y > mine); }
        }
        for (uint32_t offset = 1; offset < parts; offset *= 2) beaten_by += __shfl_xor(beaten_by, int(offset));
        if (member < band && part == 0 && (uint32_t(mine >> 32) <= floor || beaten_by >= room))
            held_list[0xffffffffu - uint32_t(mine)] = -1;                          // not kept: a score of -inf never is
        __syncthreads();
        // ordered compaction of what is kept
        uint32_t slot = 0;
        for (uint32_t base = 0; base < candidates; base += TOPK_THREADS * 4) {
            int32_t mine[4];
            uint32_t kept = 0;
            #pragma unroll
            for (int i = 0; i < 4; ++i) { const uint32_t at = base + 4 * t + i; mine[i] = at < candidates ? held_list[at] : -1; kept += mine[i] >= 0; }
            uint32_t all;
            uint32_t at = slot + block_scan(kept, wave_sums, all);
            #pragma unroll
            for (int i = 0; i < 4; ++i) if (mine[i] >= 0) row_out[at++] = mine[i];
            slot += all;
            __syncthreads();
        }
        for (size_t i = slot + t; i < k; i += TOPK_THREADS) row_out[i] = -1;
        return;
    }
    if (held) top_k_row([&](size_t v) { return held_scores[v]; }, [&](size_t v) { return held_list[v]; }, candidates, k, row_out);
    else top_k_row([=](size_t v) { return row_scores[v]; }, [=](size_t v) { return row_list[v]; }, candidates, k, row_out);
}

// All of a row's histograms to zero: after a call that only wanted the bounds.
__global__ void __launch_bounds__(256) radix_clear_kernel(uint32_t* histogram, size_t words) {
    for (size_t i = size_t(blockIdx.x) * 256 + threadIdx.x; i < words; i += size_t(gridDim.x) * 256) histogram[i] = 0u;
}

__global__ void widen_bf16_kernel(const uint16_t* from, float* to, size_t count) {
    for (size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x; i < count; i += size_t(gridDim.x) * blockDim.x) to[i] = bf16_value(from[i]);
}

void widen_bf16(Device& d, const void* from, float* to, size_t count) {
    widen_bf16_kernel<<<unsigned(std::min<size_t>(checked_blocks(count), 65536)), 256, 0, d.stream>>>(static_cast<const uint16_t*>(from), to, count);
    SD_CHECK(hipGetLastError());
}

void launch_scores(Device& d, const float* q, const void* keys, bool bf16, size_t key_batch_stride, const float* weights, const int32_t* visible,
                   size_t rows, size_t groups, size_t heads, size_t dim, float scale, float* scores, size_t score_stride,
                   const int32_t* candidates, size_t blocks, size_t block) {
    const size_t scored = candidates ? blocks * block : groups;
    const dim3 grid(checked_blocks(scored), unsigned(rows));
#define SD_SCORES(H, B) index_scores_kernel<H, B><<<grid, 256, 0, d.stream>>>(q, keys, key_batch_stride, weights, visible, groups, heads, dim, scale, \
                                                                              scores, score_stride, candidates, blocks, block)
    if (heads <= 32) { if (bf16) SD_SCORES(32, true); else SD_SCORES(32, false); }
    else { if (bf16) SD_SCORES(64, true); else SD_SCORES(64, false); }
#undef SD_SCORES
    SD_CHECK(hipGetLastError());
}


// The matrix-core indexer of the batched sparse path (scores are not returned by it): see the kernels above.
bool index_fast_supported(uint64_t heads, uint64_t dim) { return dim == 128 && heads % 16 == 0 && heads >= 16 && heads <= 64; }

struct FastIndexSpace { float *lower, *upper, *scores, *flat_scores; uint32_t* counts; int32_t *list, *flat_list; size_t segments; };
size_t fast_index_bytes(size_t batch, size_t groups) {
    const size_t segments = (groups + INTERVAL_KEYS - 1) / INTERVAL_KEYS;
    return 4 * (6 * batch * groups + batch * segments) + 8 * 256;
}
FastIndexSpace fast_index_space(void* base, size_t batch, size_t groups) {
    uint8_t* at = static_cast<uint8_t*>(base);
    const auto take = [&](size_t words) { void* p = at; at += (4 * words + 255) & ~size_t(255); return p; };
    FastIndexSpace s{};
    s.segments = (groups + INTERVAL_KEYS - 1) / INTERVAL_KEYS;
    s.lower = static_cast<float*>(take(batch * groups)); s.upper = static_cast<float*>(take(batch * groups));
    s.scores = static_cast<float*>(take(batch * groups)); s.list = static_cast<int32_t*>(take(batch * groups));
    s.flat_scores = static_cast<float*>(take(batch * groups)); s.flat_list = static_cast<int32_t*>(take(batch * groups));
    s.counts = static_cast<uint32_t*>(take(batch * s.segments));
    return s;
}

// The radix histograms of the handle: [lower | upper][level][row][bin], all zero between calls (the kernel after their last reader zeroes them; a call that failed part-way leaves them marked, and the next call clears them first).  They
// live apart from the workspace, which other ops overwrite.
uint32_t* index_histograms(Device& d, size_t batch) {
    const size_t words = size_t(RADIX_LEVELS) * RADIX_BINS + 1;        // a row's histograms and its widest margin
    if (batch > d.index_bins_rows) {
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        SD_CHECK(hipStreamIsCapturing(d.stream, &capturing));
        if (capturing != hipStreamCaptureStatusNone) throw std::runtime_error("Straydog index histograms cannot grow while a graph is recorded");
        if (d.index_bins) {
            drop_recorded_graphs(d);
            release(d, d.index_bins);
            d.index_bins = nullptr; d.index_bins_rows = 0;
        }
        d.index_bins = static_cast<uint32_t*>(allocate(d, words * batch * 4, true));
        d.index_bins_rows = batch;
        d.index_bins_dirty = false;
    }
    if (d.index_bins_dirty) {
        radix_clear_kernel<<<64, 256, 0, d.stream>>>(d.index_bins, words * d.index_bins_rows);
        SD_CHECK(hipGetLastError());
        d.index_bins_dirty = false;
    }
    return d.index_bins;
}

template<int HEADS>
void fast_index_bounds(Device& d, const void* q_index, const void* keys, const float* weights, const int32_t* visible, size_t batch, size_t groups, float scale,
                       float* lower, float* upper, uint32_t* histogram) {
    timed_launch(d, &index_interval_kernel<HEADS>, dim3(unsigned((groups + BRACKET_KEYS - 1) / BRACKET_KEYS), unsigned(batch)), dim3(BRACKET_WAVES * 64), 0,
                 static_cast<const uint16_t*>(q_index), static_cast<const uint16_t*>(keys), weights, visible, groups, scale, lower, upper, histogram, d.index_bins_rows);
    SD_CHECK(hipGetLastError());
}

template<int HEADS>
void fast_index_top_k(Device& d, const FastIndexSpace& s, const void* q_index, const void* keys, const float* weights, const int32_t* visible, size_t batch,
                      size_t groups, float scale, size_t k, int32_t* indices) {
    uint32_t* const histogram = index_histograms(d, batch);
    d.index_bins_dirty = true;           // until the last kernel, which zeroes them again, is queued
    const unsigned segments = unsigned(s.segments);
    fast_index_bounds<HEADS>(d, q_index, keys, weights, visible, batch, groups, scale, s.lower, s.upper, histogram);
    const uint32_t rank = uint32_t(std::min<size_t>(k, 0xffffffffu));
    radix_histogram_kernel<<<dim3(segments, unsigned(batch)), 256, 0, d.stream>>>(s.lower, groups, d.index_bins_rows, rank, histogram);
    candidate_segments_kernel<HEADS><<<dim3(segments, unsigned(batch)), 256, 0, d.stream>>>(s.lower, s.upper, groups, d.index_bins_rows, rank, histogram, s.list, s.counts,
                                                                                          static_cast<const uint16_t*>(q_index), static_cast<const uint16_t*>(keys), weights,
                                                                                          scale, s.scores);
    index_finish_kernel<<<unsigned(batch), TOPK_THREADS, 0, d.stream>>>(s.scores, s.list, s.counts, s.segments, groups, k, s.flat_scores, s.flat_list, indices, histogram,
                                                                        d.index_bins_rows);
    SD_CHECK(hipGetLastError());
    d.index_bins_dirty = false;
}


// The indexer's projection (one decode row): weights[h] = row h of a heads x cols matrix . x, the matrix rows BF16 (kind 30) or
// ggml Q8_0 blocks (kind 8: an FP16 scale d, then 32 int8; reference gpu/core.hpp:1290-1294).  The reference forms these with its
// GEMV stack, whose summation order follows a per-device lane count (gpu/gemv_common.hpp:785-812, gpu/gemv.hpp:1-60); here the
// order is fixed for wave64 and stated, so the bits are reproducible on the CPU: a wave per head; lane L takes the units L,
// L + 64, ... (a unit = 8 BF16 columns, or one Q8_0 block of 32); a unit's value is one chain of fused multiply-adds over its
// columns in order, started from zero (for Q8_0 over float(q) * x, the chain then multiplied by the block's scale); a lane adds
// its units' values in order; the lanes' sums are added by exchanges at distances 32, 16, 8, 4, 2, 1.
template<int KIND>
__global__ void __launch_bounds__(256) index_projection_kernel(const uint8_t* matrix, size_t row_bytes, size_t cols, const float* x, size_t heads,
                                                               float* weights) {
    const size_t head = size_t(blockIdx.x) * 4 + threadIdx.x / 64;
    if (head >= heads) return;
    const unsigned lane = threadIdx.x % 64;
    const uint8_t* row = matrix + head * row_bytes;
    constexpr size_t UNIT = KIND == 30 ? 8 : 32;
    float sum = 0.0f;
    for (size_t unit = lane; unit < cols / UNIT; unit += 64) {
        const float* in = x + unit * UNIT;
        float chain = 0.0f;
        if (KIND == 30) {
            const uint4 packed = *reinterpret_cast<const uint4*>(row + unit * 16);
            const uint32_t words[4] = {packed.x, packed.y, packed.z, packed.w};
            #pragma unroll
            for (int i = 0; i < 4; ++i) {
                chain = fmaf(__uint_as_float(words[i] << 16), in[2 * i], chain);
                chain = fmaf(__uint_as_float(words[i] & 0xffff0000u), in[2 * i + 1], chain);
            }
        } else {
            const uint8_t* blockp = row + unit * 34;
            const float d = __half2float(*reinterpret_cast<const __half*>(blockp));
            #pragma unroll
            for (int i = 0; i < 32; ++i) chain = fmaf(float(reinterpret_cast<const int8_t*>(blockp + 2)[i]), in[i], chain);
            chain *= d;
        }
        sum = rounded_sum(sum, chain);
    }
    #pragma unroll
    for (int offset = 32; offset; offset /= 2) sum = rounded_sum(sum, __shfl_xor(sum, offset));
    if (lane == 0) weights[head] = sum;
}

// Every check of the projection's arguments; returns the bytes of a weight row.
size_t index_projection_check(Device& value, const void* proj_weights, int proj_kind, uint64_t proj_cols, const float* x, uint64_t heads, float* weights) {
    if (!proj_weights || !proj_cols || proj_cols > 8192 || !heads || heads > 64) throw std::runtime_error("invalid Straydog index shape");
    if (proj_kind != 30 && proj_kind != 8) throw std::runtime_error("the index projection takes BF16 (kind 30) or Q8_0 (kind 8) rows");
    if (proj_cols % (proj_kind == 30 ? 8 : 32)) throw std::runtime_error("invalid Straydog index shape");
    const size_t row_bytes = proj_kind == 30 ? size_t(proj_cols) * 2 : size_t(proj_cols) / 32 * 34;
    op_span(value, proj_weights, checked_product({heads, row_bytes}), "a weight matrix");
    op_span(value, x, checked_floats({proj_cols}), "a linear input");
    op_span(value, weights, checked_floats({heads}), "index weights");
    if (proj_kind == 30 && reinterpret_cast<uintptr_t>(proj_weights) % 16) throw std::runtime_error("BF16 projection rows must be 16-byte aligned");
    return row_bytes;
}

void index_projection_launch(Device& value, const void* proj_weights, int proj_kind, uint64_t proj_cols, const float* x, uint64_t heads, float* weights,
                             size_t row_bytes) {
    const unsigned grid = unsigned((heads + 3) / 4);
    const auto* matrix = static_cast<const uint8_t*>(proj_weights);
    if (proj_kind == 30) index_projection_kernel<30><<<grid, 256, 0, value.stream>>>(matrix, row_bytes, size_t(proj_cols), x, size_t(heads), weights);
    else index_projection_kernel<8><<<grid, 256, 0, value.stream>>>(matrix, row_bytes, size_t(proj_cols), x, size_t(heads), weights);
}

void index_projection(Device& value, const void* proj_weights, int proj_kind, uint64_t proj_cols, const float* x, uint64_t heads, float* weights) {
    index_projection_launch(value, proj_weights, proj_kind, proj_cols, x, heads, weights,
                            index_projection_check(value, proj_weights, proj_kind, proj_cols, x, heads, weights));
}

// Every check of the fused indexer's arguments (nothing is queued before all of them have passed, as gpu/kernels.cpp:5626-5640).
void index_select_check(Device& value, const float* q, const float* keys, const float* weights, const int32_t* visible, uint64_t rows,
                        uint64_t groups, uint64_t heads, uint64_t dim, uint64_t rope_dims, const int32_t* positions,
                        const float* frequencies, float* scores, uint64_t k, int32_t* out, const int32_t* candidates, uint64_t blocks,
                        uint64_t block) {
    if (!rows || rows > 65535 || !groups || groups > (uint64_t(1) << 31) || !heads || heads > 64 || !dim || !k || k > (uint64_t(1) << 31) ||
        rope_dims % 2 || rope_dims > dim || rope_dims > 128)
        throw std::runtime_error("invalid Straydog index shape");
    uint64_t scored = groups;
    if (candidates) {
        if (!blocks || !block || blocks > (uint64_t(1) << 20) || block > 4096) throw std::runtime_error("invalid Straydog index candidates");
        op_span(value, candidates, checked_floats({rows, blocks}), "index candidates");
        scored = blocks * block;
    }
    op_span(value, q, checked_floats({rows, heads, dim}), "index queries");
    op_state_span(value, keys, checked_product({groups, dim}), "index keys");
    op_span(value, weights, checked_floats({rows, heads}), "index weights");
    op_span(value, visible, checked_floats({rows}), "visible counts");
    op_span(value, positions, checked_floats({rows}), "query positions");
    if (rope_dims) op_span(value, frequencies, checked_floats({rope_dims / 2}), "rope frequencies");
    op_span(value, scores, checked_floats({rows, std::max(groups, scored)}), "index scores");
    op_span(value, out, checked_floats({rows, k}), "top-k indices");
}

void index_select_launch(Device& value, const float* q, const float* keys, const float* weights, const int32_t* visible, uint64_t rows,
                         uint64_t groups, uint64_t heads, uint64_t dim, float scale, uint64_t rope_dims, const int32_t* positions,
                         const float* frequencies, float* scores, uint64_t k, int32_t* out, const int32_t* candidates, uint64_t blocks,
                         uint64_t block) {
    const uint64_t scored = candidates ? blocks * block : groups;
    const float* rotated = q;
    if (rope_dims) {
        // q itself stays as it was: the rotated copy lives in the device's workspace
        const size_t count = checked_product({rows, heads, dim});
        float* copy = static_cast<float*>(workspace(value, count * 4));
        rope_kernel<<<checked_blocks(count), 256, 0, value.stream>>>(q, copy, count, size_t(heads), size_t(dim), size_t(rope_dims / 2), positions,
                                                                     frequencies, 0, 1);
        SD_CHECK(hipGetLastError());
        rotated = copy;
    }
    // scores rows are `scored` wide with candidates (candidate order), `groups` wide without
    const size_t stride = candidates ? size_t(scored) : size_t(groups);
    launch_scores(value, rotated, state_base(keys), state_bf16(keys), 0, weights, visible, size_t(rows), size_t(groups), size_t(heads), size_t(dim),
                  scale, scores, stride, candidates, size_t(blocks), size_t(block ? block : 1));
    if (candidates)
        top_k_candidates_kernel<<<unsigned(rows), TOPK_THREADS, 0, value.stream>>>(scores, stride, size_t(groups), candidates, size_t(blocks),
                                                                                   size_t(block), size_t(k), out);
    else
        top_k_kernel<<<unsigned(rows), TOPK_THREADS, 0, value.stream>>>(scores, size_t(groups), stride, size_t(k), out);
    SD_CHECK(hipGetLastError());
}

void index_select(Device& value, const float* q, const float* keys, const float* weights, const int32_t* visible, uint64_t rows,
                  uint64_t groups, uint64_t heads, uint64_t dim, float scale, uint64_t rope_dims, const int32_t* positions,
                  const float* frequencies, float* scores, uint64_t k, int32_t* out, const int32_t* candidates, uint64_t blocks,
                  uint64_t block) {
    index_select_check(value, q, keys, weights, visible, rows, groups, heads, dim, rope_dims, positions, frequencies, scores, k, out, candidates, blocks, block);
    index_select_launch(value, q, keys, weights, visible, rows, groups, heads, dim, scale, rope_dims, positions, frequencies, scores, k, out, candidates,
                        blocks, block);
}

}  // namespace

extern "C" {

int sd_op_to_bf16(void* handle, const float* x, uint64_t count, void* out) {
    SD_OP_BEGIN
    if (!count) return 0;
    op_span(value, x, checked_floats({count}), "values to round");
    op_span(value, out, checked_product({count, 2}), "BF16 values");
    to_bf16_kernel<<<unsigned(std::min<size_t>(checked_blocks(size_t(count)), 65536)), 256, 0, value.stream>>>(x, size_t(count), static_cast<uint16_t*>(out));
    SD_OP_END
}

int sd_op_compress(void* handle, const float* kv, const float* gate, uint64_t groups, uint64_t ratio, uint64_t dim, float* out) {
    SD_OP_BEGIN
    if (!groups || !ratio || !dim) throw std::runtime_error("invalid Straydog compress shape");
    op_span(value, kv, checked_floats({groups, ratio, dim}), "rows to compress");
    if (gate) op_span(value, gate, checked_floats({groups, ratio, dim}), "a compression gate");
    op_span(value, out, checked_floats({groups, dim}), "compressed rows");
    const size_t values = checked_product({groups, dim});
    const auto aligned = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
    if (dim % 4 == 0 && aligned(kv) && aligned(gate) && aligned(out))
        compress_kernel<4><<<checked_blocks(values / 4), 256, 0, value.stream>>>(kv, gate, values / 4, size_t(ratio), size_t(dim), out);
    else
        compress_kernel<1><<<checked_blocks(values), 256, 0, value.stream>>>(kv, gate, values, size_t(ratio), size_t(dim), out);
    SD_OP_END
}

/* reference straydog_gpu.h:271 (gpu/kernels.cpp:4942-4956, kernel gpu/ops.hpp:107-120) */
int sd_op_rope(void* handle, float* x, uint64_t rows, uint64_t vectors, uint64_t width, uint64_t rope_dims, const int32_t* positions,
               const float* frequencies, int inverse) {
    SD_OP_BEGIN
    if (!rows || !vectors || !rope_dims || rope_dims % 2 || rope_dims > width) throw std::runtime_error("invalid Straydog rope shape");
    op_span(value, x, checked_floats({rows, vectors, width}), "a rotated buffer");
    op_span(value, positions, checked_floats({rows}), "rope positions");
    op_span(value, frequencies, checked_floats({rope_dims / 2}), "rope frequencies");
    const size_t count = checked_product({rows, vectors, rope_dims / 2});
    rope_kernel<<<checked_blocks(count), 256, 0, value.stream>>>(x, x, count, size_t(vectors), size_t(width), size_t(rope_dims / 2), positions,
                                                                 frequencies, inverse, 0);
    SD_OP_END
}

int sd_op_index_scores(void* handle, const float* q, const float* keys, const float* weights, const int32_t* visible, uint64_t rows,
                       uint64_t groups, uint64_t heads, uint64_t dim, float scale, float* scores) {
    SD_OP_BEGIN
    if (!rows || rows > 65535 || !groups || groups > (uint64_t(1) << 31) || !heads || heads > 64 || !dim) throw std::runtime_error("invalid Straydog index shape");
    op_span(value, q, checked_floats({rows, heads, dim}), "index queries");
    op_state_span(value, keys, checked_product({groups, dim}), "index keys");
    op_span(value, weights, checked_floats({rows, heads}), "index weights");
    op_span(value, visible, checked_floats({rows}), "visible counts");
    op_span(value, scores, checked_floats({rows, groups}), "index scores");
    launch_scores(value, q, state_base(keys), state_bf16(keys), 0, weights, visible, size_t(rows), size_t(groups), size_t(heads), size_t(dim), scale,
                  scores, size_t(groups), nullptr, 0, 1);
    SD_OP_END
}

int sd_op_top_k(void* handle, const float* scores, uint64_t rows, uint64_t groups, uint64_t k, int32_t* out) {
    SD_OP_BEGIN
    if (!rows || rows > 0x7fffffffu || !groups || !k || groups > (uint64_t(1) << 31) || k > (uint64_t(1) << 31)) throw std::runtime_error("invalid Straydog top-k shape");
    op_span(value, scores, checked_floats({rows, groups}), "scores");
    op_span(value, out, checked_floats({rows, k}), "top-k indices");
    top_k_kernel<<<unsigned(rows), TOPK_THREADS, 0, value.stream>>>(scores, size_t(groups), size_t(groups), size_t(k), out);
    SD_OP_END
}

int sd_op_index_candidates(void* handle, const float* scores, const int32_t* visible, uint64_t rows, uint64_t groups, uint64_t blocks,
                           uint64_t block, int32_t* out, float* scratch, uint64_t scratch_bytes) {
    SD_OP_BEGIN
    if (!rows || rows > 65535 || !groups || groups > (uint64_t(1) << 31) || !blocks || blocks > (uint64_t(1) << 20) || !block || block > 4096)
        throw std::runtime_error("invalid Straydog index candidates");
    const uint64_t count = (groups + block - 1) / block;
    op_span(value, scores, checked_floats({rows, groups}), "index scores");
    op_span(value, visible, checked_floats({rows}), "visible counts");
    op_span(value, out, checked_floats({rows, blocks}), "index candidates");
    if (checked_floats({rows, count}) > scratch_bytes) throw std::runtime_error("Straydog index candidates need more scratch");
    op_span(value, scratch, checked_floats({rows, count}), "index candidates' scratch");
    block_tops_kernel<<<dim3(checked_blocks(size_t(count), 4), unsigned(rows)), 256, 0, value.stream>>>(scores, visible, size_t(groups), size_t(block),
                                                                                                 size_t(count), scratch);
    SD_CHECK(hipGetLastError());
    top_k_kernel<<<unsigned(rows), TOPK_THREADS, 0, value.stream>>>(scratch, size_t(count), size_t(count), size_t(blocks), out);
    SD_OP_END
}

int sd_op_index_select(void* handle, const float* q, const float* keys, const float* weights, const int32_t* visible, uint64_t rows,
                       uint64_t groups, uint64_t heads, uint64_t dim, float scale, uint64_t rope_dims, const int32_t* positions,
                       const float* frequencies, float* scores, uint64_t k, int32_t* out, const int32_t* candidates, uint64_t blocks,
                       uint64_t block) {
    SD_OP_BEGIN
    index_select(value, q, keys, weights, visible, rows, groups, heads, dim, scale, rope_dims, positions, frequencies, scores, k, out, candidates,
                 blocks, block);
    SD_OP_END
}

int sdx_index_projection(void* handle, const void* proj_weights, int proj_kind, uint64_t proj_cols, const float* x, uint64_t heads, float* weights) {
    SD_OP_BEGIN
    index_projection(value, proj_weights, proj_kind, proj_cols, x, heads, weights);
    SD_OP_END
}

/* reference straydog_gpu.h:422 (gpu/kernels.cpp:5620-5667, kernel gpu/ops.hpp:2267-2300): one decode row's indexer with the
 * projection of x into the heads' weights ahead of it; the weights are left in `weights`. */
int sd_op_index_select_proj(void* handle, const void* proj_weights, int proj_kind, uint64_t proj_cols, const float* x, const float* q,
                            const float* keys, float* weights, const int32_t* visible, uint64_t groups, uint64_t heads, uint64_t dim, float scale,
                            uint64_t rope_dims, const int32_t* positions, const float* frequencies, float* scores, uint64_t k, int32_t* out,
                            const int32_t* candidates, uint64_t blocks, uint64_t block) {
    SD_OP_BEGIN
    // every argument of both halves is checked before the projection, which overwrites `weights`, is queued
    const size_t row_bytes = index_projection_check(value, proj_weights, proj_kind, proj_cols, x, heads, weights);
    index_select_check(value, q, keys, weights, visible, 1, groups, heads, dim, rope_dims, positions, frequencies, scores, k, out, candidates, blocks, block);
    index_projection_launch(value, proj_weights, proj_kind, proj_cols, x, heads, weights, row_bytes);
    SD_CHECK(hipGetLastError());
    index_select_launch(value, q, keys, weights, visible, 1, groups, heads, dim, scale, rope_dims, positions, frequencies, scores, k, out, candidates, blocks,
                        block);
    SD_OP_END
}

int sdx_index_top_k(void* handle, const void* q_index, const void* keys, const float* weights, const int32_t* visible, uint64_t batch,
                    uint64_t groups, uint64_t heads, uint64_t dim, float scale, float* scores, uint64_t k, int32_t* indices) {
    SD_OP_BEGIN
    if (!batch || batch > 65535 || !groups || groups > (uint64_t(1) << 31) || !heads || heads > 64 || !dim || !k || k > (uint64_t(1) << 31))
        throw std::runtime_error("invalid Straydog index shape");
    op_span(value, q_index, checked_product({batch, heads, dim, 2}), "index queries");
    op_span(value, keys, checked_product({batch, groups, dim, 2}), "index keys");
    op_span(value, weights, checked_floats({batch, heads}), "index weights");
    op_span(value, visible, checked_floats({batch}), "visible counts");
    op_span(value, indices, checked_floats({batch, k}), "top-k indices");
    const bool whole_pieces = (uintptr_t(q_index) | uintptr_t(keys)) % 16 == 0;        // the matrix-core path reads 16 bytes at a time
    if (!scores && index_fast_supported(heads, dim) && whole_pieces) {
        // the matrix cores bracket the scores; the canonical arithmetic runs on the few groups near the k-th only
        const FastIndexSpace space = fast_index_space(workspace(value, fast_index_bytes(batch, groups)), batch, groups);
        switch (heads) {
            case 16: fast_index_top_k<16>(value, space, q_index, keys, weights, visible, batch, groups, scale, k, indices); break;
            case 32: fast_index_top_k<32>(value, space, q_index, keys, weights, visible, batch, groups, scale, k, indices); break;
            case 48: fast_index_top_k<48>(value, space, q_index, keys, weights, visible, batch, groups, scale, k, indices); break;
            default: fast_index_top_k<64>(value, space, q_index, keys, weights, visible, batch, groups, scale, k, indices); break;
        }
        return 0;
    }
    // workspace: the queries widened to FP32 (exact), and the scores when the caller does not want them
    const size_t q_bytes = checked_floats({batch, heads, dim}), score_bytes = checked_floats({batch, groups});
    uint8_t* space = static_cast<uint8_t*>(workspace(value, q_bytes + 256 + (scores ? 0 : score_bytes)));
    float* wide_q = reinterpret_cast<float*>(space);
    float* row_scores = scores ? scores : reinterpret_cast<float*>(space + ((q_bytes + 255) & ~size_t(255)));
    if (scores) op_span(value, scores, score_bytes, "index scores");
    widen_bf16(value, q_index, wide_q, size_t(batch * heads * dim));
    launch_scores(value, wide_q, keys, true, size_t(groups * dim), weights, visible, size_t(batch), size_t(groups), size_t(heads), size_t(dim), scale,
                  row_scores, size_t(groups), nullptr, 0, 1);
    top_k_kernel<<<unsigned(batch), TOPK_THREADS, 0, value.stream>>>(row_scores, size_t(groups), size_t(groups), size_t(k), indices);
    SD_OP_END
}

int sdx_index_score_bounds(void* handle, const void* q_index, const void* keys, const float* weights, const int32_t* visible, uint64_t batch,
                           uint64_t groups, uint64_t heads, uint64_t dim, float scale, float* lower, float* upper) {
    SD_OP_BEGIN
    if (!batch || batch > 65535 || !groups || groups > (uint64_t(1) << 31) || !index_fast_supported(heads, dim))
        throw std::runtime_error("invalid Straydog index shape");
    if ((uintptr_t(q_index) | uintptr_t(keys)) % 16) throw std::runtime_error("Straydog index queries and keys must lie on 16-byte boundaries here");
    op_span(value, q_index, checked_product({batch, heads, dim, 2}), "index queries");
    op_span(value, keys, checked_product({batch, groups, dim, 2}), "index keys");
    op_span(value, weights, checked_floats({batch, heads}), "index weights");
    op_span(value, visible, checked_floats({batch}), "visible counts");
    op_span(value, lower, checked_floats({batch, groups}), "score bounds");
    op_span(value, upper, checked_floats({batch, groups}), "score bounds");
    // (no histograms: the bounds alone)
    switch (heads) {
        case 16: fast_index_bounds<16>(value, q_index, keys, weights, visible, batch, groups, scale, lower, upper, nullptr); break;
        case 32: fast_index_bounds<32>(value, q_index, keys, weights, visible, batch, groups, scale, lower, upper, nullptr); break;
        case 48: fast_index_bounds<48>(value, q_index, keys, weights, visible, batch, groups, scale, lower, upper, nullptr); break;
        default: fast_index_bounds<64>(value, q_index, keys, weights, visible, batch, groups, scale, lower, upper, nullptr); break;
    }
    SD_OP_END
}

}  // extern "C"

