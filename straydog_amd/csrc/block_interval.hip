// Qwen's block selection for a prompt chunk from FP16 matrix products with a proven error bound: the selection the exact
// kernels make (block_index.hip), block for block, ties and order included, at a fraction of their arithmetic.
//
// The reference does this on RDNA4 WMMA (gpu/qsa_interval.hpp:1-36 states the bound, :152 the key pass, :218 the scan, :323 the
// threshold, :419 the selection); this is the same idea laid out for gfx950: v_mfma_f32_16x16x32_f16, wave64, a chunk's
// queries resident in LDS as B operands, keys pre-packed as A operands so a wave's load is 1 KB of consecutive bytes.
//
// The bound.  h(x) rounds an element to FP16 (below the smallest normal FP16: zero, so no denormal ever reaches the matrix
// unit), r(x) = x - h(x) is exact in FP32.  For a pooled key k and the four query heads q_h the matrix unit forms
// a = sum_h max(h(k).h(q_h), 0).  The exact score e = sum_h max(fl(k.q_h), 0) (128 fused multiply-adds in order) differs by
//     |e - a| <= kappa (M + eps N) + rho (N + M),   kappa = |h(k)|, rho = |r(k)|, N = sum_h |h(q_h)|, M = sum_h |r(q_h)|
// (Cauchy-Schwarz on h.r + r.h + r.r; max(., 0) is 1-Lipschitz; eps = 2^-14 covers the FP32 rounding of the exact chain,
// 2^-17 of the magnitudes, and of the matrix unit's accumulation, which is taken to stay within 2^-15 of them; the whole is
// inflated by 2 % for the rounding of the bound's own arithmetic).  So e lies in [a - d, a + d].
//
// The selection.  T = the 512th highest exact score of a row.  A threshold t is guessed from a sample (every 32nd block, the
// 40th highest lower bound: about the 1280th best block); the scan over all blocks keeps, as a bit per (row, block) and the
// matrix unit's score, every block whose upper bound reaches t, and a second bit where the lower bound does.  If at least 512
// lower bounds reach t then T >= t and every block of the best 512 is among the kept ones; otherwise, or when a row keeps more
// than CAP blocks or must rescore more than BAND, or an input is beyond FP16 or not a number, the row is flagged and the exact
// kernels, launched behind this for flagged rows only, decide it: the guess costs time when it is wrong, never a different
// result.  Among the kept blocks the 512th highest lower bound Lk and upper bound Uk split them: lower bound above Uk is
// certainly selected, upper bound below Lk certainly not, the rest (the band) is scored exactly, in the exact kernels' order of
// operations, and T is the (512 - certain)th highest of those; ties at T go to the earliest blocks, the list is in block order.
#include "device.hpp"
#include "../../include/straydog_gpu_ext.h"

#include <algorithm>
#include <type_traits>

using namespace sd;

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int HEADS = 4, COLUMNS = 128, KEEP = 512;
constexpr int GROUP = 64;                 // blocks a wave scans at a time: four tiles of 16
constexpr int ROWS = 128;                 // rows a scan workgroup holds in LDS: eight tiles of 16
constexpr int SCAN_WAVES = 8;
constexpr int STRIDE = 32, AIM = 40;      // one block in 32 is sampled; the threshold is the sample's 40th highest lower bound
constexpr int SAMPLE_ROOM = 2112;         // sampled blocks a row can have (65536 / 32, rounded up to whole groups)
constexpr int CAP = 3072, BAND = 1024;    // kept blocks and rescored blocks a row may have
constexpr int GROUP_OPS = 4 * 4 * 64;     // a group's keys as A operands: [tile][32 columns][lane] x 16 bytes
constexpr int ROWS_OPS = 8 * 16 * 64;     // a workgroup's queries as B operands: [tile][head x 32 columns][lane] x 16 bytes
constexpr float HALF_MIN = 6.103515625e-05f, HALF_MAX = 65504.0f;
constexpr float ACCUMULATION = 6.103515625e-05f;   // 2^-14
constexpr float SLACK = 1.02f;

__device__ __forceinline__ float as_half(float x) { return fabsf(x) < HALF_MIN ? 0.0f : float(_Float16(x)); }

// Order-preserving keys of floats (no NaN reaches them).
__device__ __forceinline__ uint32_t ordered(float value) {
    const uint32_t bits = __float_as_uint(value);
    return bits >> 31 ? ~bits : bits | 0x80000000u;
}
__device__ __forceinline__ float unordered(uint32_t key) { return __uint_as_float(key >> 31 ? key ^ 0x80000000u : ~key); }

__device__ __forceinline__ float positive_sum(const float (&dot)[HEADS]) {
    float total = fmaxf(dot[0], 0.0f) + fmaxf(dot[1], 0.0f);
    total += fmaxf(dot[2], 0.0f);
    total += fmaxf(dot[3], 0.0f);
    return total;
}

// The same sum for the matrix unit's products, where any form of the positive part does: as integers a negative float is a
// negative number, so one integer maximum takes the positive part.
__device__ __forceinline__ float positive(float x) { return __int_as_float(max(__float_as_int(x), 0)); }
__device__ __forceinline__ float positive_sum(float a, float b, float c, float d) { return ((positive(a) + positive(b)) + positive(c)) + positive(d); }

// Eight elements as a piece of an operand; their squares and their residuals' squares added to hh and rr.
__device__ __forceinline__ uint4 pack8(const float (&x)[8], float& hh, float& rr, bool& bad) {
    half8 piece;
    #pragma unroll
    for (int j = 0; j < 8; ++j) {
        bad |= !(fabsf(x[j]) <= HALF_MAX);
        const float h = as_half(x[j]), r = x[j] - h;
        hh = fmaf(h, h, hh); rr = fmaf(r, r, rr);
        piece[j] = _Float16(h);
    }
    return __builtin_bit_cast(uint4, piece);
}

// ---- the keys as A operands, with each block's kappa and rho -------------------------------------------------------------------
// A workgroup packs one group of 64 blocks: the group's [128 columns][64 blocks] tile goes through LDS (the reads from the
// column-major keys are 256 consecutive bytes a wave), then lane (block i of tile m, column group kg) gathers its eight columns of
// each of the four 32-column steps.  Every 32nd block is the sample's: its pieces and norms go to the sample's operands as well
// (sampled block v / 32 of the sample's groups).  The tile also leaves as an FP32 copy in block order, [block][128 columns], which
// the selection rescans a block of in one piece.
__device__ __forceinline__ void pack_queries(unsigned part, const float* __restrict__ queries, size_t stride, size_t base, size_t steps, size_t pool,
                                             unsigned padded_rows, uint4* __restrict__ ops, float4* __restrict__ info, uint32_t* __restrict__ flags);

__global__ void __launch_bounds__(256) interval_pack_kernel(const float* __restrict__ blocks, size_t pool, unsigned count, unsigned first_group,
                                                            unsigned groups, uint4* __restrict__ ops, float2* __restrict__ stats,
                                                            uint4* __restrict__ sample_ops, float2* __restrict__ sample_stats, float* __restrict__ copy,
                                                            const float* __restrict__ queries, size_t stride, size_t base, size_t steps,
                                                            unsigned padded_rows, uint4* __restrict__ query_ops, float4* __restrict__ info,
                                                            uint32_t* __restrict__ flags) {
    __shared__ float tile[COLUMNS][GROUP + 1];
    if (blockIdx.x >= groups) {         // the workgroups behind the keys' pack the queries, four rows each
        pack_queries(blockIdx.x - groups, queries, stride, base, steps, pool, padded_rows, query_ops, info, flags);
        return;
    }
    const unsigned t = threadIdx.x, group = first_group + blockIdx.x, lane = t % 64;
    {
        const unsigned v = group * GROUP + lane;
        #pragma unroll 8
        for (unsigned c = t / 64; c < COLUMNS; c += 4) tile[c][lane] = v < count ? blocks[size_t(c) * pool + v] : 0.0f;
    }
    __syncthreads();
    const unsigned m = t / 64, i = m * 16 + lane % 16, kg = lane / 16, v = group * GROUP + i;
    const bool sampled = v % STRIDE == 0;
    const unsigned sv = v / STRIDE;
    float hh = 0.0f, rr = 0.0f;
    bool bad = false;
    #pragma unroll
    for (unsigned s = 0; s < 4; ++s) {
        float x[8];
        #pragma unroll
        for (int j = 0; j < 8; ++j) x[j] = tile[s * 32 + kg * 8 + j][i];
        const uint4 piece = pack8(x, hh, rr, bad);
        ops[size_t(group) * GROUP_OPS + (m * 4 + s) * 64 + lane] = piece;
        if (sampled) sample_ops[size_t(sv / GROUP) * GROUP_OPS + ((sv % GROUP / 16) * 4 + s) * 64 + kg * 16 + sv % 16] = piece;
    }
    hh += __shfl_xor(hh, 16); hh += __shfl_xor(hh, 32);
    rr += __shfl_xor(rr, 16); rr += __shfl_xor(rr, 32);
    if (kg == 0) {
        const float2 norms = make_float2(sqrtf(hh), sqrtf(rr));
        stats[v] = norms;
        if (sampled) sample_stats[sv] = norms;
    }
    (void)bad;      // (a key beyond FP16 leaves norms that are not numbers: the scan keeps such a block, the selection sees it)
    // the copy: a wave writes a block's 128 columns as 512 consecutive bytes
    for (unsigned b = t / 32; b < GROUP; b += 8) {
        const unsigned c = (t % 32) * 4;
        *reinterpret_cast<float4*>(copy + (size_t(group) * GROUP + b) * COLUMNS + c) = make_float4(tile[c][b], tile[c + 1][b], tile[c + 2][b], tile[c + 3][b]);
    }
}

// ---- the queries as B operands, with each row's bound factors ------------------------------------------------------------------
// A wave per row: lane (head, 32-column step, column group) packs eight columns.  info[row] = (threshold, to come; the factor of
// kappa; the factor of rho; the row's complete blocks as bits).  Also clears the row's flag and the count of flagged rows.
__device__ __forceinline__ void pack_queries(unsigned part, const float* __restrict__ queries, size_t stride, size_t base, size_t steps, size_t pool,
                                             unsigned padded_rows, uint4* __restrict__ ops, float4* __restrict__ info, uint32_t* __restrict__ flags) {
    const unsigned lane = threadIdx.x % 64, row = part * 4 + threadIdx.x / 64;
    const unsigned head = lane / 16, s = (lane / 4) % 4, kg = lane % 4;
    const bool live = row < steps;
    float x[8];
    #pragma unroll
    for (int j = 0; j < 8; ++j) x[j] = live ? queries[size_t(row) * stride + head * COLUMNS + s * 32 + kg * 8 + j] : 0.0f;
    float hh = 0.0f, rr = 0.0f;
    bool bad = false;
    ops[(size_t(row / ROWS) * 8 + (row % ROWS) / 16) * (16 * 64) + (head * 4 + s) * 64 + kg * 16 + row % 16] = pack8(x, hh, rr, bad);
    #pragma unroll
    for (int offset = 1; offset < 16; offset *= 2) { hh += __shfl_xor(hh, offset); rr += __shfl_xor(rr, offset); }
    float n = sqrtf(hh), m = sqrtf(rr);
    n += __shfl_xor(n, 16); n += __shfl_xor(n, 32);
    m += __shfl_xor(m, 16); m += __shfl_xor(m, 32);
    const bool any_bad = __any(bad);
    if (lane == 0) {
        const unsigned complete = live ? unsigned(min((base + row + 1) / 4, pool)) : 0u;
        info[row] = make_float4(INFINITY, SLACK * fmaf(ACCUMULATION, n, m), SLACK * (n + m), __uint_as_float(complete));
        flags[row] = any_bad ? 1u : 0u;
        if (row == 0) flags[padded_rows] = 0u;         // (the count of rows left to the exact kernels)
    }
}

// ---- the scan ------------------------------------------------------------------------------------------------------------------
// A product tile gives lane (row n = lane % 16, blocks 4g .. 4g + 3 of each of the group's four 16-block tiles): the lane bounds its
// sixteen scores with the row's factors and the blocks' norms.
struct ScanTask {
    half8 a[4][4];              // the group's keys: [tile][32-column step]
    float kappa[4][4], rho[4][4];
};

__device__ __forceinline__ void load_task(ScanTask& task, const uint4* __restrict__ key_ops, const float2* __restrict__ key_stats, unsigned group, unsigned lane) {
    #pragma unroll
    for (int m = 0; m < 4; ++m) {
        #pragma unroll
        for (int s = 0; s < 4; ++s) task.a[m][s] = __builtin_bit_cast(half8, key_ops[size_t(group) * GROUP_OPS + (m * 4 + s) * 64 + lane]);
    }
    #pragma unroll
    for (int m = 0; m < 4; ++m) {
        #pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float2 norms = key_stats[size_t(group) * GROUP + m * 16 + 4 * (lane / 16) + r];
            task.kappa[m][r] = norms.x; task.rho[m][r] = norms.y;
        }
    }
}

// The 64 products of a group with a row tile, whose B operands `fetch(head * 4 + step)` yields.
template<class Fetch>
__device__ __forceinline__ void multiply(const ScanTask& task, floatx4 (&acc)[4][HEADS], Fetch fetch) {
    #pragma unroll
    for (int m = 0; m < 4; ++m) {
        #pragma unroll
        for (int h = 0; h < HEADS; ++h) acc[m][h] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
    }
    #pragma unroll
    for (int h = 0; h < HEADS; ++h) {
        #pragma unroll
        for (int s = 0; s < 4; ++s) {
            const half8 b = fetch(h * 4 + s);
            #pragma unroll
            for (int m = 0; m < 4; ++m) acc[m][h] = __builtin_amdgcn_mfma_f32_16x16x32_f16(task.a[m][s], b, acc[m][h], 0, 0, 0);
        }
    }
}

// The sample: a workgroup per sampled group, a wave per row tile (operands straight from global memory: there is no reuse to stage
// them for); the lower bounds go to sample[row][v].
__global__ void __launch_bounds__(64 * SCAN_WAVES) interval_sample_kernel(const uint4* __restrict__ key_ops, const float2* __restrict__ key_stats,
                                                                           const uint4* __restrict__ query_ops, const float4* __restrict__ info,
                                                                           unsigned count, unsigned steps, float* __restrict__ sample) {
    const unsigned lane = threadIdx.x % 64, tile = blockIdx.y * SCAN_WAVES + threadIdx.x / 64, group = blockIdx.x;
    if (tile * 16 >= steps) return;
    ScanTask task;
    load_task(task, key_ops, key_stats, group, lane);
    floatx4 acc[4][HEADS];
    multiply(task, acc, [&](int piece) { return __builtin_bit_cast(half8, query_ops[(size_t(tile) * 16 + piece) * 64 + lane]); });
    const unsigned row = tile * 16 + lane % 16;
    const float4 mine = info[row];
    if (row >= steps) return;
    #pragma unroll
    for (int m = 0; m < 4; ++m) {
        #pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float score = positive_sum(acc[m][0][r], acc[m][1][r], acc[m][2][r], acc[m][3][r]);
            const float d = fmaf(task.kappa[m][r], mine.y, task.rho[m][r] * mine.z);
            const unsigned v = group * GROUP + m * 16 + 4 * (lane / 16) + r;
            sample[size_t(row) * SAMPLE_ROOM + v] = v < count ? score - d : -INFINITY;
        }
    }
}

// The scan proper: a workgroup of eight waves holds 128 rows' queries in LDS; each wave takes one group of 64 blocks and multiplies
// it with the row tiles that have rows.  Bits "upper bound reaches the row's threshold" and "lower bound does" go to
// kept[row][group] and sure[row][group] (64 blocks a word, assembled from the four lanes of a row), and the kept blocks' scores to
// scores[row][block].
__global__ void __launch_bounds__(64 * SCAN_WAVES) interval_scan_kernel(const uint4* __restrict__ key_ops, const float2* __restrict__ key_stats,
                                                                         const uint4* __restrict__ query_ops, const float4* __restrict__ info,
                                                                         unsigned tasks, unsigned steps, size_t pool,
                                                                         float* __restrict__ out, uint64_t* __restrict__ kept, uint64_t* __restrict__ sure,
                                                                         unsigned words) {
    extern __shared__ uint4 staged[];
    float4* row_info = reinterpret_cast<float4*>(staged + ROWS_OPS);
    const unsigned t = threadIdx.x, lane = t % 64, wave = t / 64, first_row = blockIdx.y * ROWS;
    const unsigned tiles = (min(steps - first_row, unsigned(ROWS)) + 15) / 16;
    // the wave's keys are asked for first: their trip overlaps the staging of the queries
    const unsigned group = blockIdx.x * SCAN_WAVES + wave;
    ScanTask task;
    load_task(task, key_ops, key_stats, min(group, tasks - 1), lane);
    {
        const uint4* source = query_ops + size_t(blockIdx.y) * ROWS_OPS;
        for (unsigned i = t; i < tiles * 16 * 64; i += 64 * SCAN_WAVES) staged[i] = source[i];
        if (t < ROWS) row_info[t] = info[first_row + t];
    }
    __syncthreads();
    if (group >= tasks) return;
    #pragma unroll 1
    for (unsigned j = 0; j < tiles; ++j) {
        floatx4 acc[4][HEADS];
        multiply(task, acc, [&](int piece) { return __builtin_bit_cast(half8, staged[(j * 16 + piece) * 64 + lane]); });
        const float4 mine = row_info[j * 16 + lane % 16];
        const unsigned row = first_row + j * 16 + lane % 16, complete = __float_as_uint(mine.w);
        // every row of the tile exists and every block of the group is before the complete count of its first row, the lowest
        const bool all_visible = first_row + j * 16 + 16 <= steps &&
                                 group * GROUP + GROUP <= __builtin_amdgcn_readfirstlane(__float_as_uint(row_info[j * 16].w));
        float* const at = out + size_t(row) * pool + group * GROUP + 4 * (lane / 16);
        uint32_t kept_low = 0, kept_high = 0, sure_low = 0, sure_high = 0;
        const auto bound = [&](auto checked) {
            #pragma unroll
            for (int m = 0; m < 4; ++m) {
                #pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float score = positive_sum(acc[m][0][r], acc[m][1][r], acc[m][2][r], acc[m][3][r]);
                    const float d = fmaf(task.kappa[m][r], mine.y, task.rho[m][r] * mine.z), over = score - mine.x;
                    // (a block whose bound is not a number -- a key beyond FP16 -- is kept: the selection sees it and leaves the row
                    // to the exact kernels, also when its operands came from an earlier call)
                    bool reaches = !(over < -d), surely = over >= d;
                    if (decltype(checked)::value) {
                        const bool visible = group * GROUP + m * 16 + 4 * (lane / 16) + r < complete;
                        reaches = reaches && visible; surely = surely && visible;
                    }
                    const uint32_t bit = 1u << ((m % 2) * 16 + r);
                    (m < 2 ? kept_low : kept_high) |= reaches ? bit : 0u;
                    (m < 2 ? sure_low : sure_high) |= surely ? bit : 0u;
                    if (reaches) at[m * 16 + r] = score;
                }
            }
        };
        if (all_visible) bound(std::false_type{}); else bound(std::true_type{});
        kept_low <<= 4 * (lane / 16); kept_high <<= 4 * (lane / 16); sure_low <<= 4 * (lane / 16); sure_high <<= 4 * (lane / 16);
        kept_low |= __shfl_xor(kept_low, 16); kept_low |= __shfl_xor(kept_low, 32);
        kept_high |= __shfl_xor(kept_high, 16); kept_high |= __shfl_xor(kept_high, 32);
        sure_low |= __shfl_xor(sure_low, 16); sure_low |= __shfl_xor(sure_low, 32);
        sure_high |= __shfl_xor(sure_high, 16); sure_high |= __shfl_xor(sure_high, 32);
        if (lane < 16 && row < steps) {
            kept[size_t(row) * words + group] = uint64_t(kept_low) | uint64_t(kept_high) << 32;
            sure[size_t(row) * words + group] = uint64_t(sure_low) | uint64_t(sure_high) << 32;
        }
    }
}

// ---- pieces of the per-row kernels (256 or 512 threads) --------------------------------------------------------------------------------
// The sum of `value` over the threads before this one; the workgroup's total in `total`.  `sums` is 8 words, free to rewrite
// after the next barrier of the caller (up to 16 waves).
__device__ __forceinline__ uint32_t before_me(uint32_t value, uint32_t* sums, uint32_t& total) {
    const unsigned lane = threadIdx.x % 64, wave = threadIdx.x / 64;
    uint32_t running = value;
    #pragma unroll
    for (int offset = 1; offset < 64; offset *= 2) {
        const uint32_t other = __shfl_up(running, offset);
        if (lane >= unsigned(offset)) running += other;
    }
    __syncthreads();
    if (lane == 63) sums[wave] = running;
    __syncthreads();
    uint32_t before = 0;
    total = 0;
    for (unsigned w = 0; w < blockDim.x / 64; ++w) { before += w < wave ? sums[w] : 0u; total += sums[w]; }
    return before + running - value;
}

// The k-th highest (1 <= k <= n) of n keys in LDS to their first 8 * PASSES bits (the other bits zero: a value the k-th highest
// reaches, and that fewer than k keys exceed by a whole step of those bits): passes of eight bits over a histogram of 256 counts.
template<int PASSES>
__device__ uint32_t kth_highest(const uint32_t* keys, unsigned n, unsigned k, uint32_t* counts, uint32_t* state, uint32_t* sums) {
    const unsigned t = threadIdx.x;
    uint32_t prefix = 0, mask = 0, want = k;
    for (unsigned pass = 0; pass < unsigned(PASSES); ++pass) {
        const unsigned shift = 24 - 8 * pass;
        counts[t] = 0;
        __syncthreads();
        for (unsigned i = t; i < n; i += 256) {
            const uint32_t x = keys[i];
            if ((x & mask) == prefix) atomicAdd(&counts[(x >> shift) & 255], 1u);
        }
        __syncthreads();
        const uint32_t mine = counts[255 - t];
        uint32_t total;
        const uint32_t above = before_me(mine, sums, total);
        if (above < want && above + mine >= want) { state[0] = prefix | ((255 - t) << shift); state[1] = want - above; }
        __syncthreads();
        prefix = state[0]; want = state[1];
        mask |= 255u << shift;
        __syncthreads();
    }
    return prefix;
}

// The first 22 bits (the rest zero) of the k-th highest of a[] and of b[] (n keys each, in LDS), found in step: two passes of
// eleven bits over two histograms of 2048 counts; a thread owns eight neighbouring counts of each, from the highest down.
template<int THREADS>
__device__ void kth_pair(const uint32_t* a, const uint32_t* b, unsigned n, unsigned k, uint32_t (*bins)[2048], uint32_t* state, uint32_t* sums,
                         uint32_t& found_a, uint32_t& found_b) {
    const unsigned t = threadIdx.x;
    uint32_t prefix_a = 0, prefix_b = 0, mask = 0, want_a = k, want_b = k;
    for (unsigned pass = 0; pass < 2; ++pass) {
        const unsigned shift = pass ? 10 : 21;
        constexpr unsigned MINE = 2048 / THREADS;      // neighbouring counts a thread owns
        #pragma unroll
        for (unsigned i = 0; i < MINE; ++i) { bins[0][t * MINE + i] = 0; bins[1][t * MINE + i] = 0; }
        __syncthreads();
        for (unsigned i = t; i < n; i += THREADS) {
            const uint32_t x = a[i], y = b[i];
            if ((x & mask) == prefix_a) atomicAdd(&bins[0][(x >> shift) & 2047], 1u);
            if ((y & mask) == prefix_b) atomicAdd(&bins[1][(y >> shift) & 2047], 1u);
        }
        __syncthreads();
        uint32_t mine_a[MINE], mine_b[MINE], sum = 0;
        #pragma unroll
        for (unsigned i = 0; i < MINE; ++i) {
            mine_a[i] = bins[0][2047 - (t * MINE + i)]; mine_b[i] = bins[1][2047 - (t * MINE + i)];
            sum += mine_a[i] | mine_b[i] << 16;         // (two counts of at most CAP each, scanned in one)
        }
        uint32_t total;
        const uint32_t above = before_me(sum, sums, total);
        uint32_t above_a = above & 0xffffu, above_b = above >> 16;
        #pragma unroll
        for (unsigned i = 0; i < MINE; ++i) {
            const uint32_t bin = 2047 - (t * MINE + i);
            if (above_a < want_a && above_a + mine_a[i] >= want_a) { state[0] = prefix_a | bin << shift; state[1] = want_a - above_a; }
            if (above_b < want_b && above_b + mine_b[i] >= want_b) { state[2] = prefix_b | bin << shift; state[3] = want_b - above_b; }
            above_a += mine_a[i]; above_b += mine_b[i];
        }
        __syncthreads();
        prefix_a = state[0]; want_a = state[1]; prefix_b = state[2]; want_b = state[3];
        mask |= 2047u << shift;
        __syncthreads();
    }
    found_a = prefix_a; found_b = prefix_b;
}

// ---- the threshold of a row: the sample's AIM-th highest lower bound ------------------------------------------------------------
__global__ void __launch_bounds__(256) interval_threshold_kernel(const float* __restrict__ sample, unsigned sampled, float4* __restrict__ info) {
    __shared__ uint32_t keys[SAMPLE_ROOM];
    __shared__ uint32_t counts[256], state[2], sums[8];
    const unsigned t = threadIdx.x, row = blockIdx.x;
    for (unsigned i = t; i < sampled; i += 256) keys[i] = ordered(sample[size_t(row) * SAMPLE_ROOM + i]);
    __syncthreads();
    const uint32_t found = kth_highest<2>(keys, sampled, AIM, counts, state, sums);       // (a guess: its first 16 bits do)
    if (t == 0) info[row].x = unordered(found);
}

// ---- the selection of a row ----------------------------------------------------------------------------------------------------
constexpr int SELECT = 512;         // threads of a row's selection
__global__ void __launch_bounds__(SELECT) interval_select_kernel(const float* __restrict__ queries, size_t stride, const float* __restrict__ blocks, size_t pool,
                                                              size_t base, size_t selected, const float* __restrict__ scores, const float* __restrict__ copy,
                                                              const float2* __restrict__ key_stats, const float4* __restrict__ info,
                                                              const uint64_t* __restrict__ kept, const uint64_t* __restrict__ sure, unsigned words,
                                                              uint32_t* __restrict__ flags, unsigned gate, float* __restrict__ indices,
                                                              float* __restrict__ counts_out) {
    __shared__ uint32_t block_of[CAP], low[CAP], high[CAP];
    __shared__ uint32_t exact[BAND];
    __shared__ uint16_t band_of[BAND];
    __shared__ float query[HEADS * COLUMNS];
    __shared__ uint32_t bins[2][2048], state[4], sums[16];
    const unsigned t = threadIdx.x, row = blockIdx.x;
    if (flags[row]) {           // (a query element beyond FP16 or not a number)
        if (t == 0) atomicAdd(&flags[gate], 1u);
        return;
    }
    const float4 mine = info[row];
    const unsigned complete = __float_as_uint(mine.w);
    const size_t position = base + row;
    for (unsigned i = t; i < HEADS * COLUMNS; i += SELECT) query[i] = queries[size_t(row) * stride + i];
    // the kept blocks in block order: a run of words per thread
    const unsigned used = (complete + GROUP - 1) / GROUP, per = (used + SELECT - 1) / SELECT;
    const unsigned first_word = min(t * per, used), last_word = min(first_word + per, used);
    uint32_t mine_kept = 0, mine_sure = 0;
    for (unsigned w = first_word; w < last_word; ++w) {
        mine_kept += __popcll(kept[size_t(row) * words + w]);
        mine_sure += __popcll(sure[size_t(row) * words + w]);
    }
    uint32_t n, surely;
    uint32_t at = before_me(mine_kept, sums, n);
    (void)before_me(mine_sure, sums, surely);
    if (surely < unsigned(KEEP) || n > unsigned(CAP)) {
        if (t == 0) { flags[row] = 1u; atomicAdd(&flags[gate], 1u); }
        return;
    }
    for (unsigned w = first_word; w < last_word; ++w) {
        uint64_t bits = kept[size_t(row) * words + w];
        while (bits) {
            block_of[at++] = w * GROUP + unsigned(__ffsll((unsigned long long)bits)) - 1;
            bits &= bits - 1;
        }
    }
    __syncthreads();
    bool odd = false;
    #pragma unroll 6
    for (unsigned i = t; i < n; i += SELECT) {
        const unsigned block = block_of[i];
        const float score = scores[size_t(row) * pool + block];
        const float2 norms = key_stats[block];
        const float d = fmaf(norms.x, mine.y, norms.y * mine.z);
        odd |= !(fabsf(score) + d < INFINITY);
        low[i] = ordered(score - d); high[i] = ordered(score + d);
    }
    if (__syncthreads_or(odd)) {
        if (t == 0) { flags[row] = 1u; atomicAdd(&flags[gate], 1u); }
        return;
    }
    // to 22 bits: the 512th highest lower bound rounded down, the 512th highest upper bound rounded up (either way the safe side)
    uint32_t low_kth, high_kth;
    kth_pair<SELECT>(low, high, n, KEEP, bins, state, sums, low_kth, high_kth);
    high_kth |= 0x3ffu;
    // a run of kept blocks per thread: certain ones counted, the band listed in block order
    const unsigned run = (n + SELECT - 1) / SELECT, c0 = min(t * run, n), c1 = min(c0 + run, n);
    uint32_t my_certain = 0, my_band = 0;
    for (unsigned c = c0; c < c1; ++c) {
        if (low[c] > high_kth) ++my_certain;
        else if (high[c] >= low_kth) ++my_band;
    }
    uint32_t certain, band;
    (void)before_me(my_certain, sums, certain);
    uint32_t band_at = before_me(my_band, sums, band);
    if (band > unsigned(BAND)) {
        if (t == 0) { flags[row] = 1u; atomicAdd(&flags[gate], 1u); }
        return;
    }
    for (unsigned c = c0; c < c1; ++c)
        if (low[c] <= high_kth && high[c] >= low_kth) band_of[band_at++] = uint16_t(c);
    __syncthreads();
    // the band's exact scores: four neighbouring lanes take a block's four heads, each its chain of 128 fused multiply-adds in
    // column order; the first of them adds the positive parts in head order
    for (unsigned i = t / 4; i < ((band + SELECT / 4 - 1) / (SELECT / 4)) * (SELECT / 4); i += SELECT / 4) {
        const unsigned head = t % 4;
        float dot = 0.0f;
        if (i < band) {
            // (all of the block's 512 bytes asked for at once: one trip to memory, then the chain)
            const float4* key = reinterpret_cast<const float4*>(copy + size_t(block_of[band_of[i]]) * COLUMNS);
            const float* q = query + head * COLUMNS;
            float4 four[COLUMNS / 4];
            #pragma unroll
            for (unsigned c = 0; c < COLUMNS / 4; ++c) four[c] = key[c];
            #pragma unroll
            for (unsigned c = 0; c < COLUMNS / 4; ++c) {
                dot = fmaf(four[c].x, q[4 * c], dot); dot = fmaf(four[c].y, q[4 * c + 1], dot);
                dot = fmaf(four[c].z, q[4 * c + 2], dot); dot = fmaf(four[c].w, q[4 * c + 3], dot);
            }
        }
        const unsigned lane = t % 64, first = lane & ~3u;
        const float four[HEADS] = {__shfl(dot, first), __shfl(dot, first + 1), __shfl(dot, first + 2), __shfl(dot, first + 3)};
        if (head == 0 && i < band) exact[i] = __float_as_uint(positive_sum(four));
    }
    __syncthreads();
    // the (512 - certain)th highest of the band's exact scores, by counting: the band is short
    const uint32_t need = unsigned(KEEP) - certain;
    for (unsigned i = t; i < band; i += SELECT) {
        const uint32_t x = exact[i];
        uint32_t higher = 0, same = 0;
        for (unsigned j = 0; j < band; ++j) { const uint32_t y = exact[j]; higher += y > x; same += y == x; }
        if (higher < need && need <= higher + same) state[0] = x;
    }
    __syncthreads();
    const uint32_t limit = state[0];
    uint32_t my_above = 0;
    for (unsigned i = t; i < band; i += SELECT) my_above += exact[i] > limit;
    uint32_t above;
    (void)before_me(my_above, sums, above);
    const uint32_t ties = need - above;         // blocks at the limit that are taken: the earliest
    uint32_t my_equal = 0;
    {
        unsigned i = band_at - my_band;
        for (unsigned c = c0; c < c1; ++c)
            if (low[c] <= high_kth && high[c] >= low_kth) my_equal += exact[i++] == limit;
    }
    uint32_t equal_total;
    uint32_t equal_before = before_me(my_equal, sums, equal_total);
    uint32_t my_taken = 0;
    {
        unsigned i = band_at - my_band, seen = equal_before;
        for (unsigned c = c0; c < c1; ++c) {
            if (low[c] > high_kth) ++my_taken;
            else if (high[c] >= low_kth) {
                const uint32_t score = exact[i++];
                if (score > limit || (score == limit && seen++ < ties)) ++my_taken;
            }
        }
    }
    uint32_t taken_total;
    uint32_t out_at = before_me(my_taken, sums, taken_total);
    float* out = indices + size_t(row) * selected;
    {
        unsigned i = band_at - my_band, seen = equal_before;
        for (unsigned c = c0; c < c1; ++c) {
            bool take = low[c] > high_kth;
            if (!take && high[c] >= low_kth) {
                const uint32_t score = exact[i++];
                take = score > limit || (score == limit && seen++ < ties);
            }
            if (take && out_at < unsigned(KEEP)) {
                const float4 four = make_float4(float(block_of[c] * 4), float(block_of[c] * 4 + 1), float(block_of[c] * 4 + 2), float(block_of[c] * 4 + 3));
                out[size_t(out_at) * 4] = four.x; out[size_t(out_at) * 4 + 1] = four.y; out[size_t(out_at) * 4 + 2] = four.z; out[size_t(out_at) * 4 + 3] = four.w;
                ++out_at;
            }
        }
    }
    const size_t head = size_t(KEEP) * 4;
    for (size_t i = t; size_t(complete) * 4 + i <= position; i += SELECT) out[head + i] = float(size_t(complete) * 4 + i);
    if (t == 0) counts_out[row] = float(head + position + 1 - size_t(complete) * 4);
}

struct IntervalSpace {
    uint4* key_ops; float2* key_stats; float* copy; uint4* sample_ops; float2* sample_stats; uint4* query_ops; float4* info; float* sample;
    uint64_t* kept; uint64_t* sure; uint32_t* flags;
    size_t bytes;
};

IntervalSpace lay_out(void* scratch, size_t steps, size_t pool) {
    const size_t groups = (pool + GROUP - 1) / GROUP, sample_groups = SAMPLE_ROOM / GROUP, rows = (steps + ROWS - 1) / ROWS * ROWS;
    uint8_t* at = static_cast<uint8_t*>(scratch);
    const auto take = [&](size_t bytes) { uint8_t* here = at; at += (bytes + 255) & ~size_t(255); return here; };
    IntervalSpace s{};
    s.key_ops = reinterpret_cast<uint4*>(take(groups * GROUP_OPS * sizeof(uint4)));
    s.key_stats = reinterpret_cast<float2*>(take(groups * GROUP * sizeof(float2)));
    s.copy = reinterpret_cast<float*>(take(groups * GROUP * COLUMNS * sizeof(float)));
    s.sample_ops = reinterpret_cast<uint4*>(take(sample_groups * GROUP_OPS * sizeof(uint4)));
    s.sample_stats = reinterpret_cast<float2*>(take(sample_groups * GROUP * sizeof(float2)));
    s.query_ops = reinterpret_cast<uint4*>(take(rows / ROWS * ROWS_OPS * sizeof(uint4)));
    s.info = reinterpret_cast<float4*>(take(rows * sizeof(float4)));
    s.sample = reinterpret_cast<float*>(take(rows * SAMPLE_ROOM * sizeof(float)));
    s.kept = reinterpret_cast<uint64_t*>(take(rows * groups * sizeof(uint64_t)));
    s.sure = reinterpret_cast<uint64_t*>(take(rows * groups * sizeof(uint64_t)));
    s.flags = reinterpret_cast<uint32_t*>(take((rows + 64) * sizeof(uint32_t)));
    s.bytes = size_t(at - static_cast<uint8_t*>(scratch));
    return s;
}

}  // namespace

namespace sd {

size_t interval_scratch_bytes(size_t steps, size_t pool) { return lay_out(nullptr, steps, pool).bytes; }

// Whether the interval scheme serves a span: the sample must be large enough for its 40th highest value to mean something.
bool interval_serves(size_t base) { return (base + 1) / 4 / STRIDE >= 256; }

// Queues the selection of rows base .. base + steps - 1 by intervals.  Afterwards (in stream order) flags[row] != 0 names the rows
// that the exact kernels must decide, flags[*gate] counts them; every other row has its indices and count.  `valid`: blocks whose operands the scratch
// still holds from the call before it on the same keys (0: none); left at this call's complete blocks.
const uint32_t* interval_select(Device& d, const float* queries, size_t stride, const float* blocks, size_t pool, size_t base, size_t steps,
                                size_t selected, float* scores, float* indices, float* counts, void* scratch, uint64_t* valid, unsigned* gate) {
    const IntervalSpace s = lay_out(scratch, steps, pool);
    const unsigned most = unsigned((base + steps) / 4), first_complete = unsigned((base + 1) / 4), sampled = first_complete / STRIDE;
    const unsigned tasks = (most + GROUP - 1) / GROUP, sample_tasks = (sampled + GROUP - 1) / GROUP;
    const unsigned rows = unsigned((steps + ROWS - 1) / ROWS * ROWS), row_groups = rows / ROWS, words = unsigned((pool + GROUP - 1) / GROUP);
    const size_t held = valid ? std::min<size_t>(size_t(*valid), most) : 0;
    const unsigned from = unsigned(held / GROUP);
    const unsigned packed = tasks > from ? tasks - from : 0;
    interval_pack_kernel<<<packed + rows / 4, 256, 0, d.stream>>>(blocks, pool, most, from, packed, s.key_ops, s.key_stats, s.sample_ops, s.sample_stats, s.copy,
                                                                  queries, stride, base, steps, rows, s.query_ops, s.info, s.flags);
    if (valid) *valid = most;
    const size_t shared = ROWS_OPS * sizeof(uint4) + ROWS * sizeof(float4);
    raise_shared_limit(d, reinterpret_cast<const void*>(&interval_scan_kernel), shared);
    interval_sample_kernel<<<dim3(sample_tasks, (rows / 16 + SCAN_WAVES - 1) / SCAN_WAVES), 64 * SCAN_WAVES, 0, d.stream>>>(
        s.sample_ops, s.sample_stats, s.query_ops, s.info, sampled, unsigned(steps), s.sample);
    interval_threshold_kernel<<<unsigned(steps), 256, 0, d.stream>>>(s.sample, sampled, s.info);
    timed_launch(d, &interval_scan_kernel, dim3((tasks + SCAN_WAVES - 1) / SCAN_WAVES, row_groups), dim3(64 * SCAN_WAVES), shared,
                 s.key_ops, s.key_stats, s.query_ops, s.info, tasks, unsigned(steps), pool, scores, s.kept, s.sure, words);
    interval_select_kernel<<<unsigned(steps), SELECT, 0, d.stream>>>(queries, stride, blocks, pool, base, selected, scores, s.copy, s.key_stats, s.info, s.kept,
                                                                  s.sure, words, s.flags, rows, indices, counts);
    SD_CHECK(hipGetLastError());
    *gate = rows;
    return s.flags;
}

// The rows the last interval_select on this scratch left to the exact kernels (waits for the stream).
size_t interval_undecided(Device& d, const void* scratch, size_t steps, size_t pool) {
    const IntervalSpace s = lay_out(const_cast<void*>(scratch), steps, pool);
    std::vector<uint32_t> flags(steps);
    download(d, flags.data(), s.flags, steps * sizeof(uint32_t));
    size_t undecided = 0;
    for (const uint32_t flag : flags) undecided += flag != 0;
    return undecided;
}

}  // namespace sd
