// Qwen's block indexer: the index inputs' normalisation and rotation, the pooled keys of four-position blocks, the exact block
// scores and the choice of the 512 best blocks per row.
//
// The arithmetic is the reference's (gpu/sparse_attention.hpp:2-23 qsa_rope/qsa_normalize, :87-139 qsa_pool/qsa_save_history,
// :141-155 qsa_block_scores, :172-241 qsa_select, :314-400 qsa_select_rows, :403-414 qsa_index_exact):
//   score(block) = sum over the 4 index heads, in order, of max(dot_h, 0), dot_h a chain of fused multiply-adds over the 128
//   columns in order (the bits do not depend on the tiling); a row with more than 512 complete blocks keeps the 512 whose raw
//   score bits are highest, ties to the earliest blocks, listed in block order with their four positions each, then the
//   positions of the incomplete block; a row with at most 512 complete blocks keeps every causal position.  Positions and the
//   count are stored as floats.
// The layout is the reference's too: pooled keys column-major blocks[column * pool + block], pool = context / 4 + 1, so a wave
// reading 64 neighbouring blocks of one column reads 256 contiguous bytes.
//
// Wave64 forms: one lane per block and all of a span's rows per lane while the span is short (decode, verification: the keys
// are read once from HBM, 512 bytes a block); a 32-row x 256-block tile per workgroup with operands staged through LDS for a
// prefill chunk (FP32 FMA-bound); a 1024-thread workgroup per row for the selection, the row's scores read once and held in LDS (and registers,
// beyond 32768 blocks), four 8-bit radix passes over per-wave LDS histograms (the first, where nearly all values share a digit, counted by ballots), and
// one ordered pass whose slots come from 64-wide ballots and a scan over (run, wave) counts.
#include "device.hpp"
#include "kv_codec.hpp"
#include "tree_sum.hpp"
#include "../../include/straydog_gpu_ext.h"

using namespace sd;

namespace {

constexpr int HEADS = 4, COLUMNS = 128, KEEP = 512, RING = 16;

__device__ __forceinline__ float turn(float own, float partner, unsigned column, size_t position) {
    if (column >= 64) return own;
    const float angle = float(position) / powf(1e7f, float(column % 32) / 32.0f);
    return own * cosf(angle) + (column < 32 ? -partner : partner) * sinf(angle);
}

// A vector of `width` values (128 or 256), one per thread c < width: x * norm / sqrt(mean(x^2) + 1e-6), the first 64 columns turned
// for `position`.  Every thread of the workgroup calls it (the sum has barriers); values and sums are 256 floats of LDS each.
__device__ __forceinline__ float normalized(float x, const float* norm, unsigned width, size_t position, float* values, float* sums) {
    const unsigned c = threadIdx.x;
    if (c < width) values[c] = x * norm[c];
    const float denominator = sqrtf(tree_sum(c < width ? x * x : 0.0f, sums, width) / float(width) + 1e-6f);
    const float own = c < width ? values[c] / denominator : 0.0f;
    const float partner = c < 64 ? values[(c + 32) % 64] / denominator : 0.0f;
    const float value = turn(own, partner, c, position);
    __syncthreads();        // (values may be written again at once)
    return value;
}

// One workgroup of `width` threads per (row, head).
__global__ void __launch_bounds__(256) normalize_kernel(const float* source, const float* norm, unsigned heads, unsigned width, size_t stride,
                                                        size_t position, float* target) {
    __shared__ float values[256], sums[256];
    const size_t head = blockIdx.x, token = head / heads;
    const unsigned c = threadIdx.x;
    target[head * width + c] = normalized(source[head * stride + c], norm, width, position + token, values, sums);
}

// The mean of a block's four index-key inputs as a thread's column: taps in position order, earlier ones from the ring.
__device__ __forceinline__ float pooled_mean(const float* incoming, size_t incoming_stride, const float* history, size_t begin, size_t base, unsigned c) {
    float x = 0.0f;
    #pragma unroll
    for (size_t tap = 0; tap < 4; ++tap) {
        const size_t pos = begin + tap;
        x += pos < base ? history[(pos % RING) * COLUMNS + c] : incoming[(pos - base) * incoming_stride + c];
    }
    return x / 4.0f;
}

// One workgroup of 128 threads per block completed by the span.
__global__ void __launch_bounds__(COLUMNS) pool_kernel(const float* incoming, size_t incoming_stride, const float* history, const float* norm, size_t pool,
                                                       size_t base, float* blocks) {
    __shared__ float values[256], sums[256];
    const size_t block = base / 4 + blockIdx.x, begin = block * 4;
    const unsigned c = threadIdx.x;
    blocks[c * pool + block] = normalized(pooled_mean(incoming, incoming_stride, history, begin, base, c), norm, COLUMNS, begin, values, sums);
}

__global__ void __launch_bounds__(256) save_history_kernel(const float* incoming, size_t incoming_stride, size_t base, size_t steps, float* history) {
    const size_t i = threadIdx.x + size_t(blockIdx.x) * 256, kept = steps < 4 ? steps : 4;
    if (i >= kept * COLUMNS) return;
    const size_t token = steps - kept + i / COLUMNS;
    history[((base + token) % RING) * COLUMNS + i % COLUMNS] = incoming[token * incoming_stride + i % COLUMNS];
}

__device__ __forceinline__ float positive_sum(const float (&dot)[HEADS]) {
    float total = fmaxf(dot[0], 0.0f) + fmaxf(dot[1], 0.0f);
    total += fmaxf(dot[2], 0.0f);
    total += fmaxf(dot[3], 0.0f);
    return total;
}

// ---- scores of a short span: a lane per block, a wave per head, T rows per lane ----------------------------------------------
// The chains of a block's four heads run in four waves of the workgroup (the same 64 blocks, the keys read by each: the second
// to fourth find them in the cache), so a compute unit holds four times the waves to hide the loads behind; the four sums meet
// in LDS and are added in head order.  The queries sit in LDS as [row][head][column]: a wave-uniform read a column.
template<int T>
__global__ void __launch_bounds__(64 * HEADS) scores_rows_kernel(const float* __restrict__ queries, size_t query_stride, const float* __restrict__ blocks,
                                                                size_t pool, size_t base, const uint32_t* dynamic, unsigned steps, float* __restrict__ scores) {
    __shared__ float q[T][HEADS][COLUMNS];
    __shared__ float sums[HEADS][T][64];
    if (dynamic) base = *dynamic;
    const size_t most = min((base + steps) / 4, pool), first = size_t(blockIdx.x) * 64;   // the last row's complete blocks
    const unsigned lane = threadIdx.x % 64, head = threadIdx.x / 64;
    if (most <= KEEP || first >= most) return;
    for (unsigned i = threadIdx.x; i < T * HEADS * COLUMNS; i += 64 * HEADS) {
        const unsigned row = i / (HEADS * COLUMNS);
        q[row][i / COLUMNS % HEADS][i % COLUMNS] = row < steps ? queries[row * query_stride + i % (HEADS * COLUMNS)] : 0.0f;
    }
    __syncthreads();
    const float* column = blocks + min(first + lane, pool - 1);
    float dot[T] = {};
    #pragma unroll 1
    for (unsigned c0 = 0; c0 < COLUMNS; c0 += 16) {
        float key[16];
        #pragma unroll
        for (unsigned j = 0; j < 16; ++j) key[j] = column[size_t(c0 + j) * pool];
        #pragma unroll
        for (unsigned j = 0; j < 16; ++j)
            #pragma unroll
            for (int row = 0; row < T; ++row) dot[row] = fmaf(key[j], q[row][head][c0 + j], dot[row]);
    }
    #pragma unroll
    for (int row = 0; row < T; ++row) sums[head][row][lane] = dot[row];
    __syncthreads();
    for (unsigned row = head; row < unsigned(T); row += HEADS) {
        const size_t complete = (base + row + 1) / 4;
        const float four[HEADS] = {sums[0][row][lane], sums[1][row][lane], sums[2][row][lane], sums[3][row][lane]};
        if (row < steps && complete > KEEP && first + lane < min(complete, pool)) scores[row * pool + first + lane] = positive_sum(four);
    }
}

// ---- scores of a prefill chunk: 32 rows x 256 blocks per workgroup ---------------------------------------------------------
// Eight waves; a lane owns 4 neighbouring blocks, a wave 4 rows, so a thread carries 4 x 4 x 4 chains.  Sixteen columns of
// keys [column][block] and queries [column][row * 4 + head] are staged at a time: the key read is 16 bytes a lane without
// bank conflicts, the query read is wave-uniform.  The next sixteen columns travel from global memory into registers while
// the current ones are multiplied.
constexpr int TILE_ROWS = 32, TILE_BLOCKS = 256, TILE_COLUMNS = 16, TILE_THREADS = 512, QUERY_PITCH = TILE_ROWS * HEADS + 4;
// One tile of 32 rows x 256 blocks (every thread of the workgroup calls it; `most`: the complete blocks of the tile's last row).
__device__ __forceinline__ void scores_tile(const float* __restrict__ queries, size_t query_stride, const float* __restrict__ blocks, size_t pool,
                                            size_t base, size_t steps, float* __restrict__ scores, size_t first_row, size_t first_block,
                                            float (&keys)[2][TILE_COLUMNS][TILE_BLOCKS], float (&query)[2][TILE_COLUMNS][QUERY_PITCH]) {
    const unsigned t = threadIdx.x, lane = t % 64, wave = t / 64;
    constexpr int KEY_LOADS = TILE_COLUMNS * TILE_BLOCKS / TILE_THREADS, QUERY_LOADS = TILE_COLUMNS * TILE_ROWS * HEADS / TILE_THREADS;
    float key_next[KEY_LOADS], query_next[QUERY_LOADS];
    const size_t key_block = min(first_block + t % TILE_BLOCKS, pool - 1);
    const auto fetch = [&](unsigned k) {
        #pragma unroll
        for (int j = 0; j < KEY_LOADS; ++j) key_next[j] = blocks[size_t(k + t / TILE_BLOCKS + j * (TILE_THREADS / TILE_BLOCKS)) * pool + key_block];
        #pragma unroll
        for (int j = 0; j < QUERY_LOADS; ++j) {
            const unsigned i = t + j * TILE_THREADS, c = i % TILE_COLUMNS, slot = i / TILE_COLUMNS;      // slot = row * 4 + head
            const size_t row = first_row + slot / HEADS;
            query_next[j] = row < steps ? queries[row * query_stride + (slot % HEADS) * COLUMNS + k + c] : 0.0f;
        }
    };
    const auto place = [&](int buffer) {
        #pragma unroll
        for (int j = 0; j < KEY_LOADS; ++j) keys[buffer][t / TILE_BLOCKS + j * (TILE_THREADS / TILE_BLOCKS)][t % TILE_BLOCKS] = key_next[j];
        #pragma unroll
        for (int j = 0; j < QUERY_LOADS; ++j) {
            const unsigned i = t + j * TILE_THREADS;
            query[buffer][i % TILE_COLUMNS][i / TILE_COLUMNS] = query_next[j];
        }
    };
    float sums[4][HEADS][4] = {};   // row, head, block
    fetch(0);
    place(0);
    __syncthreads();
    #pragma unroll 1
    for (unsigned k = 0; k < COLUMNS; k += TILE_COLUMNS) {
        const int buffer = (k / TILE_COLUMNS) & 1;
        if (k + TILE_COLUMNS < COLUMNS) fetch(k + TILE_COLUMNS);
        #pragma unroll 2
        for (unsigned c = 0; c < TILE_COLUMNS; ++c) {
            const float4 four = *reinterpret_cast<const float4*>(&keys[buffer][c][lane * 4]);
            const float key[4] = {four.x, four.y, four.z, four.w};
            #pragma unroll
            for (unsigned i = 0; i < 4; ++i) {
                const float4 heads = *reinterpret_cast<const float4*>(&query[buffer][c][(wave * 4 + i) * HEADS]);
                const float qh[HEADS] = {heads.x, heads.y, heads.z, heads.w};
                #pragma unroll
                for (unsigned h = 0; h < HEADS; ++h) {
                    #pragma unroll
                    for (unsigned b = 0; b < 4; ++b) sums[i][h][b] = fmaf(key[b], qh[h], sums[i][h][b]);
                }
            }
        }
        if (k + TILE_COLUMNS < COLUMNS) place(buffer ^ 1);      // the other buffer was last read before the barrier below, an iteration ago
        __syncthreads();
    }
    #pragma unroll
    for (unsigned i = 0; i < 4; ++i) {
        const size_t row = first_row + wave * 4 + i, complete = min((base + row + 1) / 4, pool);
        if (row >= steps || complete <= KEEP) continue;
        #pragma unroll
        for (unsigned b = 0; b < 4; ++b) {
            const size_t block = first_block + lane * 4 + b;
            const float dot[HEADS] = {sums[i][0][b], sums[i][1][b], sums[i][2][b], sums[i][3][b]};
            if (block < complete) scores[row * pool + block] = positive_sum(dot);
        }
    }
}

// ONLY = false: a workgroup per tile.  ONLY = true (behind the interval selection): the tiles of the rows it left undecided, which
// only[row] marks and only[gate] counts; a launch has fewer workgroups than tiles of blocks, each takes every gridDim.x-th, and
// every workgroup leaves at once when no row is marked.
template<bool ONLY>
__global__ void __launch_bounds__(TILE_THREADS) scores_tiled_kernel(const float* __restrict__ queries, size_t query_stride,
                                                                    const float* __restrict__ blocks, size_t pool, size_t base, size_t steps,
                                                                    float* __restrict__ scores, const uint32_t* __restrict__ only, unsigned gate) {
    __shared__ __align__(16) float keys[2][TILE_COLUMNS][TILE_BLOCKS];
    __shared__ __align__(16) float query[2][TILE_COLUMNS][QUERY_PITCH];
    const size_t first_row = size_t(blockIdx.y) * TILE_ROWS;
    const size_t most = min((base + min(steps, first_row + TILE_ROWS)) / 4, pool);        // complete blocks of the tile's last row
    if (most <= KEEP) return;
    if (ONLY) {
        if (!only[gate]) return;
        bool any = false;
        for (size_t r = first_row; r < min(steps, first_row + TILE_ROWS); ++r) any |= only[r] != 0;
        if (!any) return;
        for (size_t first_block = size_t(blockIdx.x) * TILE_BLOCKS; first_block < most; first_block += size_t(gridDim.x) * TILE_BLOCKS)
            scores_tile(queries, query_stride, blocks, pool, base, steps, scores, first_row, first_block, keys, query);
    } else {
        const size_t first_block = size_t(blockIdx.x) * TILE_BLOCKS;
        if (first_block < most) scores_tile(queries, query_stride, blocks, pool, base, steps, scores, first_row, first_block, keys, query);
    }
}

// ---- the selection ----------------------------------------------------------------------------------------------------------
constexpr int SELECT_THREADS = 1024, SELECT_WAVES = SELECT_THREADS / 64;

// Exclusive prefix of `value` over the workgroup in thread order, and the workgroup's sum.
__device__ __forceinline__ uint32_t group_scan(uint32_t value, uint32_t* wave_sums, uint32_t& total) {
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
    for (int w = 0; w < SELECT_WAVES; ++w) {
        const uint32_t c = wave_sums[w];
        before += unsigned(w) < wave ? c : 0u;
        sum += c;
    }
    total = sum;
    return before + inclusive - value;
}

// What the selection keeps between its steps, in LDS.
struct SelectShared {
    uint32_t bins[SELECT_WAVES * 256];      // a histogram per wave; at other times the (run, wave) counts or the sample's histogram
    uint32_t wave_sums[SELECT_WAVES], threshold, remaining;
};

// The choice itself over values a thread holds as (run i, thread t) in ascending block order: each_run(body) calls
// body(i, bits, valid) for the thread's value of every run, block_of(i) names its block.  Values below `guess` are known
// not to be among the 512 highest; should fewer than 512 be left, the guess is dropped.  Four 8-bit radix passes find the 512th
// highest value (a per-wave histogram; the first pass, where nearly all values share the digit, adds once per digit by a
// ballot), then one ordered pass gives every kept value its slot: ballots rank the lanes of a wave, a scan over the (run, wave)
// counts ranks the waves, and the values equal to the 512th are taken from the earliest blocks on.
template<class Each, class BlockOf>
__device__ __forceinline__ void choose_blocks(SelectShared& sh, Each each_run, BlockOf block_of, unsigned runs, unsigned most_runs, uint32_t guess,
                                              float* out) {
    const unsigned t = threadIdx.x, lane = t % 64, wave = t / 64;
    uint32_t prefix = 0, wanted = KEEP, mask = 0;
    uint32_t* own = sh.bins + wave * 256;
    #pragma unroll 1
    for (int shift = 24; shift >= 0; shift -= 8) {
        for (unsigned i = t; i < SELECT_WAVES * 256; i += SELECT_THREADS) sh.bins[i] = 0;
        __syncthreads();
        each_run([&](unsigned, uint32_t bits, bool valid) {
            const bool live = valid && bits >= guess && (bits & mask) == prefix;
            const uint32_t digit = (bits >> shift) & 255u;
            if (shift == 24) {
                uint64_t todo = __ballot(live);
                while (todo) {
                    const int leader = __ffsll(static_cast<long long>(todo)) - 1;
                    const uint32_t d = uint32_t(__builtin_amdgcn_readlane(int(digit), leader));
                    const uint64_t same = __ballot(live && digit == d);
                    if (int(lane) == leader) atomicAdd(own + d, uint32_t(__popcll(same)));
                    todo &= ~same;
                }
            } else if (live) {
                atomicAdd(own + digit, 1u);
            }
        });
        __syncthreads();
        // thread i < 256 holds bin 255 - i: the scan counts the values in higher bins
        const uint32_t bucket = 255u - (t & 255u);
        uint32_t count = 0, every;
        if (t < 256)
            for (int w = 0; w < SELECT_WAVES; ++w) count += sh.bins[w * 256 + bucket];
        const uint32_t above = group_scan(count, sh.wave_sums, every);
        if (shift == 24 && every < KEEP) {                   // the guess was too high: once more, over every value
            guess = 0;
            shift += 8;
            continue;
        }
        if (t < 256 && above < wanted && above + count >= wanted) { sh.threshold = prefix | (bucket << shift); sh.remaining = wanted - above; }
        __syncthreads();
        prefix = sh.threshold; wanted = sh.remaining;
        mask |= 255u << shift;
    }
    // Kept: every value above `prefix` and the first `wanted` equal to it, in block order.
    uint32_t* greater = sh.bins;
    uint32_t* equal = sh.bins + most_runs * SELECT_WAVES;
    each_run([&](unsigned i, uint32_t bits, bool valid) {
        const uint64_t above = __ballot(valid && bits > prefix), same = __ballot(valid && bits == prefix);
        if (lane == 0) { greater[i * SELECT_WAVES + wave] = uint32_t(__popcll(above)); equal[i * SELECT_WAVES + wave] = uint32_t(__popcll(same)); }
    });
    __syncthreads();
    const unsigned entries = runs * SELECT_WAVES;           // at most 1024: one per thread
    const uint32_t g = t < entries ? greater[t] : 0u, e = t < entries ? equal[t] : 0u;
    uint32_t every;
    const uint32_t greater_before = group_scan(g, sh.wave_sums, every);
    const uint32_t equal_before = group_scan(e, sh.wave_sums, every);
    if (t < entries) { greater[t] = greater_before; equal[t] = equal_before; }
    __syncthreads();
    const uint64_t below = (uint64_t(1) << lane) - 1;
    each_run([&](unsigned i, uint32_t bits, bool valid) {
        const bool above = valid && bits > prefix, same = valid && bits == prefix;
        const uint64_t above_mask = __ballot(above), same_mask = __ballot(same);
        if (!above && !same) return;
        const uint32_t equal_seen = equal[i * SELECT_WAVES + wave] + uint32_t(__popcll(same_mask & below));
        if (same && equal_seen >= wanted) return;
        const size_t at = size_t(greater[i * SELECT_WAVES + wave] + uint32_t(__popcll(above_mask & below)) + min(equal_seen, wanted)) * 4;
        const size_t block = block_of(i);
        #pragma unroll
        for (size_t tap = 0; tap < 4; ++tap) out[at + tap] = float(block * 4 + tap);
    });
}

// A short span's rows (a decode step, a verification span) would leave all but a few compute units idle while one workgroup a
// row sweeps 60K values.  For those the thinning is spread out: THIN_SEGMENTS workgroups a row each find the same guess from the
// same sample of the row (the R-th highest of 4096 values spread evenly over it, to 24 bits) and list, in block order, the values
// of their own stretch of the row that reach it; the row's workgroup then only gathers the lists.  A stretch whose list does
// not fit says so and the row's workgroup does all the work itself, as it does for rows too short to be worth it.
constexpr int THIN_SEGMENTS = 32, THIN_THREADS = 256, THIN_CAP = 256, THIN_ROWS = 8, THIN_SAMPLE = 4096;
constexpr uint32_t THIN_NONE = 0xffffffffu;
__global__ void __launch_bounds__(THIN_THREADS) thin_kernel(const float* __restrict__ scores, size_t pool, size_t base, const uint32_t* dynamic,
                                                            uint2* __restrict__ listed, uint32_t* __restrict__ listed_counts) {
    __shared__ uint32_t bins[THIN_SAMPLE];
    __shared__ uint32_t wave_sums[THIN_THREADS / 64], found[2];
    if (dynamic) base = *dynamic;
    const size_t token = blockIdx.y, position = base + token, complete = (position + 1) / 4;
    const unsigned t = threadIdx.x, lane = t % 64, wave = t / 64, segment = blockIdx.x;
    uint32_t* const count_out = listed_counts + token * THIN_SEGMENTS + segment;
    if (position + 1 > 4 * pool || complete < size_t(8) * SELECT_THREADS) {          // (the row's workgroup decides the same way)
        if (t == 0) *count_out = THIN_NONE;
        return;
    }
    const uint32_t* row = reinterpret_cast<const uint32_t*>(scores + token * pool);   // scores are sums of max(., 0): their bits order as they do
    constexpr unsigned MINE = THIN_SAMPLE / THIN_THREADS;
    uint32_t sample[MINE];
    #pragma unroll
    for (unsigned k = 0; k < MINE; ++k) sample[k] = row[size_t(t + THIN_THREADS * k) * complete / THIN_SAMPLE];
    uint32_t guess = 0, rank = uint32_t(3 * size_t(KEEP) * THIN_SAMPLE / (2 * complete)) + 16;
    #pragma unroll 1
    for (int shift = 20; shift >= 8; shift -= 12) {          // the sample's rank-th highest value to 24 bits: 12 bits a level
        for (unsigned i = t; i < unsigned(THIN_SAMPLE); i += THIN_THREADS) bins[i] = 0;
        __syncthreads();
        #pragma unroll
        for (unsigned k = 0; k < MINE; ++k)
            if (shift == 20 || (sample[k] >> 20) == (guess >> 20)) atomicAdd(bins + ((sample[k] >> shift) & 4095u), 1u);
        __syncthreads();
        // thread t holds the 16 bins below 4096 - 16 t, highest first: a scan in thread order counts the values in higher bins
        uint32_t mine[MINE], sum = 0;
        #pragma unroll
        for (unsigned j = 0; j < MINE; ++j) { mine[j] = bins[4095 - MINE * t - j]; sum += mine[j]; }
        uint32_t inclusive = sum;
        #pragma unroll
        for (unsigned offset = 1; offset < 64; offset *= 2) { const uint32_t other = __shfl_up(inclusive, offset); if (lane >= offset) inclusive += other; }
        if (lane == 63) wave_sums[wave] = inclusive;
        __syncthreads();
        uint32_t above = inclusive - sum;
        for (unsigned w = 0; w < wave; ++w) above += wave_sums[w];
        #pragma unroll
        for (unsigned j = 0; j < MINE; ++j) {
            if (above < rank && above + mine[j] >= rank) { found[0] = guess | ((4095 - MINE * t - j) << shift); found[1] = rank - above; }
            above += mine[j];
        }
        __syncthreads();
        guess = found[0]; rank = found[1];
    }
    // the stretch's values that reach the guess, in block order
    const size_t stretch = (complete + THIN_SEGMENTS - 1) / THIN_SEGMENTS, first = segment * stretch, last = min(first + stretch, complete);
    uint2* const out = listed + (token * THIN_SEGMENTS + segment) * THIN_CAP;
    uint32_t written = 0;
    const uint64_t below = (uint64_t(1) << lane) - 1;
    for (size_t at = first; at < last; at += THIN_THREADS) {
        const size_t block = at + t;
        const uint32_t bits = block < last ? row[block] : 0u;
        const bool reaches = block < last && bits >= guess;
        const uint64_t reaching = __ballot(reaches);
        __syncthreads();                                     // the counts of the round before are read
        if (lane == 0) wave_sums[wave] = uint32_t(__popcll(reaching));
        __syncthreads();
        uint32_t before = written, round = 0;
        #pragma unroll
        for (unsigned w = 0; w < THIN_THREADS / 64; ++w) { before += w < wave ? wave_sums[w] : 0u; round += wave_sums[w]; }
        const uint32_t slot = before + uint32_t(__popcll(reaching & below));
        if (reaches && slot < uint32_t(THIN_CAP)) out[slot] = make_uint2(bits, uint32_t(block));
        written += round;
    }
    if (t == 0) *count_out = written <= uint32_t(THIN_CAP) ? written : THIN_NONE;
}

// One workgroup per row; block i * 1024 + t is thread t's value i.  The row is read once and stays on the chip: its first
// LDS_RUNS runs of 1024 values in LDS (as many as the row has: the launch sizes the array), the runs beyond, for the longest
// rows, in REGS registers a thread.
//
// A long row is thinned first, since every sweep over 64 values a thread costs about as much as all the rest: the R-th
// highest of a sample of four values a thread (spread over the runs in LDS; R: one and a half times the sample's share of 512, and
// a margin), found to 24 bits by two 4096-bin histograms, is a guess below the 512th highest value of the row.  Two light sweeps count and list, in block order, the values that reach the guess; when they are
// at least 512 and fit the list, the choice runs over the list alone, otherwise over the whole row.
constexpr int LDS_RUNS = 31, LIST_RUNS = 2, LIST = LIST_RUNS * SELECT_THREADS;
template<int REGS>
__global__ void __launch_bounds__(SELECT_THREADS) select_kernel(const float* __restrict__ scores, size_t pool, size_t base, const uint32_t* dynamic,
                                                                size_t selected, unsigned held_runs, float* __restrict__ indices,
                                                                float* __restrict__ counts, const uint2* __restrict__ thinned,
                                                                const uint32_t* __restrict__ thinned_counts, const uint32_t* __restrict__ only) {
    extern __shared__ uint32_t held[];                       // [run][1024]
    if (only && !only[blockIdx.x]) return;
    __shared__ SelectShared sh;
    __shared__ uint2 list[LIST];                             // (score bits, block) of the values that reach the guess
    if (dynamic) base = *dynamic;
    const size_t token = blockIdx.x, position = base + token, complete = (position + 1) / 4;
    const unsigned t = threadIdx.x, lane = t % 64, wave = t / 64;
    float* out = indices + token * selected;
    if (position + 1 > 4 * pool || complete > size_t(held_runs + REGS) * SELECT_THREADS) {   // a position this key pool (or this launch) cannot hold
        if (t == 0) counts[token] = 0.0f;
        return;
    }
    if (complete <= KEEP) {
        for (size_t i = t; i <= position; i += SELECT_THREADS) out[i] = float(i);
        if (t == 0) counts[token] = float(position + 1);
        return;
    }
    const float* row = scores + token * pool;
    const unsigned runs = unsigned((complete + SELECT_THREADS - 1) / SELECT_THREADS), lds_runs = min(runs, held_runs);
    uint32_t values[REGS ? REGS : 1];
    uint32_t guess = 0;
    bool listed = false;
    uint32_t list_count = 0;
    // The row thinned by thin_kernel: its stretches' lists, one after the other, are the row's list -- when every stretch's
    // fitted and they hold at least 512 values and no more than the list does; the row itself is then not read at all.
    if (thinned && runs >= 8) {
        const uint32_t mine = t < unsigned(THIN_SEGMENTS) ? thinned_counts[token * THIN_SEGMENTS + t] : 0u;
        const bool none = __syncthreads_or(mine == THIN_NONE);
        const uint32_t before = group_scan(none ? 0u : mine, sh.wave_sums, list_count);
        listed = !none && list_count >= KEEP && list_count <= LIST;
        if (listed) {
            if (t < unsigned(THIN_SEGMENTS)) { sh.bins[2 * t] = before; sh.bins[2 * t + 1] = mine; }
            __syncthreads();
            for (unsigned slot = t; slot < unsigned(THIN_SEGMENTS * THIN_CAP); slot += SELECT_THREADS) {
                const unsigned segment = slot / THIN_CAP, entry = slot % THIN_CAP;
                if (entry < sh.bins[2 * segment + 1]) list[sh.bins[2 * segment] + entry] = thinned[(token * THIN_SEGMENTS + segment) * THIN_CAP + entry];
            }
            __syncthreads();
        }
    }
    if (!listed) {
    #pragma unroll 8
    for (unsigned i = 0; i < lds_runs; ++i) {
        const size_t block = size_t(i) * SELECT_THREADS + t;
        held[i * SELECT_THREADS + t] = block < complete ? __float_as_uint(row[block]) : 0u;
    }
    if constexpr (REGS > 0) {
        #pragma unroll
        for (int j = 0; j < REGS; ++j) {
            const size_t block = size_t(LDS_RUNS + j) * SELECT_THREADS + t;
            values[j] = block < complete ? __float_as_uint(row[block]) : 0u;
        }
    }
    }
    // body(run, bits, valid) for every run of the row, in run order (every thread reads back only what it wrote)
    const auto each_run = [&](auto body) {
        unsigned i = 0;
        for (; i + 4 <= lds_runs; i += 4) {                  // four reads in flight at a time
            uint32_t four[4];
            #pragma unroll
            for (unsigned j = 0; j < 4; ++j) four[j] = held[(i + j) * SELECT_THREADS + t];
            #pragma unroll
            for (unsigned j = 0; j < 4; ++j) body(i + j, four[j], size_t(i + j) * SELECT_THREADS + t < complete);
        }
        for (; i < lds_runs; ++i) body(i, held[i * SELECT_THREADS + t], size_t(i) * SELECT_THREADS + t < complete);
        if constexpr (REGS > 0) {
            #pragma unroll
            for (int j = 0; j < REGS; ++j)
                if (unsigned(LDS_RUNS + j) < runs) body(unsigned(LDS_RUNS + j), values[j], size_t(LDS_RUNS + j) * SELECT_THREADS + t < complete);
        }
    };
    if (!listed && runs >= 8) {
        constexpr unsigned SAMPLES = 4;                      // values a thread gives to the sample
        uint32_t sample[SAMPLES];
        bool sampled[SAMPLES];
        #pragma unroll
        for (unsigned k = 0; k < SAMPLES; ++k) {
            const unsigned run = (t + 7 * k) % lds_runs;
            sampled[k] = size_t(run) * SELECT_THREADS + t < complete;
            sample[k] = held[run * SELECT_THREADS + t];
        }
        uint32_t rank = uint32_t(3 * size_t(KEEP) * SAMPLES * SELECT_THREADS / (2 * complete)) + 16;
        #pragma unroll 1
        for (int shift = 20; shift >= 8; shift -= 12) {     // the sample's rank-th highest value to 24 bits: 12 bits a level
            for (unsigned i = t; i < SELECT_WAVES * 256; i += SELECT_THREADS) sh.bins[i] = 0;
            if (t == 0) { sh.threshold = guess; sh.remaining = rank; }
            __syncthreads();
            #pragma unroll
            for (unsigned k = 0; k < SAMPLES; ++k)
                if (sampled[k] && (shift == 20 || (sample[k] >> 20) == (guess >> 20))) atomicAdd(sh.bins + ((sample[k] >> shift) & 4095u), 1u);
            __syncthreads();
            uint32_t four[4], sum = 0, every;
            #pragma unroll
            for (unsigned j = 0; j < 4; ++j) { four[j] = sh.bins[4095 - 4 * t - j]; sum += four[j]; }
            uint32_t above = group_scan(sum, sh.wave_sums, every);
            #pragma unroll
            for (unsigned j = 0; j < 4; ++j) {
                if (above < rank && above + four[j] >= rank) { sh.threshold = guess | ((4095 - 4 * t - j) << shift); sh.remaining = rank - above; }
                above += four[j];
            }
            __syncthreads();
            guess = sh.threshold; rank = sh.remaining;
            __syncthreads();
        }
        // how many values reach the guess, per (run, wave) in block order
        uint32_t* reach = sh.bins;
        each_run([&](unsigned i, uint32_t bits, bool valid) {
            const uint64_t reaching = __ballot(valid && bits >= guess);
            if (lane == 0) reach[i * SELECT_WAVES + wave] = uint32_t(__popcll(reaching));
        });
        __syncthreads();
        const unsigned entries = runs * SELECT_WAVES;
        const uint32_t mine = t < entries ? reach[t] : 0u;
        const uint32_t before = group_scan(mine, sh.wave_sums, list_count);
        if (t < entries) reach[t] = before;
        __syncthreads();
        if (list_count < KEEP) guess = 0;                    // too high a guess: the whole row, every value
        listed = list_count >= KEEP && list_count <= LIST;
        if (listed) {
            const uint64_t below = (uint64_t(1) << lane) - 1;
            each_run([&](unsigned i, uint32_t bits, bool valid) {
                const bool reaches = valid && bits >= guess;
                const uint64_t reaching = __ballot(reaches);
                if (reaches) list[reach[i * SELECT_WAVES + wave] + uint32_t(__popcll(reaching & below))] = make_uint2(bits, i * SELECT_THREADS + t);
            });
        }
        __syncthreads();
    }
    if (listed) {
        uint2 mine[LIST_RUNS];
        #pragma unroll
        for (int j = 0; j < LIST_RUNS; ++j) mine[j] = unsigned(j) * SELECT_THREADS + t < list_count ? list[j * SELECT_THREADS + t] : make_uint2(0u, 0u);
        const unsigned list_runs = (list_count + SELECT_THREADS - 1) / SELECT_THREADS;
        choose_blocks(sh, [&](auto body) {
            #pragma unroll
            for (int j = 0; j < LIST_RUNS; ++j)
                if (unsigned(j) < list_runs) body(unsigned(j), mine[j].x, unsigned(j) * SELECT_THREADS + t < list_count);
        }, [&](unsigned j) { return size_t(j == 0 ? mine[0].y : mine[1].y); }, list_runs, LIST_RUNS, 0u, out);
    } else {
        choose_blocks(sh, each_run, [&](unsigned i) { return size_t(i) * SELECT_THREADS + t; }, runs, LDS_RUNS + REGS, guess, out);
    }
    const size_t head = size_t(KEEP) * 4;
    for (size_t i = t; complete * 4 + i <= position; i += SELECT_THREADS) out[head + i] = float(complete * 4 + i);
    if (t == 0) counts[token] = float(head + position + 1 - complete * 4);
}

template<int REGS>
void launch_select(Device& d, const float* scores, size_t pool, size_t base, const uint32_t* dynamic, size_t selected, size_t most, unsigned rows,
                   float* indices, float* counts, const uint2* thinned, const uint32_t* thinned_counts, const uint32_t* only = nullptr) {
    const unsigned held_runs = unsigned(std::min<size_t>((most + SELECT_THREADS - 1) / SELECT_THREADS, LDS_RUNS));
    const size_t shared = size_t(std::max(held_runs, 1u)) * SELECT_THREADS * 4;
    if (shared > 48 * 1024) raise_shared_limit(d, reinterpret_cast<const void*>(&select_kernel<REGS>), LDS_RUNS * SELECT_THREADS * 4);
    select_kernel<REGS><<<rows, SELECT_THREADS, shared, d.stream>>>(scores, pool, base, dynamic, selected, held_runs, indices, counts, thinned, thinned_counts, only);
}

// ---- a decode or verification pass's inputs in one launch --------------------------------------------------------------
// The reference's qsa_normalize_rows (gpu/qsa_decode.hpp:86-111): blockIdx.y = row; blockIdx.x = a query head (normalised and turned
// into `queries`), then a K/V head (the key normalised and turned, key and value rows encoded into the cache at the row's
// position), then the four index-query heads (in place), then one workgroup that pools the index keys of all rows in turn
// (a row completes a block from the ring the rows before it wrote).  Positions and rope positions are read on the device.
struct StageArgs {
    float* projections;            // row r at r * stride: heads x [query 256 | gate 256], kv x key 256, kv x value 256, 4 x index query 128, index key 128
    size_t stride;
    const float *q_norm, *k_norm, *index_q_norm, *index_k_norm;
    unsigned heads, kv_heads, steps;
    const uint32_t *positions, *ropes;   // device-resident positions of the rows, or null: row r is at base + r
    size_t base;
    uint8_t* pages;
    unsigned page_tokens, row_bytes;
    const int32_t* page_table;
    size_t page_count;
    size_t context;
    float* queries;                // [steps][heads][256]
    float *blocks, *history;
    size_t pool;
};
__global__ void __launch_bounds__(256) stage_prepare_kernel(StageArgs a) {
    __shared__ float values[256], sums[256];
    __shared__ __align__(16) float key[256];
    const unsigned block = blockIdx.x, c = threadIdx.x;
    const size_t row = blockIdx.y, pos = a.positions ? a.positions[row] : a.base + row, rope = a.ropes ? a.ropes[row] : a.base + row;
    float* own = a.projections + row * a.stride;
    const size_t keys_at = size_t(a.heads) * 512, values_at = keys_at + size_t(a.kv_heads) * 256, index_at = keys_at + size_t(a.kv_heads) * 512;
    if (block < a.heads) {
        a.queries[(row * a.heads + block) * 256 + c] = normalized(own[size_t(block) * 512 + c], a.q_norm, 256, rope, values, sums);
    } else if (block < a.heads + a.kv_heads) {
        const unsigned head = block - a.heads;
        key[c] = normalized(own[keys_at + head * 256 + c], a.k_norm, 256, rope, values, sums);
        __syncthreads();
        if (pos >= a.context || c >= 128) return;           // a position outside the cache writes no row; two waves encode
        const long long entry = a.page_table ? a.page_table[pos / a.page_tokens] : 0;
        if (entry < 0 || size_t(entry) >= a.page_count) return;   // nor does a table entry that names no page of the pool
        const size_t page = size_t(entry), in_page = a.page_table ? pos % a.page_tokens : pos;
        const bool is_value = c >= 64;
        const unsigned quad = c % 64;                       // four columns a thread: a wave holds the row, 8 lanes a 32-column block
        uint8_t* target = a.pages + ((page * 2 * a.kv_heads + (is_value ? a.kv_heads : 0) + head) * a.page_tokens + in_page) * a.row_bytes;
        const float* from = is_value ? own + values_at + head * 256 + 4 * quad : key + 4 * quad;
        const float x[4] = {from[0], from[1], from[2], from[3]};
        kv_store_quad(target, quad, 256, a.row_bytes != 512, x, true);
    } else if (block < a.heads + a.kv_heads + HEADS) {
        const unsigned head = block - a.heads - a.kv_heads;
        float* vector = own + index_at + head * COLUMNS;
        const float value = normalized(c < COLUMNS ? vector[c] : 0.0f, a.index_q_norm, COLUMNS, rope, values, sums);
        if (c < COLUMNS) vector[c] = value;
    } else if (row == 0) {
        for (size_t r = 0; r < a.steps; ++r) {
            const size_t at = a.positions[r];
            if (c < COLUMNS) a.history[(at % RING) * COLUMNS + c] = a.projections[r * a.stride + index_at + HEADS * COLUMNS + c];
            if ((at + 1) % 4 == 0 && at / 4 < a.pool) {
                float x = 0.0f;
                if (c < COLUMNS) {
                    #pragma unroll
                    for (size_t tap = 0; tap < 4; ++tap) x += a.history[((at - 3 + tap) % RING) * COLUMNS + c];
                    x /= 4.0f;
                }
                const float value = normalized(x, a.index_k_norm, COLUMNS, size_t(a.ropes[r]) - 3, values, sums);
                if (c < COLUMNS) a.blocks[c * a.pool + at / 4] = value;
            }
        }
    }
}

template<int T>
void launch_rows(Device& d, const float* queries, size_t stride, const float* blocks, size_t pool, size_t base, const uint32_t* dynamic, size_t steps,
                 size_t most, float* scores) {
    timed_launch(d, &scores_rows_kernel<T>, dim3(checked_blocks(most, 64)), dim3(64 * HEADS), 0, queries, stride, blocks, pool, base, dynamic, unsigned(steps), scores);
}

}  // namespace

namespace sd {
void validate_pool(Device& d, const sdx_kv_pool* pool);     // kv_write.hip
// block_interval.hip
size_t interval_scratch_bytes(size_t steps, size_t pool);
bool interval_serves(size_t base);
const uint32_t* interval_select(Device& d, const float* queries, size_t stride, const float* blocks, size_t pool, size_t base, size_t steps,
                                size_t selected, float* scores, float* indices, float* counts, void* scratch, uint64_t* valid, unsigned* gate);
size_t interval_undecided(Device& d, const void* scratch, size_t steps, size_t pool);
// The lists of a short span's thinned rows: allocated once per handle, never while a graph is being recorded (sd_graph_begin
// calls this first, so that a recorded pass takes the same path as an eager one).
constexpr size_t thin_list_bytes = size_t(THIN_ROWS) * THIN_SEGMENTS * THIN_CAP * sizeof(uint2);
void select_thin_reserve(Device& d) {
    if (d.select_thin) return;
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    SD_CHECK(hipStreamIsCapturing(d.stream, &capturing));
    if (capturing == hipStreamCaptureStatusNone) d.select_thin = allocate(d, thin_list_bytes + size_t(THIN_ROWS) * THIN_SEGMENTS * 4, true);
}
}  // namespace sd

extern "C" {

int sdx_qsa_normalize(void* handle, const float* source, const float* norm, uint64_t rows, uint64_t heads, uint64_t width, uint64_t stride,
                      uint64_t position, float* target) {
    SD_OP_BEGIN
    if (!rows || !heads || (width != 128 && width != 256) || stride < width) throw std::runtime_error("sdx_qsa_normalize: rows and heads >= 1, width 128 or 256, stride >= width");
    const size_t vectors = checked_product({rows, heads});
    op_span(value, source, checked_floats({uint64_t(vectors - 1), stride}) + width * 4, "sdx_qsa_normalize source");
    op_span(value, norm, width * 4, "sdx_qsa_normalize norm");
    op_span(value, target, checked_floats({uint64_t(vectors), width}), "sdx_qsa_normalize target");
    if (position + rows > (uint64_t(1) << 24)) throw std::runtime_error("sdx_qsa_normalize: positions beyond 2^24");
    normalize_kernel<<<checked_blocks(vectors, 1), unsigned(width), 0, value.stream>>>(source, norm, unsigned(heads), unsigned(width), stride, position, target);
    SD_OP_END
}

int sdx_qsa_pool(void* handle, const float* incoming, float* history, const float* norm, uint64_t pool, uint64_t base, uint64_t steps, float* blocks) {
    SD_OP_BEGIN
    if (!steps || !pool || (base + steps) / 4 > pool || base + steps > (uint64_t(1) << 24)) throw std::runtime_error("sdx_qsa_pool: steps >= 1 and (base + steps) / 4 blocks must fit the pool");
    op_span(value, incoming, checked_floats({steps, uint64_t(COLUMNS)}), "sdx_qsa_pool incoming");
    op_span(value, history, size_t(RING) * COLUMNS * 4, "sdx_qsa_pool history");
    op_span(value, norm, COLUMNS * 4, "sdx_qsa_pool norm");
    op_span(value, blocks, checked_floats({pool, uint64_t(COLUMNS)}), "sdx_qsa_pool blocks");
    const size_t completed = (base + steps) / 4 - base / 4;
    if (completed) pool_kernel<<<checked_blocks(completed, 1), COLUMNS, 0, value.stream>>>(incoming, COLUMNS, history, norm, pool, base, blocks);
    save_history_kernel<<<checked_blocks(std::min<size_t>(steps, 4) * COLUMNS), 256, 0, value.stream>>>(incoming, COLUMNS, base, steps, history);
    SD_OP_END
}

int sdx_qsa_index(void* handle, const float* queries, uint64_t query_stride, const float* blocks, uint64_t pool, uint64_t base,
                  const uint32_t* dynamic_base, uint64_t steps, uint64_t selected, float* scores, float* indices, float* counts) {
    SD_OP_BEGIN
    constexpr size_t widest = size_t(64) * SELECT_THREADS;      // complete blocks a row's selection can hold in registers
    if (!steps || !pool || query_stride < HEADS * COLUMNS) throw std::runtime_error("sdx_qsa_index: steps and pool >= 1, query stride >= 512");
    if (pool > widest + 1) throw std::runtime_error("sdx_qsa_index: a pool of more than 65537 blocks (a context beyond 262144)");
    if (!dynamic_base && ((base + steps) / 4 > pool || base + steps > 4 * pool)) throw std::runtime_error("sdx_qsa_index: the span's blocks must fit the pool");
    const size_t needed = dynamic_base ? std::min<size_t>(4 * pool, 2052) : std::min<size_t>(base + steps, 2052);
    if (selected < needed) throw std::runtime_error("sdx_qsa_index: `selected` is smaller than a row's selection can be");
    op_span(value, queries, checked_floats({steps - 1, query_stride}) + HEADS * COLUMNS * 4, "sdx_qsa_index queries");
    op_span(value, blocks, checked_floats({pool, uint64_t(COLUMNS)}), "sdx_qsa_index blocks");
    op_span(value, scores, checked_floats({steps, pool}), "sdx_qsa_index scores");
    op_span(value, indices, checked_floats({steps, selected}), "sdx_qsa_index indices");
    op_span(value, counts, checked_floats({steps}), "sdx_qsa_index counts");
    if (dynamic_base) op_span(value, dynamic_base, 4, "sdx_qsa_index position");
    const size_t most = dynamic_base ? size_t(pool) : size_t((base + steps) / 4);       // complete blocks of the last row, at most
    {
        if (most > KEEP) {
            if (steps <= 1) launch_rows<1>(value, queries, query_stride, blocks, pool, base, dynamic_base, steps, most, scores);
            else if (steps <= 2) launch_rows<2>(value, queries, query_stride, blocks, pool, base, dynamic_base, steps, most, scores);
            else if (steps <= 4) launch_rows<4>(value, queries, query_stride, blocks, pool, base, dynamic_base, steps, most, scores);
            else if (steps <= 8) launch_rows<8>(value, queries, query_stride, blocks, pool, base, dynamic_base, steps, most, scores);
            else {
                if (dynamic_base) throw std::runtime_error("sdx_qsa_index: a device-resident position serves spans of up to 8 rows");
                timed_launch(value, &scores_tiled_kernel<false>, dim3(checked_blocks(most, TILE_BLOCKS), checked_blocks(steps, TILE_ROWS)), dim3(TILE_THREADS), 0,
                             queries, query_stride, blocks, pool, base, steps, scores, static_cast<const uint32_t*>(nullptr), 0u);
            }
        }
    }
    const unsigned rows = checked_blocks(steps, 1);
    // a few long rows: the thinning goes to many workgroups first (their lists live in a small buffer the handle keeps from
    // the first such call, or from the first sd_graph_begin, on: a call recorded into a graph finds it there)
    const uint2* thinned = nullptr;
    const uint32_t* thinned_counts = nullptr;
    if (rows <= unsigned(THIN_ROWS) && most >= size_t(8) * SELECT_THREADS) {
        constexpr size_t lists = thin_list_bytes;
        select_thin_reserve(value);
        if (value.select_thin) {
            uint2* listed = static_cast<uint2*>(value.select_thin);
            uint32_t* listed_counts = reinterpret_cast<uint32_t*>(static_cast<uint8_t*>(value.select_thin) + lists);
            thin_kernel<<<dim3(THIN_SEGMENTS, rows), THIN_THREADS, 0, value.stream>>>(scores, pool, base, dynamic_base, listed, listed_counts);
            thinned = listed; thinned_counts = listed_counts;
        }
    }
    if (most <= size_t(LDS_RUNS) * SELECT_THREADS) launch_select<0>(value, scores, pool, base, dynamic_base, selected, most, rows, indices, counts, thinned, thinned_counts);
    else launch_select<33>(value, scores, pool, base, dynamic_base, selected, most, rows, indices, counts, thinned, thinned_counts);
    SD_OP_END
}

uint64_t sdx_qsa_index_interval_scratch(uint64_t steps, uint64_t pool) {
    try { return interval_scratch_bytes(size_t(checked_product({steps, 1})), size_t(checked_product({pool, 1}))); } catch (const std::exception&) { return 0; }
}

int sdx_qsa_index_interval(void* handle, const float* queries, uint64_t query_stride, const float* blocks, uint64_t pool, uint64_t base, uint64_t steps,
                           uint64_t selected, float* scores, float* indices, float* counts, void* scratch, uint64_t scratch_bytes, uint64_t* valid) {
    if (handle && !interval_serves(size_t(base))) {
        // a short context: the exact kernels' time is small, and a sample of it says little
        if (valid) *valid = 0;
        return sdx_qsa_index(handle, queries, query_stride, blocks, pool, base, nullptr, steps, selected, scores, indices, counts);
    }
    SD_OP_BEGIN
    if (!steps || steps > 4096 || !pool || query_stride < HEADS * COLUMNS) throw std::runtime_error("sdx_qsa_index_interval: 1 to 4096 steps, pool >= 1, query stride >= 512");
    if (pool > size_t(64) * SELECT_THREADS + 1) throw std::runtime_error("sdx_qsa_index_interval: a pool of more than 65537 blocks (a context beyond 262144)");
    if ((base + steps) / 4 > pool || base + steps > 4 * pool) throw std::runtime_error("sdx_qsa_index_interval: the span's blocks must fit the pool");
    if (selected < 2052) throw std::runtime_error("sdx_qsa_index_interval: `selected` is smaller than a row's selection can be");
    op_span(value, queries, checked_floats({steps - 1, query_stride}) + HEADS * COLUMNS * 4, "sdx_qsa_index_interval queries");
    op_span(value, blocks, checked_floats({pool, uint64_t(COLUMNS)}), "sdx_qsa_index_interval blocks");
    op_span(value, scores, checked_floats({steps, pool}), "sdx_qsa_index_interval scores");
    op_span(value, indices, checked_floats({steps, selected}), "sdx_qsa_index_interval indices");
    op_span(value, counts, checked_floats({steps}), "sdx_qsa_index_interval counts");
    const size_t need = interval_scratch_bytes(steps, pool);
    if (scratch_bytes < need) throw std::runtime_error("sdx_qsa_index_interval: scratch too small (see sdx_qsa_index_interval_scratch)");
    op_span(value, scratch, need, "sdx_qsa_index_interval scratch");
    unsigned gate = 0;
    const uint32_t* undecided = interval_select(value, queries, query_stride, blocks, pool, base, steps, selected, scores, indices, counts, scratch, valid, &gate);
    // the rows the intervals left undecided, by the exact kernels (workgroups of other rows leave at once)
    const size_t most = size_t((base + steps) / 4);
    scores_tiled_kernel<true><<<dim3(std::min(checked_blocks(most, TILE_BLOCKS), 64u), checked_blocks(steps, TILE_ROWS)), TILE_THREADS, 0, value.stream>>>(
        queries, query_stride, blocks, pool, base, steps, scores, undecided, gate);
    const unsigned rows = checked_blocks(steps, 1);
    if (most <= size_t(LDS_RUNS) * SELECT_THREADS) launch_select<0>(value, scores, pool, base, nullptr, selected, most, rows, indices, counts, nullptr, nullptr, undecided);
    else launch_select<33>(value, scores, pool, base, nullptr, selected, most, rows, indices, counts, nullptr, nullptr, undecided);
    SD_OP_END
}

int sdx_qsa_index_interval_undecided(void* handle, const void* scratch, uint64_t steps, uint64_t pool, uint64_t* rows) {
    SD_OP_BEGIN
    if (!rows || !steps || steps > 4096 || !pool) throw std::runtime_error("sdx_qsa_index_interval_undecided: steps, pool, rows");
    op_span(value, scratch, interval_scratch_bytes(steps, pool), "sdx_qsa_index_interval scratch");
    *rows = interval_undecided(value, scratch, steps, pool);
    SD_OP_END
}

uint64_t sdx_qsa_decode_attend_scratch(uint64_t steps, uint64_t heads, uint64_t kv_heads, uint64_t context) {
    try {
        const uint64_t pool = context / 4 + 1;
        return checked_floats({steps, heads * 256 + pool + 2052 + 1}) + 256 + sdx_selected_attention_scratch(steps, kv_heads, 2052);
    } catch (const std::exception&) { return 0; }
}

int sdx_qsa_decode_attend(void* handle, const sdx_qsa_state* state, float* projections, uint64_t stride, uint64_t steps, const uint32_t* positions,
                          const uint32_t* ropes, void* scratch, uint64_t scratch_bytes, float* attended) {
    {
        SD_OP_BEGIN
        if (!state || !state->kv) throw std::runtime_error("sdx_qsa_decode_attend: no state");
        const sdx_kv_pool& kv = *state->kv;
        const uint64_t heads = state->heads, context = state->context, pool = context / 4 + 1;
        if (kv.dim != 256 || !heads || heads % kv.kv_heads || heads / kv.kv_heads > 16 || !steps || steps > 8 || !context || context > (uint64_t(1) << 24) ||
            stride < heads * 512 + uint64_t(kv.kv_heads) * 512 + HEADS * COLUMNS + COLUMNS)
            throw std::runtime_error("sdx_qsa_decode_attend: 1..8 rows of heads x 512 + K/V heads x 512 + 640 projections, K/V rows of 256 columns");
        if (!state->page_table && kv.page_tokens < context) throw std::runtime_error("sdx_qsa_decode_attend: without a page table one page must hold the context");
        if (state->page_table) op_span(value, state->page_table, checked_floats({(context + kv.page_tokens - 1) / kv.page_tokens}), "a page table");
        validate_pool(value, state->kv);        // (the rows are written below: page moves queued so far come first)
        op_span(value, state->blocks, checked_floats({pool, uint64_t(COLUMNS)}), "pooled index keys");
        op_span(value, state->history, size_t(RING) * COLUMNS * 4, "the index history");
        op_span(value, state->q_norm, 256 * 4, "a query norm weight");
        op_span(value, state->k_norm, 256 * 4, "a key norm weight");
        op_span(value, state->index_q_norm, COLUMNS * 4, "an index query norm weight");
        op_span(value, state->index_k_norm, COLUMNS * 4, "an index key norm weight");
        op_span(value, projections, checked_floats({steps - 1, stride}) + (heads * 512 + uint64_t(kv.kv_heads) * 512 + 640) * 4, "projections");
        op_span(value, positions, checked_floats({steps}), "positions");
        op_span(value, ropes, checked_floats({steps}), "rope positions");
        op_span(value, attended, checked_floats({steps, heads, 256}), "an attention output");
        const uint64_t need = sdx_qsa_decode_attend_scratch(steps, heads, kv.kv_heads, context);
        if (!need || scratch_bytes < need) throw std::runtime_error("sdx_qsa_decode_attend: scratch too small (see sdx_qsa_decode_attend_scratch)");
        op_span(value, scratch, need, "stage scratch");
        StageArgs args{};
        args.projections = projections; args.stride = stride;
        args.q_norm = state->q_norm; args.k_norm = state->k_norm; args.index_q_norm = state->index_q_norm; args.index_k_norm = state->index_k_norm;
        args.heads = unsigned(heads); args.kv_heads = kv.kv_heads; args.steps = unsigned(steps); args.positions = positions; args.ropes = ropes;
        args.pages = static_cast<uint8_t*>(kv.pages); args.page_tokens = kv.page_tokens; args.row_bytes = kv.row_bytes; args.page_table = state->page_table; args.page_count = size_t(kv.page_count);
        args.context = context; args.queries = static_cast<float*>(scratch); args.blocks = state->blocks; args.history = state->history; args.pool = pool;
        stage_prepare_kernel<<<dim3(unsigned(heads + kv.kv_heads + HEADS + 1), unsigned(steps)), 256, 0, value.stream>>>(args);
        SD_CHECK(hipGetLastError());
    } catch (const std::exception& e) { ::sd::last_error = e.what(); return -1; }
    }
    // the two stages behind it, on the position the device holds
    const uint64_t heads = state->heads, pool = state->context / 4 + 1;
    float* queries = static_cast<float*>(scratch);
    float* scores = queries + steps * heads * 256;
    float* indices = scores + steps * pool;
    float* counts = indices + steps * 2052;
    uint8_t* partial = reinterpret_cast<uint8_t*>((reinterpret_cast<uintptr_t>(counts + steps) + 255) & ~uintptr_t(255));
    const size_t index_at = heads * 512 + size_t(state->kv->kv_heads) * 512;
    if (sdx_qsa_index(handle, projections + index_at, stride, state->blocks, pool, 0, positions, steps, 2052, scores, indices, counts) < 0) return -1;
    return sdx_selected_attention(handle, state->kv, state->page_table, state->context, 0, positions, indices, 2052, counts, queries, 0, steps, heads, 0.0625f,
                                  projections + 256, 512, stride, attended, 0, partial, sdx_selected_attention_scratch(steps, state->kv->kv_heads, 2052));
}

uint64_t sdx_qsa_prefill_attend_scratch(uint64_t steps, uint64_t heads, uint64_t kv_heads, uint64_t context) {
    try {
        const uint64_t pool = context / 4 + 1;
        const uint64_t first = (checked_floats({steps, heads * 256 + pool + 2052 + 1}) + 255) & ~uint64_t(255);
        const uint64_t partial = (sdx_selected_attention_scratch(steps, kv_heads, 2052) + 255) & ~uint64_t(255);
        return first + partial + sdx_qsa_index_interval_scratch(steps, pool);
    } catch (const std::exception&) { return 0; }
}

int sdx_qsa_prefill_attend(void* handle, const sdx_qsa_state* state, float* projections, uint64_t stride, uint64_t steps, uint64_t base, void* scratch,
                           uint64_t scratch_bytes, uint64_t* valid, float* attended) {
    size_t index_at = 0;
    uint64_t pool = 0;
    {
        SD_OP_BEGIN
        if (!state || !state->kv) throw std::runtime_error("sdx_qsa_prefill_attend: no state");
        const sdx_kv_pool& kv = *state->kv;
        const uint64_t heads = state->heads, context = state->context;
        pool = context / 4 + 1;
        if (kv.dim != 256 || !heads || heads % kv.kv_heads || heads / kv.kv_heads > 16 || !steps || steps > 4096 || !context || context > (uint64_t(1) << 24) ||
            base + steps > context || stride < heads * 512 + uint64_t(kv.kv_heads) * 512 + HEADS * COLUMNS + COLUMNS)
            throw std::runtime_error("sdx_qsa_prefill_attend: 1..4096 rows of heads x 512 + K/V heads x 512 + 640 projections inside the context, K/V rows of 256 columns");
        if (!state->page_table && kv.page_tokens < context) throw std::runtime_error("sdx_qsa_prefill_attend: without a page table one page must hold the context");
        if (state->page_table) op_span(value, state->page_table, checked_floats({(context + kv.page_tokens - 1) / kv.page_tokens}), "a page table");
        validate_pool(value, state->kv);
        op_span(value, state->blocks, checked_floats({pool, uint64_t(COLUMNS)}), "pooled index keys");
        op_span(value, state->history, size_t(RING) * COLUMNS * 4, "the index history");
        op_span(value, state->q_norm, 256 * 4, "a query norm weight");
        op_span(value, state->k_norm, 256 * 4, "a key norm weight");
        op_span(value, state->index_q_norm, COLUMNS * 4, "an index query norm weight");
        op_span(value, state->index_k_norm, COLUMNS * 4, "an index key norm weight");
        op_span(value, projections, checked_floats({steps - 1, stride}) + (heads * 512 + uint64_t(kv.kv_heads) * 512 + 640) * 4, "projections");
        op_span(value, attended, checked_floats({steps, heads, 256}), "an attention output");
        const uint64_t need = sdx_qsa_prefill_attend_scratch(steps, heads, kv.kv_heads, context);
        if (!need || scratch_bytes < need) throw std::runtime_error("sdx_qsa_prefill_attend: scratch too small (see sdx_qsa_prefill_attend_scratch)");
        if (uintptr_t(scratch) % 256) throw std::runtime_error("sdx_qsa_prefill_attend: the scratch must lie on a 256-byte boundary");
        op_span(value, scratch, need, "stage scratch");
        StageArgs args{};
        args.projections = projections; args.stride = stride;
        args.q_norm = state->q_norm; args.k_norm = state->k_norm; args.index_q_norm = state->index_q_norm; args.index_k_norm = state->index_k_norm;
        args.heads = unsigned(heads); args.kv_heads = kv.kv_heads; args.steps = unsigned(steps); args.positions = nullptr; args.ropes = nullptr; args.base = size_t(base);
        args.pages = static_cast<uint8_t*>(kv.pages); args.page_tokens = kv.page_tokens; args.row_bytes = kv.row_bytes; args.page_table = state->page_table; args.page_count = size_t(kv.page_count);
        args.context = context; args.queries = static_cast<float*>(scratch); args.blocks = state->blocks; args.history = state->history; args.pool = pool;
        // 1. rows normalised and turned, K/V rows appended (no workgroup of the grid pools: the span's blocks are pooled at once below)
        stage_prepare_kernel<<<dim3(unsigned(heads + kv.kv_heads + HEADS), unsigned(steps)), 256, 0, value.stream>>>(args);
        SD_CHECK(hipGetLastError());
        // 2. the blocks the span completes, and the ring's newest rows
        index_at = heads * 512 + size_t(kv.kv_heads) * 512;
        const float* incoming = projections + index_at + HEADS * COLUMNS;
        const size_t completed = size_t((base + steps) / 4 - base / 4);
        if (completed) pool_kernel<<<checked_blocks(completed, 1), COLUMNS, 0, value.stream>>>(incoming, size_t(stride), state->history, state->index_k_norm, size_t(pool), size_t(base), state->blocks);
        save_history_kernel<<<checked_blocks(std::min<size_t>(steps, 4) * COLUMNS), 256, 0, value.stream>>>(incoming, size_t(stride), size_t(base), size_t(steps), state->history);
        SD_CHECK(hipGetLastError());
    } catch (const std::exception& e) { ::sd::last_error = e.what(); return -1; }
    }
    // 3. the rows' selections (by intervals past 32768 positions, the packed keys carried from chunk to chunk in the scratch);
    // 4. each row over its selection, gated
    const uint64_t heads = state->heads, kv_heads = state->kv->kv_heads;
    float* queries = static_cast<float*>(scratch);
    float* scores = queries + steps * heads * 256;
    float* indices = scores + steps * pool;
    float* counts = indices + steps * 2052;
    uint8_t* partial = reinterpret_cast<uint8_t*>((reinterpret_cast<uintptr_t>(counts + steps) + 255) & ~uintptr_t(255));
    const uint64_t partial_bytes = sdx_selected_attention_scratch(steps, kv_heads, 2052);
    uint8_t* interval = partial + ((partial_bytes + 255) & ~uint64_t(255));
    if (sdx_qsa_index_interval(handle, projections + index_at, stride, state->blocks, pool, base, steps, 2052, scores, indices, counts, interval,
                               sdx_qsa_index_interval_scratch(steps, pool), valid) < 0) return -1;
    return sdx_selected_attention(handle, state->kv, state->page_table, state->context, base, nullptr, indices, 2052, counts, queries, 0, steps, heads, 0.0625f,
                                  projections + 256, 512, stride, attended, 0, partial, partial_bytes);
}

}  // extern "C"
