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
// prefill chunk (FP32 FMA-bound); a 1024-thread workgroup per row for the selection, the row's scores held in registers, four
// 8-bit radix passes over per-wave LDS histograms (the first, where nearly all values share a digit, counted by ballots), and
// one ordered pass whose slots come from 64-wide ballots and a scan over (run, wave) counts.
#include "device.hpp"
#include "../../include/straydog_gpu_ext.h"

using namespace sd;

namespace {

constexpr int HEADS = 4, COLUMNS = 128, KEEP = 512, RING = 16;

__device__ __forceinline__ float turn(float own, float partner, unsigned column, size_t position) {
    if (column >= 64) return own;
    const float angle = float(position) / powf(1e7f, float(column % 32) / 32.0f);
    return own * cosf(angle) + (column < 32 ? -partner : partner) * sinf(angle);
}

// The sum over the workgroup's `width` threads in the order of a halving tree, sums[c] += sums[c + offset], which is the
// reference's order; the last six levels are lane shifts inside the first wave.
__device__ __forceinline__ float tree_sum(float mine, float* sums, unsigned width) {
    const unsigned c = threadIdx.x;
    sums[c] = mine;
    __syncthreads();
    for (unsigned offset = width / 2; offset >= 64; offset /= 2) {
        if (c < offset) sums[c] += sums[c + offset];
        __syncthreads();
    }
    if (c < 64) {
        float v = sums[c];
        #pragma unroll
        for (unsigned offset = 32; offset; offset /= 2) v += __shfl_down(v, offset);
        if (c == 0) sums[0] = v;
    }
    __syncthreads();
    return sums[0];
}

// One workgroup of `width` threads per (row, head).
__global__ void __launch_bounds__(256) normalize_kernel(const float* source, const float* norm, unsigned heads, unsigned width, size_t stride,
                                                        size_t position, float* target) {
    __shared__ float values[256], sums[256];
    const size_t head = blockIdx.x, token = head / heads;
    const unsigned c = threadIdx.x;
    const float x = source[head * stride + c];
    values[c] = x * norm[c];
    const float denominator = sqrtf(tree_sum(x * x, sums, width) / float(width) + 1e-6f);
    const float own = values[c] / denominator;
    const float partner = c < 64 ? values[(c + 32) % 64] / denominator : 0.0f;
    target[head * width + c] = turn(own, partner, c, position + token);
}

// One workgroup of 128 threads per block completed by the span.
__global__ void __launch_bounds__(COLUMNS) pool_kernel(const float* incoming, const float* history, const float* norm, size_t pool, size_t base,
                                                       float* blocks) {
    __shared__ float values[COLUMNS], sums[COLUMNS];
    const size_t block = base / 4 + blockIdx.x, begin = block * 4;
    const unsigned c = threadIdx.x;
    float x = 0.0f;
    #pragma unroll
    for (size_t tap = 0; tap < 4; ++tap) {
        const size_t pos = begin + tap;
        x += pos < base ? history[(pos % RING) * COLUMNS + c] : incoming[(pos - base) * COLUMNS + c];
    }
    x /= 4.0f;
    values[c] = x * norm[c];
    const float denominator = sqrtf(tree_sum(x * x, sums, COLUMNS) / float(COLUMNS) + 1e-6f);
    const float own = values[c] / denominator;
    const float partner = c < 64 ? values[(c + 32) % 64] / denominator : 0.0f;
    blocks[c * pool + block] = turn(own, partner, c, begin);
}

__global__ void __launch_bounds__(256) save_history_kernel(const float* incoming, size_t base, size_t steps, float* history) {
    const size_t i = threadIdx.x + size_t(blockIdx.x) * 256, kept = steps < 4 ? steps : 4;
    if (i >= kept * COLUMNS) return;
    const size_t token = steps - kept + i / COLUMNS;
    history[((base + token) % RING) * COLUMNS + i % COLUMNS] = incoming[token * COLUMNS + i % COLUMNS];
}

__device__ __forceinline__ float positive_sum(const float (&dot)[HEADS]) {
    float total = fmaxf(dot[0], 0.0f) + fmaxf(dot[1], 0.0f);
    total += fmaxf(dot[2], 0.0f);
    total += fmaxf(dot[3], 0.0f);
    return total;
}

// ---- scores of a short span: a lane per block, T rows per lane ------------------------------------------------------------
// The queries sit in LDS as [row][column][head], so the four heads of a column come by one wave-uniform 16-byte read.
template<int T>
__global__ void __launch_bounds__(64) scores_rows_kernel(const float* __restrict__ queries, size_t query_stride, const float* __restrict__ blocks,
                                                         size_t pool, size_t base, const uint32_t* dynamic, unsigned steps, float* __restrict__ scores) {
    __shared__ __align__(16) float q[T][COLUMNS][HEADS];
    if (dynamic) base = *dynamic;
    const size_t most = min((base + steps) / 4, pool), first = size_t(blockIdx.x) * 64;   // the last row's complete blocks
    const unsigned lane = threadIdx.x;
    if (most <= KEEP || first >= most) return;
    for (unsigned i = lane; i < T * HEADS * COLUMNS; i += 64) {
        const unsigned row = i / (HEADS * COLUMNS), h = i / COLUMNS % HEADS, c = i % COLUMNS;
        q[row][c][h] = row < steps ? queries[row * query_stride + h * COLUMNS + c] : 0.0f;
    }
    __syncthreads();
    const float* column = blocks + min(first + lane, pool - 1);
    float dot[T][HEADS] = {};
    #pragma unroll 1
    for (unsigned c0 = 0; c0 < COLUMNS; c0 += 16) {
        float key[16];
        #pragma unroll
        for (unsigned j = 0; j < 16; ++j) key[j] = column[size_t(c0 + j) * pool];
        #pragma unroll
        for (unsigned j = 0; j < 16; ++j) {
            #pragma unroll
            for (int row = 0; row < T; ++row) {
                const float4 heads = *reinterpret_cast<const float4*>(q[row][c0 + j]);
                dot[row][0] = fmaf(key[j], heads.x, dot[row][0]);
                dot[row][1] = fmaf(key[j], heads.y, dot[row][1]);
                dot[row][2] = fmaf(key[j], heads.z, dot[row][2]);
                dot[row][3] = fmaf(key[j], heads.w, dot[row][3]);
            }
        }
    }
    #pragma unroll
    for (int row = 0; row < T; ++row) {
        const size_t complete = (base + row + 1) / 4;
        if (unsigned(row) < steps && complete > KEEP && first + lane < min(complete, pool)) scores[row * pool + first + lane] = positive_sum(dot[row]);
    }
}

// ---- scores of a prefill chunk: 32 rows x 256 blocks per workgroup ---------------------------------------------------------
// Eight waves; a lane owns 4 neighbouring blocks, a wave 4 rows, so a thread carries 4 x 4 x 4 chains.  Sixteen columns of
// keys [column][block] and queries [column][row * 4 + head] are staged at a time: the key read is 16 bytes a lane without
// bank conflicts, the query read is wave-uniform.  The next sixteen columns travel from global memory into registers while
// the current ones are multiplied.
constexpr int TILE_ROWS = 32, TILE_BLOCKS = 256, TILE_COLUMNS = 16, TILE_THREADS = 512, QUERY_PITCH = TILE_ROWS * HEADS + 4;
__global__ void __launch_bounds__(TILE_THREADS) scores_tiled_kernel(const float* __restrict__ queries, size_t query_stride,
                                                                    const float* __restrict__ blocks, size_t pool, size_t base, size_t steps,
                                                                    float* __restrict__ scores) {
    __shared__ __align__(16) float keys[2][TILE_COLUMNS][TILE_BLOCKS];
    __shared__ __align__(16) float query[2][TILE_COLUMNS][QUERY_PITCH];
    const size_t first_row = size_t(blockIdx.y) * TILE_ROWS, first_block = size_t(blockIdx.x) * TILE_BLOCKS;
    const size_t most = min((base + min(steps, first_row + TILE_ROWS)) / 4, pool);        // complete blocks of the tile's last row
    if (most <= KEEP || first_block >= most) return;
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

// body(i) for every run of 1024 blocks the row has: unrolled over the registers that hold the row, or a plain loop.
template<int RUN, bool HELD, class Body>
__device__ __forceinline__ void each_run(unsigned runs, Body body) {
    if constexpr (HELD) {
        #pragma unroll
        for (int i = 0; i < RUN; ++i)
            if (unsigned(i) < runs) body(i);
    } else {
        for (unsigned i = 0; i < runs; ++i) body(int(i));
    }
}

// One workgroup per row of up to RUN * 1024 complete blocks; block i * 1024 + t is thread t's value i.  HELD: the row is read
// once into registers (a prefill chunk's many rows); otherwise every pass reads it again, from L2 (the longest rows, whose
// 64 values a thread would not fit beside the rest at sixteen waves).
template<int RUN, bool HELD>
__global__ void __launch_bounds__(SELECT_THREADS) select_kernel(const float* __restrict__ scores, size_t pool, size_t base, const uint32_t* dynamic,
                                                                size_t selected, float* __restrict__ indices, float* __restrict__ counts) {
    __shared__ uint32_t bins[SELECT_WAVES * 256];            // a histogram per wave; later the (run, wave) counts
    __shared__ uint32_t wave_sums[SELECT_WAVES], threshold, remaining;
    if (dynamic) base = *dynamic;
    const size_t token = blockIdx.x, position = base + token, complete = (position + 1) / 4;
    const unsigned t = threadIdx.x, lane = t % 64, wave = t / 64;
    float* out = indices + token * selected;
    if (position + 1 > 4 * pool || complete > size_t(RUN) * SELECT_THREADS) {   // a position this key pool (or this variant) cannot hold
        if (t == 0) counts[token] = 0.0f;
        return;
    }
    if (complete <= KEEP) {
        for (size_t i = t; i <= position; i += SELECT_THREADS) out[i] = float(i);
        if (t == 0) counts[token] = float(position + 1);
        return;
    }
    const float* row = scores + token * pool;
    const unsigned runs = unsigned((complete + SELECT_THREADS - 1) / SELECT_THREADS);
    uint32_t values[HELD ? RUN : 1];
    if constexpr (HELD) {
        #pragma unroll
        for (int i = 0; i < RUN; ++i) {
            const size_t block = size_t(i) * SELECT_THREADS + t;
            values[i] = block < complete ? __float_as_uint(row[block]) : 0u;
        }
    }
    const auto value_of = [&](int i, bool valid) -> uint32_t {
        if constexpr (HELD) return values[i];
        else return valid ? __float_as_uint(row[size_t(i) * SELECT_THREADS + t]) : 0u;
    };
    // The 512th highest value, eight bits a pass.
    uint32_t prefix = 0, wanted = KEEP, mask = 0;
    uint32_t* own = bins + wave * 256;
    #pragma unroll 1
    for (int shift = 24; shift >= 0; shift -= 8) {
        for (unsigned i = t; i < SELECT_WAVES * 256; i += SELECT_THREADS) bins[i] = 0;
        __syncthreads();
        each_run<RUN, HELD>(runs, [&](int i) {
            const bool valid = size_t(i) * SELECT_THREADS + t < complete;
            const uint32_t bits = value_of(i, valid);
            const bool live = valid && (bits & mask) == prefix;
            const uint32_t digit = (bits >> shift) & 255u;
            if (shift == 24) {
                // nearly every score shares its top byte: the lanes of a digit add once, by a ballot
                uint64_t todo = __ballot(live);
                while (todo) {
                    const int leader = __ffsll(static_cast<long long>(todo)) - 1;
                    const uint32_t d = __shfl(digit, leader);
                    const uint64_t same = __ballot(live && digit == d);
                    if (int(lane) == leader) own[d] += uint32_t(__popcll(same));
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
            for (int w = 0; w < SELECT_WAVES; ++w) count += bins[w * 256 + bucket];
        const uint32_t above = group_scan(count, wave_sums, every);
        if (t < 256 && above < wanted && above + count >= wanted) { threshold = prefix | (bucket << shift); remaining = wanted - above; }
        __syncthreads();
        prefix = threshold; wanted = remaining;
        mask |= 255u << shift;
    }
    // Kept: every value above `prefix` and the first `wanted` equal to it, in block order.
    uint32_t* greater = bins;
    uint32_t* equal = bins + RUN * SELECT_WAVES;
    each_run<RUN, HELD>(runs, [&](int i) {
        const bool valid = size_t(i) * SELECT_THREADS + t < complete;
        const uint32_t bits = value_of(i, valid);
        const uint64_t above = __ballot(valid && bits > prefix), same = __ballot(valid && bits == prefix);
        if (lane == 0) { greater[i * SELECT_WAVES + wave] = uint32_t(__popcll(above)); equal[i * SELECT_WAVES + wave] = uint32_t(__popcll(same)); }
    });
    __syncthreads();
    const unsigned entries = runs * SELECT_WAVES;           // at most 1024: one per thread
    const uint32_t g = t < entries ? greater[t] : 0u, e = t < entries ? equal[t] : 0u;
    uint32_t every;
    const uint32_t greater_before = group_scan(g, wave_sums, every);
    const uint32_t equal_before = group_scan(e, wave_sums, every);
    if (t < entries) { greater[t] = greater_before; equal[t] = equal_before; }
    __syncthreads();
    const uint64_t below = (uint64_t(1) << lane) - 1;
    each_run<RUN, HELD>(runs, [&](int i) {
        const size_t block = size_t(i) * SELECT_THREADS + t;
        const bool valid = block < complete;
        const uint32_t bits = value_of(i, valid);
        const bool above = valid && bits > prefix, same = valid && bits == prefix;
        const uint64_t above_mask = __ballot(above), same_mask = __ballot(same);
        if (!above && !same) return;
        const uint32_t equal_seen = equal[i * SELECT_WAVES + wave] + uint32_t(__popcll(same_mask & below));
        if (same && equal_seen >= wanted) return;
        const size_t at = size_t(greater[i * SELECT_WAVES + wave] + uint32_t(__popcll(above_mask & below)) + min(equal_seen, wanted)) * 4;
        #pragma unroll
        for (size_t tap = 0; tap < 4; ++tap) out[at + tap] = float(block * 4 + tap);
    });
    const size_t head = size_t(KEEP) * 4;
    for (size_t i = t; complete * 4 + i <= position; i += SELECT_THREADS) out[head + i] = float(complete * 4 + i);
    if (t == 0) counts[token] = float(head + position + 1 - complete * 4);
}

template<int T>
void launch_rows(Device& d, const float* queries, size_t stride, const float* blocks, size_t pool, size_t base, const uint32_t* dynamic, size_t steps,
                 size_t most, float* scores) {
    scores_rows_kernel<T><<<checked_blocks(most, 64), 64, 0, d.stream>>>(queries, stride, blocks, pool, base, dynamic, unsigned(steps), scores);
}

}  // namespace

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
    if (completed) pool_kernel<<<checked_blocks(completed, 1), COLUMNS, 0, value.stream>>>(incoming, history, norm, pool, base, blocks);
    save_history_kernel<<<checked_blocks(std::min<size_t>(steps, 4) * COLUMNS), 256, 0, value.stream>>>(incoming, base, steps, history);
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
        KernelTimer timer(value);
        if (most > KEEP) {
            if (steps <= 1) launch_rows<1>(value, queries, query_stride, blocks, pool, base, dynamic_base, steps, most, scores);
            else if (steps <= 2) launch_rows<2>(value, queries, query_stride, blocks, pool, base, dynamic_base, steps, most, scores);
            else if (steps <= 4) launch_rows<4>(value, queries, query_stride, blocks, pool, base, dynamic_base, steps, most, scores);
            else if (steps <= 8) launch_rows<8>(value, queries, query_stride, blocks, pool, base, dynamic_base, steps, most, scores);
            else {
                if (dynamic_base) throw std::runtime_error("sdx_qsa_index: a device-resident position serves spans of up to 8 rows");
                scores_tiled_kernel<<<dim3(checked_blocks(most, TILE_BLOCKS), checked_blocks(steps, TILE_ROWS)), TILE_THREADS, 0, value.stream>>>(
                    queries, query_stride, blocks, pool, base, steps, scores);
            }
        }
    }
    const unsigned rows = checked_blocks(steps, 1);
    if (most <= size_t(4) * SELECT_THREADS) select_kernel<4, true><<<rows, SELECT_THREADS, 0, value.stream>>>(scores, pool, base, dynamic_base, selected, indices, counts);
    else if (most <= size_t(16) * SELECT_THREADS) select_kernel<16, true><<<rows, SELECT_THREADS, 0, value.stream>>>(scores, pool, base, dynamic_base, selected, indices, counts);
    else select_kernel<64, false><<<rows, SELECT_THREADS, 0, value.stream>>>(scores, pool, base, dynamic_base, selected, indices, counts);
    SD_OP_END
}

}  // extern "C"
