// The batched gather attention of the sparse top-k path on matrix cores: every sequence's query heads attend the BF16
// latent rows its selection lists, keys being a row's kdim columns and values its first vdim columns.  The arithmetic is
// op_sparse_attention_kernel's (reference gpu/ops.hpp:1240-1297) without window or sink, with BF16 operands and FP32
// sums, as the reference's WMMA prompt path does it (gpu/ds_attention_wmma.hpp:26-340).
//
// Shape of the work on gfx950 (wave64, v_mfma_f32_16x16x32_bf16):
//   * a workgroup (4 waves) owns one sequence, 64 or 128 of its selected rows and 32 heads; a wave takes 16 of the heads and
//     half of the value columns (the two waves of a head tile form the same scores and weights, each for itself: the partial
//     results, and not the products, are what this kernel's time goes into, and 32 heads a workgroup let a chunk be twice as
//     long, and the partial results half as many, with the same number of workgroups);
//   * 32 rows at a time are gathered (16-byte pieces, every row whole) into a padded tile in LDS, two tiles in turn, read
//     without bank conflicts as MFMA operands by all four waves: as rows for the scores, and for the values a lane takes
//     eight neighbouring columns of its eight rows (16 bytes each) and sorts them into eight operands with v_perm -- which
//     value column a lane's place in an operand stands for is free to choose, so nothing is transposed through LDS;
//   * S^T = K . Q^T (rows x heads) leaves the weights in the B-operand layout of O^T += V^T . P^T, so they never move
//     between lanes (the layout notes of paged_rows.hpp apply);
//   * the chunks' (maximum, sum, unnormalised output) are merged by a second kernel.
#include "paged_rows.hpp"

using namespace sd;
using namespace sd::paged;

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int CHUNK = 64, CHUNK_MAX = 128, BLOCK_HEADS = 32;           // selected rows per workgroup (the shorter kind, the longer), heads

struct GatherArgs {
    const uint16_t* q;              // [batch][heads][kdim] BF16
    const uint16_t* latents;        // [batch][groups][kdim] BF16
    const int32_t* selected;        // [batch][k], entries outside 0..groups-1 are skipped
    unsigned groups, k, heads, chunks, chunk_rows;
    float scale_log2;
    float* partial;                 // [batch][chunk][heads][vdim], then [batch][chunk][heads] (maximum, sum)
    float* out;                     // [batch][heads][vdim]
};

__device__ __forceinline__ uint32_t bf16_pair(float low, float high) {
    // round to nearest even, as the reference's to_bf16 (gpu/token_mixing.hpp:729-735) does for finite values
    const uint32_t a = __float_as_uint(low), b = __float_as_uint(high);
    return ((a + 0x7fffu + ((a >> 16) & 1u)) >> 16) | ((b + 0x7fffu + ((b >> 16) & 1u)) & 0xffff0000u);
}

template<int KDIM, int VDIM>
__global__ void __launch_bounds__(256) latent_gather_kernel(GatherArgs a) {
    constexpr int KSTEPS = KDIM / 32, TILES = VDIM / 16, KP = 2 * KDIM + 16, PIECES = KDIM / 8;
    const int chunk = blockIdx.x, batch = blockIdx.z, thread = threadIdx.x;
    const int lane = thread & 63, wave = __builtin_amdgcn_readfirstlane(thread >> 6), li = lane & 15, g = lane >> 4;
    const int tile_of_heads = wave & 1, half = wave >> 1;                                  // the wave's 16 heads and its half of the columns
    const int head = int(blockIdx.y) * BLOCK_HEADS + tile_of_heads * 16 + li;
    const bool real = head < int(a.heads);
    extern __shared__ uint8_t lds[];
    uint8_t* tiles = lds;                                     // two of [32 rows][KP]
    uint32_t* seen = reinterpret_cast<uint32_t*>(tiles + 2 * STEP * KP);   // two of [32]: 1 where the step's row exists
    int32_t* chosen = reinterpret_cast<int32_t*>(seen + 2 * STEP);         // [CHUNK_MAX]: the workgroup's selected rows, -1 where there is none
    const int first = chunk * int(a.chunk_rows), last = min(int(a.k), first + int(a.chunk_rows));
    // the selection is read once, ahead of everything else: a step's rows then wait for one load, not for two in a row
    if (thread < CHUNK_MAX) chosen[thread] = first + thread < last ? a.selected[size_t(batch) * a.k + first + thread] : -1;

    bf16x8 qf[KSTEPS];
    #pragma unroll
    for (int b = 0; b < KSTEPS; ++b) {
        uint4 bits = {0u, 0u, 0u, 0u};
        if (real) bits = *reinterpret_cast<const uint4*>(a.q + (size_t(batch) * a.heads + head) * KDIM + 32 * b + 8 * g);
        qf[b] = __builtin_bit_cast(bf16x8, bits);
    }
    constexpr int MY_TILES = TILES / 2;
    floatx4 acc[MY_TILES];
    #pragma unroll
    for (int j = 0; j < MY_TILES; ++j) acc[j] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
    float m = NEG_BIG, l = 0.0f;

    __syncthreads();
    // gather: a row is PIECES pieces of 16 bytes, a thread takes every 256th piece of a step; a missing row is read from row 0
    // and masked.  The pieces of the step after this one are fetched into registers before this one is multiplied.  (Two steps
    // ahead was measured and is slower: the registers it takes cost more than the trip to memory it hides.)
    constexpr int MINE = (STEP * PIECES + 255) / 256;
    uint4 fetched[MINE];
    uint32_t present = 0;                                     // bit j: the row of the thread's j-th piece exists
    // (the sequence's rows from an address all lanes share and a 32-bit offset a lane: two vector instructions an address)
    const uint8_t* rows = reinterpret_cast<const uint8_t*>(a.latents + size_t(batch) * a.groups * KDIM);
    const auto fetch = [&](int key0) {
        present = 0;
        #pragma unroll
        for (int j = 0; j < MINE; ++j) {
            const int piece = thread + 256 * j, row = piece / PIECES, part = piece % PIECES;
            fetched[j] = uint4{0u, 0u, 0u, 0u};
            if (piece < STEP * PIECES) {
                const uint32_t index = uint32_t(chosen[key0 - first + row]);
                const bool exists = index < a.groups;                       // (a negative entry is a large unsigned one)
                fetched[j] = *reinterpret_cast<const uint4*>(rows + size_t((exists ? index : 0u) * uint32_t(2 * KDIM) + uint32_t(16 * part)));
                present |= exists ? 1u << j : 0u;
            }
        }
    };
    if (first < last) fetch(first);
    for (int key0 = first, turn = 0; key0 < last; key0 += STEP, turn ^= 1) {
        // (the tile of the step before last is done with: every wave has passed the barrier of the step between)
        uint8_t* ktile = tiles + turn * STEP * KP;
        uint32_t* here = seen + turn * STEP;
        #pragma unroll
        for (int j = 0; j < MINE; ++j) {
            const int piece = thread + 256 * j, row = piece / PIECES, part = piece % PIECES;
            if (piece < STEP * PIECES) {
                *reinterpret_cast<uint4*>(ktile + row * KP + 16 * part) = fetched[j];
                if (part == 0) here[row] = (present >> j) & 1u;
            }
        }
        if (key0 + STEP < last) fetch(key0 + STEP);
        __syncthreads();
        // S^T tiles: rows of the step (4 per lane group) x heads (lane li)
        floatx4 s[2] = {floatx4{0.0f, 0.0f, 0.0f, 0.0f}, floatx4{0.0f, 0.0f, 0.0f, 0.0f}};
        #pragma unroll
        for (int b = 0; b < KSTEPS; ++b)
            #pragma unroll
            for (int t = 0; t < 2; ++t) {
                const bf16x8 ka = *reinterpret_cast<const bf16x8*>(ktile + (16 * t + li) * KP + 64 * b + 16 * g);
                s[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka, qf[b], s[t], 0, 0, 0);
            }
        float top = NEG_BIG;
        #pragma unroll
        for (int t = 0; t < 2; ++t) {
            const uint4 flags = *reinterpret_cast<const uint4*>(here + 16 * t + 4 * g);
            const uint32_t flag[4] = {flags.x, flags.y, flags.z, flags.w};
            #pragma unroll
            for (int r = 0; r < 4; ++r) {
                if (!flag[r]) s[t][r] = -INFINITY;
                top = fmaxf(top, s[t][r]);
            }
        }
        top = row_max(top);
        // The reference maximum moves only when some head's maximum has outgrown it by more than 2^8 (weights stay below 2^8,
        // and 128 accumulator registers are not multiplied through at every step); the first step sets it, nothing is summed yet.
        if (key0 == first) m = top;
        else if (__any((top - m) * a.scale_log2 > 8.0f)) {
            asm volatile("; new reference maxima" ::: "memory");
            const float m_new = fmaxf(m, top), alpha = __builtin_amdgcn_exp2f((m - m_new) * a.scale_log2);
            m = m_new;
            l *= alpha;
            #pragma unroll
            for (int j = 0; j < MY_TILES; ++j) acc[j] *= alpha;
        }
        const float offset = -m * a.scale_log2;
        float w[8], sum = 0.0f;
        #pragma unroll
        for (int t = 0; t < 2; ++t)
            #pragma unroll
            for (int r = 0; r < 4; ++r) {
                w[4 * t + r] = __builtin_amdgcn_exp2f(fmaf(s[t][r], a.scale_log2, offset));
                sum += w[4 * t + r];
            }
        l += sum;
        // The weights as two BF16 terms (the value and what its rounding left), so the products keep 16 bits of each weight.
        float rest[8];
        #pragma unroll
        for (int i = 0; i < 8; ++i) rest[i] = w[i] - __uint_as_float(bf16_pair(0.0f, w[i]) & 0xffff0000u);
        const uint4 high = {bf16_pair(w[0], w[1]), bf16_pair(w[2], w[3]), bf16_pair(w[4], w[5]), bf16_pair(w[6], w[7])};
        const uint4 low = {bf16_pair(rest[0], rest[1]), bf16_pair(rest[2], rest[3]), bf16_pair(rest[4], rest[5]), bf16_pair(rest[6], rest[7])};
        const bf16x8 pb = __builtin_bit_cast(bf16x8, high), pl = __builtin_bit_cast(bf16x8, low);
        // O^T tiles, the wave's half of them.  The lane's place li in an A operand stands for value column
        // 128 (2 half + q) + 8 li + c in tile 8 q + c: its eight k-slots are that column of the lane's rows {4g..4g+3, 16+4g..}, and
        // one 16-byte read a row brings the eight columns c = 0..7 at once.
        #pragma unroll
        for (int q = 0; q < MY_TILES / 8; ++q) {
            uint4 rows8[8];
            #pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int row = 4 * g + (e < 4 ? e : 12 + e);
                rows8[e] = *reinterpret_cast<const uint4*>(ktile + row * KP + 2 * (128 * (2 * half + q) + 8 * li));
            }
            #pragma unroll
            for (int c = 0; c < 8; ++c) {
                const uint32_t sel = (c & 1) ? 0x07060302u : 0x05040100u;
                uint32_t words[4];
                #pragma unroll
                for (int w = 0; w < 4; ++w) {
                    const uint4 &low = rows8[2 * w], &high = rows8[2 * w + 1];
                    const uint32_t lo = c / 2 == 0 ? low.x : c / 2 == 1 ? low.y : c / 2 == 2 ? low.z : low.w;
                    const uint32_t hi = c / 2 == 0 ? high.x : c / 2 == 1 ? high.y : c / 2 == 2 ? high.z : high.w;
                    words[w] = byte_perm(hi, lo, sel);
                }
                const bf16x8 va = __builtin_bit_cast(bf16x8, uint4{words[0], words[1], words[2], words[3]});
                acc[8 * q + c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va, pb, acc[8 * q + c], 0, 0, 0);
                acc[8 * q + c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va, pl, acc[8 * q + c], 0, 0, 0);
            }
        }
    }
    l = row_sum(l);
    // The partial results leave through LDS: an accumulator's four values are columns 8 apart (rows 4g + r of the tile are the
    // places li = 4g + r of the A operand), and a store should be a stretch of one head's row.  A wave uses a stretch of LDS of
    // its own, written and read back by itself; the barrier is for the tiles that the stretches lie over.
    constexpr int MY_COLUMNS = VDIM / 2, ROW_WORDS = MY_COLUMNS + 4;
    static_assert(MY_COLUMNS == 4 * 64 && MY_TILES == 16, "a lane stores 16 bytes of a head's half row");
    __syncthreads();
    float* mine = reinterpret_cast<float*>(lds) + wave * 16 * ROW_WORDS;
    #pragma unroll
    for (int j = 0; j < MY_TILES; ++j)
        #pragma unroll
        for (int r = 0; r < 4; ++r) mine[li * ROW_WORDS + 128 * (j / 8) + 8 * (4 * g + r) + j % 8] = acc[j][r];
    const size_t item = (size_t(batch) * a.chunks + chunk) * a.heads;
    const int head0 = int(blockIdx.y) * BLOCK_HEADS + tile_of_heads * 16;
    #pragma unroll 4
    for (int h = 0; h < 16; ++h)
        if (head0 + h < int(a.heads))
            *reinterpret_cast<floatx4*>(a.partial + (item + head0 + h) * VDIM + half * MY_COLUMNS + 4 * lane) = *reinterpret_cast<const floatx4*>(mine + h * ROW_WORDS + 4 * lane);
    if (real && g == 0 && half == 0) {
        float* stats = a.partial + size_t(gridDim.z) * a.chunks * a.heads * VDIM + (item + head) * 2;
        stats[0] = m; stats[1] = l;
    }
}

// One block per (sequence, head): the chunks merged under their common maximum and normalised; a head none of whose
// rows exists gives zeros.  The chunks' pieces are asked for eight at a time, so that eight loads are in flight and not one.
template<int VDIM>
__global__ void __launch_bounds__(VDIM / 4) latent_merge_kernel(GatherArgs a) {
    const size_t item = blockIdx.x, batch = item / a.heads, head = item % a.heads;
    const float* base = a.partial + (batch * a.chunks * a.heads + head) * VDIM;
    const float* stats = a.partial + size_t(gridDim.x) * a.chunks * VDIM + (batch * a.chunks * a.heads + head) * 2;      // (behind all the values)
    const size_t step = size_t(a.heads) * VDIM, stats_step = size_t(a.heads) * 2;
    constexpr unsigned AT_ONCE = 8;
    float top = NEG_BIG;
    for (unsigned c0 = 0; c0 < a.chunks; c0 += AT_ONCE) {
        float tops[AT_ONCE];
        #pragma unroll
        for (unsigned i = 0; i < AT_ONCE; ++i) tops[i] = stats[min(c0 + i, a.chunks - 1) * stats_step];
        #pragma unroll
        for (unsigned i = 0; i < AT_ONCE; ++i) top = fmaxf(top, tops[i]);
    }
    floatx4 value = {0.0f, 0.0f, 0.0f, 0.0f};
    float sum = 0.0f;
    for (unsigned c0 = 0; c0 < a.chunks; c0 += AT_ONCE) {
        floatx4 values[AT_ONCE];
        float tops[AT_ONCE], sums[AT_ONCE];
        #pragma unroll
        for (unsigned i = 0; i < AT_ONCE; ++i) {
            const size_t chunk = min(c0 + i, a.chunks - 1);
            values[i] = *reinterpret_cast<const floatx4*>(base + chunk * step + 4 * threadIdx.x);
            tops[i] = stats[chunk * stats_step];
            sums[i] = stats[chunk * stats_step + 1];
        }
        #pragma unroll
        for (unsigned i = 0; i < AT_ONCE; ++i) {
            const float weight = c0 + i < a.chunks ? __builtin_amdgcn_exp2f((tops[i] - top) * a.scale_log2) : 0.0f;
            sum += sums[i] * weight;
            value += values[i] * weight;
        }
    }
    if (sum > 0.0f) value *= 1.0f / sum; else value = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
    *reinterpret_cast<floatx4*>(a.out + item * VDIM + 4 * threadIdx.x) = value;
}

}  // namespace

namespace sd {

// The shapes the matrix-core path takes (the batched entry falls back to the general kernel otherwise).
bool latent_gather_supported(uint64_t kdim, uint64_t vdim) { return kdim == 576 && vdim == 512; }

uint64_t latent_gather_scratch(uint64_t batch, uint64_t k, uint64_t heads, uint64_t vdim) {
    return batch * ((k + CHUNK - 1) / CHUNK) * heads * (vdim + 2) * 4;
}

void latent_gather(Device& d, const void* q, const void* latents, const int32_t* selected, uint64_t batch, uint64_t groups, uint64_t k,
                   uint64_t heads, float scale, float* out, float* partial) {
    constexpr int KDIM = 576, VDIM = 512;
    GatherArgs args{};
    args.q = static_cast<const uint16_t*>(q); args.latents = static_cast<const uint16_t*>(latents); args.selected = selected;
    args.groups = unsigned(groups); args.k = unsigned(k); args.heads = unsigned(heads);
    // the longer chunks when they still give every compute unit a workgroup: half the partial results to write and to merge
    const uint64_t head_parts = (heads + BLOCK_HEADS - 1) / BLOCK_HEADS;
    args.chunk_rows = batch * ((k + CHUNK_MAX - 1) / CHUNK_MAX) * head_parts >= uint64_t(d.compute_units) ? CHUNK_MAX : CHUNK;
    args.chunks = unsigned((k + args.chunk_rows - 1) / args.chunk_rows);
    args.scale_log2 = scale * 1.44269504088896341f; args.partial = partial; args.out = out;
    constexpr size_t shared = 2 * size_t(STEP) * (2 * KDIM + 16) + 2 * STEP * 4 + CHUNK_MAX * 4;
    raise_shared_limit(d, reinterpret_cast<const void*>(&latent_gather_kernel<KDIM, VDIM>), shared);
    timed_launch(d, &latent_gather_kernel<KDIM, VDIM>, dim3(args.chunks, unsigned(head_parts), unsigned(batch)), dim3(256), shared, args);
    SD_CHECK(hipGetLastError());
    latent_merge_kernel<VDIM><<<unsigned(batch * heads), VDIM / 4, 0, d.stream>>>(args);
}

}  // namespace sd
