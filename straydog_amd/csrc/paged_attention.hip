// Causal grouped-query attention over the paged Q8_0 / FP16 K/V cache for few query rows per sequence:
// single-token decode and speculative verify spans.  Stands in for the reference's split-K decode pair
// qsa_decode_parts + qsa_decode_merge (gpu/sparse_attention_compute.hpp:41-170) with the dense selection
// 0..position and the reference's FP16-operand convention (Q8_0 -> exact integer in FP16, one rounding by the
// block scale, FP32 sums: gpu/qsa_prompt_attention.hpp:15-33, :144-150).
//
// Shape of the work on gfx950 (wave64, v_mfma_f32_16x16x32_f16):
//   * the batch's cached tokens, all K/V heads, are cut on the device into equal shares, one per workgroup (4 waves) and as
//     many workgroups as are resident at once: all start together and end together, whatever the mix of lengths.  A share
//     that crosses from one (sequence, K/V head) into the next is worked in segments, one partial result each;
//   * the waves take alternate 32-token steps, each with its own online softmax, and merge through LDS at the end of a
//     segment; a second kernel merges the segments of a sequence;
//   * a step's K and V slabs (32 contiguous rows of a page plane) are copied by coalesced, non-temporal 16-byte
//     global->LDS loads into the wave's own LDS stage, operands are read from there in MFMA layout, and the next step's
//     copy is in flight while this step is computed;
//   * operand layouts and the Q8_0 -> FP16 conversion: paged_rows.hpp.
#include "paged_rows.hpp"

#include <cstdlib>

namespace sd {
void validate_pool(Device& d, const sdx_kv_pool* pool);
void prefill_attention(Device& d, const sdx_kv_pool* pool, const int32_t* page_table, uint64_t table_stride, const int32_t* positions,
                       uint64_t max_context, const void* q, int q_f16, uint64_t seqs, uint64_t span, uint64_t heads, float scale, void* out,
                       int out_f16);
void prefill_chunk(Device& d, const sdx_kv_pool* pool, const int32_t* page_table, uint64_t table_stride, const int32_t* positions,
                   uint64_t max_context, const void* keys, const void* values, int kv_f16, const void* q, int q_f16, uint64_t seqs, uint64_t span,
                   uint64_t heads, float scale, void* out, int out_f16, void* tiles, const int32_t* valid);
uint64_t prefill_tiles_bytes(uint64_t seqs, uint64_t kv_heads, uint64_t max_context);
}
using namespace sd;
using namespace sd::paged;

namespace {

// The batch's work is counted in units of 128 tokens (one step of each of the four waves): a sequence of n tokens has
// ceil(n / 128) units per K/V head, laid out sequence by sequence and, within one, K/V head by K/V head.  Workgroup w of G
// takes the units floor(w U / G) up to floor((w + 1) U / G): G is as many workgroups as are resident at once (fewer when
// that would leave a workgroup less than share_min units).  Every wave finds the same numbers from the positions alone.
constexpr unsigned UNIT = STEP * WAVES;
struct Share { unsigned units, groups; };
__device__ __forceinline__ Share batch_share(const PagedArgs& args, int lane) {
    unsigned units = 0;
    for (unsigned s = lane; s < args.seqs; s += 64) units += unsigned(min(first_position(args.positions, s, args.max_context) + int(args.span), args.max_context) + int(UNIT) - 1) / UNIT;
    #pragma unroll
    for (int d = 32; d; d >>= 1) units += __shfl_xor(units, d);
    units = __builtin_amdgcn_readfirstlane(units * args.kv_heads);
    return Share{units, min(args.groups_max, max(1u, units / args.share_min))};
}
__device__ __forceinline__ unsigned share_begin(const Share& share, unsigned w) { return unsigned(uint64_t(w) * share.units / share.groups); }
// the workgroup that takes unit u: the w with floor(w U / G) <= u < floor((w + 1) U / G)
__device__ __forceinline__ unsigned share_owner(const Share& share, unsigned u) { return unsigned((uint64_t(u + 1) * share.groups - 1) / share.units); }

// Where unit u lies: its sequence and K/V head, how many units into them, and how many they have (a running count over 64
// sequences at a time; `before` = the units of the sequences before).
// (The lane number is taken afresh, by an instruction the compiler may not move: what is derived from it here would
// otherwise be kept in registers all through the caller's loop over the tokens.)
__device__ __forceinline__ int fresh_lane() {
    int lane;
    asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(lane));
    return lane;
}
// (Likewise the kernel's arguments, read afresh for each segment through a pointer the compiler cannot see through: fields
// that only a segment's start or end needs do not then occupy scalar registers through the loop over the tokens.)
typedef __attribute__((address_space(4))) const PagedArgs* args_ptr;
__device__ __forceinline__ PagedArgs fresh_args() {
    args_ptr at = (args_ptr)__builtin_amdgcn_kernarg_segment_ptr();
    asm volatile("" : "+s"(at));
    PagedArgs args;
    args.pages = at->pages; args.page_tokens = at->page_tokens; args.kv_heads = at->kv_heads; args.heads = at->heads; args.group = at->group;
    args.span = at->span; args.page_table = at->page_table; args.table_stride = at->table_stride; args.positions = at->positions; args.q = at->q;
    args.q_f16 = at->q_f16; args.scale_log2 = at->scale_log2; args.partial = at->partial; args.rows = at->rows; args.seqs = at->seqs;
    args.groups_max = at->groups_max; args.share_min = at->share_min; args.max_context = at->max_context; args.page_last = at->page_last;
    return args;
}
struct Segment { int seq, kvh, position, total; unsigned unit, units, before; };
__device__ __forceinline__ bool locate(const PagedArgs& args, unsigned u, Segment& seg) {
    const int lane = fresh_lane();
    unsigned before = 0;
    for (unsigned first = 0; first < args.seqs; first += 64) {
        const unsigned s = first + lane;
        const int position = s < args.seqs ? first_position(args.positions, s, args.max_context) : 0;
        const int total = s < args.seqs ? min(position + int(args.span), args.max_context) : 0;
        const unsigned units = unsigned(total + int(UNIT) - 1) / UNIT;
        unsigned upto = units * args.kv_heads;      // units of this and the earlier sequences of the 64
        #pragma unroll
        for (int d = 1; d < 64; d <<= 1) { const unsigned other = __shfl_up(upto, d); if (lane >= d) upto += other; }
        const unsigned all = __shfl(upto, 63);
        if (u < before + all) {
            const int owner = __popcll(__ballot(before + upto <= u));
            seg.units = __shfl(units, owner);
            seg.before = before + __shfl(upto - units * args.kv_heads, owner);
            const unsigned within = u - seg.before;
            seg.seq = int(first) + owner;
            seg.total = __shfl(total, owner);
            seg.position = __shfl(position, owner);
            seg.kvh = int(within / seg.units);
            seg.unit = within % seg.units;
            return true;
        }
        before += all;
    }
    return false;
}

constexpr float SLACK = 8.0f;     // how far (base-2 exponent) a row's true maximum may run ahead of its reference maximum
constexpr int stages_per_wave(int slab, int occupancy) { return occupancy <= 2 && WAVES * 2 * 2 * slab * occupancy <= 160 * 1024 ? 2 : 1; }
// s_waitcnt for the vector-memory counter alone: wait until at most N of the wave's loads are outstanding.
template<int N> __device__ __forceinline__ void wait_loads() { __builtin_amdgcn_s_waitcnt(0x0f70 | (N & 15) | ((N >> 4) << 14)); }

// A step's K and V slabs (32 contiguous rows each) are copied by fully coalesced 16-byte global->LDS loads into the wave's
// own LDS stage; operands are then read from LDS in MFMA layout while the next step's copy is in flight.  OCC = the waves per
// SIMD the variant is compiled for (its register budget).
template<int DIM, int QT, bool Q8, int OCC>
__global__ void __launch_bounds__(WAVES * 64) __attribute__((amdgpu_waves_per_eu(OCC, OCC))) paged_attention_kernel(PagedArgs given) {
    constexpr int ROW = Q8 ? DIM + DIM / 16 : 2 * DIM, BLOCKS = DIM / 32, W = DIM / 16, TILES = DIM / 16;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const Share share = batch_share(given, threadIdx.x & 63);
    if (blockIdx.x >= share.groups) return;
    extern __shared__ float lds[];
    const unsigned share_end = share_begin(share, blockIdx.x + 1);
    for (unsigned unit = share_begin(share, blockIdx.x); unit < share_end;) {
    // (a fresh lane number per segment: what a segment's start and end derive from it is then worked out there, not kept in
    // registers through every other segment's loop over the tokens)
    const int lane = fresh_lane(), li = lane & 15, g = lane >> 4;
    const PagedArgs args = fresh_args();                    // (the kernel's only argument: it lies at the segment's start)
    Segment found;
    if (!locate(args, unit, found)) return;            // (cannot happen: the units were counted from the same positions)
    const int seq = __builtin_amdgcn_readfirstlane(found.seq), kvh = __builtin_amdgcn_readfirstlane(found.kvh);
    const int total = __builtin_amdgcn_readfirstlane(found.total), position = __builtin_amdgcn_readfirstlane(found.position);
    const unsigned first_unit = __builtin_amdgcn_readfirstlane(found.unit);
    const unsigned take = min(share_end - unit, unsigned(__builtin_amdgcn_readfirstlane(found.units)) - first_unit);
    const int segment_begin = int(first_unit * UNIT), segment_end = min(total, int((first_unit + take) * UNIT));
    const table_ptr table = (table_ptr)(args.page_table + size_t(seq) * args.table_stride);
    const size_t plane_bytes = size_t(args.page_tokens) * ROW;

    // With several query tiles the kernel is bound by its vector instructions and the matrix cores have time to spare: a row's sum
    // of weights is then one more product a tile and step -- the weights against a block of ones, every row of the result the sum,
    // every one of a row's four lanes holding all of it -- instead of eight additions a tile.
    constexpr bool SUMS_BY_PRODUCT = QT >= 2 && DIM == 128;      // (at 256 columns the registers are all taken)
    floatx4 acc[QT][TILES], sums[SUMS_BY_PRODUCT ? QT : 1];
    float m[QT], l[QT];
    #pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
        m[qt] = NEG_BIG; l[qt] = 0.0f;
        if (SUMS_BY_PRODUCT) sums[qt] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
        #pragma unroll
        for (int jj = 0; jj < TILES; ++jj) acc[qt][jj] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
    }

    constexpr int SLAB = STEP * ROW;                       // one step's rows of one plane: contiguous in the page
    // Stages per wave: with few waves per SIMD one step in flight per wave does not cover the memory latency, so a wave then
    // keeps two (where the workgroups resident at once still fit the 160 KiB of LDS).
    constexpr int DEPTH = stages_per_wave(SLAB, OCC), LOADS = 2 * ((SLAB + 1023) / 1024);
    uint8_t* const stages = reinterpret_cast<uint8_t*>(lds) + wave * (DEPTH * 2 * SLAB);
    // A step's rows from the wave's stage into operand registers.  The rows past the sequence's end in its last step hold
    // whatever the page held: they are cleared first (their scores are masked, but a stray scale must not meet a zero weight).
    const auto request = [&](RowLoad<DIM, Q8>& rows, uint8_t* stage, int token0) {
        const int valid = total - token0;
        if (valid < STEP)
            #pragma unroll
            for (int part = 0; part < 2; ++part)
                for (int at = valid * ROW + 4 * lane; at < SLAB; at += 256) *reinterpret_cast<uint32_t*>(stage + part * SLAB + at) = 0u;
        load_step<DIM>(rows, stage, stage + SLAB, li, g);
    };
    // The step's two slabs copied into the stage, 1 KiB per instruction and up to four instructions a run (the slab's address is
    // the wave's: scalar registers; a lane adds 16 * lane), lanes past a slab's end switched off.
    const uint32_t lane_bytes = 16 * lane;
    const auto copy_in = [&](uint8_t* stage, int page, int in_page) {
        const uint8_t* base = args.pages + (size_t(pool_page(page, args.page_last)) * 2 * args.kv_heads + kvh) * plane_bytes + size_t(in_page) * ROW;
        const uint32_t to = __builtin_amdgcn_readfirstlane(lds_address(stage));
        constexpr int WHOLE = SLAB / 1024, REST = SLAB % 1024;
        #pragma unroll
        for (int part = 0; part < 2; ++part) {
            const uint8_t* from = base + size_t(part ? args.kv_heads : 0) * plane_bytes;
            #pragma unroll
            for (int j = 0; j < WHOLE; j += 4) {
                if (WHOLE - j >= 4) load_run_to_lds<true, 4>(from + 1024 * j, to + part * SLAB + 1024 * j, lane_bytes);
                else if (WHOLE - j == 3) load_run_to_lds<true, 3>(from + 1024 * j, to + part * SLAB + 1024 * j, lane_bytes);
                else if (WHOLE - j == 2) load_run_to_lds<true, 2>(from + 1024 * j, to + part * SLAB + 1024 * j, lane_bytes);
                else load_run_to_lds<true, 1>(from + 1024 * j, to + part * SLAB + 1024 * j, lane_bytes);
            }
            if (REST && int(lane_bytes) < REST) load_run_to_lds<true, 1>(from + 1024 * WHOLE, to + part * SLAB + 1024 * WHOLE, lane_bytes);
        }
    };

    // Where the step to copy next lies: page_index-th page of the sequence, in_page rows into it.  Its page number is fetched
    // (a scalar load) a step before its copy is issued.
    int token0 = segment_begin + STEP * wave;
    const int last_page = (total - 1) / int(args.page_tokens);
    int page_index = token0 / int(args.page_tokens), in_page = token0 % int(args.page_tokens);
    const auto advance = [&] {
        in_page += STEP * WAVES;
        while (in_page >= int(args.page_tokens)) { in_page -= int(args.page_tokens); ++page_index; }
    };
    // The first steps' copies are asked for first, then the queries: both are on their way together, and one wait for every
    // load so far stands before the loop (the compiler's own wait for the queries would otherwise sit at their first use
    // inside the loop and wait for the copies issued by then as well).
    settle_loads();
    #pragma unroll
    for (int ahead = 0; ahead < DEPTH; ++ahead) {
        if (token0 + ahead * STEP * WAVES < segment_end) copy_in(stages + ahead * (2 * SLAB), table[min(page_index, last_page)], in_page);
        advance();
    }
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

    settle_loads();
    int page_ahead = table[min(page_index, last_page)];
    for (int buffer = 0; token0 < segment_end; token0 += STEP * WAVES, buffer = DEPTH == 2 ? buffer ^ 1 : 0) {
        uint8_t* const stage = stages + buffer * (2 * SLAB);
        const bool more = token0 + DEPTH * STEP * WAVES < segment_end;      // a step to copy into this stage once it is read
        const int page_now = page_ahead, in_page_now = in_page;
        advance();
        page_ahead = table[min(page_index, last_page)];
        RowLoad<DIM, Q8> current;
        // the stage holds this step when only the step after it is still on its way
        if (DEPTH == 2 && token0 + STEP * WAVES < segment_end) wait_loads<LOADS>(); else wait_loads<0>();
        request(current, stage, token0);
        __builtin_amdgcn_s_waitcnt(0xc07f);          // lgkmcnt(0): operands are in registers, the stage is free again
        __builtin_amdgcn_sched_barrier(0);
        if (more) copy_in(stage, page_now, in_page_now);
        __builtin_amdgcn_sched_barrier(0);
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
        // Scores stay unscaled (the scale goes into the exponent's multiply-add); m is a row's reference maximum in unscaled
        // units.  It follows the true maximum only when that has grown by more than SLACK (in base-2 exponent units): weights
        // then stay below 2^SLACK, far inside FP16 and FP32 range, and the accumulators are rescaled a few times per row
        // instead of at every new maximum.  The quotient acc/sum does not depend on the reference.
        if (token0 + STEP - 1 > position) {          // wave-uniform: some token of the step is past the first row's position
            #pragma unroll
            for (int qt = 0; qt < QT; ++qt)
                #pragma unroll
                for (int t = 0; t < 2; ++t)
                    #pragma unroll
                    for (int r = 0; r < 4; ++r)
                        if (token0 + 16 * t + 4 * g + r > limit[qt]) s[qt][t][r] = -INFINITY;
        }
        // (whether a row has outgrown its reference is seen by the lane that holds its largest score: the row's four lanes
        // compare their own eight scores, and only a step that moves a reference reduces the maxima across them)
        float top[QT];
        bool grown = false;
        #pragma unroll
        for (int qt = 0; qt < QT; ++qt) {
            top[qt] = fmaxf(fmaxf(fmaxf(s[qt][0][0], s[qt][0][1]), fmaxf(s[qt][0][2], s[qt][0][3])),
                            fmaxf(fmaxf(s[qt][1][0], s[qt][1][1]), fmaxf(s[qt][1][2], s[qt][1][3])));
            grown |= (top[qt] - m[qt]) * args.scale_log2 > SLACK;
        }
        if (__any(grown)) {
            #pragma unroll
            for (int qt = 0; qt < QT; ++qt) {
                top[qt] = row_max(top[qt]);
                const float m_new = fmaxf(m[qt], top[qt]);
                const float alpha = __builtin_amdgcn_exp2f((m[qt] - m_new) * args.scale_log2);
                m[qt] = m_new;
                l[qt] *= alpha;
                if (SUMS_BY_PRODUCT) sums[qt] *= alpha;
                #pragma unroll
                for (int jj = 0; jj < TILES; ++jj) acc[qt][jj] *= alpha;
            }
        }
        half8 pb[QT];
        #pragma unroll
        for (int qt = 0; qt < QT; ++qt) {
            const float offset = -m[qt] * args.scale_log2;
            float sum = 0.0f;
            half8 p;
            #pragma unroll
            for (int t = 0; t < 2; ++t)
                #pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float w = __builtin_amdgcn_exp2f(fmaf(s[qt][t][r], args.scale_log2, offset));
                    if (!SUMS_BY_PRODUCT) sum += w;
                    p[4 * t + r] = (_Float16)w;
                }
            pb[qt] = p;
            if (SUMS_BY_PRODUCT) {
                const _Float16 one = (_Float16)1.0f;
                sums[qt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(half8{one, one, one, one, one, one, one, one}, p, sums[qt], 0, 0, 0);
            } else l[qt] += sum;
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
    }

    // Merge the waves, two by two, through LDS: waves 2 and 3 hand their maxima, sums and unnormalised outputs to waves 0 and
    // 1, then wave 1 hands its own to wave 0.  Corresponding lanes hold corresponding elements, so a value goes from lane to
    // lane ([register][lane] in LDS, no bank conflicts), and the area is two waves' registers: it fits the stages it overlays.
    if (SUMS_BY_PRODUCT)
        #pragma unroll
        for (int qt = 0; qt < QT; ++qt) l[qt] = sums[qt][0];
    __syncthreads();    // the stages are free
    constexpr int STRIDE = DIM + 2, HELD = QT * (TILES * 4 + 2);
    const int lane_after = fresh_lane(), li_after = lane_after & 15, g_after = lane_after >> 4;   // (again: nothing of this is worked out before the loop)
    const auto hand_over = [&](int slot) {
        float* to = lds + size_t(slot) * HELD * 64 + lane_after;
        #pragma unroll
        for (int qt = 0; qt < QT; ++qt) {
            float* mine = to + qt * (TILES * 4 + 2) * 64;
            mine[0] = m[qt]; mine[64] = l[qt];
            #pragma unroll
            for (int jj = 0; jj < TILES; ++jj)
                #pragma unroll
                for (int r = 0; r < 4; ++r) mine[(2 + 4 * jj + r) * 64] = acc[qt][jj][r];
        }
    };
    const auto take_in = [&](int slot) {
        const float* from = lds + size_t(slot) * HELD * 64 + lane_after;
        #pragma unroll
        for (int qt = 0; qt < QT; ++qt) {
            const float* theirs = from + qt * (TILES * 4 + 2) * 64;
            const float m_other = theirs[0], m_new = fmaxf(m[qt], m_other);
            const float keep = __builtin_amdgcn_exp2f((m[qt] - m_new) * args.scale_log2), add = __builtin_amdgcn_exp2f((m_other - m_new) * args.scale_log2);
            m[qt] = m_new;
            l[qt] = l[qt] * keep + theirs[64] * add;
            #pragma unroll
            for (int jj = 0; jj < TILES; ++jj)
                #pragma unroll
                for (int r = 0; r < 4; ++r) acc[qt][jj][r] = acc[qt][jj][r] * keep + theirs[(2 + 4 * jj + r) * 64] * add;
        }
    };
    if (wave >= 2) hand_over(wave - 2);
    __syncthreads();
    if (wave < 2) take_in(wave);
    __syncthreads();
    if (wave == 1) hand_over(0);
    __syncthreads();
    if (wave == 0) {
        take_in(0);
        // a partial result per (workgroup, sequence and K/V head) met: both only grow along the units, so their sum numbers
        // them.  Row layout: DIM outputs, the maximum in exponent units, the sum; a lane holds 4 runs of 8 columns of its row.
        float* out = args.partial + (size_t(blockIdx.x) + size_t(seq) * args.kv_heads + kvh) * args.rows * STRIDE;
        #pragma unroll
        for (int qt = 0; qt < QT; ++qt) {
            const float sum = SUMS_BY_PRODUCT ? l[qt] : row_sum(l[qt]);       // (a sum formed by products is whole in each of the row's lanes)
            const int row = qt * 16 + li_after;
            if (row < int(args.rows)) {
                float* to = out + size_t(row) * STRIDE;
                if (g_after == 0) *reinterpret_cast<float2*>(to + DIM) = make_float2(m[qt] * args.scale_log2, sum);
                #pragma unroll
                for (int r = 0; r < 4; ++r)
                    #pragma unroll
                    for (int jj = 0; jj < TILES; jj += 2)
                        *reinterpret_cast<float2*>(to + W * (4 * g_after + r) + jj) = make_float2(acc[qt][jj][r], acc[qt][jj + 1][r]);
            }
        }
    }
    unit += take;
    if (unit < share_end) __syncthreads();                  // the next segment's stages overlay what wave 0 has just read
    }
}

// A wave per (sequence, span row, head): the segments' partial results merged and normalised (the algebra of the
// reference's qsa_decode_merge, gpu/sparse_attention_compute.hpp:139-170).  A lane takes two columns of every segment and
// every lane reads the segments' maxima and sums for itself (one address a wave: a broadcast), so nothing is exchanged
// between lanes and nothing waits on LDS or a barrier: the segments are asked for sixteen at a time, all loads in flight at
// once, under a running maximum.  Four rows a workgroup.
template<int DIM, bool F16_OUT>
__global__ void __launch_bounds__(256) paged_merge_kernel(PagedArgs args, void* out, unsigned outputs) {
    constexpr int STRIDE = DIM + 2, PER = DIM / 128, AT_ONCE = 16;
    static_assert(DIM % 128 == 0, "a lane takes two columns of every run of 128");
    const unsigned item = blockIdx.x * 4 + threadIdx.x / 64;
    if (item >= outputs) return;
    const unsigned head = item % args.heads, span_row = item / args.heads % args.span, seq = item / args.heads / args.span;
    const unsigned kvh = head / args.group, row = span_row * args.group + head % args.group;
    // the workgroups whose shares met this sequence and K/V head
    const int lane = int(threadIdx.x & 63);
    const Share share = batch_share(args, lane);
    unsigned before = 0;
    for (unsigned s = lane; s < seq; s += 64) before += unsigned(min(first_position(args.positions, s, args.max_context) + int(args.span), args.max_context) + int(UNIT) - 1) / UNIT;
    #pragma unroll
    for (int d = 32; d; d >>= 1) before += __shfl_xor(before, d);
    const unsigned units = unsigned(min(first_position(args.positions, seq, args.max_context) + int(args.span), args.max_context) + int(UNIT) - 1) / UNIT;
    const unsigned begin = (before * args.kv_heads + kvh * units), owner = share_owner(share, begin);
    const unsigned used = share_owner(share, begin + units - 1) - owner + 1;
    const float* base = args.partial + (size_t(owner) + size_t(seq) * args.kv_heads + kvh) * args.rows * STRIDE + size_t(row) * STRIDE;
    const size_t step = size_t(args.rows) * STRIDE;
    float top = NEG_BIG, sum = 0.0f;
    float2 value[PER];
    #pragma unroll
    for (int i = 0; i < PER; ++i) value[i] = make_float2(0.0f, 0.0f);
    for (unsigned first = 0; first < used; first += AT_ONCE) {
        float2 stats[AT_ONCE], v[AT_ONCE][PER];
        #pragma unroll
        for (int c = 0; c < AT_ONCE; ++c) {
            const float* from = base + size_t(min(first + c, used - 1)) * step;
            stats[c] = *reinterpret_cast<const float2*>(from + DIM);
            #pragma unroll
            for (int i = 0; i < PER; ++i) v[c][i] = *reinterpret_cast<const float2*>(from + 128 * i + 2 * lane);
        }
        float higher = top;
        #pragma unroll
        for (int c = 0; c < AT_ONCE; ++c) if (first + c < used) higher = fmaxf(higher, stats[c].x);
        const float keep = __builtin_amdgcn_exp2f(top - higher);
        top = higher;
        sum *= keep;
        #pragma unroll
        for (int i = 0; i < PER; ++i) { value[i].x *= keep; value[i].y *= keep; }
        #pragma unroll
        for (int c = 0; c < AT_ONCE; ++c) {
            const float w = first + c < used ? __builtin_amdgcn_exp2f(stats[c].x - top) : 0.0f;
            sum += stats[c].y * w;
            #pragma unroll
            for (int i = 0; i < PER; ++i) { value[i].x += v[c][i].x * w; value[i].y += v[c][i].y * w; }
        }
    }
    #pragma unroll
    for (int i = 0; i < PER; ++i) {
        const float2 result = make_float2(value[i].x / sum, value[i].y / sum);
        const size_t at = size_t(item) * DIM + 128 * i + 2 * lane;
        if (F16_OUT) *reinterpret_cast<__half2*>(static_cast<__half*>(out) + at) = __floats2half2_rn(result.x, result.y);
        else *reinterpret_cast<float2*>(static_cast<float*>(out) + at) = result;
    }
}

// Tuning switch read once from the environment, as the reference reads its hot-path switches (STRAYDOG_QSA_MMA,
// gpu/sparse_attention_compute.hpp:594): STRAYDOG_DECODE_GROUPS = the most workgroups a batch is shared among (0: as many as
// are resident at once).
unsigned tuned_groups() {
    static const unsigned value = [] {
        const char* text = std::getenv("STRAYDOG_DECODE_GROUPS");
        return text ? unsigned(std::strtoul(text, nullptr, 10)) : 0u;
    }();
    return value;
}

// A share is at least 256 tokens; the host knows only max_context, which bounds the units a batch can have and so the
// workgroups worth launching.
constexpr unsigned smallest_share = 2;
uint64_t most_groups(uint64_t seqs, uint64_t kv_heads, uint64_t max_context) {
    return seqs * kv_heads * ((max_context + smallest_share * UNIT - 1) / (smallest_share * UNIT));
}

template<int DIM, int QT, bool Q8, int OCC>
void launch(Device& d, const PagedArgs& args, dim3 grid) {
    constexpr int slab = STEP * (Q8 ? DIM + DIM / 16 : 2 * DIM);
    const size_t shared = std::max(size_t(2) * QT * (DIM / 16 * 4 + 2) * 64 * 4, size_t(WAVES) * stages_per_wave(slab, OCC) * 2 * slab);
    if (shared > 160 * 1024) throw std::runtime_error("Straydog paged attention: too many query rows per K/V head for the decode kernel");
    if (shared > 64 * 1024) raise_shared_limit(d, reinterpret_cast<const void*>(&paged_attention_kernel<DIM, QT, Q8, OCC>), shared);
    timed_launch(d, &paged_attention_kernel<DIM, QT, Q8, OCC>, grid, dim3(WAVES * 64), shared, args);
}

// The variants that exist: (columns, query tiles, format) -> waves per SIMD the kernel is compiled for.  One query tile is
// the decode shape (4 waves/SIMD at 128 columns of Q8_0); more tiles hold more accumulators.
constexpr int variant_occupancy(int dim, bool q8, unsigned query_tiles) {
    const bool small = dim == 128;
    return query_tiles == 1 ? (small && q8 ? 4 : small ? 2 : 1) : query_tiles == 2 ? (small ? 2 : 1) : query_tiles == 3 ? (small && q8 ? 2 : 1) : 1;
}
template<int DIM, bool Q8>
void launch_tiles(Device& d, const PagedArgs& args, unsigned query_tiles, dim3 grid) {
    constexpr bool small = DIM == 128;
    switch (query_tiles) {
        case 1: launch<DIM, 1, Q8, variant_occupancy(DIM, Q8, 1)>(d, args, grid); break;
        case 2: launch<DIM, 2, Q8, variant_occupancy(DIM, Q8, 2)>(d, args, grid); break;
        case 3: if constexpr (small) { launch<DIM, 3, Q8, variant_occupancy(DIM, Q8, 3)>(d, args, grid); break; }
        case 4: if constexpr (small) { launch<DIM, 4, Q8, variant_occupancy(DIM, Q8, 4)>(d, args, grid); break; }
        default: throw std::runtime_error("Straydog paged attention: too many query rows per K/V head for the decode kernel");
    }
}
// Workgroups resident at once: as many per compute unit as the variant's waves per SIMD and its LDS allow.
unsigned resident_slots(const Device& d, unsigned dim, bool q8, unsigned query_tiles) {
    const int occupancy = variant_occupancy(int(dim), q8, query_tiles), slab = STEP * int(q8 ? dim + dim / 16 : 2 * dim);
    const size_t shared = std::max(size_t(2) * query_tiles * (dim / 16 * 4 + 2) * 64 * 4, size_t(WAVES) * stages_per_wave(slab, occupancy) * 2 * slab);
    return d.compute_units * unsigned(std::max<size_t>(1, std::min<size_t>(size_t(occupancy), (160 * 1024) / shared)));
}


// The partial results of the entry point that allocates nothing: device memory of the library itself, one copy per GPU,
// held until the process ends.
constexpr size_t static_scratch_bytes = size_t(16) << 20;
static __device__ __align__(256) float scratch[static_scratch_bytes / 4];

// What both entry points do once their partial-result area is known.  `timed`: the main kernel may go through the extended
// launch when the handle is being profiled (that creates events, which the entry point that allocates nothing must not).
void paged_attention(Device& value, const sdx_kv_pool* pool, const int32_t* page_table, uint64_t table_stride, const int32_t* positions,
                     uint64_t max_context, const void* q, int q_f16, uint64_t seqs, uint64_t span, uint64_t heads, float scale, void* out,
                     int out_f16, float* partial, uint64_t partial_bytes, bool own_partial) {
    validate_pool(value, pool);
    if (!(scale > 0.0f) || !seqs || seqs > 65535 || !span || !heads || heads % pool->kv_heads || !max_context || max_context > (uint64_t(1) << 30) ||
        !table_stride || max_context > table_stride * pool->page_tokens)
        throw std::runtime_error("invalid Straydog paged attention shape");
    const uint64_t group = heads / pool->kv_heads, rows = span * group;
    const unsigned query_tiles = unsigned((rows + 15) / 16);
    op_span(value, page_table, checked_floats({seqs, table_stride}), "a page table");
    op_span(value, positions, checked_floats({seqs}), "query positions");
    op_span(value, q, checked_product({seqs, span, heads, pool->dim, q_f16 ? 2u : 4u}), "attention queries");
    op_span(value, out, checked_product({seqs, span, heads, pool->dim, out_f16 ? 2u : 4u}), "an attention output");
    if (query_tiles > (pool->dim == 128 ? 4u : 2u)) {
        if (own_partial) throw std::runtime_error("Straydog paged attention: too many query rows per K/V head for the entry point that allocates nothing");
        // many rows per K/V head (a prefill chunk): every workgroup walks the keys once for a run of rows, nothing to merge
        prefill_attention(value, pool, page_table, table_stride, positions, max_context, q, q_f16, seqs, span, heads, scale, out, out_f16);
        SD_CHECK(hipGetLastError());
        return;
    }
    PagedArgs args{};
    args.pages = static_cast<const uint8_t*>(pool->pages);
    args.page_tokens = pool->page_tokens; args.kv_heads = pool->kv_heads; args.heads = unsigned(heads); args.group = unsigned(group);
    args.span = unsigned(span); args.page_table = page_table; args.table_stride = size_t(table_stride); args.positions = positions;
    args.q = q; args.q_f16 = q_f16; args.scale_log2 = scale * 1.44269504088896341f;
    args.rows = unsigned(rows); args.seqs = unsigned(seqs);
    args.max_context = int(max_context);
    args.page_last = unsigned(std::min<uint64_t>(pool->page_count - 1, 0x7fffffffu));
    const uint64_t items = checked_product({seqs, pool->kv_heads});
    if (checked_product({items, (max_context + UNIT - 1) / UNIT}) > 0x7fffffffu) throw std::runtime_error("invalid Straydog paged attention shape");
    const unsigned slots = resident_slots(value, pool->dim, pool->row_bytes != 2 * pool->dim, query_tiles);
    args.groups_max = unsigned(std::min<uint64_t>(tuned_groups() ? tuned_groups() : slots, most_groups(seqs, pool->kv_heads, max_context)));
    args.share_min = smallest_share;
    const size_t need = checked_floats({uint64_t(args.groups_max) + items, rows, uint64_t(pool->dim) + 2});
    if (own_partial) {
        if (need > partial_bytes)
            throw std::runtime_error("Straydog paged attention: this batch needs " + std::to_string(need) + " bytes of partial results, the entry point that allocates nothing holds " +
                                     std::to_string(partial_bytes));
    } else {
        if (!partial || partial_bytes < need) throw std::runtime_error("Straydog paged attention scratch too small");
        op_span(value, partial, need, "attention scratch");
    }
    args.partial = partial;
    const bool profiled = value.profile;
    if (own_partial) value.profile = false;
    struct Restore { Device& d; bool profile; ~Restore() { d.profile = profile; } } restore{value, profiled};
    const dim3 grid(args.groups_max);
    const bool q8 = pool->row_bytes != 2 * pool->dim;
    if (pool->dim == 128) { if (q8) launch_tiles<128, true>(value, args, query_tiles, grid); else launch_tiles<128, false>(value, args, query_tiles, grid); }
    else { if (q8) launch_tiles<256, true>(value, args, query_tiles, grid); else launch_tiles<256, false>(value, args, query_tiles, grid); }
    SD_CHECK(hipGetLastError());
    const unsigned outputs = unsigned(checked_product({seqs, span, heads})), merge_groups = (outputs + 3) / 4;
    if (pool->dim == 128) {
        if (out_f16) paged_merge_kernel<128, true><<<merge_groups, 256, 0, value.stream>>>(args, out, outputs);
        else paged_merge_kernel<128, false><<<merge_groups, 256, 0, value.stream>>>(args, out, outputs);
    } else {
        if (out_f16) paged_merge_kernel<256, true><<<merge_groups, 256, 0, value.stream>>>(args, out, outputs);
        else paged_merge_kernel<256, false><<<merge_groups, 256, 0, value.stream>>>(args, out, outputs);
    }
}


}  // namespace

namespace sd {
// Called by sd_create with the handle's device current: the address this device holds the library's partial-result area at
// (each GPU has its own copy of the array at its own address; the array's name is not a device address in host code).
void paged_attention_setup(Device& d) {
    float* address = nullptr;
    SD_CHECK(hipGetSymbolAddress(reinterpret_cast<void**>(&address), HIP_SYMBOL(scratch)));
    d.paged_static = address;
}
}  // namespace sd

extern "C" {

uint64_t sdx_paged_attention_scratch(uint64_t seqs, uint64_t span, uint64_t heads, uint64_t dim, uint64_t max_context) {
    // a partial result per workgroup and one more per (sequence, K/V head); at most a workgroup per 256 tokens of a sequence
    const uint64_t shares = (max_context + smallest_share * UNIT - 1) / (smallest_share * UNIT);
    return seqs * span * heads * (shares + 1) * (dim + 2) * 4;
}

int sdx_paged_attention(void* handle, const sdx_kv_pool* pool, const int32_t* page_table, uint64_t table_stride,
                        const int32_t* positions, uint64_t max_context, const void* q, int q_f16, uint64_t seqs, uint64_t span,
                        uint64_t heads, float scale, void* out, int out_f16, void* scratch, uint64_t scratch_bytes) {
    SD_OP_BEGIN
    paged_attention(value, pool, page_table, table_stride, positions, max_context, q, q_f16, seqs, span, heads, scale, out, out_f16,
                    static_cast<float*>(scratch), scratch_bytes, false);
    SD_OP_END
}

uint64_t sdx_prefill_tiles_bytes(uint64_t seqs, uint64_t kv_heads, uint64_t dim, uint64_t max_context) {
    try { return dim == 128 && seqs && kv_heads && max_context ? prefill_tiles_bytes(seqs, kv_heads, max_context) : 0; }
    catch (const std::exception&) { return 0; }
}

int sdx_prefill_wave_rows(void* handle, uint64_t rows) {
    SD_OP_BEGIN
    if (rows != 32 && rows != 64) throw std::runtime_error("a wave of the Straydog prompt kernel holds 32 or 64 rows");
    value.prefill_wave_rows = uint32_t(rows);
    SD_OP_END
}

int sdx_prefill_chunk(void* handle, const sdx_kv_pool* pool, const int32_t* page_table, uint64_t table_stride, const int32_t* positions,
                      uint64_t max_context, const void* keys, const void* values, int kv_f16, const void* q, int q_f16, uint64_t seqs, uint64_t span,
                      uint64_t heads, float scale, void* out, int out_f16, void* tiles, uint64_t tiles_bytes, const int32_t* valid) {
    SD_OP_BEGIN
    validate_pool(value, pool);
    if (pool->dim != 128) throw std::runtime_error("Straydog prefill chunk: rows of 128 columns only");
    if (!(scale > 0.0f) || !seqs || seqs > 65535 || !span || !heads || heads % pool->kv_heads || !max_context || max_context > (uint64_t(1) << 30) ||
        !table_stride || max_context > table_stride * pool->page_tokens || !keys != !values)
        throw std::runtime_error("invalid Straydog prefill chunk shape");
    op_span(value, page_table, checked_floats({seqs, table_stride}), "a page table");
    op_span(value, positions, checked_floats({seqs}), "query positions");
    if (valid) op_span(value, valid, checked_floats({seqs}), "valid tile positions");
    if (keys) {
        op_span(value, keys, checked_product({seqs, span, pool->kv_heads, pool->dim, kv_f16 ? 2u : 4u}), "new keys");
        op_span(value, values, checked_product({seqs, span, pool->kv_heads, pool->dim, kv_f16 ? 2u : 4u}), "new values");
    }
    op_span(value, q, checked_product({seqs, span, heads, pool->dim, q_f16 ? 2u : 4u}), "attention queries");
    op_span(value, out, checked_product({seqs, span, heads, pool->dim, out_f16 ? 2u : 4u}), "an attention output");
    const uint64_t need = prefill_tiles_bytes(seqs, pool->kv_heads, max_context);
    if (!tiles || tiles_bytes < need) throw std::runtime_error("Straydog prefill chunk: the tile buffer is too small");
    if (uintptr_t(tiles) % 16) throw std::runtime_error("Straydog prefill chunk: the tile buffer must lie on a 16-byte boundary");
    op_span(value, tiles, size_t(need), "prefill tiles");
    prefill_chunk(value, pool, page_table, table_stride, positions, max_context, keys, values, kv_f16, q, q_f16, seqs, span, heads, scale, out, out_f16,
                  tiles, valid);
    SD_OP_END
}

uint64_t sdx_paged_attention_static_bytes(void) { return static_scratch_bytes; }

int sdx_paged_attention_static(void* handle, const sdx_kv_pool* pool, const int32_t* page_table, uint64_t table_stride,
                               const int32_t* positions, uint64_t max_context, const void* q, int q_f16, uint64_t seqs, uint64_t span,
                               uint64_t heads, float scale, void* out, int out_f16) {
    SD_OP_BEGIN
    if (!value.paged_static) throw std::runtime_error("Straydog paged attention: the library's own partial-result area was not found on this device");
    paged_attention(value, pool, page_table, table_stride, positions, max_context, q, q_f16, seqs, span, heads, scale, out, out_f16,
                    value.paged_static, static_scratch_bytes, true);
    SD_OP_END
}

}  // extern "C"
