// Causal grouped-query attention over the paged Q8_0 / FP16 K/V cache for many query rows per sequence: chunked
// prefill (a span of new tokens attends the cache, which already holds the span's own K/V rows, and is causal within
// the span).  Stands in for the reference's per-token prompt attention qsa_prompt_attention
// (gpu/qsa_prompt_attention.hpp:47-213: S^T = K . Q^T and O^T += V^T . P^T on matrix cores, Q8_0 -> FP16 operands,
// base-2 online softmax in FP32) and its multi-token qsa_flash (gpu/sparse_attention_compute.hpp:176-279) with the
// dense selection 0..position.
//
// Shape of the work on gfx950 (wave64, v_mfma_f32_16x16x32_f16).  Query rows are ordered (span row, head in group), so a
// run of consecutive rows is a run of consecutive tokens with all their grouped heads and every K/V row read serves all of
// them.  A workgroup of 8 waves (two per SIMD) walks the keys 64 at a time, the next steps' operands travelling by 16-byte
// global->LDS loads into a ring of stages while this one is computed; one barrier per 64 keys; steps that lie wholly after
// a wave's rows are skipped.  Two kernels:
//   * prefill_dense_kernel (128 columns, the headline shape): a pass before it unpacks the cached rows once per call into
//     FP16 tiles in a workspace, laid out as LDS wants them, so the kernel's loop converts nothing: it copies a tile, reads
//     operands without bank conflicts, multiplies and exponentiates, every wave's stream pipelined by hand.  A workgroup
//     owns two runs of 128 rows, one from the end of the span and its mirror image from the start, so every workgroup does
//     about the same work, and writes its outputs normalised, with no merge (details at the kernels);
//   * prefill_attention_kernel (256 columns): 4 x QT x 16 rows per workgroup; every wave builds its own operands from the
//     raw rows in the stage (paged_rows.hpp); a quarter of the rows belongs to a pair of waves, one taking the first 32
//     keys of every step and one the last 32, each with its own online softmax, merged through LDS at the end; the
//     workgroups with the longest walks are dispatched first.
#include "paged_rows.hpp"
#include "kv_codec.hpp"

#include <cstdlib>
#include <type_traits>

using namespace sd;
using namespace sd::paged;

namespace {

constexpr float SLACK = 8.0f;     // how far (base-2 exponent) a row's true maximum may run ahead of its reference maximum
// The ring of K/V stages: the copies of STAGES - 1 steps are in flight or landed; as many as fit beside nothing else, at most 4.
constexpr int stages_for(int stage_bytes) { return 150 * 1024 / stage_bytes < 4 ? 150 * 1024 / stage_bytes : 4; }
constexpr int GROUPS = 4, HALVES = 2, TEAM = GROUPS * HALVES;   // row quarters x key halves = waves of a workgroup
constexpr int WALK = HALVES * STEP;                            // keys per step of the workgroup

// s_waitcnt for the vector-memory counter alone: wait until at most N of the wave's loads are outstanding.
template<int N> __device__ __forceinline__ void wait_loads() { __builtin_amdgcn_s_waitcnt(0x0f70 | (N & 15) | ((N >> 4) << 14)); }

struct PrefillArgs {
    const uint8_t* pages;
    unsigned page_tokens, kv_heads, heads, group, span;
    const int32_t* page_table;
    size_t table_stride;
    const int32_t* positions;
    const void* q;
    int q_f16;
    float scale_log2;      // softmax scale * log2(e): scores live in the base-2 domain
    unsigned rows;         // span * group: query rows per K/V head
    int max_context;       // positions[s] + span is clipped to this
    unsigned page_last;    // the pool's last page (table entries outside the pool are taken as the nearest page of it)
    void* out;
    int out_f16;
    // The union walk (UNION kernels only): each tile of query rows walks the list of positions that some token of the tile
    // selected, union_pos[tile][entry] in ascending order, union_count[tile] of them; bit (token - the tile's first token) of
    // union_mask[tile][entry] says whether that token selected the entry.  One sequence, whose first row is at `base`; a null
    // page table means one page holds the context.  gate (or null): the output is multiplied by sigmoid(gate[token][head][column]).
    const int32_t* union_pos;
    const uint32_t* union_mask;
    const uint32_t* union_count;
    unsigned union_cap;
    int base;
    const float* gate;
    size_t gate_stride, gate_row_stride;
};

template<int DIM, int QT, bool Q8, int OCC, bool UNION = false>
__global__ void __launch_bounds__(TEAM * 64) __attribute__((amdgpu_waves_per_eu(OCC, OCC))) prefill_attention_kernel(PrefillArgs args) {
    constexpr int ROW = Q8 ? DIM + DIM / 16 : 2 * DIM, BLOCKS = DIM / 32, W = DIM / 16, TILES = DIM / 16;
    constexpr int SLAB = WALK * ROW, UNITS = (SLAB + 1023) / 1024;     // a slab is copied 1 KiB (one instruction of a wave) at a time
    constexpr int WAVE_ROWS = QT * 16, GROUP_ROWS = GROUPS * WAVE_ROWS, STAGES = stages_for(2 * SLAB);
    static_assert(STAGES >= 2, "a step is copied while the one before is computed");
    const int tile = int(gridDim.x) - 1 - int(blockIdx.x), kvh = blockIdx.y, seq = blockIdx.z;   // later rows walk further: first
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), li = lane & 15, g = lane >> 4;
    const int position = UNION ? args.base : first_position(args.positions, unsigned(seq), args.max_context);
    // rows of the sequence the cache holds; of a union walk: the entries of the tile's list, which `keys` then counts
    const int cached = UNION ? int(args.union_count[tile]) : min(position + int(args.span), args.max_context);
    const int quarter = wave % GROUPS, half = wave / GROUPS;                      // waves w and w + 4 share a SIMD and the rows
    const int row0 = tile * GROUP_ROWS + quarter * WAVE_ROWS;                     // the wave's first query row
    const int group_last = min(int(args.rows), (tile + 1) * GROUP_ROWS) - 1;
    const int keys = UNION ? cached : min(position + group_last / int(args.group) + 1, cached);    // the workgroup walks keys 0..keys-1
    const bool idle = row0 >= int(args.rows);                                     // a wave past the last row only helps copying
    const int wave_first = UNION ? -1 : position + row0 / int(args.group);        // the smallest and largest position of
    const int wave_last = UNION ? 0x7fffffff : position + (min(int(args.rows), row0 + WAVE_ROWS) - 1) / int(args.group);   // the wave's rows
    const int tile_token = tile * GROUP_ROWS / int(args.group);                  // (union walk) the first token with a row in the tile
    const int32_t* const listed = UNION ? args.union_pos + size_t(tile) * args.union_cap : nullptr;
    const uint32_t* const marks = UNION ? args.union_mask + size_t(tile) * args.union_cap : nullptr;
    const table_ptr table = (table_ptr)(args.page_table + size_t(seq) * args.table_stride);
    const size_t plane_bytes = size_t(args.page_tokens) * ROW;
    extern __shared__ uint8_t stages[];                                           // [STAGES][K slab | V slab]
    constexpr int MOST = (2 * UNITS + TEAM - 1) / TEAM, LEAST = 2 * UNITS / TEAM;   // copy instructions a wave issues per step
    const bool most = wave < 2 * UNITS - LEAST * TEAM;

    // The step's two slabs into a stage: 2 * UNITS pieces of 1 KiB, every fourth one by this wave.
    // (Pages of fewer tokens than a step: the step's rows lie in two pages, and every lane looks up the page of its own
    // 16 bytes; rows past the cached ones are the last cached row again, and never read.)
    const bool split_pages = UNION || args.page_tokens % WALK != 0;
    // (union walk) where the rows of the wave's pieces of one step lie, in 16-byte units from the pool's start (K plane of K/V
    // head 0): read from the list a step before the pieces themselves are asked for, so that the wait for them does not also
    // wait for the copies in flight.  Entries past the list's last are the last again (masked).
    uint32_t held[MOST] = {};
    const auto look_up = [&](int token0, uint32_t (&places)[MOST]) {
        #pragma unroll
        for (int k = 0; k < MOST; ++k) {
            const int unit = wave + TEAM * k, part = unit >= UNITS ? 1 : 0, j = unit - part * UNITS, at = 16 * lane + 1024 * j;
            places[k] = unit < 2 * UNITS && at < SLAB ? uint32_t(listed[min(token0 + at / ROW, cached - 1)]) : 0u;
        }
    };
    const auto copy_in = [&](int buffer, int token0, const uint32_t (&places)[MOST] = {}) {
        uint8_t* stage = stages + buffer * (2 * SLAB);
        if (UNION) {
            #pragma unroll
            for (int k = 0; k < MOST; ++k) {
                const int unit = wave + TEAM * k, part = unit >= UNITS ? 1 : 0, j = unit - part * UNITS, at = 16 * lane + 1024 * j;
                if (unit < 2 * UNITS && at < SLAB) {
                    const uint8_t* from = args.pages + size_t(places[k]) * 16 + (size_t(part ? args.kv_heads : 0) + kvh) * plane_bytes + at % ROW;
                    __builtin_amdgcn_global_load_lds((global_ptr)from, (lds_ptr)(stage + part * SLAB + 1024 * j), 16, 0, 0);
                }
            }
            return;
        }
        if (split_pages) {
            #pragma unroll
            for (int k = 0; k < MOST; ++k) {
                const int unit = wave + TEAM * k, part = unit >= UNITS ? 1 : 0, j = unit - part * UNITS, at = 16 * lane + 1024 * j;
                if (unit < 2 * UNITS && at < SLAB) {
                    const int token = min(token0 + at / ROW, cached - 1);
                    const int page = pool_page(args.page_table[size_t(seq) * args.table_stride + token / int(args.page_tokens)], args.page_last);
                    const uint8_t* from = args.pages + (size_t(page) * 2 * args.kv_heads + (part ? args.kv_heads : 0) + kvh) * plane_bytes +
                                          size_t(token % int(args.page_tokens)) * ROW + at % ROW;
                    __builtin_amdgcn_global_load_lds((global_ptr)from, (lds_ptr)(stage + part * SLAB + 1024 * j), 16, 0, 0);
                }
            }
            return;
        }
        const int page = pool_page(table[token0 / int(args.page_tokens)], args.page_last);
        const uint8_t* base = args.pages + (size_t(page) * 2 * args.kv_heads + kvh) * plane_bytes + size_t(token0 % int(args.page_tokens)) * ROW + 16 * lane;
        #pragma unroll
        for (int k = 0; k < MOST; ++k) {
            const int unit = wave + TEAM * k, part = unit >= UNITS ? 1 : 0, j = unit - part * UNITS;
            if (unit < 2 * UNITS && 16 * lane + 1024 * j < SLAB)
                __builtin_amdgcn_global_load_lds((global_ptr)(base + size_t(part ? args.kv_heads : 0) * plane_bytes + 1024 * j),
                                                 (lds_ptr)(stage + part * SLAB + 1024 * j), 16, 0, 0);
        }
    };
    // Steps past the last one are copied again from the last one's rows (and never read), so that the count of loads in flight
    // is the same at every step.
    const int last_step = (keys - 1) / WALK * WALK;
    #pragma unroll
    for (int ahead = 0; ahead < STAGES - 1; ++ahead) {
        if (UNION) look_up(min(ahead * WALK, last_step), held);
        copy_in(ahead, min(ahead * WALK, last_step), held);
    }
    if (UNION) look_up(min((STAGES - 1) * WALK, last_step), held);

    // Query rows: row = span_row * group + head_in_group; a lane holds row row0 + qt*16 + li as B operands.  A row past the
    // last real one holds zeros and is never stored.
    half8 qf[QT][BLOCKS];
    int limit[QT];
    #pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
        const int row = row0 + qt * 16 + li;
        const bool real = row < int(args.rows);
        const int span_row = real ? row / int(args.group) : 0, head = kvh * int(args.group) + (real ? row % int(args.group) : 0);
        // (union walk: the bit of the row's token in an entry's mask; a padding row has none)
        limit[qt] = UNION ? (real ? span_row - tile_token : 31) : real ? position + span_row : 0x7fffffff;
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

    for (int walk0 = 0, buffer = 0; walk0 < keys; walk0 += WALK, buffer = buffer + 1 == STAGES ? 0 : buffer + 1) {
        // this wave's pieces of the step have landed when only the later steps' are outstanding
        // (union walk: between two steps' copies lie the look-ups of the step after them, as many loads again)
        constexpr int BETWEEN = UNION ? 2 : 1;
        if (most) wait_loads<BETWEEN * MOST * (STAGES - 2)>(); else wait_loads<BETWEEN * LEAST * (STAGES - 2)>();
        __syncthreads();                             // ... and everybody's; the stage of the step before is no longer being read
        if (UNION) {
            // the copies of the step three ahead use the places looked up a step ago; the next step's are looked up first, so
            // that waiting for them later leaves these copies in flight
            uint32_t next[MOST];
            look_up(min(walk0 + STAGES * WALK, last_step), next);
            copy_in(buffer == 0 ? STAGES - 1 : buffer - 1, 0, held);
            #pragma unroll
            for (int k = 0; k < MOST; ++k) held[k] = next[k];
        } else
        copy_in(buffer == 0 ? STAGES - 1 : buffer - 1, min(walk0 + (STAGES - 1) * WALK, last_step));
        uint8_t* stage = stages + buffer * (2 * SLAB);
        if (!UNION && cached - walk0 < WALK) {
            // the sequence's last rows: the stage's tail holds whatever the page held.  It is cleared (those scores are masked,
            // but a stray scale must not meet a zero weight).
            #pragma unroll
            for (int part = 0; part < 2; ++part)
                for (int at = (cached - walk0) * ROW + 4 * int(threadIdx.x); at < SLAB; at += 4 * TEAM * 64)
                    *reinterpret_cast<uint32_t*>(stage + part * SLAB + at) = 0u;
            __syncthreads();
        }
        const int token0 = walk0 + half * STEP;      // the wave's 32 keys of the step
        if (idle || token0 > wave_last || token0 >= keys) continue;    // none of them is visible to the wave's rows
        RowLoad<DIM, Q8> current;
        load_step<DIM>(current, stage + half * STEP * ROW, stage + SLAB + half * STEP * ROW, li, g);
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
        // Scores stay unscaled; the scale goes into the exponent's multiply-add.  m is a row's reference maximum in unscaled units.
        if (UNION) {
            // an entry counts for a row when the row's token selected it: the lane's eight entries' masks, the row's bit
            const uint4 low = *reinterpret_cast<const uint4*>(marks + token0 + 4 * g), high = *reinterpret_cast<const uint4*>(marks + token0 + 16 + 4 * g);
            const uint32_t mask[2][4] = {{low.x, low.y, low.z, low.w}, {high.x, high.y, high.z, high.w}};
            #pragma unroll
            for (int qt = 0; qt < QT; ++qt)
                #pragma unroll
                for (int t = 0; t < 2; ++t)
                    #pragma unroll
                    for (int r = 0; r < 4; ++r)
                        if (token0 + 16 * t + 4 * g + r >= keys || !((mask[t][r] >> limit[qt]) & 1u)) s[qt][t][r] = -INFINITY;
        } else if (token0 + STEP - 1 > wave_first) {          // wave-uniform: some token of the step is past some row's position
            #pragma unroll
            for (int qt = 0; qt < QT; ++qt)
                #pragma unroll
                for (int t = 0; t < 2; ++t)
                    #pragma unroll
                    for (int r = 0; r < 4; ++r)
                        if (token0 + 16 * t + 4 * g + r > limit[qt]) s[qt][t][r] = -INFINITY;
        }
        half8 pb[QT];
        #pragma unroll
        for (int qt = 0; qt < QT; ++qt) {
            float top = fmaxf(fmaxf(fmaxf(s[qt][0][0], s[qt][0][1]), fmaxf(s[qt][0][2], s[qt][0][3])),
                              fmaxf(fmaxf(s[qt][1][0], s[qt][1][1]), fmaxf(s[qt][1][2], s[qt][1][3])));
            top = fmaxf(top, __shfl_xor(top, 16));
            top = fmaxf(top, __shfl_xor(top, 32));
            // The reference maximum follows the true one only when that has grown by more than SLACK (in base-2 exponent
            // units): weights then stay below 2^SLACK, far inside FP16 and FP32 range, and the accumulators are rescaled
            // a few times per row instead of at every new maximum.  The quotient sum/acc does not depend on the reference.
            if (__any((top - m[qt]) * args.scale_log2 > SLACK)) {
                const float m_new = fmaxf(m[qt], top);
                const float alpha = __builtin_amdgcn_exp2f((m[qt] - m_new) * args.scale_log2);
                m[qt] = m_new;
                l[qt] *= alpha;
                #pragma unroll
                for (int jj = 0; jj < TILES; ++jj) acc[qt][jj] *= alpha;
            }
            const float offset = -m[qt] * args.scale_log2;
            float sum = 0.0f;
            half8 p;
            #pragma unroll
            for (int t = 0; t < 2; ++t)
                #pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float w = __builtin_amdgcn_exp2f(fmaf(s[qt][t][r], args.scale_log2, offset));
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
    }

    // The pair of waves that shares rows merges: the second half's wave leaves its state in LDS (the stages are done with),
    // register by register with the lane innermost, and the first half's wave adds it in under the common reference maximum.
    #pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
        l[qt] += __shfl_xor(l[qt], 16);
        l[qt] += __shfl_xor(l[qt], 32);
    }
    __syncthreads();
    float* mine = reinterpret_cast<float*>(stages) + size_t(quarter) * (QT * (TILES * 4 + 2)) * 64 + lane;
    if (half == 1) {
        #pragma unroll
        for (int qt = 0; qt < QT; ++qt) {
            float* at = mine + size_t(qt) * (TILES * 4 + 2) * 64;
            at[0] = m[qt]; at[64] = l[qt];
            #pragma unroll
            for (int jj = 0; jj < TILES; ++jj)
                #pragma unroll
                for (int r = 0; r < 4; ++r) at[(2 + 4 * jj + r) * 64] = acc[qt][jj][r];
        }
    }
    __syncthreads();
    if (half == 1) return;
    #pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
        const float* at = mine + size_t(qt) * (TILES * 4 + 2) * 64;
        const float other = at[0], top = fmaxf(m[qt], other);
        const float keep = __builtin_amdgcn_exp2f((m[qt] - top) * args.scale_log2), add = __builtin_amdgcn_exp2f((other - top) * args.scale_log2);
        l[qt] = l[qt] * keep + at[64] * add;
        #pragma unroll
        for (int jj = 0; jj < TILES; ++jj)
            #pragma unroll
            for (int r = 0; r < 4; ++r) acc[qt][jj][r] = acc[qt][jj][r] * keep + at[(2 + 4 * jj + r) * 64] * add;
    }

    // A lane holds, of its query row, the columns W*(4g + r) + jj: for each r a run of W consecutive ones.
    #pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
        const int row = row0 + qt * 16 + li;
        if (row >= int(args.rows)) continue;
        const float inverse = UNION && !(l[qt] > 0.0f) ? 0.0f : 1.0f / l[qt];     // (a row whose list names no position it may see: zeros)
        const int span_row = row / int(args.group), head = kvh * int(args.group) + row % int(args.group);
        const size_t at = ((size_t(seq) * args.span + span_row) * args.heads + head) * DIM;
        if (UNION && args.gate) {
            #pragma unroll
            for (int r = 0; r < 4; ++r)
                #pragma unroll
                for (int jj = 0; jj < TILES; ++jj) {
                    const float x = args.gate[size_t(span_row) * args.gate_row_stride + size_t(head) * args.gate_stride + W * (4 * g + r) + jj];
                    const float e = expf(-fabsf(x));
                    acc[qt][jj][r] *= x >= 0.0f ? 1.0f / (1.0f + e) : e / (1.0f + e);
                }
        }
        #pragma unroll
        for (int r = 0; r < 4; ++r) {
            const size_t first = at + W * (4 * g + r);
            if (args.out_f16) {
                #pragma unroll
                for (int part = 0; part < TILES / 8; ++part) {
                    half8 packed;
                    #pragma unroll
                    for (int jj = 0; jj < 8; ++jj) packed[jj] = (_Float16)(acc[qt][8 * part + jj][r] * inverse);
                    *reinterpret_cast<half8*>(static_cast<_Float16*>(args.out) + first + 8 * part) = packed;
                }
            } else {
                #pragma unroll
                for (int part = 0; part < TILES / 4; ++part) {
                    floatx4 packed;
                    #pragma unroll
                    for (int jj = 0; jj < 4; ++jj) packed[jj] = acc[qt][4 * part + jj][r] * inverse;
                    *reinterpret_cast<floatx4*>(static_cast<float*>(args.out) + first + 4 * part) = packed;
                }
            }
        }
    }
}

// ---- the form for 128 columns: K/V unpacked once per call into FP16 tiles in a workspace -----------------------------------
// A pass before the attention turns the cached rows of every (sequence, K/V head) into tiles of 64 keys, each a K block
// [64 keys][128 columns] and a V^T block [128 columns][64 keys] of FP16, 32 KiB together, laid out in the order LDS wants them:
// the 16-byte pieces of a K row sit at piece ^ (key % 16); a V^T row keeps the eight keys a lane multiplies at once (keys 4g.. and
// 16 + 4g.. of a 32-key half) side by side as one 16-byte piece, at piece ^ (column / 2 % 8): the sixteen lanes of an operand
// read then fall on sixteen different bank groups without any padding, and an operand is one 16-byte read.  The attention
// kernel then copies a step's tile by plain 1 KiB global->LDS loads and has no conversion in its loop at all; the tiles are
// read by every workgroup of the K/V head (from L2), the pass itself costs a few microseconds per call.
constexpr int TILE_KEYS = 64;
typedef float float2v __attribute__((ext_vector_type(2)));
template<int DIM> constexpr int tile_bytes() { return 2 * TILE_KEYS * DIM * 2; }

// A chunk's new rows may come with the call (IN: 1 FP32, 2 FP16; 0: none): then the kernel is also the K/V writer -- a new row
// is encoded (kv_encode's bits) into its page and, from the same bytes, into the tile, where otherwise it would be read back from
// the page.  `valid` (device, may be null): the leading positions of each sequence whose tiles the buffer still holds from
// earlier chunks; a tile that lies wholly below it is left as it is.
struct AppendArgs {
    const void* keys;
    const void* values;
    const int32_t* valid;
};
// A workgroup builds a quarter of a tile: the K block's or the V^T block's share of 32 of the tile's 64 keys.
constexpr int PART_KEYS = 32, TILE_PARTS = 2 * (TILE_KEYS / PART_KEYS);
template<int DIM, bool Q8, int IN>
__global__ void __launch_bounds__(256) unpack_tiles_kernel(PrefillArgs args, uint8_t* tiles_out, unsigned tiles_per_seq, AppendArgs append) {
    constexpr int ROW = Q8 ? DIM + DIM / 16 : 2 * DIM, KT = TILE_KEYS * DIM * 2, PIECES = DIM / 8;
    static_assert(DIM == 128 && PART_KEYS == 32, "a K row is 16 pieces, a V^T row 16 units; a 16-byte piece of V^T holds keys of one half");
    const int tile = blockIdx.x / TILE_PARTS, value = blockIdx.x / 2 % 2, half = blockIdx.x % 2, kvh = blockIdx.y, seq = blockIdx.z, t = threadIdx.x;
    const int position = first_position(args.positions, unsigned(seq), args.max_context);
    const int cached = min(position + int(args.span), args.max_context), key0 = tile * TILE_KEYS + half * PART_KEYS;
    if (tile * TILE_KEYS >= cached) return;
    if (append.valid && (tile + 1) * TILE_KEYS <= min(max(append.valid[seq], 0), position)) return;
    const int32_t* table = args.page_table + size_t(seq) * args.table_stride;
    const size_t plane_bytes = size_t(args.page_tokens) * ROW, plane = (value ? args.kv_heads : 0) + kvh;
    uint8_t* out = tiles_out + ((size_t(seq) * args.kv_heads + kvh) * tiles_per_seq + tile) * tile_bytes<DIM>();
    // The part's raw rows come into LDS first, by 8-byte words that follow one another through a row and from row to row of
    // a page (the small pieces the layouts below are made of would each be a memory access of their own otherwise).  Rows past
    // the sequence's end are never read: they become zeros below.
    __shared__ __attribute__((aligned(16))) uint8_t raw[PART_KEYS][ROW];
    const auto row_in_pool = [&](int token) {
        return const_cast<uint8_t*>(args.pages) + (size_t(pool_page(table[token / int(args.page_tokens)], args.page_last)) * 2 * args.kv_heads + plane) * plane_bytes +
               size_t(token % int(args.page_tokens)) * ROW;
    };
    constexpr int WORDS = ROW / 8, ALL = PART_KEYS * WORDS, MINE = (ALL + 255) / 256;
    uint2 held[MINE];
    bool old[MINE];
    #pragma unroll
    for (int j = 0; j < MINE; ++j) {                        // all of a thread's words are asked for before the first is stored
        const int word = min(t + 256 * j, ALL - 1), key = word / WORDS, at = word % WORDS, token = key0 + key;
        old[j] = t + 256 * j < ALL && token < cached && !(IN && token >= position);            // (a new row is not in its page yet)
        held[j] = old[j] ? *reinterpret_cast<const uint2*>(row_in_pool(token) + 8 * at) : uint2{0u, 0u};
    }
    [[maybe_unused]] float x[PART_KEYS * (DIM / 4) / 256][4];
    if (IN) {
        // the new rows among the part's keys: four values a thread, the eight threads of a 32-value block side by side
        constexpr int QUADS = DIM / 4;
        const void* source = value ? append.values : append.keys;
        #pragma unroll
        for (int j = 0; j < PART_KEYS * QUADS / 256; ++j) {
            const int index = t + 256 * j, key = index / QUADS, quad = index % QUADS, token = key0 + key;
            const bool live = token >= position && token < cached;
            const size_t first = ((size_t(seq) * args.span + size_t(live ? token - position : 0)) * args.kv_heads + kvh) * DIM + 4 * quad;
            if (IN == 2) {
                const uint2 bits = *reinterpret_cast<const uint2*>(static_cast<const __half*>(source) + first);
                const __half2 a = *reinterpret_cast<const __half2*>(&bits.x), b = *reinterpret_cast<const __half2*>(&bits.y);
                x[j][0] = __low2float(a); x[j][1] = __high2float(a); x[j][2] = __low2float(b); x[j][3] = __high2float(b);
            } else {
                const float4 four = *reinterpret_cast<const float4*>(static_cast<const float*>(source) + first);
                x[j][0] = four.x; x[j][1] = four.y; x[j][2] = four.z; x[j][3] = four.w;
            }
        }
    }
    #pragma unroll
    for (int j = 0; j < MINE; ++j)
        if (old[j]) *reinterpret_cast<uint2*>(&raw[0][0] + 8 * (t + 256 * j)) = held[j];
    if (IN) {
        constexpr int QUADS = DIM / 4;
        #pragma unroll
        for (int j = 0; j < PART_KEYS * QUADS / 256; ++j) {
            const int index = t + 256 * j, key = index / QUADS, quad = index % QUADS, token = key0 + key;
            const bool live = token >= position && token < cached;
            uint8_t* page_row = row_in_pool(live ? token : position);
            if (Q8) {
                uint32_t word;
                __half scale16;
                kv_quad_q8(x[j], word, scale16);
                if (live) {
                    *reinterpret_cast<uint32_t*>(page_row + quad * 4) = word;
                    *reinterpret_cast<uint32_t*>(raw[key] + quad * 4) = word;
                    if (quad % 8 == 0) {
                        *reinterpret_cast<__half*>(page_row + DIM + quad / 8 * 2) = scale16;
                        *reinterpret_cast<__half*>(raw[key] + DIM + quad / 8 * 2) = scale16;
                    }
                }
            } else {
                kv_store_quad(page_row, unsigned(quad), DIM, false, x[j], live);
                kv_store_quad(raw[key], unsigned(quad), DIM, false, x[j], live);
            }
        }
    }
    __syncthreads();
    typedef _Float16 half4 __attribute__((ext_vector_type(4)));
    if (!value) {
        // K: a thread takes pieces of 8 columns; rows past the sequence's end become zeros
        #pragma unroll
        for (int j = 0; j < PART_KEYS * PIECES / 256; ++j) {
            const int piece = t + 256 * j, key = piece / PIECES, c = piece % PIECES, tile_key = half * PART_KEYS + key;
            const uint8_t* row = raw[key];
            half8 values;
            if (Q8) {
                const uint2 bytes = *reinterpret_cast<const uint2*>(row + 8 * c);
                const _Float16 scale = *reinterpret_cast<const _Float16*>(row + DIM + 2 * (c / 4));
                #pragma unroll
                for (int i = 0; i < 8; ++i) values[i] = (_Float16)float(int8_t((i < 4 ? bytes.x : bytes.y) >> (8 * (i & 3)))) * scale;
            } else values = *reinterpret_cast<const half8*>(row + 16 * c);
            if (key0 + key >= cached) values = half8{};
            *reinterpret_cast<half8*>(out + tile_key * (2 * DIM) + ((c ^ (tile_key & 15)) * 16)) = values;
        }
        return;
    }
    // V^T: a thread takes 4 keys x 4 columns
    static_assert((PART_KEYS / 4) * (DIM / 4) == 256, "one block of 4 keys x 4 columns a thread");
    const int keys4 = t % (PART_KEYS / 4), cols4 = t / (PART_KEYS / 4);
    _Float16 v[4][4];       // [key][column]
    #pragma unroll
    for (int e = 0; e < 4; ++e) {
        const uint8_t* row = raw[4 * keys4 + e];
        const bool live = key0 + 4 * keys4 + e < cached;
        if (Q8) {
            const uint32_t bytes = *reinterpret_cast<const uint32_t*>(row + 4 * cols4);
            const _Float16 scale = *reinterpret_cast<const _Float16*>(row + DIM + 2 * (cols4 / 8));
            #pragma unroll
            for (int c = 0; c < 4; ++c) v[e][c] = live ? (_Float16)float(int8_t(bytes >> (8 * c))) * scale : (_Float16)0.0f;
        } else {
            const half4 four = *reinterpret_cast<const half4*>(row + 8 * cols4);
            #pragma unroll
            for (int c = 0; c < 4; ++c) v[e][c] = live ? four[c] : (_Float16)0.0f;
        }
    }
    #pragma unroll
    for (int c = 0; c < 4; ++c) {
        const int column = 4 * cols4 + c;
        // keys 32 half + 16 h + 4 g + (0..3) go to piece 4 half + g, its first (h = 0) or second 8 bytes
        const int piece = 4 * half + keys4 % 4, second = keys4 / 4;
        *reinterpret_cast<half4*>(out + KT + column * (2 * TILE_KEYS) + ((piece ^ ((column >> 1) & 7)) * 16) + 8 * second) = half4{v[0][c], v[1][c], v[2][c], v[3][c]};
    }
}

// Two runs of 4 x QT x 16 rows per workgroup: one counted from the end of the span on waves 0-3 (its rows see the most keys) and
// its mirror image from the start on waves 4-7, so every workgroup walks about the same number of (row, key) pairs and every
// SIMD hosts one wave of each run.  A tile of 64 keys arrives by 32 global->LDS loads of 1 KiB, four a wave, into a ring of
// four stages; the workgroup meets once a tile.
//
// Every wave holds 32 rows and its own instruction stream is pipelined by hand: a step of the wave is 32 keys, and while the
// weights of step u are formed (exponentials) the scores of step u + 1 are multiplied, the K operands of step u + 2 and the
// V^T operands of step u are on their way from LDS, and the products O^T += V^T . P^T of step u follow -- one matrix
// instruction, then the one or two vector instructions that fit beside it, in an order that is written out and fenced, since
// a wave issues in order and the matrix core idles whenever the wave at its head has something else to do first.  Measured
// on this hardware, a matrix instruction leaves room for about three plain vector instructions or one exponential; so
// there are as few vector instructions as the arithmetic allows:
//   * the queries carry the softmax scale (times log2 e), and the products S^T = K . Q^T start from minus the rows'
//     reference maxima instead of zero: a score leaves the matrix core ready to be exponentiated;
//   * the causal mask is -inf in those starting values (set up only for the one or two steps of a wave that cross its
//     diagonal), so a masked score leaves the matrix core as -inf and costs the loop nothing;
//   * whether some row has outgrown its reference maximum by more than the slack is one comparison per lane of the largest
//     score a lane holds; only then (rarely) are row maxima reduced across lanes, the references moved, the sums so far
//     scaled down, and the step's scores multiplied again from the new references -- the score registers are only ever
//     written by the matrix cores.
template<int DIM, int QT>
__global__ void __launch_bounds__(TEAM * 64) __attribute__((amdgpu_waves_per_eu(2, 2))) prefill_dense_kernel(PrefillArgs args, const uint8_t* tiles_in,
                                                                                                       unsigned tiles_per_seq) {
    constexpr int BLOCKS = DIM / 32, TILES = DIM / 16, KT = TILE_KEYS * DIM * 2, TILE = tile_bytes<DIM>();
    constexpr int WAVE_ROWS = QT * 16, GROUP_ROWS = GROUPS * WAVE_ROWS, RING = 4, PER = TILE / 1024 / TEAM, SUB = 32;
    static_assert(TILE % (1024 * TEAM) == 0 && RING * TILE <= 160 * 1024 - 1024 && TILE_KEYS == 2 * SUB, "a tile is two steps of a wave");
    const int kvh = blockIdx.y, seq = blockIdx.z;
    const int thread = threadIdx.x, lane = thread & 63, wave = __builtin_amdgcn_readfirstlane(thread >> 6), li = lane & 15, g = lane >> 4;
    const int position = first_position(args.positions, unsigned(seq), args.max_context);
    const int cached = min(position + int(args.span), args.max_context);
    const int quarter = wave % GROUPS, half = wave / GROUPS;
    const int runs = (int(args.rows) + GROUP_ROWS - 1) / GROUP_ROWS;
    const int late = runs - 1 - int(blockIdx.x), early = int(blockIdx.x), run = half == 0 ? late : early;
    const int row0 = run * GROUP_ROWS + quarter * WAVE_ROWS;
    const int group_last = min(int(args.rows), (late + 1) * GROUP_ROWS) - 1;
    const int keys = min(position + group_last / int(args.group) + 1, cached);
    const bool idle = row0 >= int(args.rows) || (half == 1 && early == late);
    const int wave_first = position + row0 / int(args.group);
    const int wave_last = min(position + (min(int(args.rows), row0 + WAVE_ROWS) - 1) / int(args.group), keys - 1);
    const int steps = idle ? 0 : wave_last / SUB + 1;                              // the wave's own steps of 32 keys
    extern __shared__ __attribute__((aligned(16))) uint8_t stages[];              // [RING][K block | V^T block]
    const uint8_t* const source = tiles_in + (size_t(seq) * args.kv_heads + kvh) * tiles_per_seq * TILE + 1024 * PER * wave + 16 * lane;
    const int last_tile = (keys - 1) / TILE_KEYS;
    const auto copy_in = [&](int tile) {
        const uint8_t* from = source + size_t(min(tile, last_tile)) * TILE;
        uint8_t* stage = stages + (tile % RING) * TILE + 1024 * PER * wave;
        #pragma unroll
        for (int k = 0; k < PER; ++k) load_to_lds<false>(from + 1024 * k, stage + 1024 * k);
    };

    // the first tiles are on their way while the queries are fetched (the compiler's wait for the queries, which it places
    // before their conversion right below, covers these loads too: they are older)
    #pragma unroll
    for (int ahead = 0; ahead < RING - 1; ++ahead) copy_in(ahead);
    half8 qf[QT][BLOCKS];          // the queries times scale * log2 e: a score is a base-2 exponent
    int limit[QT];
    #pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
        const int row = row0 + qt * 16 + li;
        const bool real = row < int(args.rows);
        const int span_row = real ? row / int(args.group) : 0, head = kvh * int(args.group) + (real ? row % int(args.group) : 0);
        limit[qt] = real ? position + span_row : 0x7fffffff;                      // a padding row masks nothing
        const size_t at = ((size_t(seq) * args.span + span_row) * args.heads + head) * DIM;
        #pragma unroll
        for (int b = 0; b < BLOCKS; ++b) {
            half8 value = {};
            if (real) {
                if (args.q_f16) {
                    const half8 raw = *reinterpret_cast<const half8*>(static_cast<const _Float16*>(args.q) + at + 32 * b + 8 * g);
                    #pragma unroll
                    for (int i = 0; i < 8; ++i) value[i] = (_Float16)(float(raw[i]) * args.scale_log2);
                } else {
                    const float* from = static_cast<const float*>(args.q) + at + 32 * b + 8 * g;
                    #pragma unroll
                    for (int i = 0; i < 8; ++i) value[i] = (_Float16)(from[i] * args.scale_log2);
                }
            }
            qf[qt][b] = value;
        }
    }
    // start: where the score products of a step begin instead of zero: minus the row's reference maximum, or -inf for a key
    // after the row's own position -- the causal mask costs the loop nothing, a masked score leaves the matrix core as -inf
    floatx4 acc[QT][TILES], start[QT][2];
    float l[QT], ref[QT];
    #pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
        l[qt] = 0.0f; ref[qt] = 0.0f;
        start[qt][0] = start[qt][1] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
        #pragma unroll
        for (int jj = 0; jj < TILES; ++jj) acc[qt][jj] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
    }
    const auto crosses = [&](int u) { return SUB * u + SUB - 1 > wave_first; };
    // the starting values of a step that crosses the wave's diagonal (every later step of the wave does)
    const auto veil = [&](int u) {
        asm volatile("; the step crosses the diagonal" ::: "memory");
        #pragma unroll
        for (int qt = 0; qt < QT; ++qt)
            #pragma unroll
            for (int t = 0; t < 2; ++t)
                #pragma unroll
                for (int r = 0; r < 4; ++r) start[qt][t][r] = SUB * u + 16 * t + 4 * g + r > limit[qt] ? -INFINITY : ref[qt];
    };
    // K operands of step u and the scores they give, relative to the references
    const auto scores = [&](int u, floatx4 (&s)[QT][2]) {
        const uint8_t* const kblock = stages + ((u >> 1) % RING) * TILE + (u & 1) * (SUB * 2 * DIM);
        half8 ka[2][BLOCKS];
        #pragma unroll
        for (int t = 0; t < 2; ++t)
            #pragma unroll
            for (int b = 0; b < BLOCKS; ++b) ka[t][b] = *reinterpret_cast<const half8*>(kblock + (16 * t + li) * (2 * DIM) + (((4 * b + g) ^ li) * 16));
        #pragma unroll
        for (int b = 0; b < BLOCKS; ++b)
            #pragma unroll
            for (int t = 0; t < 2; ++t)
                #pragma unroll
                for (int qt = 0; qt < QT; ++qt) s[qt][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka[t][b], qf[qt][b], b == 0 ? start[qt][t] : s[qt][t], 0, 0, 0);
    };
    // The rows' maxima of step u's scores (of the keys a row may see) become (FIRST) or raise (otherwise) the references: what
    // has been summed so far is scaled down, and the step's scores are multiplied again from the new references -- the
    // score registers are only ever written by the matrix cores, which keeps them where they are.
    const auto raise = [&](auto first, int u, floatx4 (&s)[QT][2]) {
        asm volatile("; new reference maxima" ::: "memory");
        #pragma unroll
        for (int qt = 0; qt < QT; ++qt) {
            float most = s[qt][0][0];
            #pragma unroll
            for (int t = 0; t < 2; ++t)
                #pragma unroll
                for (int r = 0; r < 4; ++r) most = fmaxf(most, s[qt][t][r]);
            const float top = row_max(most);
            const float delta = decltype(first)::value ? top : fmaxf(top, 0.0f);
            ref[qt] -= delta;
            start[qt][0] -= delta; start[qt][1] -= delta;
            if (!decltype(first)::value) {
                const float alpha = __builtin_amdgcn_exp2f(-delta);
                l[qt] *= alpha;
                #pragma unroll
                for (int jj = 0; jj < TILES; ++jj) acc[qt][jj] *= alpha;
            }
        }
        scores(u, s);
    };
    // One step: weights of step u from `now`, scores of step u + 1 into `next`, the products of step u, the maxima of step
    // u + 1.  The order of issue is written out: between two fences the compiler finds one product and the few vector
    // instructions that run beside it, nothing crosses a fence.
    static_assert(QT == 2 && BLOCKS == 4 && TILES == 8, "the interleaving below is written for 32 rows x 32 keys x 128 columns");
    half8 ka[2][BLOCKS];           // the K operands of the step after the one whose weights are being formed: read a step ahead
    const auto read_k = [&](int u, int t, int b) {
        const uint8_t* const kblock = stages + ((u >> 1) % RING) * TILE + (u & 1) * (SUB * 2 * DIM);
        ka[t][b] = *reinterpret_cast<const half8*>(kblock + (16 * t + li) * (2 * DIM) + (((4 * b + g) ^ li) * 16));
    };
    // the workgroup's meeting once a tile: the next tile has landed (the wave's own pieces: only the tile after it is still
    // outstanding; everybody's: the barrier), and everybody is done with the tile before this one, whose stage the tile
    // three ahead now goes to
    const auto meet = [&](int tile) {
        wait_loads<PER * (RING - 3)>();
        ring_barrier();
        copy_in(tile + RING - 1);
    };
    const auto advance = [&](auto even, int u, floatx4 (&now)[QT][2], floatx4 (&next)[QT][2]) {
        if (crosses(u + 1)) veil(u + 1);
        const uint8_t* const vblock = stages + ((u >> 1) % RING) * TILE + KT;
        const int part = u & 1;
        half8 va[TILES];
        __builtin_amdgcn_sched_barrier(0);
        words4 pw[QT];
        float w0[8], w1[8];
        const auto weight = [&](float score) { return __builtin_amdgcn_exp2f(score); };
        const auto packed = [&](float first, float second) { return __builtin_bit_cast(uint32_t, __builtin_convertvector(float2v{first, second}, half2v)); };
        #pragma unroll
        for (int i = 0; i < 16; ++i) {
            // the product: column block b of key tile t for row tile qt (past the wave's last step: of whatever the stage holds, never used)
            const int b = i / 4, t = (i / 2) % 2, qt = i % 2;
            next[qt][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka[t][b], qf[qt][b], b == 0 ? start[qt][t] : next[qt][t], 0, 0, 0);
            // beside it: a weight of this step's first row tile, or its sum and packing and a V^T operand
            const int e = i / 2;
            if (i % 2 == 0) w0[e] = weight(now[0][e / 4][e % 4]);
            else {
                l[0] += w0[e];
                if (e % 2) pw[0][e / 2] = packed(w0[e - 1], w0[e]);
            }
            if (i < 8) {
                va[i] = *reinterpret_cast<const half8*>(vblock + (16 * i + li) * (2 * TILE_KEYS) + (((4 * part + g) ^ (li >> 1)) * 16));
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        if (decltype(even)::value) meet(u >> 1);        // the step after the next reads the next tile
        __builtin_amdgcn_sched_barrier(0);
        #pragma unroll
        for (int j = 0; j < 8; ++j) {       // the first row tile's products, the second's weights, the K operands of the step after the next
            acc[0][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va[j], __builtin_bit_cast(half8, pw[0]), acc[0][j], 0, 0, 0);
            w1[j] = weight(now[1][j / 4][j % 4]);
            if (j % 2) pw[1][j / 2] = packed(w1[j - 1], w1[j]);
            read_k(u + 2, j % 2, j / 2);
            __builtin_amdgcn_sched_barrier(0);
        }
        float most = next[0][0][0];
        #pragma unroll
        for (int j = 0; j < 8; ++j) {       // the second row tile's products, its weights' sum, the next step's largest score
            acc[1][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va[j], __builtin_bit_cast(half8, pw[1]), acc[1][j], 0, 0, 0);
            l[1] += w1[j];
            most = fmaxf(fmaxf(most, next[j / 4][(j / 2) % 2][2 * (j % 2)]), next[j / 4][(j / 2) % 2][2 * (j % 2) + 1]);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (__any(most > SLACK) && u + 1 < steps) raise(std::false_type{}, u + 1, next);
    };


    floatx4 even[QT][2], odd[QT][2];
    wait_loads<PER * (RING - 2)>();
    ring_barrier();
    if (steps > 0) {
        if (crosses(0)) veil(0);
        scores(0, even);
        raise(std::true_type{}, 0, even);
        #pragma unroll
        for (int b = 0; b < BLOCKS; ++b)
            #pragma unroll
            for (int t = 0; t < 2; ++t) read_k(1, t, b);
    }
    for (int tile = 0; tile <= last_tile; ++tile) {
        if (2 * tile < steps) advance(std::true_type{}, 2 * tile, even, odd); else meet(tile);
        if (2 * tile + 1 < steps) advance(std::false_type{}, 2 * tile + 1, odd, even);
    }

    if (idle) return;
    #pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
        const int row = row0 + qt * 16 + li;
        const float inverse = 1.0f / row_sum(l[qt]);
        if (row >= int(args.rows)) continue;
        const int span_row = row / int(args.group), head = kvh * int(args.group) + row % int(args.group);
        const size_t first = ((size_t(seq) * args.span + span_row) * args.heads + head) * DIM + 4 * g;
        #pragma unroll
        for (int jj = 0; jj < TILES; ++jj) {
            const floatx4 value = acc[qt][jj] * inverse;
            if (args.out_f16) {
                typedef _Float16 half4 __attribute__((ext_vector_type(4)));
                *reinterpret_cast<half4*>(static_cast<_Float16*>(args.out) + first + 16 * jj) = half4{(_Float16)value[0], (_Float16)value[1], (_Float16)value[2], (_Float16)value[3]};
            } else *reinterpret_cast<floatx4*>(static_cast<float*>(args.out) + first + 16 * jj) = value;
        }
    }
}

// ---- the same walk with 64 rows a wave ---------------------------------------------------------------------------------------
// One wave a SIMD (four a workgroup) holds four 16-row tiles: two of the run counted from the span's end and two of its mirror
// image from the start, so a wave is its own pair and every SIMD has work as long as the workgroup has.  An operand read from
// LDS then feeds four products where it fed two: what a compute unit reads from LDS per product is halved, and LDS traffic
// (operand reads and the tiles' arrival) is what the products compete with.  The wave needs about 330 registers; which of them
// live in the accumulation half of the register file is said here, by writing the products as instructions with register
// classes: the queries (only ever a B operand) and the output accumulators (only ever written by products) do, everything the
// vector arithmetic touches does not -- left to itself the compiler puts every product's result there and copies scores back
// and forth (2.6 copies a product, measured).  The compiler then does not know these instructions for products, so what it would
// have kept apart is kept apart here: a vector instruction's result waits two states before a product reads it (s_nop 1 ahead of
// the first product that follows one), a product's result is read by vector instructions only a step later (or after a wait
// written out), and a product that adds to another's result comes at least three products after it.
template<bool AFTER_VECTOR>
__device__ __forceinline__ void score_first(floatx4& d, const half8& k, const half8& q, const floatx4& c) {
    if (AFTER_VECTOR) asm volatile("s_nop 1\n\tv_mfma_f32_16x16x32_f16 %0, %1, %2, %3" : "=&v"(d) : "v"(k), "a"(q), "v"(c));
    else asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %3" : "=&v"(d) : "v"(k), "a"(q), "v"(c));
}
__device__ __forceinline__ void score_more(floatx4& d, const half8& k, const half8& q) { asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(d) : "v"(k), "a"(q)); }
template<bool AFTER_VECTOR>
__device__ __forceinline__ void output_more(floatx4& d, const half8& v, const words4& p) {
    if (AFTER_VECTOR) asm volatile("s_nop 1\n\tv_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(d) : "v"(v), "v"(p));
    else asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(d) : "v"(v), "v"(p));
}
// (after products whose results vector instructions read at once: longer than any product takes)
__device__ __forceinline__ void products_done() { asm volatile("s_nop 15\n\ts_nop 15" ::: "memory"); }

template<int DIM>
__global__ void __launch_bounds__(GROUPS * 64) __attribute__((amdgpu_waves_per_eu(1, 1))) prefill_dense64_kernel(PrefillArgs args, const uint8_t* tiles_in,
                                                                                                            unsigned tiles_per_seq) {
    constexpr int QT = 4, BLOCKS = DIM / 32, TILES = DIM / 16, KT = TILE_KEYS * DIM * 2, TILE = tile_bytes<DIM>();
    constexpr int PAIR_ROWS = 32, GROUP_ROWS = GROUPS * PAIR_ROWS, RING = 4, PER = TILE / 1024 / GROUPS, SUB = 32;
    static_assert(TILE % (1024 * GROUPS) == 0 && RING * TILE <= 160 * 1024 - 1024 && TILE_KEYS == 2 * SUB && BLOCKS == 4 && TILES == 8, "a tile is two steps of a wave");
    const int kvh = blockIdx.y, seq = blockIdx.z;
    const int thread = threadIdx.x, lane = thread & 63, wave = __builtin_amdgcn_readfirstlane(thread >> 6), li = lane & 15, g = lane >> 4;
    const int runs = (int(args.rows) + GROUP_ROWS - 1) / GROUP_ROWS;
    const int late = runs - 1 - int(blockIdx.x), early = int(blockIdx.x);
    // The queries are asked for first: where they lie does not depend on the sequence's position, whose own trip from memory
    // everything else waits for.  (Tiles 0 and 1 are the late run's, 2 and 3 the early run's; a row past the last stands for the last.)
    half8 raw16[QT][BLOCKS];
    float raw32[QT][BLOCKS][8];
    #pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
        const int row = min(((qt / 2 == 0 ? late : early) * GROUP_ROWS + wave * PAIR_ROWS) + (qt % 2) * 16 + li, int(args.rows) - 1);
        const int span_row = row / int(args.group), head = kvh * int(args.group) + row % int(args.group);
        const size_t at = ((size_t(seq) * args.span + span_row) * args.heads + head) * DIM;
        #pragma unroll
        for (int b = 0; b < BLOCKS; ++b) {
            if (args.q_f16) raw16[qt][b] = *reinterpret_cast<const half8*>(static_cast<const _Float16*>(args.q) + at + 32 * b + 8 * g);
            else {
                const float* from = static_cast<const float*>(args.q) + at + 32 * b + 8 * g;
                #pragma unroll
                for (int i = 0; i < 8; ++i) raw32[qt][b][i] = from[i];
            }
        }
    }
    const int position = first_position(args.positions, unsigned(seq), args.max_context);
    const int cached = min(position + int(args.span), args.max_context);
    const int group_last = min(int(args.rows), (late + 1) * GROUP_ROWS) - 1;
    const int keys = min(position + group_last / int(args.group) + 1, cached);
    // the wave's two pairs of tiles: pair 0 of the late run, pair 1 of the early one
    int row0[2], wave_first[2], steps[2];
    #pragma unroll
    for (int p = 0; p < 2; ++p) {
        row0[p] = (p == 0 ? late : early) * GROUP_ROWS + wave * PAIR_ROWS;
        const bool idle = row0[p] >= int(args.rows) || (p == 1 && early == late);
        wave_first[p] = position + row0[p] / int(args.group);
        const int wave_last = min(position + (min(int(args.rows), row0[p] + PAIR_ROWS) - 1) / int(args.group), keys - 1);
        steps[p] = idle ? 0 : wave_last / SUB + 1;
    }
    const bool swapped = steps[0] < steps[1];
    if (swapped) {      // (the late run's quarter may lie past the span's last row: the longer walk is pair 0's)
        const int r = row0[0], f = wave_first[0], n = steps[0];
        row0[0] = row0[1]; wave_first[0] = wave_first[1]; steps[0] = steps[1];
        row0[1] = r; wave_first[1] = f; steps[1] = n;
    }
    extern __shared__ __attribute__((aligned(16))) uint8_t stages[];              // [RING][K block | V^T block]
    const uint8_t* const source = tiles_in + (size_t(seq) * args.kv_heads + kvh) * tiles_per_seq * TILE;        // (the wave's: scalar)
    const int last_tile = (keys - 1) / TILE_KEYS;
    // A tile's eight pieces of a wave as one run of instructions: the tile's address is the wave's (scalar registers), a lane adds
    // its own constant offset, the pieces differ by the instruction's offset, which moves both ends.
    static_assert(PER == 8, "two runs of four pieces");
    const uint32_t lane_offset = 1024 * PER * wave + 16 * lane, lane_offset_high = lane_offset + 4096;
    const uint32_t wave_stage = __builtin_amdgcn_readfirstlane(lds_address(stages)) + 1024 * PER * wave;
    const auto copy_in = [&](int tile) {
        const uint64_t from = uint64_t(source + size_t(min(tile, last_tile)) * TILE);
        const uint32_t to = wave_stage + (tile % RING) * TILE;
        uint32_t keep;
        asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\t"
                     "global_load_lds_dwordx4 %3, %2\n\tglobal_load_lds_dwordx4 %3, %2 offset:1024\n\t"
                     "global_load_lds_dwordx4 %3, %2 offset:2048\n\tglobal_load_lds_dwordx4 %3, %2 offset:3072\n\t"
                     "s_add_u32 m0, %1, 0x1000\n\ts_nop 0\n\t"
                     "global_load_lds_dwordx4 %4, %2\n\tglobal_load_lds_dwordx4 %4, %2 offset:1024\n\t"
                     "global_load_lds_dwordx4 %4, %2 offset:2048\n\tglobal_load_lds_dwordx4 %4, %2 offset:3072\n\t"
                     "s_mov_b32 m0, %0"
                     : "=&s"(keep) : "s"(to), "s"(from), "v"(lane_offset), "v"(lane_offset_high) : "memory", "scc");
    };
    #pragma unroll
    for (int ahead = 0; ahead < RING - 1; ++ahead) copy_in(ahead);
    half8 qf[QT][BLOCKS];          // the queries times scale * log2 e: a score is a base-2 exponent
    int limit[QT];
    #pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
        const int row = row0[qt / 2] + (qt % 2) * 16 + li;
        const bool real = row < int(args.rows) && steps[qt / 2] > 0;
        limit[qt] = real ? position + row / int(args.group) : 0x7fffffff;         // a padding row masks nothing
        #pragma unroll
        for (int b = 0; b < BLOCKS; ++b) {
            half8 value = {};
            if (real) {
                if (args.q_f16) {
                    const half8 raw = swapped ? raw16[qt ^ 2][b] : raw16[qt][b];
                    #pragma unroll
                    for (int i = 0; i < 8; ++i) value[i] = (_Float16)(float(raw[i]) * args.scale_log2);
                } else {
                    #pragma unroll
                    for (int i = 0; i < 8; ++i) value[i] = (_Float16)((swapped ? raw32[qt ^ 2][b][i] : raw32[qt][b][i]) * args.scale_log2);
                }
            }
            // (the queries are only ever a product's B operand: they live in the accumulation registers, where a product reads them
            // as well, and leave the vector registers to what the vector arithmetic touches)
            asm volatile("; queries of tile %1 block %2" : "=a"(qf[qt][b]) : "n"(qt), "n"(b), "0"(value));
        }
    }
    floatx4 acc[QT][TILES], start[QT][2];
    float l[QT], ref[QT];
    #pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
        l[qt] = 0.0f; ref[qt] = 0.0f;
        start[qt][0] = start[qt][1] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
        #pragma unroll
        for (int jj = 0; jj < TILES; ++jj) asm volatile("; zero" : "=a"(acc[qt][jj]) : "0"(floatx4{0.0f, 0.0f, 0.0f, 0.0f}));
    }
    const auto crosses = [&](int p, int u) { return SUB * u + SUB - 1 > wave_first[p]; };
    // the starting values of a pair's step that crosses its diagonal (every later step of the pair does)
    const auto veil = [&](int p, int u) {
        asm volatile("; the step crosses the diagonal" ::: "memory");
        #pragma unroll
        for (int q = 0; q < 2; ++q)
            #pragma unroll
            for (int t = 0; t < 2; ++t)
                #pragma unroll
                for (int r = 0; r < 4; ++r) start[2 * p + q][t][r] = SUB * u + 16 * t + 4 * g + r > limit[2 * p + q] ? -INFINITY : ref[2 * p + q];
        asm volatile("s_nop 1" ::: "memory");      // (the products that read these come right behind)
    };
    // K operands of step u and the scores they give a pair, relative to its references (not pipelined: the start and the rare raise)
    const auto scores = [&](int p, int u, floatx4 (&s)[QT][2]) {
        const uint8_t* const kblock = stages + ((u >> 1) % RING) * TILE + (u & 1) * (SUB * 2 * DIM);
        half8 k[2][BLOCKS];
        #pragma unroll
        for (int t = 0; t < 2; ++t)
            #pragma unroll
            for (int b = 0; b < BLOCKS; ++b) k[t][b] = *reinterpret_cast<const half8*>(kblock + (16 * t + li) * (2 * DIM) + (((4 * b + g) ^ li) * 16));
        #pragma unroll
        for (int b = 0; b < BLOCKS; ++b)
            #pragma unroll
            for (int t = 0; t < 2; ++t)
                #pragma unroll
                for (int q = 0; q < 2; ++q) {
                    if (b == 0) score_first<true>(s[2 * p + q][t], k[t][b], qf[2 * p + q][b], start[2 * p + q][t]);      // (the starting values may have been written just now)
                    else score_more(s[2 * p + q][t], k[t][b], qf[2 * p + q][b]);
                }
        products_done();
    };
    const auto raise = [&](auto first, int p, int u, floatx4 (&s)[QT][2]) {
        asm volatile("; new reference maxima" ::: "memory");
        if (!decltype(first)::value) products_done();       // (the accumulators scaled below were written by products just now)
        #pragma unroll
        for (int q = 0; q < 2; ++q) {
            const int qt = 2 * p + q;
            float most = s[qt][0][0];
            #pragma unroll
            for (int t = 0; t < 2; ++t)
                #pragma unroll
                for (int r = 0; r < 4; ++r) most = fmaxf(most, s[qt][t][r]);
            const float top = row_max(most);
            const float delta = decltype(first)::value ? top : fmaxf(top, 0.0f);
            ref[qt] -= delta;
            start[qt][0] -= delta; start[qt][1] -= delta;
            if (!decltype(first)::value) {
                const float alpha = __builtin_amdgcn_exp2f(-delta);
                l[qt] *= alpha;
                #pragma unroll
                for (int jj = 0; jj < TILES; ++jj) {
                    const floatx4 scaled = acc[qt][jj] * alpha;
                    asm volatile("; scaled" : "=a"(acc[qt][jj]) : "0"(scaled));     // (back into the accumulation registers)
                }
            }
        }
        scores(p, u, s);
    };
    half8 ka[2][BLOCKS];           // the K operands of the step after the one whose weights are being formed: read a step ahead
    const auto read_k = [&](int u, int t, int b) {
        const uint8_t* const kblock = stages + ((u >> 1) % RING) * TILE + (u & 1) * (SUB * 2 * DIM);
        ka[t][b] = *reinterpret_cast<const half8*>(kblock + (16 * t + li) * (2 * DIM) + (((4 * b + g) ^ li) * 16));
    };
    half8 va[TILES];               // the V^T operands of the step whose weights are being formed
    const auto meet = [&](int tile) {
        wait_loads<PER * (RING - 3)>();
        ring_barrier();
        copy_in(tile + RING - 1);
    };
    // One step of one pair p: weights of step u from `now`, scores of step u + 1 into `next`, the products of step u, the largest
    // score of step u + 1.  READS_V: this pair is the step's first (it fetches the V^T operands and, on even steps, meets the
    // workgroup); READS_K: it is the step's last (it fetches the K operands of the step after the next).
    const auto advance = [&](auto reads_v, auto reads_k, auto even, int p, int u, floatx4 (&now)[QT][2], floatx4 (&next)[QT][2]) {
        constexpr bool READS_V = decltype(reads_v)::value, READS_K = decltype(reads_k)::value;
        if (crosses(p, u + 1)) veil(p, u + 1);
        const uint8_t* const vblock = stages + ((u >> 1) % RING) * TILE + KT;
        const int part = u & 1, q0 = 2 * p, q1 = 2 * p + 1;
        __builtin_amdgcn_sched_barrier(0);
        words4 pw[2];
        float w0[8], w1[8];
        const auto packed = [&](float first, float second) { return __builtin_bit_cast(uint32_t, __builtin_convertvector(float2v{first, second}, half2v)); };
        // (the weights' exponentials are written as instructions too: the compiler then keeps no wait state after each for the vector
        // instruction that reads it -- a product always lies between them here)
        const auto weight = [&](float score) { float w; asm volatile("v_exp_f32 %0, %1" : "=v"(w) : "v"(score)); return w; };
        #pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int b = i / 4, t = (i / 2) % 2, q = i % 2;
            if (b == 0) score_first<false>(next[q0 + q][t], ka[t][b], qf[q0 + q][b], start[q0 + q][t]); else score_more(next[q0 + q][t], ka[t][b], qf[q0 + q][b]);
            const int e = i / 2;
            if (i % 2 == 0) w0[e] = weight(now[q0][e / 4][e % 4]);
            else {
                __builtin_amdgcn_sched_barrier(0);      // (the exponential of the slot before and the sum that reads it: the product between them)
                if (e % 2) pw[0][e / 2] = packed(w0[e - 1], w0[e]);
                l[q0] += w0[e];
            }
            if (READS_V && i < 8) va[i] = *reinterpret_cast<const half8*>(vblock + (16 * i + li) * (2 * TILE_KEYS) + (((4 * part + g) ^ (li >> 1)) * 16));
            __builtin_amdgcn_sched_barrier(0);
        }
        if (READS_V && decltype(even)::value) meet(u >> 1);        // the step after the next reads the next tile
        __builtin_amdgcn_sched_barrier(0);
        #pragma unroll
        for (int j = 0; j < 8; ++j) {
            w1[j] = weight(now[q1][j / 4][j % 4]);
            __builtin_amdgcn_sched_barrier(0);
            // (the first product reads weights packed two instructions ago: more wait states)
            if (j == 0) output_more<true>(acc[q0][j], va[j], pw[0]); else output_more<false>(acc[q0][j], va[j], pw[0]);
            __builtin_amdgcn_sched_barrier(0);
            if (j % 2) pw[1][j / 2] = packed(w1[j - 1], w1[j]);
            if (READS_K) read_k(u + 2, j % 2, j / 2);
            __builtin_amdgcn_sched_barrier(0);
        }
        float most = next[q0][0][0];
        #pragma unroll
        for (int j = 0; j < 8; ++j) {
            l[q1] += w1[j];
            most = fmaxf(fmaxf(most, next[q0 + j / 4][(j / 2) % 2][2 * (j % 2)]), next[q0 + j / 4][(j / 2) % 2][2 * (j % 2) + 1]);
            if (j == 0) __builtin_amdgcn_sched_barrier(0);      // (the first product reads weights packed just now: the two instructions above first)
            output_more<false>(acc[q1][j], va[j], pw[1]);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (__builtin_expect(__any(most > SLACK), 0)) raise(std::false_type{}, p, u + 1, next);
    };
    floatx4 even[QT][2], odd[QT][2];
    wait_loads<PER * (RING - 2)>();
    ring_barrier();
    #pragma unroll
    for (int p = 0; p < 2; ++p)
        if (steps[p] > 0) {
            if (crosses(p, 0)) veil(p, 0);
            scores(p, 0, even);
            raise(std::true_type{}, p, 0, even);
        }
    #pragma unroll
    for (int b = 0; b < BLOCKS; ++b)
        #pragma unroll
        for (int t = 0; t < 2; ++t) read_k(1, t, b);
    // Whole tiles (two steps each): first those both pairs walk, then those only the longer pair walks.  A pair's last tile may
    // hold a step past its rows' last key: every score of it is masked, it adds nothing, and the loops stay free of branches.
    const int both = steps[1] == 0 ? 0 : min((steps[1] + 1) / 2, last_tile + 1);
    int tile = 0;
    for (; tile < both; ++tile) {
        advance(std::true_type{}, std::false_type{}, std::true_type{}, 0, 2 * tile, even, odd);
        advance(std::false_type{}, std::true_type{}, std::true_type{}, 1, 2 * tile, even, odd);
        advance(std::true_type{}, std::false_type{}, std::false_type{}, 0, 2 * tile + 1, odd, even);
        advance(std::false_type{}, std::true_type{}, std::false_type{}, 1, 2 * tile + 1, odd, even);
    }
    // A pair's rows normalised and written.  The shorter pair's leave as soon as it is done, while the longer one walks on: the
    // launch's outputs then do not all reach memory at once as every workgroup ends.
    const auto deliver = [&](int p) {
        #pragma unroll
        for (int q = 0; q < 2; ++q) {
            const int qt = 2 * p + q, row = row0[p] + q * 16 + li;
            const float inverse = 1.0f / row_sum(l[qt]);
            if (steps[p] == 0 || row >= int(args.rows)) continue;
            const int span_row = row / int(args.group), head = kvh * int(args.group) + row % int(args.group);
            const size_t first = ((size_t(seq) * args.span + span_row) * args.heads + head) * DIM + 4 * g;
            #pragma unroll
            for (int jj = 0; jj < TILES; ++jj) {
                const floatx4 value = acc[qt][jj] * inverse;
                if (args.out_f16) {
                    typedef _Float16 half4 __attribute__((ext_vector_type(4)));
                    *reinterpret_cast<half4*>(static_cast<_Float16*>(args.out) + first + 16 * jj) = half4{(_Float16)value[0], (_Float16)value[1], (_Float16)value[2], (_Float16)value[3]};
                } else *reinterpret_cast<floatx4*>(static_cast<float*>(args.out) + first + 16 * jj) = value;
            }
        }
    };
    const bool early_leaves = tile <= last_tile;        // (the longer pair has tiles of its own left)
    if (early_leaves) {
        products_done();
        deliver(1);
    }
    for (; tile <= last_tile; ++tile) {
        advance(std::true_type{}, std::true_type{}, std::true_type{}, 0, 2 * tile, even, odd);
        advance(std::true_type{}, std::true_type{}, std::false_type{}, 0, 2 * tile + 1, odd, even);
    }

    products_done();
    deliver(0);
    if (!early_leaves) deliver(1);
}

// `tiles`: where the cached rows' FP16 tiles go -- the device's workspace, rebuilt whole on every call, or a buffer the caller
// keeps between the chunks of a prompt (then `append` may carry the chunk's new rows and the count of positions still valid).
template<int DIM, int QT, bool Q8>
void launch_dense(Device& d, const PrefillArgs& args, unsigned seqs, uint8_t* tiles, const AppendArgs& append, int input) {
    const unsigned tiles_per_seq = unsigned((args.max_context + TILE_KEYS - 1) / TILE_KEYS);
    if (!tiles) tiles = static_cast<uint8_t*>(workspace(d, checked_product({seqs, args.kv_heads, tiles_per_seq, uint64_t(tile_bytes<DIM>())})));
    constexpr int shared = 4 * tile_bytes<DIM>();
    raise_shared_limit(d, reinterpret_cast<const void*>(&prefill_dense_kernel<DIM, QT>), shared);
    const dim3 grid(tiles_per_seq * TILE_PARTS, args.kv_heads, seqs);
    if (input == 2) unpack_tiles_kernel<DIM, Q8, 2><<<grid, 256, 0, d.stream>>>(args, tiles, tiles_per_seq, append);
    else if (input == 1) unpack_tiles_kernel<DIM, Q8, 1><<<grid, 256, 0, d.stream>>>(args, tiles, tiles_per_seq, append);
    else unpack_tiles_kernel<DIM, Q8, 0><<<grid, 256, 0, d.stream>>>(args, tiles, tiles_per_seq, append);
    const unsigned runs = (args.rows + GROUPS * QT * 16 - 1) / (GROUPS * QT * 16);
    if (d.prefill_wave_rows == 64) {        // (the same rows a workgroup, the same tiles, the same grid: four waves of 64 rows for eight of 32)
        raise_shared_limit(d, reinterpret_cast<const void*>(&prefill_dense64_kernel<DIM>), shared);
        timed_launch(d, &prefill_dense64_kernel<DIM>, dim3((runs + 1) / 2, args.kv_heads, seqs), dim3(GROUPS * 64), shared, args, tiles, tiles_per_seq);
    } else timed_launch(d, &prefill_dense_kernel<DIM, QT>, dim3((runs + 1) / 2, args.kv_heads, seqs), dim3(TEAM * 64), shared, args, tiles, tiles_per_seq);
}

template<int DIM, int QT, bool Q8, int OCC>
void launch(Device& d, const PrefillArgs& args, unsigned seqs) {
    constexpr size_t merge = size_t(GROUPS) * QT * (DIM / 16 * 4 + 2) * 64 * 4;
    constexpr size_t stage = size_t(2) * WALK * (Q8 ? DIM + DIM / 16 : 2 * DIM), ring = stages_for(int(stage)) * stage;
    constexpr size_t shared = ring > merge ? ring : merge;
    static_assert(shared <= 160 * 1024, "the stages and the merge area share the compute unit's LDS");
    if (shared > 64 * 1024) raise_shared_limit(d, reinterpret_cast<const void*>(&prefill_attention_kernel<DIM, QT, Q8, OCC>), shared);
    const unsigned tiles = (args.rows + GROUPS * QT * 16 - 1) / (GROUPS * QT * 16);
    timed_launch(d, &prefill_attention_kernel<DIM, QT, Q8, OCC>, dim3(tiles, args.kv_heads, seqs), dim3(TEAM * 64), shared, args);
}

}  // namespace

namespace sd {

// Called by sdx_paged_attention (which has validated the arguments) when a sequence has more query rows per K/V head than
// the decode kernel's workgroup takes.
void prefill_attention(Device& d, const sdx_kv_pool* pool, const int32_t* page_table, uint64_t table_stride, const int32_t* positions,
                       uint64_t max_context, const void* q, int q_f16, uint64_t seqs, uint64_t span, uint64_t heads, float scale, void* out,
                       int out_f16) {
    PrefillArgs args{};
    args.pages = static_cast<const uint8_t*>(pool->pages);
    args.page_tokens = pool->page_tokens; args.kv_heads = pool->kv_heads; args.heads = unsigned(heads);
    args.group = unsigned(heads / pool->kv_heads); args.span = unsigned(span);
    args.page_table = page_table; args.table_stride = size_t(table_stride); args.positions = positions;
    args.q = q; args.q_f16 = q_f16; args.scale_log2 = scale * 1.44269504088896341f;
    args.rows = unsigned(span * args.group); args.max_context = int(max_context);
    args.page_last = unsigned(std::min<uint64_t>(pool->page_count - 1, 0x7fffffffu));
    args.out = out; args.out_f16 = out_f16;
    const bool q8 = pool->row_bytes != 2 * pool->dim;
    if (pool->dim == 128) {
        if (q8) launch_dense<128, 2, true>(d, args, unsigned(seqs), nullptr, AppendArgs{}, 0); else launch_dense<128, 2, false>(d, args, unsigned(seqs), nullptr, AppendArgs{}, 0);
    } else { if (q8) launch<256, 1, true, 2>(d, args, unsigned(seqs)); else launch<256, 1, false, 2>(d, args, unsigned(seqs)); }
}

// A prompt chunk in one call: the chunk's K/V rows appended (when given) and its queries attended, the cached rows' tiles kept in
// the caller's buffer from chunk to chunk.  128 columns.
void prefill_chunk(Device& d, const sdx_kv_pool* pool, const int32_t* page_table, uint64_t table_stride, const int32_t* positions,
                   uint64_t max_context, const void* keys, const void* values, int kv_f16, const void* q, int q_f16, uint64_t seqs, uint64_t span,
                   uint64_t heads, float scale, void* out, int out_f16, void* tiles, const int32_t* valid) {
    PrefillArgs args{};
    args.pages = static_cast<const uint8_t*>(pool->pages);
    args.page_tokens = pool->page_tokens; args.kv_heads = pool->kv_heads; args.heads = unsigned(heads);
    args.group = unsigned(heads / pool->kv_heads); args.span = unsigned(span);
    args.page_table = page_table; args.table_stride = size_t(table_stride); args.positions = positions;
    args.q = q; args.q_f16 = q_f16; args.scale_log2 = scale * 1.44269504088896341f;
    args.rows = unsigned(span * args.group); args.max_context = int(max_context);
    args.page_last = unsigned(std::min<uint64_t>(pool->page_count - 1, 0x7fffffffu));
    args.out = out; args.out_f16 = out_f16;
    const AppendArgs append{keys, values, valid};
    const int input = keys ? (kv_f16 ? 2 : 1) : 0;
    if (pool->row_bytes != 2 * pool->dim) launch_dense<128, 2, true>(d, args, unsigned(seqs), static_cast<uint8_t*>(tiles), append, input);
    else launch_dense<128, 2, false>(d, args, unsigned(seqs), static_cast<uint8_t*>(tiles), append, input);
}

uint64_t prefill_tiles_bytes(uint64_t seqs, uint64_t kv_heads, uint64_t max_context) {
    return checked_product({seqs, kv_heads, (max_context + TILE_KEYS - 1) / TILE_KEYS, uint64_t(tile_bytes<128>())});
}

// The union walk of a prompt chunk (256 columns): `tokens` rows of one sequence from position `base`, each tile of 64 query rows
// (16 x the heads of a K/V head) walking its own list of positions (see PrefillArgs).  Lists and masks are device memory.
unsigned union_tile_rows() { return GROUPS * 16; }
void prefill_union(Device& d, const sdx_kv_pool* pool, const int32_t* page_table, uint64_t base, const void* q, int q_f16, uint64_t tokens,
                   uint64_t heads, float scale, const float* gate, uint64_t gate_stride, uint64_t gate_row_stride, void* out, int out_f16,
                   const int32_t* union_pos, const uint32_t* union_mask, const uint32_t* union_count, unsigned union_cap) {
    PrefillArgs args{};
    args.pages = static_cast<const uint8_t*>(pool->pages);
    args.page_tokens = pool->page_tokens; args.kv_heads = pool->kv_heads; args.heads = unsigned(heads);
    args.group = unsigned(heads / pool->kv_heads); args.span = unsigned(tokens);
    args.page_table = page_table; args.table_stride = 0; args.positions = nullptr;
    args.q = q; args.q_f16 = q_f16; args.scale_log2 = scale * 1.44269504088896341f;
    args.rows = unsigned(tokens * args.group); args.max_context = 0;
    args.page_last = unsigned(std::min<uint64_t>(pool->page_count - 1, 0x7fffffffu));
    args.out = out; args.out_f16 = out_f16;
    args.union_pos = union_pos; args.union_mask = union_mask; args.union_count = union_count; args.union_cap = union_cap;
    args.base = int(base); args.gate = gate; args.gate_stride = size_t(gate_stride); args.gate_row_stride = size_t(gate_row_stride);
    const bool q8 = pool->row_bytes != 2 * pool->dim;
    const auto go = [&](auto kernel, size_t stage_bytes) {
        const size_t merge = size_t(GROUPS) * (256 / 16 * 4 + 2) * 64 * 4, ring = stages_for(int(stage_bytes)) * stage_bytes;
        const size_t shared = ring > merge ? ring : merge;
        if (shared > 64 * 1024) raise_shared_limit(d, reinterpret_cast<const void*>(kernel), shared);
        const unsigned tiles = (args.rows + GROUPS * 16 - 1) / (GROUPS * 16);
        timed_launch(d, kernel, dim3(tiles, args.kv_heads, 1), dim3(TEAM * 64), shared, args);
    };
    if (q8) go(&prefill_attention_kernel<256, 1, true, 2, true>, size_t(2) * WALK * (256 + 16));
    else go(&prefill_attention_kernel<256, 1, false, 2, true>, size_t(2) * WALK * 512);
}

}  // namespace sd
