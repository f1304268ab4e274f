// Selection-list attention over Q8_0 / FP16 K/V rows of 256 columns: every query row attends the positions its own list
// names.  Stands in for the reference's qsa_attention / qsa_attention_rows (gpu/sparse_attention_compute.hpp:609-647:
// qsa_decode_parts :41-135, block = 32 selected keys x 1 K/V head x all grouped query heads, and qsa_decode_merge :139-170),
// with the validity rule of attention_scores (gpu/kernels.cpp:100-165: an entry counts iff 0 <= raw <= position and
// raw < context) and the output gate qsa_gate (gpu/sparse_attention.hpp:439-442, sigmoid as gpu/core.hpp:1108-1111).
//
// Shape of the work on gfx950: a workgroup of 4 waves owns (row, K/V head, 128 entries of the row's list); a wave takes 32
// entries, one per lane for the address arithmetic (list entry -> position -> page -> row address), and gathers the 32 K rows
// and 32 V rows into its LDS stage by 16-byte global->LDS loads whose lanes each name their own piece of a row (a row is 17 or
// 32 such pieces), so a gathered step lands in the stage exactly as a contiguous step of the paged decode kernel does and the
// operand code (paged_rows.hpp) is shared: S^T = K . Q^T and O^T += V^T . P^T on v_mfma_f32_16x16x32_f16 with the group's
// query heads (up to 16) as one tile.  The four waves merge through LDS; the workgroups' partial results (maximum, sum,
// unnormalised output) are merged, normalised and gated by a second kernel, a block per (row, head).
#include "paged_rows.hpp"

using namespace sd;
using namespace sd::paged;

namespace sd {
void validate_pool(Device& d, const sdx_kv_pool* pool);
}

namespace {

constexpr int DIM = 256, CHUNK = WAVES * STEP;       // list entries per workgroup

struct SelectedArgs {
    const uint8_t* pages;
    unsigned page_tokens, kv_heads, heads, group;
    const int32_t* page_table;     // null: one page holds the context
    unsigned page_last;            // the pool's last page (table entries outside the pool are taken as the nearest page of it)
    size_t context, base;
    const uint32_t* dynamic_base;
    const float* indices;
    size_t selected;
    const float* counts;
    const void* q;
    int q_f16;
    float scale_log2;
    float* partial;                // [row][kv head][chunk][16][DIM + 2]
    unsigned chunks;
};

__device__ __forceinline__ unsigned list_length(const SelectedArgs& a, size_t row) {
    const float c = a.counts[row];
    return c > 0.0f ? unsigned(min(size_t(c), a.selected)) : 0u;
}

template<bool Q8>
__global__ void __launch_bounds__(WAVES * 64) selected_attention_kernel(SelectedArgs a) {
    constexpr int ROW = Q8 ? DIM + DIM / 16 : 2 * DIM, BLOCKS = DIM / 32, W = DIM / 16, TILES = DIM / 16;
    constexpr int SLAB = STEP * ROW, PIECES = ROW / 16, UNITS = (STEP * PIECES + 63) / 64, STRIDE = DIM + 2;
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), li = lane & 15, g = lane >> 4;
    const unsigned chunk = blockIdx.x, kvh = blockIdx.y;
    const size_t row = blockIdx.z, position = (a.dynamic_base ? size_t(*a.dynamic_base) : a.base) + row;
    const unsigned count = list_length(a, row);
    if (chunk * CHUNK >= count) return;                 // (the merge knows how many chunks a row has)
    extern __shared__ float lds[];
    uint8_t* const stage = reinterpret_cast<uint8_t*>(lds) + wave * (2 * SLAB);
    const unsigned first = chunk * CHUNK + wave * STEP;  // the wave's entries: first + (0..31)

    floatx4 acc[TILES];
    #pragma unroll
    for (int jj = 0; jj < TILES; ++jj) acc[jj] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
    float m = NEG_BIG, l = 0.0f;
    if (first < count) {
        // the group's query heads as B operands: lane li holds head li (zeros past the group)
        half8 qf[BLOCKS];
        const bool real = li < int(a.group);
        const size_t at = (row * a.heads + kvh * a.group + (real ? li : 0)) * DIM;
        #pragma unroll
        for (int b = 0; b < BLOCKS; ++b) {
            half8 value = {};
            if (real) {
                if (a.q_f16) value = *reinterpret_cast<const half8*>(static_cast<const _Float16*>(a.q) + at + 32 * b + 8 * g);
                else {
                    const float* from = static_cast<const float*>(a.q) + at + 32 * b + 8 * g;
                    #pragma unroll
                    for (int i = 0; i < 8; ++i) value[i] = (_Float16)from[i];
                }
            }
            qf[b] = value;
        }
        // lane e < 32: entry first + e.  An entry that does not count is read from the row's own position (a written row:
        // its score is masked, its weight is zero).
        float raw = -1.0f;
        if (lane < STEP && first + lane < count) raw = a.indices[row * a.selected + first + lane];
        const bool counts_in = raw >= 0.0f && raw <= float(position) && raw < float(a.context);
        const uint64_t usable = __ballot(counts_in);
        const size_t token = counts_in ? size_t(raw) : min(position, a.context - 1);
        const size_t page = a.page_table ? size_t(pool_page(a.page_table[token / a.page_tokens], a.page_last)) : 0, in_page = a.page_table ? token % a.page_tokens : token;
        const size_t plane_bytes = size_t(a.page_tokens) * ROW;
        const uint8_t* const krow = a.pages + (page * 2 * a.kv_heads + kvh) * plane_bytes + in_page * ROW;
        settle_loads();
        #pragma unroll
        for (int part = 0; part < 2; ++part) {
            #pragma unroll
            for (int j = 0; j < UNITS; ++j) {
                const int piece = 64 * j + lane, entry = piece / PIECES, within = piece % PIECES;
                const uint64_t from = __shfl(uint64_t(reinterpret_cast<uintptr_t>(krow)), entry & 31);
                if (64 * j + 64 <= STEP * PIECES || piece < STEP * PIECES)
                    load_to_lds<false>(reinterpret_cast<const uint8_t*>(from) + size_t(part ? a.kv_heads : 0) * plane_bytes + 16 * within,
                                       stage + part * SLAB + 1024 * j);
            }
        }
        __builtin_amdgcn_s_waitcnt(0x0f70);             // vmcnt(0): the gathered rows have landed
        RowLoad<DIM, Q8> current;
        load_step<DIM>(current, stage, stage + SLAB, li, g);
        floatx4 s[2];
        #pragma unroll
        for (int t = 0; t < 2; ++t) {
            s[t] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
            #pragma unroll
            for (int b = 0; b < BLOCKS; ++b) s[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(key_operand<DIM>(current, t, b), qf[b], s[t], 0, 0, 0);
            #pragma unroll
            for (int r = 0; r < 4; ++r)
                if (!((usable >> (16 * t + 4 * g + r)) & 1)) s[t][r] = -INFINITY;
        }
        const float top = row_max(fmaxf(fmaxf(fmaxf(s[0][0], s[0][1]), fmaxf(s[0][2], s[0][3])), fmaxf(fmaxf(s[1][0], s[1][1]), fmaxf(s[1][2], s[1][3]))));
        m = fmaxf(m, top);
        const float offset = -m * a.scale_log2;
        half8 p;
        #pragma unroll
        for (int t = 0; t < 2; ++t)
            #pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float w = __builtin_amdgcn_exp2f(fmaf(s[t][r], a.scale_log2, offset));
                l += w;
                p[4 * t + r] = (_Float16)w;
            }
        ValueScales<DIM> vs;
        value_scales<DIM>(current, vs);
        #pragma unroll
        for (int jj = 0; jj < TILES; ++jj) acc[jj] = __builtin_amdgcn_mfma_f32_16x16x32_f16(value_operand<DIM>(current, vs, jj), p, acc[jj], 0, 0, 0);
    }

    // Merge the waves through LDS: per wave and query head the maximum, the sum and the unnormalised output.
    __syncthreads();    // the merge area overlays the stages
    {
        const float sum = row_sum(l);
        float* mine = lds + (size_t(wave) * 16 + li) * STRIDE;
        if (g == 0) { mine[DIM] = m * a.scale_log2; mine[DIM + 1] = sum; }      // maxima leave in exponent units
        #pragma unroll
        for (int jj = 0; jj < TILES; ++jj)
            #pragma unroll
            for (int r = 0; r < 4; ++r) mine[W * (4 * g + r) + jj] = acc[jj][r];
    }
    __syncthreads();
    float* out = a.partial + ((row * a.kv_heads + kvh) * a.chunks + chunk) * 16 * STRIDE;
    for (unsigned i = threadIdx.x; i < a.group * STRIDE; i += WAVES * 64) {
        const unsigned head = i / STRIDE, col = i % STRIDE;
        float top = NEG_BIG;
        #pragma unroll
        for (int w = 0; w < WAVES; ++w) top = fmaxf(top, lds[(size_t(w) * 16 + head) * STRIDE + DIM]);
        float value;
        if (col == DIM) value = top;
        else {
            value = 0.0f;
            #pragma unroll
            for (int w = 0; w < WAVES; ++w) {
                const float* other = lds + (size_t(w) * 16 + head) * STRIDE;
                value += other[col] * __builtin_amdgcn_exp2f(other[DIM] - top);
            }
        }
        out[i] = value;
    }
}

// A block per (row, head), a thread per column: the row's chunks merged, normalised, gated.
template<bool F16_OUT>
__global__ void __launch_bounds__(DIM) selected_merge_kernel(SelectedArgs a, const float* gate, size_t gate_stride, size_t gate_row_stride, void* out) {
    constexpr int STRIDE = DIM + 2;
    const size_t row = blockIdx.x / a.heads;
    const unsigned head = blockIdx.x % a.heads, kvh = head / a.group, col = threadIdx.x;
    const unsigned used = (list_length(a, row) + CHUNK - 1) / CHUNK;
    const float* base = a.partial + ((row * a.kv_heads + kvh) * a.chunks) * 16 * STRIDE + size_t(head % a.group) * STRIDE;
    // the chunks' pieces are asked for eight at a time: eight loads in flight, not one after the other
    constexpr unsigned AT_ONCE = 8;
    float top = NEG_BIG;
    for (unsigned c0 = 0; c0 < used; c0 += AT_ONCE) {
        float tops[AT_ONCE];
        #pragma unroll
        for (unsigned i = 0; i < AT_ONCE; ++i) tops[i] = base[size_t(min(c0 + i, used - 1)) * 16 * STRIDE + DIM];
        #pragma unroll
        for (unsigned i = 0; i < AT_ONCE; ++i) top = fmaxf(top, tops[i]);
    }
    float sum = 0.0f, value = 0.0f;
    for (unsigned c0 = 0; c0 < used; c0 += AT_ONCE) {
        float tops[AT_ONCE], sums[AT_ONCE], values[AT_ONCE];
        #pragma unroll
        for (unsigned i = 0; i < AT_ONCE; ++i) {
            const float* part = base + size_t(min(c0 + i, used - 1)) * 16 * STRIDE;
            tops[i] = part[DIM]; sums[i] = part[DIM + 1]; values[i] = part[col];
        }
        #pragma unroll
        for (unsigned i = 0; i < AT_ONCE; ++i) {
            const float weight = c0 + i < used ? __builtin_amdgcn_exp2f(tops[i] - top) : 0.0f;
            sum += sums[i] * weight;
            value += values[i] * weight;
        }
    }
    value = sum > 0.0f ? value / sum : 0.0f;
    if (gate) {
        const float x = gate[row * gate_row_stride + head * gate_stride + col], e = expf(-fabsf(x));
        value *= x >= 0.0f ? 1.0f / (1.0f + e) : e / (1.0f + e);
    }
    const size_t at = (row * a.heads + head) * DIM + col;
    if (F16_OUT) static_cast<_Float16*>(out)[at] = (_Float16)value;
    else static_cast<float*>(out)[at] = value;
}

uint64_t scratch_bytes_for(uint64_t rows, uint64_t kv_heads, uint64_t selected) {
    return checked_floats({rows, kv_heads, (selected + CHUNK - 1) / CHUNK, 16, uint64_t(DIM) + 2});
}

template<bool Q8>
void launch(Device& d, const SelectedArgs& args, size_t rows) {
    constexpr int ROW = Q8 ? DIM + DIM / 16 : 2 * DIM;
    const size_t shared = std::max<size_t>(size_t(WAVES) * 2 * STEP * ROW, size_t(WAVES) * 16 * (DIM + 2) * 4);
    raise_shared_limit(d, reinterpret_cast<const void*>(&selected_attention_kernel<Q8>), shared);
    timed_launch(d, &selected_attention_kernel<Q8>, dim3(args.chunks, args.kv_heads, unsigned(rows)), dim3(WAVES * 64), shared, args);
}

}  // namespace

extern "C" {

uint64_t sdx_selected_attention_scratch(uint64_t rows, uint64_t kv_heads, uint64_t selected) {
    try { return scratch_bytes_for(rows, kv_heads, selected); } catch (const std::exception&) { return 0; }
}

int sdx_selected_attention(void* handle, const sdx_kv_pool* pool, const int32_t* page_table, uint64_t context, uint64_t base,
                           const uint32_t* dynamic_base, const float* indices, uint64_t selected, const float* counts, const void* q, int q_f16,
                           uint64_t rows, uint64_t heads, float scale, const float* gate, uint64_t gate_stride, uint64_t gate_row_stride, void* out, int out_f16,
                           void* scratch, uint64_t scratch_bytes) {
    SD_OP_BEGIN
    validate_pool(value, pool);
    if (pool->dim != DIM) throw std::runtime_error("sdx_selected_attention: rows of 256 columns");
    if (!(scale > 0.0f) || !rows || rows > 65535 || !heads || heads % pool->kv_heads || heads / pool->kv_heads > 16 || !selected || !context ||
        context > (uint64_t(1) << 24) || pool->kv_heads > 65535)
        throw std::runtime_error("sdx_selected_attention: rows, heads (a multiple of the K/V heads, at most 16 each), selected and context >= 1, scale > 0");
    const uint64_t pages = (context + pool->page_tokens - 1) / pool->page_tokens;
    if (page_table) op_span(value, page_table, checked_floats({pages}), "a page table");
    else if (pool->page_tokens < context) throw std::runtime_error("sdx_selected_attention: without a page table one page must hold the context");
    if (!dynamic_base && base + rows > context) throw std::runtime_error("sdx_selected_attention: rows past the context");
    if (dynamic_base) op_span(value, dynamic_base, 4, "a position");
    op_span(value, indices, checked_floats({rows, selected}), "selection lists");
    op_span(value, counts, checked_floats({rows}), "selection counts");
    op_span(value, q, checked_product({rows, heads, uint64_t(DIM), q_f16 ? 2u : 4u}), "attention queries");
    op_span(value, out, checked_product({rows, heads, uint64_t(DIM), out_f16 ? 2u : 4u}), "an attention output");
    if (gate) {
        if (!gate_row_stride) gate_row_stride = heads * gate_stride;
        if (gate_stride < DIM || gate_row_stride < (heads - 1) * gate_stride + DIM) throw std::runtime_error("sdx_selected_attention: gate strides below a head's 256 values or a row's heads");
        op_span(value, gate, checked_floats({rows - 1, gate_row_stride}) + ((heads - 1) * gate_stride + DIM) * 4, "an attention gate");
    }
    const size_t need = scratch_bytes_for(rows, pool->kv_heads, selected);
    if (scratch_bytes < need) throw std::runtime_error("sdx_selected_attention: scratch too small (see sdx_selected_attention_scratch)");
    op_span(value, scratch, need, "attention scratch");
    SelectedArgs args{};
    args.pages = static_cast<const uint8_t*>(pool->pages);
    args.page_tokens = pool->page_tokens; args.kv_heads = pool->kv_heads; args.heads = unsigned(heads); args.group = unsigned(heads / pool->kv_heads);
    args.page_table = page_table; args.page_last = unsigned(std::min<uint64_t>(pool->page_count - 1, 0x7fffffffu)); args.context = context; args.base = base; args.dynamic_base = dynamic_base;
    args.indices = indices; args.selected = selected; args.counts = counts; args.q = q; args.q_f16 = q_f16;
    args.scale_log2 = scale * 1.4426950408889634f;
    args.partial = static_cast<float*>(scratch);
    args.chunks = unsigned((selected + CHUNK - 1) / CHUNK);
    if (pool->row_bytes != 2 * pool->dim) launch<true>(value, args, rows); else launch<false>(value, args, rows);
    SD_CHECK(hipGetLastError());
    if (out_f16) selected_merge_kernel<true><<<unsigned(rows * heads), DIM, 0, value.stream>>>(args, gate, gate_stride, gate_row_stride, out);
    else selected_merge_kernel<false><<<unsigned(rows * heads), DIM, 0, value.stream>>>(args, gate, gate_stride, gate_row_stride, out);
    SD_OP_END
}

}  // extern "C"
