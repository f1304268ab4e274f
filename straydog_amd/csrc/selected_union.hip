// Selection-list attention for the rows of a prompt chunk as a union walk: the tokens whose query rows share a tile of the
// attention kernel (64 rows: 16 x the heads of a K/V head, five or six tokens of Qwen's 12 heads a K/V head) walk the union of
// their selections once, each entry's K/V row converted once for all of them, with a bit per (entry, token) saying whose it is.
//
// The reference's form of this is qsa_flash_wmma over qsa_mark_blocks / qsa_union_blocks (gpu/sparse_attention_compute.hpp:744-755,
// 841-896, 906-1041: groups of 16 tokens, blocks of four positions, 24 waves), which it measured slower than its per-token kernel
// on its cards.  Here the walk is the 256-column prefill kernel itself (prefill_attention.hip) with two switches -- the step's
// rows come from a list, the mask from the list's bits -- so the matrix cores' room is what pays for the entries a token did not
// select: consecutive tokens of a real prompt select mostly the same blocks, and a K/V row is then converted once for 64 query
// rows instead of once for 16.  On selections that do not overlap (random queries) it has nothing to gain over
// sdx_selected_attention.
//
// Three launches before the walk: marks[tile][position] |= bit(token) for every entry that counts (at most the token's own
// position, inside the context; sdx_selected_attention's rule); the counts of marked positions per 4096-position segment;
// the ordered lists (position, mask) of every tile.  Any list does, sorted or not; an entry named twice counts once.
#include "device.hpp"
#include "../../include/straydog_gpu_ext.h"

#include <algorithm>

using namespace sd;

namespace sd {
void validate_pool(Device& d, const sdx_kv_pool* pool);
unsigned union_tile_rows();
void prefill_union(Device& d, const sdx_kv_pool* pool, const int32_t* page_table, uint64_t base, const void* q, int q_f16, uint64_t tokens,
                   uint64_t heads, float scale, const float* gate, uint64_t gate_stride, uint64_t gate_row_stride, void* out, int out_f16,
                   const int32_t* union_pos, const uint32_t* union_mask, const uint32_t* union_count, unsigned union_cap);
}

namespace {

constexpr int SEGMENT = 4096, PER_THREAD = SEGMENT / 256;

struct UnionSpace {
    uint32_t* marks;        // [tiles][context rounded up to segments]
    uint32_t* segment;      // [tiles][segments] marked positions of a segment
    int32_t* pos;           // [tiles][cap] where the entry's K row (K/V head 0) lies in the pool, in 16-byte units
    uint32_t* mask;         // [tiles][cap]
    uint32_t* count;        // [tiles]
    size_t tiles, segments, cap, bytes;
};

UnionSpace lay_out(void* scratch, size_t tokens, size_t group, size_t selected, size_t context) {
    UnionSpace s{};
    const size_t tile_rows = union_tile_rows();
    s.tiles = (tokens * group + tile_rows - 1) / tile_rows;
    s.segments = (context + SEGMENT - 1) / SEGMENT;
    const size_t tile_tokens = (tile_rows + group - 1) / group + 1;                // tokens with a row in one tile, at most
    s.cap = (std::min(tile_tokens * selected, context) + 63) / 64 * 64 + 64;
    uint8_t* at = static_cast<uint8_t*>(scratch);
    const auto take = [&](size_t bytes) { uint8_t* here = at; at += (bytes + 255) & ~size_t(255); return here; };
    s.marks = reinterpret_cast<uint32_t*>(take(s.tiles * s.segments * SEGMENT * 4));
    s.segment = reinterpret_cast<uint32_t*>(take(s.tiles * s.segments * 4));
    s.pos = reinterpret_cast<int32_t*>(take(s.tiles * s.cap * 4));
    s.mask = reinterpret_cast<uint32_t*>(take(s.tiles * s.cap * 4));
    s.count = reinterpret_cast<uint32_t*>(take(s.tiles * 4));
    s.bytes = size_t(at - static_cast<uint8_t*>(scratch));
    return s;
}

__global__ void __launch_bounds__(256) union_clear_kernel(uint4* marks, size_t count) {
    for (size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x; i < count; i += size_t(gridDim.x) * blockDim.x) marks[i] = make_uint4(0u, 0u, 0u, 0u);
}

// A workgroup per token: its entries that count set the token's bit at their positions, in every tile the token has rows in.
__global__ void __launch_bounds__(256) union_mark_kernel(const float* __restrict__ indices, size_t selected, const float* __restrict__ counts, size_t base,
                                                         size_t context, unsigned group, unsigned tile_rows, size_t stride, uint32_t* __restrict__ marks) {
    const size_t token = blockIdx.x, position = base + token;
    const float c = counts[token];
    const unsigned count = c > 0.0f ? unsigned(min(size_t(c), selected)) : 0u;
    const unsigned first_tile = unsigned(token * group / tile_rows), last_tile = unsigned((token * group + group - 1) / tile_rows);
    for (unsigned i = threadIdx.x; i < count; i += 256) {
        const float raw = indices[token * selected + i];
        if (!(raw >= 0.0f && raw <= float(position) && raw < float(context))) continue;
        for (unsigned tile = first_tile; tile <= last_tile; ++tile)
            atomicOr(&marks[size_t(tile) * stride + size_t(raw)], 1u << unsigned(token - size_t(tile) * tile_rows / group));
    }
}

// The marked positions of every (tile, segment), counted.
__global__ void __launch_bounds__(256) union_count_kernel(const uint32_t* __restrict__ marks, size_t stride, unsigned segments, uint32_t* __restrict__ segment) {
    __shared__ uint32_t sums[4];
    const unsigned tile = blockIdx.y, seg = blockIdx.x, t = threadIdx.x;
    const uint4* from = reinterpret_cast<const uint4*>(marks + size_t(tile) * stride + size_t(seg) * SEGMENT + t * PER_THREAD);
    uint32_t mine = 0;
    #pragma unroll
    for (int i = 0; i < PER_THREAD / 4; ++i) { const uint4 four = from[i]; mine += (four.x != 0) + (four.y != 0) + (four.z != 0) + (four.w != 0); }
    #pragma unroll
    for (int offset = 32; offset; offset /= 2) mine += __shfl_xor(mine, offset);
    if (t % 64 == 0) sums[t / 64] = mine;
    __syncthreads();
    if (t == 0) segment[size_t(tile) * segments + seg] = sums[0] + sums[1] + sums[2] + sums[3];
}

// The lists in position order: a workgroup per (tile, segment) knows how many marked positions lie before its segment, a thread
// how many before its 16 positions.  A tile without any entry gets one that nobody selected (the walk needs a row to read).
__global__ void __launch_bounds__(256) union_list_kernel(const uint32_t* __restrict__ marks, size_t stride, unsigned segments, const uint32_t* __restrict__ segment,
                                                         size_t cap, size_t base, const int32_t* __restrict__ page_table, unsigned page_tokens,
                                                         unsigned page_last, size_t plane16, unsigned row16, unsigned kv_heads,
                                                         int32_t* __restrict__ pos, uint32_t* __restrict__ mask, uint32_t* __restrict__ count) {
    __shared__ uint32_t sums[4], before_segment, total;
    const unsigned tile = blockIdx.y, seg = blockIdx.x, t = threadIdx.x, lane = t % 64, wave = t / 64;
    {
        uint32_t before = 0, all = 0;
        for (unsigned s = t; s < segments; s += 256) { const uint32_t n = segment[size_t(tile) * segments + s]; all += n; before += s < seg ? n : 0u; }
        #pragma unroll
        for (int offset = 32; offset; offset /= 2) { before += __shfl_xor(before, offset); all += __shfl_xor(all, offset); }
        if (lane == 0) { sums[wave] = before; }
        __syncthreads();
        if (t == 0) before_segment = sums[0] + sums[1] + sums[2] + sums[3];
        __syncthreads();
        if (lane == 0) sums[wave] = all;
        __syncthreads();
        if (t == 0) total = sums[0] + sums[1] + sums[2] + sums[3];
        __syncthreads();
    }
    // a position's place: its page's K plane of K/V head 0, its row in the page (16-byte units; a row is 17 or 32 of them)
    const auto place = [&](size_t position) {
        const size_t page = page_table ? size_t(min(unsigned(page_table[position / page_tokens]), page_last)) : 0, in_page = page_table ? position % page_tokens : position;
        return int32_t(page * 2 * kv_heads * plane16 + in_page * row16);
    };
    if (seg == 0 && t == 0) {
        count[tile] = max(total, 1u);
        if (total == 0) { pos[size_t(tile) * cap] = place(base); mask[size_t(tile) * cap] = 0u; }
    }
    const uint32_t* from = marks + size_t(tile) * stride + size_t(seg) * SEGMENT + t * PER_THREAD;
    uint32_t held[PER_THREAD], mine = 0;
    #pragma unroll
    for (int i = 0; i < PER_THREAD / 4; ++i) {
        const uint4 four = reinterpret_cast<const uint4*>(from)[i];
        held[4 * i] = four.x; held[4 * i + 1] = four.y; held[4 * i + 2] = four.z; held[4 * i + 3] = four.w;
    }
    #pragma unroll
    for (int i = 0; i < PER_THREAD; ++i) mine += held[i] != 0;
    uint32_t running = mine;
    #pragma unroll
    for (int offset = 1; offset < 64; offset *= 2) {
        const uint32_t other = __shfl_up(running, offset);
        if (lane >= unsigned(offset)) running += other;
    }
    __syncthreads();
    if (lane == 63) sums[wave] = running;
    __syncthreads();
    size_t at = before_segment + running - mine;
    for (unsigned w = 0; w < wave; ++w) at += sums[w];
    #pragma unroll
    for (int i = 0; i < PER_THREAD; ++i)
        if (held[i] != 0 && at < cap) {
            pos[size_t(tile) * cap + at] = place(size_t(seg) * SEGMENT + t * PER_THREAD + i);
            mask[size_t(tile) * cap + at] = held[i];
            ++at;
        }
}

}  // namespace

extern "C" {

uint64_t sdx_selected_attention_union_scratch(uint64_t rows, uint64_t heads, uint64_t kv_heads, uint64_t selected, uint64_t context) {
    try {
        if (!rows || !kv_heads || !heads || heads % kv_heads || !selected || !context) return 0;
        return lay_out(nullptr, size_t(checked_product({rows, 1})), size_t(heads / kv_heads), size_t(checked_product({selected, 1})),
                       size_t(checked_product({context, 1}))).bytes;
    } catch (const std::exception&) { return 0; }
}

int sdx_selected_attention_union(void* handle, const sdx_kv_pool* pool, const int32_t* page_table, uint64_t context, uint64_t base,
                                 const float* indices, uint64_t selected, const float* counts, const void* q, int q_f16, uint64_t rows, uint64_t heads,
                                 float scale, const float* gate, uint64_t gate_stride, uint64_t gate_row_stride, void* out, int out_f16, void* scratch,
                                 uint64_t scratch_bytes) {
    SD_OP_BEGIN
    validate_pool(value, pool);
    if (pool->dim != 256) throw std::runtime_error("sdx_selected_attention_union: rows of 256 columns");
    // (a tile of 64 query rows holds 64 / group tokens, and an entry's mask has 32 bits)
    if (!(scale > 0.0f) || !rows || rows > 65535 || !heads || heads % pool->kv_heads || heads / pool->kv_heads > 16 || heads / pool->kv_heads < 2 ||
        !selected || !context || context > (uint64_t(1) << 24) || pool->kv_heads > 65535 || selected > (uint64_t(1) << 20))
        throw std::runtime_error("sdx_selected_attention_union: rows, heads (a multiple of the K/V heads, 2 to 16 each), selected and context >= 1, scale > 0");
    const uint64_t pages = (context + pool->page_tokens - 1) / pool->page_tokens;
    if (page_table) op_span(value, page_table, checked_floats({pages}), "a page table");
    else if (pool->page_tokens < context) throw std::runtime_error("sdx_selected_attention_union: without a page table one page must hold the context");
    if (base + rows > context) throw std::runtime_error("sdx_selected_attention_union: rows past the context");
    op_span(value, indices, checked_floats({rows, selected}), "selection lists");
    op_span(value, counts, checked_floats({rows}), "selection counts");
    op_span(value, q, checked_product({rows, heads, 256, q_f16 ? 2u : 4u}), "attention queries");
    op_span(value, out, checked_product({rows, heads, 256, out_f16 ? 2u : 4u}), "an attention output");
    if (gate) {
        if (!gate_row_stride) gate_row_stride = heads * gate_stride;
        if (gate_stride < 256 || gate_row_stride < (heads - 1) * gate_stride + 256) throw std::runtime_error("sdx_selected_attention_union: gate strides below a head's 256 values or a row's heads");
        op_span(value, gate, checked_floats({rows - 1, gate_row_stride}) + ((heads - 1) * gate_stride + 256) * 4, "an attention gate");
    }
    const size_t group = size_t(heads / pool->kv_heads);
    const UnionSpace s = lay_out(scratch, rows, group, selected, context);
    if (scratch_bytes < s.bytes) throw std::runtime_error("sdx_selected_attention_union: scratch too small (see sdx_selected_attention_union_scratch)");
    op_span(value, scratch, s.bytes, "attention scratch");
    const size_t stride = s.segments * SEGMENT;
    union_clear_kernel<<<unsigned(std::min<size_t>(s.tiles * stride / 4 / 256 + 1, 4096)), 256, 0, value.stream>>>(reinterpret_cast<uint4*>(s.marks), s.tiles * stride / 4);
    union_mark_kernel<<<unsigned(rows), 256, 0, value.stream>>>(indices, selected, counts, base, context, unsigned(group), union_tile_rows(), stride, s.marks);
    union_count_kernel<<<dim3(unsigned(s.segments), unsigned(s.tiles)), 256, 0, value.stream>>>(s.marks, stride, unsigned(s.segments), s.segment);
    const size_t row_bytes = pool->row_bytes, plane_bytes = size_t(pool->page_tokens) * row_bytes;
    if (checked_product({pool->page_count, 2, pool->kv_heads, uint64_t(plane_bytes)}) / 16 > 0x7fffffffu)
        throw std::runtime_error("sdx_selected_attention_union: a pool of more than 32 GiB");
    union_list_kernel<<<dim3(unsigned(s.segments), unsigned(s.tiles)), 256, 0, value.stream>>>(
        s.marks, stride, unsigned(s.segments), s.segment, s.cap, base, page_table, pool->page_tokens,
        unsigned(std::min<uint64_t>(pool->page_count - 1, 0x7fffffffu)), plane_bytes / 16, unsigned(row_bytes / 16), pool->kv_heads, s.pos, s.mask, s.count);
    SD_CHECK(hipGetLastError());
    prefill_union(value, pool, page_table, base, q, q_f16, rows, heads, scale, gate, gate_stride, gate_row_stride, out, out_f16, s.pos, s.mask, s.count,
                  unsigned(s.cap));
    SD_OP_END
}

}  // extern "C"
