// Appending rows to the paged K/V cache.
// The Q8_0 arithmetic is the reference's kv_encode/kv_put (gpu/kernels.cpp:58-74): scale = f16(max|x| / 127) over a
// 32-value block, q = clamp(rint(x / f32(scale)), -127, 127), q = 0 when the scale is 0.
#include "device.hpp"
#include "kv_codec.hpp"
#include "../../include/straydog_gpu_ext.h"

#include <hip/hip_fp16.h>

using namespace sd;

namespace {

// A thread holds 4 consecutive values of a row; the 8 threads of a 32-value block are adjacent lanes, so the
// block's largest magnitude is three xor-shuffles away.  One 4-byte store per thread; lane 0 of a block stores the scale.
template<bool F16_IN>
__global__ void __launch_bounds__(256) kv_write_kernel(uint8_t* pages, size_t page_count, unsigned page_tokens, unsigned kv_heads, unsigned dim, unsigned row_bytes,
                                                       const int32_t* page_table, size_t table_stride, const int32_t* positions,
                                                       const void* keys, const void* values, size_t span, size_t total) {
    const size_t index = size_t(blockIdx.x) * blockDim.x + threadIdx.x;   // one per 4 values of [K|V][seq][row][head][dim/4]
    const bool live = index < total;
    const size_t quads = dim / 4, per_kind = total / 2;
    const size_t at = live ? index % per_kind : 0;
    const bool is_value = live && index >= per_kind;
    const size_t quad = at % quads, head = at / quads % kv_heads, row = at / quads / kv_heads % span, seq = at / quads / kv_heads / span;
    const void* source = is_value ? values : keys;
    float x[4];
    const size_t first = ((seq * span + row) * kv_heads + head) * dim + quad * 4;
    if (F16_IN) {
        const uint2 raw = *reinterpret_cast<const uint2*>(static_cast<const __half*>(source) + first);
        const __half2 a = *reinterpret_cast<const __half2*>(&raw.x), b = *reinterpret_cast<const __half2*>(&raw.y);
        x[0] = __low2float(a); x[1] = __high2float(a); x[2] = __low2float(b); x[3] = __high2float(b);
    } else {
        const float4 raw = *reinterpret_cast<const float4*>(static_cast<const float*>(source) + first);
        x[0] = raw.x; x[1] = raw.y; x[2] = raw.z; x[3] = raw.w;
    }
    // The positions are device-resident (a replayed graph advances them there), so the host cannot check them: a row whose
    // position is negative or past the sequence's table row, or whose table entry names no page of the pool, is not stored.
    const long long first_position = positions[seq];
    const size_t position = size_t(first_position < 0 ? 0 : first_position) + row;
    bool stored = live && first_position >= 0 && position < table_stride * page_tokens;
    const long long page = stored ? page_table[seq * table_stride + position / page_tokens] : 0;
    stored = stored && page >= 0 && size_t(page) < page_count;
    const size_t plane = is_value ? kv_heads + head : head;
    uint8_t* out = pages + ((size_t(stored ? page : 0) * 2 * kv_heads + plane) * page_tokens + position % page_tokens) * row_bytes;
    kv_store_quad(out, unsigned(quad), dim, row_bytes != 2 * dim, x, stored);
}

}  // namespace

namespace sd {
void validate_pool(Device& d, const sdx_kv_pool* pool) {
    if (!pool || !pool->pages || !pool->page_count || !pool->page_tokens || pool->page_tokens % 32 || !pool->kv_heads ||
        (pool->dim != 128 && pool->dim != 256) || (pool->row_bytes != pool->dim + pool->dim / 16 && pool->row_bytes != 2 * pool->dim))
        throw std::runtime_error("invalid Straydog K/V pool");
    op_span(d, pool->pages, checked_product({pool->page_count, 2, pool->kv_heads, pool->page_tokens, pool->row_bytes}), "a K/V pool");
    kv_settle(d);       // (every op that reads or writes pages passes here: it runs after the page moves queued so far)
}
}  // namespace sd

extern "C" {

int sdx_kv_write(void* handle, const sdx_kv_pool* pool, const int32_t* page_table, uint64_t table_stride, const int32_t* positions,
                 const void* keys, const void* values, int input_f16, uint64_t seqs, uint64_t span) {
    SD_OP_BEGIN
    validate_pool(value, pool);
    if (!seqs || !span || !table_stride) throw std::runtime_error("invalid Straydog K/V write shape");
    const size_t element = input_f16 ? 2 : 4;
    op_span(value, page_table, checked_floats({seqs, table_stride}), "a page table");
    op_span(value, positions, checked_floats({seqs}), "K/V positions");
    op_span(value, keys, checked_product({seqs, span, pool->kv_heads, pool->dim, element}), "new keys");
    op_span(value, values, checked_product({seqs, span, pool->kv_heads, pool->dim, element}), "new values");
    const size_t total = checked_product({2, seqs, span, pool->kv_heads, pool->dim / 4});
    auto* pages = static_cast<uint8_t*>(pool->pages);
    if (input_f16)
        kv_write_kernel<true><<<checked_blocks(total), 256, 0, value.stream>>>(pages, size_t(pool->page_count), pool->page_tokens, pool->kv_heads, pool->dim, pool->row_bytes,
            page_table, size_t(table_stride), positions, keys, values, size_t(span), total);
    else
        kv_write_kernel<false><<<checked_blocks(total), 256, 0, value.stream>>>(pages, size_t(pool->page_count), pool->page_tokens, pool->kv_heads, pool->dim, pool->row_bytes,
            page_table, size_t(table_stride), positions, keys, values, size_t(span), total);
    SD_OP_END
}

}  // extern "C"
