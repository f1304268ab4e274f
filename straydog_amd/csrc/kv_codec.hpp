// Device-side reading and writing of K/V rows: the reference's kv_load / kv_encode / kv_put (gpu/kernels.cpp:37-74)
// for rows of any width that is a multiple of 32.
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cstdint>

namespace sd {

// Column `column` of a row: Q8_0 (`dim` int8 then dim/32 FP16 scales) or FP16 (row_bytes == 2 * dim).
__device__ __forceinline__ float kv_value(const uint8_t* row, unsigned column, unsigned dim, bool q8) {
    if (q8) return float(reinterpret_cast<const int8_t*>(row)[column]) * __half2float(reinterpret_cast<const __half*>(row + dim)[column / 32]);
    return __half2float(reinterpret_cast<const __half*>(row)[column]);
}

// The Q8_0 encoding of four consecutive values of a 32-value block: their four bytes and the block's scale.  The 8 lanes that
// hold the block are adjacent (lane % 8 = quad within the block) and must all call this together.
__device__ __forceinline__ void kv_quad_q8(const float (&x)[4], uint32_t& word, __half& scale16) {
    float top = fmaxf(fmaxf(fabsf(x[0]), fabsf(x[1])), fmaxf(fabsf(x[2]), fabsf(x[3])));
    top = fmaxf(top, __shfl_xor(top, 1));
    top = fmaxf(top, __shfl_xor(top, 2));
    top = fmaxf(top, __shfl_xor(top, 4));
    scale16 = __float2half_rn(top / 127.0f);
    const float scale = __half2float(scale16);
    word = 0;
    #pragma unroll
    for (int i = 0; i < 4; ++i) {
        int q = scale > 0.0f ? __float2int_rn(x[i] / scale) : 0;
        q = q > 127 ? 127 : q < -127 ? -127 : q;
        word |= uint32_t(uint8_t(int8_t(q))) << (8 * i);
    }
}

// Four consecutive values (column a multiple of 4) stored into a row.  The 8 lanes that hold one 32-value block
// are adjacent (lane % 8 = quad within the block) and must all call this together.
__device__ __forceinline__ void kv_store_quad(uint8_t* row, unsigned quad, unsigned dim, bool q8, const float (&x)[4], bool live) {
    if (!q8) {
        if (!live) return;
        const __half2 a = __halves2half2(__float2half_rn(x[0]), __float2half_rn(x[1]));
        const __half2 b = __halves2half2(__float2half_rn(x[2]), __float2half_rn(x[3]));
        uint2 packed;
        packed.x = *reinterpret_cast<const uint32_t*>(&a); packed.y = *reinterpret_cast<const uint32_t*>(&b);
        *reinterpret_cast<uint2*>(row + quad * 8) = packed;
        return;
    }
    uint32_t word;
    __half scale16;
    kv_quad_q8(x, word, scale16);
    if (!live) return;
    *reinterpret_cast<uint32_t*>(row + quad * 4) = word;
    if (quad % 8 == 0) *reinterpret_cast<__half*>(row + dim + quad / 8 * 2) = scale16;
}

}  // namespace sd
