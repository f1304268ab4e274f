// The sum of one float per thread of a workgroup in the order of a halving tree -- sums[c] += sums[c + offset] for offset =
// width / 2, width / 4, ..., 1 -- which is the order the reference's block reductions use (gpu/ops.hpp:28-38,
// gpu/sparse_attention.hpp:14-17), so sums of squares come out with the same bits.  The levels below 64 are lane shifts inside
// the first wave: lane c < offset adds lane c + offset, whose value is still the tree's at that level.
#pragma once
#include <hip/hip_runtime.h>

namespace sd {

// `width` = the workgroup's threads (a power of two, 64 .. 1024); `sums` = width floats of LDS.  Every thread calls it and
// every thread gets the sum.
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
    const float total = sums[0];
    __syncthreads();       // (sums may be written again at once)
    return total;
}

}  // namespace sd
