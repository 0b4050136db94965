// Block-level sum of squares shared by the norm kernels and the fused decode kernels.
#pragma once
#include "it_device.h"

namespace itk {

// ------------------------------------------------------------------ sum of squares
// Serial f64 accumulation of f32 squares (naive.rs:633-640) by one lane, or a tree.
// `buf` holds the row in LDS.  Returns the sum to every thread of the block.
template <int THREADS>
__device__ double block_sumsq(const float* buf, int n, int exact, double* red) {
    if (exact) {
        if (threadIdx.x == 0) {
            double sum = 0.0;
            for (int i = 0; i < n; i++) sum += (double)(buf[i] * buf[i]);
            red[0] = sum;
        }
        __syncthreads();
        return red[0];
    }
    double part = 0.0;
    for (int i = threadIdx.x; i < n; i += THREADS) part += (double)(buf[i] * buf[i]);
    for (int off = 32; off > 0; off >>= 1) part += __shfl_down(part, off, 64);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = part;
    __syncthreads();
    if (threadIdx.x == 0) {
        double sum = 0.0;
        for (int w = 0; w < THREADS / 64; w++) sum += red[w];
        red[0] = sum;
    }
    __syncthreads();
    return red[0];
}


// Sum over the 8 lanes of an aligned group with data-parallel-primitive moves (no LDS crossbar):
// neighbours, then pairs, then the mirrored half.  Every lane of the group ends with the total.
IT_DEV float sum8_lanes(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xf, 0xf, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xf, 0xf, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xf, 0xf, true));
    return v;
}

}  // namespace itk
