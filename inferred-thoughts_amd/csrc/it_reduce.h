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


// ------------------------------------------------------------------ lane exchanges without LDS
// DPP moves reach the lanes of a row of 16: neighbour (quad_perm 1,0,3,2), pair (quad_perm
// 2,3,0,1), the mirrored half of 8 and the mirrored row of 16.  After the first two steps a
// quad is uniform, after three a group of 8, so the mirrors pair each lane with one of the
// other half.  Across rows (offsets 16 and 32) the exchange goes through ds_bpermute.
IT_DEV float dpp_xor1(float v) { return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xf, 0xf, true)); }
IT_DEV float dpp_xor2(float v) { return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xf, 0xf, true)); }
IT_DEV float dpp_half_mirror(float v) { return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xf, 0xf, true)); }
IT_DEV float dpp_row_mirror(float v) { return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xf, 0xf, true)); }
IT_DEV double dpp_f64(double v, int which) {
    const unsigned long long u = __builtin_bit_cast(unsigned long long, v);
    int lo = (int)(u & 0xffffffffull), hi = (int)(u >> 32);
    if (which == 0) {
        lo = __builtin_amdgcn_update_dpp(0, lo, 0xB1, 0xf, 0xf, true);
        hi = __builtin_amdgcn_update_dpp(0, hi, 0xB1, 0xf, 0xf, true);
    } else if (which == 1) {
        lo = __builtin_amdgcn_update_dpp(0, lo, 0x4E, 0xf, 0xf, true);
        hi = __builtin_amdgcn_update_dpp(0, hi, 0x4E, 0xf, 0xf, true);
    } else if (which == 2) {
        lo = __builtin_amdgcn_update_dpp(0, lo, 0x141, 0xf, 0xf, true);
        hi = __builtin_amdgcn_update_dpp(0, hi, 0x141, 0xf, 0xf, true);
    } else {
        lo = __builtin_amdgcn_update_dpp(0, lo, 0x140, 0xf, 0xf, true);
        hi = __builtin_amdgcn_update_dpp(0, hi, 0x140, 0xf, 0xf, true);
    }
    return __builtin_bit_cast(double, ((unsigned long long)(unsigned)hi << 32) | (unsigned)lo);
}

// sum (or max) over aligned groups of L lanes, L a power of two up to 64; every lane gets the result
template <int L> IT_DEV float group_sum(float v) {
    if (L >= 2) v += dpp_xor1(v);
    if (L >= 4) v += dpp_xor2(v);
    if (L >= 8) v += dpp_half_mirror(v);
    if (L >= 16) v += dpp_row_mirror(v);
    if (L >= 32) v += __shfl_xor(v, 16, 64);
    if (L >= 64) v += __shfl_xor(v, 32, 64);
    return v;
}
template <int L> IT_DEV float group_max(float v) {
    if (L >= 2) v = fmaxf(v, dpp_xor1(v));
    if (L >= 4) v = fmaxf(v, dpp_xor2(v));
    if (L >= 8) v = fmaxf(v, dpp_half_mirror(v));
    if (L >= 16) v = fmaxf(v, dpp_row_mirror(v));
    if (L >= 32) v = fmaxf(v, __shfl_xor(v, 16, 64));
    if (L >= 64) v = fmaxf(v, __shfl_xor(v, 32, 64));
    return v;
}
// The same reductions with the result only in the LAST lane of each group: across rows a row's
// total (its lane 15) is broadcast into the next row (row_bcast15 into rows 1 and 3, row_bcast31
// into rows 2 and 3), which needs no LDS crossbar at all.
IT_DEV float dpp_bcast15(float v) { return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x142, 0xa, 0xf, false)); }
IT_DEV float dpp_bcast31(float v) { return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x143, 0xc, 0xf, false)); }
template <int L> IT_DEV float group_sum_tail(float v) {
    if (L >= 2) v += dpp_xor1(v);
    if (L >= 4) v += dpp_xor2(v);
    if (L >= 8) v += dpp_half_mirror(v);
    if (L >= 16) v += dpp_row_mirror(v);
    if (L >= 32) v += dpp_bcast15(v);
    if (L >= 64) v += dpp_bcast31(v);
    return v;
}
template <int L> IT_DEV float group_max_tail(float v) {
    if (L >= 2) v = fmaxf(v, dpp_xor1(v));
    if (L >= 4) v = fmaxf(v, dpp_xor2(v));
    if (L >= 8) v = fmaxf(v, dpp_half_mirror(v));
    if (L >= 16) v = fmaxf(v, dpp_row_mirror(v));
    // a masked-off row receives 0 from the broadcast: harmless for a maximum only when values are
    // compared through max(v, t) on the rows that do receive, so the other rows keep v
    if (L >= 32) {
        const float t = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, v), __builtin_bit_cast(int, v), 0x142, 0xa, 0xf, false));
        v = fmaxf(v, t);
    }
    if (L >= 64) {
        const float t = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, v), __builtin_bit_cast(int, v), 0x143, 0xc, 0xf, false));
        v = fmaxf(v, t);
    }
    return v;
}
// total of the wave in lane 63
IT_DEV double wave_sum_f64_tail(double v) {
    v += dpp_f64(v, 0);
    v += dpp_f64(v, 1);
    v += dpp_f64(v, 2);
    v += dpp_f64(v, 3);
    {
        const unsigned long long u = __builtin_bit_cast(unsigned long long, v);
        const int lo = __builtin_amdgcn_update_dpp(0, (int)(u & 0xffffffffull), 0x142, 0xa, 0xf, false);
        const int hi = __builtin_amdgcn_update_dpp(0, (int)(u >> 32), 0x142, 0xa, 0xf, false);
        v += __builtin_bit_cast(double, ((unsigned long long)(unsigned)hi << 32) | (unsigned)lo);
    }
    {
        const unsigned long long u = __builtin_bit_cast(unsigned long long, v);
        const int lo = __builtin_amdgcn_update_dpp(0, (int)(u & 0xffffffffull), 0x143, 0xc, 0xf, false);
        const int hi = __builtin_amdgcn_update_dpp(0, (int)(u >> 32), 0x143, 0xc, 0xf, false);
        v += __builtin_bit_cast(double, ((unsigned long long)(unsigned)hi << 32) | (unsigned)lo);
    }
    return v;
}

// Sum over the 8 lanes of an aligned group with data-parallel-primitive moves (no LDS crossbar):
// neighbours, then pairs, then the mirrored half.  Every lane of the group ends with the total.
IT_DEV float sum8_lanes(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xf, 0xf, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xf, 0xf, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xf, 0xf, true));
    return v;
}

// Per-head rms_norm (weight w) and NeoX rotation at `pos` of one head's HD values, four per lane
// (lane li of the head's HD / 4 lanes holds dims 4 li .. 4 li + 3): what rms_norm_heads + rope_neox do
// for a single token (naive.rs:180-218, 633-650), with the sum of squares reduced across the lanes.
template <int HD>
IT_DEV float4 head_norm_rope(float4 v, const float* __restrict__ w, float eps, const float2* __restrict__ rope,
                             int n_rot, int pos, int li) {
    constexpr int LPH = HD / 4;
    double part = (double)(v.x * v.x);
    part += (double)(v.y * v.y);
    part += (double)(v.z * v.z);
    part += (double)(v.w * v.w);
    part += dpp_f64(part, 0);
    part += dpp_f64(part, 1);
    part += dpp_f64(part, 2);
    part += dpp_f64(part, 3);
    if (LPH >= 32) part += __shfl_xor(part, 16, 64);
    if (LPH >= 64) part += __shfl_xor(part, 32, 64);
    const float scale = 1.0f / sqrtf((float)(part / (double)HD) + eps);
    const float4 ww = ((const float4*)w)[li];
    v.x = v.x * scale * ww.x;
    v.y = v.y * scale * ww.y;
    v.z = v.z * scale * ww.z;
    v.w = v.w * scale * ww.w;
    const int half = n_rot >> 1, hl = half >> 2;  // lanes per rotated half (a power of two)
    float4 o;
    o.x = __shfl_xor(v.x, hl, 64);
    o.y = __shfl_xor(v.y, hl, 64);
    o.z = __shfl_xor(v.z, hl, 64);
    o.w = __shfl_xor(v.w, hl, 64);
    if (li < 2 * hl) {
        const float4* cs = (const float4*)(rope + (int64_t)pos * half + 4 * (li & (hl - 1)));
        const float4 c01 = cs[0], c23 = cs[1];  // (cos, sin) of dims i, i+1 and i+2, i+3
        if (li < hl) {  // x0 = mine, x1 = partner
            v = make_float4(v.x * c01.x - o.x * c01.y, v.y * c01.z - o.y * c01.w, v.z * c23.x - o.z * c23.y,
                            v.w * c23.z - o.w * c23.w);
        } else {        // x0 = partner, x1 = mine
            v = make_float4(o.x * c01.y + v.x * c01.x, o.y * c01.w + v.y * c01.z, o.z * c23.y + v.z * c23.x,
                            o.w * c23.w + v.w * c23.z);
        }
    }
    return v;
}

}  // namespace itk
