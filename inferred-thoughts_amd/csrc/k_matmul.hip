// Quantized matmuls: weight repack, the decode GEMV (dense, per-expert, fused
// gate/up), and the tiled batch kernel.
//
// Arithmetic is the reference CPU path's (/root/reference src/ops/naive.rs):
//   Q8_0  (naive.rs:691-704): per 32-block  sumf += (float)isum * (dw * dx)
//   NVFP4 (naive.rs:714-734): per 16-sub-block sumf += (dy * d) * (float)(lo + hi)
// with the f32 chain walked serially in ascending block order.  Every per-block
// term is computed by its own lane (integer dot via v_dot4_i32_i8, exact), written
// to LDS, and one lane per output row folds the terms in order — so the result is
// the CPU result bit for bit while the HBM stream stays 128-bit coalesced.
#include "it_device.h"
#include "kernels.h"
#include "it_dot.h"

namespace itk {

// ------------------------------------------------------------------ repack
// file Q8_0 block = [f16 d][32 x i8]  ->  quants[row][n_in] + scales[row][n_in/32]
__global__ void repack_q8_0_k(const uint8_t* __restrict__ raw, int8_t* __restrict__ q,
                              uint16_t* __restrict__ scales, int64_t n_blocks) {
    // 8 lanes per block, 4 bytes each
    int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t b = gid >> 3;
    int sub = (int)(gid & 7);
    if (b >= n_blocks) return;
    const uint8_t* blk = raw + b * 34;
    // 34-byte blocks are only 2-byte aligned: assemble from u16 loads
    const uint16_t* p = (const uint16_t*)(blk + 2 + sub * 4);
    uint32_t v = (uint32_t)p[0] | ((uint32_t)p[1] << 16);
    *(uint32_t*)(q + b * 32 + sub * 4) = v;
    if (sub == 0) scales[b] = *(const uint16_t*)blk;
}
void repack_q8_0(const uint8_t* raw, int8_t* q, uint16_t* scales, int64_t n_rows, int n_in, hipStream_t s) {
    int64_t n_blocks = n_rows * (n_in / 32);
    if (n_blocks <= 0) return;
    int64_t threads = n_blocks * 8;
    hipLaunchKernelGGL(repack_q8_0_k, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, s, raw, q, scales,
                       n_blocks);
}

// file NVFP4 block = [4 x ue4m3][32 nibble bytes] -> nibbles[row][n_in/2] + scales[row][n_in/16]
__global__ void repack_nvfp4_k(const uint8_t* __restrict__ raw, uint8_t* __restrict__ nib,
                               uint8_t* __restrict__ scales, int64_t n_blocks) {
    // 9 dwords per block; 8 lanes move nibbles, lane 0 also moves the scales
    int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t b = gid >> 3;
    int sub = (int)(gid & 7);
    if (b >= n_blocks) return;
    const uint32_t* blk = (const uint32_t*)(raw + b * 36);
    ((uint32_t*)nib)[b * 8 + sub] = blk[1 + sub];
    if (sub == 0) ((uint32_t*)scales)[b] = blk[0];
}
void repack_nvfp4(const uint8_t* raw, uint8_t* nib, uint8_t* scales, int64_t n_rows, int n_in, hipStream_t s) {
    int64_t n_blocks = n_rows * (n_in / 64);
    if (n_blocks <= 0) return;
    int64_t threads = n_blocks * 8;
    hipLaunchKernelGGL(repack_nvfp4_k, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, s, raw, nib,
                       scales, n_blocks);
}

// ------------------------------------------------------------------ GEMV
struct GemvP {
    const uint8_t *q, *s;     // weights (gate when GLU)
    const uint8_t *q2, *s2;   // up weights when GLU
    int64_t q_stride, s_stride;  // bytes per expert (0 for a dense matrix)
    const uint8_t* const *q_tab, *const *s_tab, *const *q2_tab, *const *s2_tab;  // expert placement tables or null
    const int32_t* ids;       // expert id per y, or null
    const float *scale2, *scale2_up;  // per-expert second scales or null
    const float* act_scales;  // [x_rows][n_in/32]
    const int8_t* act_quants; // [x_rows][n_in]
    float* out;               // [n_y][n_out]
    int n_in, n_out, rows_per_wave;
    int x_mode, n_used;       // 0: row per y, 1: row y / n_used, 2: row 0
    float out_scale;
};

constexpr int GEMV_WAVES = 4;

template <int FMT, bool GLU>
__global__ __launch_bounds__(64 * GEMV_WAVES) void gemv_k(GemvP p) {
    extern __shared__ __align__(16) float lds[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int U = p.n_in >> 5;                     // 32-element units per row
    const int TPU = (FMT == W_NVFP4) ? 2 : 1;      // terms per unit
    const int T = U * TPU;                         // terms per row
    const int R = p.rows_per_wave;
    const int tstride = T + 4;
    float* terms = lds + (size_t)wave * R * tstride * (GLU ? 2 : 1);
    float* terms2 = terms + (size_t)R * tstride;

    const int y = blockIdx.y;
    const int row0 = (blockIdx.x * GEMV_WAVES + wave) * R;
    if (row0 >= p.n_out) return;
    const int nrows = min(R, p.n_out - row0);

    int64_t e = p.ids ? (int64_t)p.ids[y] : 0;
    const uint8_t* wq = it_expert_at(p.q, p.q_tab, e, p.q_stride);
    const uint8_t* ws = it_expert_at(p.s, p.s_tab, e, p.s_stride);
    const uint8_t* wq2 = GLU ? it_expert_at(p.q2, p.q2_tab, e, p.q_stride) : nullptr;
    const uint8_t* ws2 = GLU ? it_expert_at(p.s2, p.s2_tab, e, p.s_stride) : nullptr;
    int xr = p.x_mode == 0 ? y : (p.x_mode == 1 ? y / p.n_used : 0);
    const int8_t* aq = p.act_quants + (int64_t)xr * p.n_in;
    const float* as = p.act_scales + (int64_t)xr * U;

    const int items = nrows * U;
    for (int base = 0; base < items; base += 64) {
        int it = base + lane;
        if (it < items) {
            int r = it / U, u = it - r * U;
            int64_t row = row0 + r;
            const uint4* ap = (const uint4*)(aq + u * 32);
            uint4 a0 = ap[0], a1 = ap[1];
            float dx = as[u];
            if (FMT == W_Q8_0) {
                const uint4* wp = (const uint4*)(wq + row * p.n_in + u * 32);
                uint16_t dw = ((const uint16_t*)ws)[row * U + u];
                terms[r * tstride + u] = unit_q8_0(wp[0], wp[1], dw, a0, a1, dx);
                if (GLU) {
                    const uint4* wp2 = (const uint4*)(wq2 + row * p.n_in + u * 32);
                    uint16_t dw2 = ((const uint16_t*)ws2)[row * U + u];
                    terms2[r * tstride + u] = unit_q8_0(wp2[0], wp2[1], dw2, a0, a1, dx);
                }
            } else {
                uint4 w = *(const uint4*)(wq + row * (p.n_in >> 1) + u * 16);
                uint32_t sc = ((const uint16_t*)ws)[row * U + u];
                float tA, tB;
                unit_nvfp4(w, sc, a0, a1, dx, &tA, &tB);
                terms[r * tstride + 2 * u] = tA;
                terms[r * tstride + 2 * u + 1] = tB;
                if (GLU) {
                    uint4 w2 = *(const uint4*)(wq2 + row * (p.n_in >> 1) + u * 16);
                    uint32_t sc2 = ((const uint16_t*)ws2)[row * U + u];
                    unit_nvfp4(w2, sc2, a0, a1, dx, &tA, &tB);
                    terms2[r * tstride + 2 * u] = tA;
                    terms2[r * tstride + 2 * u + 1] = tB;
                }
            }
        }
    }
    // the wave's own LDS region: a wave-level barrier is enough
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    if (lane < nrows) {
        float acc = fold_terms(terms + lane * tstride, T);
        float* o = p.out + (int64_t)y * p.n_out + row0 + lane;
        if (GLU) {
            float acc2 = fold_terms(terms2 + lane * tstride, T);
            if (p.scale2) acc *= p.scale2[e];
            if (p.scale2_up) acc2 *= p.scale2_up[e];
            *o = it_silu(acc) * acc2;
        } else {
            if (p.scale2) acc *= p.scale2[e];
            if (p.out_scale != 1.0f) acc *= p.out_scale;
            *o = acc;
        }
    }
}

static int pick_rows_per_wave(int n_out, int n_y) {
    // aim for >= ~2048 waves in flight, cap the fold's idle lanes at 16 rows per wave
    int64_t want_waves = 2048;
    int64_t r = ((int64_t)n_out * n_y) / want_waves;
    int R = 1;
    while (R < 16 && R * 2 <= r) R *= 2;
    return R;
}

template <int FMT, bool GLU>
static void launch_gemv(GemvP p, int n_y, hipStream_t s) {
    int R = pick_rows_per_wave(p.n_out, n_y);
    int T = (p.n_in / 32) * (FMT == W_NVFP4 ? 2 : 1);
    auto lds_for = [&](int r) { return (size_t)GEMV_WAVES * r * (T + 4) * sizeof(float) * (GLU ? 2 : 1); };
    while (R > 1 && lds_for(R) > 48 * 1024) R /= 2;
    p.rows_per_wave = R;
    size_t lds = lds_for(R);
    int gx = (p.n_out + R * GEMV_WAVES - 1) / (R * GEMV_WAVES);
    hipLaunchKernelGGL((gemv_k<FMT, GLU>), dim3(gx, n_y), dim3(64 * GEMV_WAVES), lds, s, p);
}

// ------------------------------------------------------------------ unquantized weights
// naive.rs:843-861: serial f32 fold over the row, one thread per output.
template <int FMT>
__global__ void dense_float_k(const uint8_t* __restrict__ w, const float* __restrict__ x, float* __restrict__ out,
                              int n_in, int n_out, int n_tok, float out_scale) {
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (int64_t)n_out * n_tok) return;
    int j = (int)(idx % n_out);
    int64_t t = idx / n_out;
    const float* xt = x + t * n_in;
    float sum = 0.0f;
    if (FMT == W_F32) {
        const float* row = (const float*)w + (int64_t)j * n_in;
        for (int i = 0; i < n_in; i++) sum += row[i] * xt[i];
    } else {
        const uint16_t* row = (const uint16_t*)w + (int64_t)j * n_in;
        for (int i = 0; i < n_in; i++)
            sum += (FMT == W_F16 ? it_f16_to_f32(row[i]) : it_bf16_to_f32(row[i])) * xt[i];
    }
    if (out_scale != 1.0f) sum *= out_scale;
    out[t * n_out + j] = sum;
}

// Unquantized weights, fast mode: the row sum is split over a wave (not the CPU path's serial order).
// Up to 8 tokens per launch row: one wave per weight row, lanes stride the row in 4-element pieces that are read
// once and used for every token.
template <int FMT>
IT_DEV float4 load_w4(const uint8_t* row, int i) {
    if (FMT == W_F32) return *(const float4*)((const float*)row + i);
    const uint2 h = *(const uint2*)((const uint16_t*)row + i);
    if (FMT == W_F16)
        return make_float4(it_f16_to_f32(h.x & 0xffffu), it_f16_to_f32(h.x >> 16), it_f16_to_f32(h.y & 0xffffu), it_f16_to_f32(h.y >> 16));
    return make_float4(it_bf16_to_f32(h.x & 0xffffu), it_bf16_to_f32(h.x >> 16), it_bf16_to_f32(h.y & 0xffffu), it_bf16_to_f32(h.y >> 16));
}

template <int FMT, int NT>
__global__ __launch_bounds__(256) void float_gemv_fast_k(const uint8_t* __restrict__ w, const float* __restrict__ x,
                                                         float* __restrict__ out, int n_in, int n_out, int n_tok, int tok0,
                                                         float out_scale) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int j = blockIdx.x * 4 + wave;
    if (j >= n_out) return;
    const uint8_t* row = w + (int64_t)j * n_in * (FMT == W_F32 ? 4 : 2);
    float acc[NT];
#pragma unroll
    for (int t = 0; t < NT; t++) acc[t] = 0.0f;
    for (int i = lane * 4; i < n_in; i += 256) {
        const float4 wv = load_w4<FMT>(row, i);
#pragma unroll
        for (int t = 0; t < NT; t++) {
            if (tok0 + t < n_tok) {
                const float4 xv = *(const float4*)(x + (int64_t)(tok0 + t) * n_in + i);
                acc[t] = fmaf(wv.x, xv.x, fmaf(wv.y, xv.y, fmaf(wv.z, xv.z, fmaf(wv.w, xv.w, acc[t]))));
            }
        }
    }
#pragma unroll
    for (int t = 0; t < NT; t++) {
        float v = acc[t];
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
        if (lane == 0 && tok0 + t < n_tok) out[(int64_t)(tok0 + t) * n_out + j] = out_scale != 1.0f ? v * out_scale : v;
    }
}

// Two matrices read with the same activations (matmul_pair: router + shared-gate logit, ssm alpha + beta) as one
// launch: rows 0 .. n0 are matrix 0's, the next n1 matrix 1's, each with its own output.  n1 = 0: one matrix.
struct FloatMats {
    const uint8_t *w0, *w1;
    float *out0, *out1;
    int n0, n1;
};
template <int FMT>
IT_DEV const uint8_t* float_row(const FloatMats& m, int j, int n_in) {
    constexpr int ESZ = FMT == W_F32 ? 4 : 2;
    const int last = m.n0 + m.n1 - 1;
    j = j < last ? j : last;
    return j < m.n0 ? m.w0 + (int64_t)j * n_in * ESZ : m.w1 + (int64_t)(j - m.n0) * n_in * ESZ;
}
IT_DEV void float_store(const FloatMats& m, int t, int j, float v) {
    if (j < m.n0) m.out0[(int64_t)t * m.n0 + j] = v;
    else if (j < m.n0 + m.n1) m.out1[(int64_t)t * m.n1 + (j - m.n0)] = v;
}

// More tokens: a block owns 64 weight rows x 64 tokens, stages 16-wide k slabs of both operands in LDS (the next
// slab's loads in flight while this one is multiplied) and every thread keeps a 4 x 4 tile of sums.
template <int FMT>
__global__ __launch_bounds__(256) void float_gemm_fast_k(FloatMats m, const float* __restrict__ x, int n_in, int n_tok,
                                                         float out_scale) {
    constexpr int KS = 16;
    __shared__ float Ws[KS][64 + 4], Xs[KS][64 + 4];
    const int tid = threadIdx.x, tr = tid & 15, tc = tid >> 4;   // rows 4 tr .. + 3, tokens 4 tc .. + 3
    const int row0 = blockIdx.x * 64, tok0 = blockIdx.y * 64;
    const int lr = tid >> 2, lk = (tid & 3) * 4;                 // staging: row (or token) lr, k lk .. + 3
    const int64_t xrow = min(tok0 + lr, n_tok - 1);
    const uint8_t* wp = float_row<FMT>(m, row0 + lr, n_in);
    const float* xp = x + xrow * n_in;
    float acc[4][4];
#pragma unroll
    for (int a = 0; a < 4; a++)
#pragma unroll
        for (int b = 0; b < 4; b++) acc[a][b] = 0.0f;
    float4 wv = load_w4<FMT>(wp, lk);
    float4 xv = *(const float4*)(xp + lk);
    for (int k0 = 0; k0 < n_in; k0 += KS) {
        __syncthreads();
        Ws[lk][lr] = wv.x; Ws[lk + 1][lr] = wv.y; Ws[lk + 2][lr] = wv.z; Ws[lk + 3][lr] = wv.w;
        Xs[lk][lr] = xv.x; Xs[lk + 1][lr] = xv.y; Xs[lk + 2][lr] = xv.z; Xs[lk + 3][lr] = xv.w;
        __syncthreads();
        if (k0 + KS < n_in) {
            wv = load_w4<FMT>(wp, k0 + KS + lk);
            xv = *(const float4*)(xp + k0 + KS + lk);
        }
#pragma unroll
        for (int k = 0; k < KS; k++) {
            const float4 a = *(const float4*)&Ws[k][4 * tr];
            const float4 b = *(const float4*)&Xs[k][4 * tc];
            const float av[4] = {a.x, a.y, a.z, a.w}, bv[4] = {b.x, b.y, b.z, b.w};
#pragma unroll
            for (int ia = 0; ia < 4; ia++)
#pragma unroll
                for (int ib = 0; ib < 4; ib++) acc[ia][ib] = fmaf(av[ia], bv[ib], acc[ia][ib]);
        }
    }
#pragma unroll
    for (int ib = 0; ib < 4; ib++) {
        const int t = tok0 + 4 * tc + ib;
        if (t >= n_tok) continue;
#pragma unroll
        for (int ia = 0; ia < 4; ia++) float_store(m, t, row0 + 4 * tr + ia, out_scale != 1.0f ? acc[ia][ib] * out_scale : acc[ia][ib]);
    }
}

// A long batch against a matrix of many rows (the F32 router of a real file over a prefill pass): 128 rows x 128
// tokens per block and an 8 x 8 tile of sums per thread, i.e. a quarter of the LDS bytes per multiply-add of the
// 4 x 4 form.  Every sum runs over k in the same order as there.
template <int FMT>
__global__ __launch_bounds__(256) void float_gemm_wide_k(FloatMats m, const float* __restrict__ x, int n_in, int n_tok,
                                                         float out_scale) {
    constexpr int KS = 16, TILE = 128;
    __shared__ __align__(16) float Ws[KS][TILE + 4], Xs[KS][TILE + 4];
    const int tid = threadIdx.x, tr = tid & 15, tc = tid >> 4;   // rows 4 tr .. + 3 and 64 + 4 tr .. + 3; tokens likewise by tc
    const int row0 = blockIdx.x * TILE, tok0 = blockIdx.y * TILE;
    const int lr = tid >> 2, lk = (tid & 3) * 4;                 // staging: rows (tokens) lr and lr + 64, k lk .. + 3
    const uint8_t* wp[2];
    const float* xp[2];
#pragma unroll
    for (int h = 0; h < 2; h++) {
        wp[h] = float_row<FMT>(m, row0 + lr + 64 * h, n_in);
        xp[h] = x + (int64_t)min(tok0 + lr + 64 * h, n_tok - 1) * n_in;
    }
    float acc[8][8];
#pragma unroll
    for (int a = 0; a < 8; a++)
#pragma unroll
        for (int b = 0; b < 8; b++) acc[a][b] = 0.0f;
    float4 wv[2], xv[2];
#pragma unroll
    for (int h = 0; h < 2; h++) {
        wv[h] = load_w4<FMT>(wp[h], lk);
        xv[h] = *(const float4*)(xp[h] + lk);
    }
    for (int k0 = 0; k0 < n_in; k0 += KS) {
        __syncthreads();
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const int c = lr + 64 * h;
            Ws[lk][c] = wv[h].x; Ws[lk + 1][c] = wv[h].y; Ws[lk + 2][c] = wv[h].z; Ws[lk + 3][c] = wv[h].w;
            Xs[lk][c] = xv[h].x; Xs[lk + 1][c] = xv[h].y; Xs[lk + 2][c] = xv[h].z; Xs[lk + 3][c] = xv[h].w;
        }
        __syncthreads();
        if (k0 + KS < n_in) {   // the next slab's loads fly while this one is multiplied
#pragma unroll
            for (int h = 0; h < 2; h++) {
                wv[h] = load_w4<FMT>(wp[h], k0 + KS + lk);
                xv[h] = *(const float4*)(xp[h] + k0 + KS + lk);
            }
        }
#pragma unroll
        for (int k = 0; k < KS; k++) {
            const float4 a0 = *(const float4*)&Ws[k][4 * tr], a1 = *(const float4*)&Ws[k][64 + 4 * tr];
            const float4 b0 = *(const float4*)&Xs[k][4 * tc], b1 = *(const float4*)&Xs[k][64 + 4 * tc];
            const float av[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
            const float bv[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
#pragma unroll
            for (int ia = 0; ia < 8; ia++)
#pragma unroll
                for (int ib = 0; ib < 8; ib++) acc[ia][ib] = fmaf(av[ia], bv[ib], acc[ia][ib]);
        }
    }
#pragma unroll
    for (int ib = 0; ib < 8; ib++) {
        const int t = tok0 + (ib < 4 ? 4 * tc + ib : 64 + 4 * tc + ib - 4);
        if (t >= n_tok) continue;
#pragma unroll
        for (int ia = 0; ia < 8; ia++) {
            const int j = row0 + (ia < 4 ? 4 * tr + ia : 64 + 4 * tr + ia - 4);
            float_store(m, t, j, out_scale != 1.0f ? acc[ia][ib] * out_scale : acc[ia][ib]);
        }
    }
}

template <int FMT>
static void float_gemm_launch(const FloatMats& m, const float* x, int n_in, int n_tok, float out_scale, hipStream_t s) {
    const int rows = m.n0 + m.n1;
    if (n_tok >= 1024 && rows >= 256)
        hipLaunchKernelGGL(float_gemm_wide_k<FMT>, dim3((rows + 127) / 128, (n_tok + 127) / 128), dim3(256), 0, s, m, x, n_in, n_tok, out_scale);
    else
        hipLaunchKernelGGL(float_gemm_fast_k<FMT>, dim3((rows + 63) / 64, (n_tok + 63) / 64), dim3(256), 0, s, m, x, n_in, n_tok, out_scale);
}

template <int FMT>
static bool float_matmul_fast(const WView& w, const float* x, int n_tok, float* out, float out_scale, hipStream_t s) {
    if (w.n_in % 16 || (reinterpret_cast<uintptr_t>(w.q) & 15) || (reinterpret_cast<uintptr_t>(x) & 15)) return false;
    const uint8_t* wp = (const uint8_t*)w.q;
    if (n_tok > 16) {
        float_gemm_launch<FMT>(FloatMats{wp, nullptr, out, nullptr, w.n_out, 0}, x, w.n_in, n_tok, out_scale, s);
        return true;
    }
    for (int t0 = 0; t0 < n_tok; t0 += 8) {
        if (n_tok - t0 == 1)
            hipLaunchKernelGGL((float_gemv_fast_k<FMT, 1>), dim3((w.n_out + 3) / 4), dim3(256), 0, s, wp, x, out, w.n_in, w.n_out,
                               n_tok, t0, out_scale);
        else
            hipLaunchKernelGGL((float_gemv_fast_k<FMT, 8>), dim3((w.n_out + 3) / 4), dim3(256), 0, s, wp, x, out, w.n_in, w.n_out,
                               n_tok, t0, out_scale);
    }
    return true;
}

// matmul_pair over a batch with two unquantized matrices of one element type (fast mode): one launch for both
bool float_matmul_pair(const WView& a, const WView& b, const float* x, int n_tok, float* out_a, float* out_b, hipStream_t s) {
    if (a.fmt != b.fmt || a.n_in != b.n_in || n_tok <= 16 || a.n_in % 16 || a.n_out <= 0 || b.n_out <= 0) return false;
    if (a.fmt != W_F32 && a.fmt != W_F16 && a.fmt != W_BF16) return false;
    if ((reinterpret_cast<uintptr_t>(a.q) & 15) || (reinterpret_cast<uintptr_t>(b.q) & 15) || (reinterpret_cast<uintptr_t>(x) & 15)) return false;
    const FloatMats m{(const uint8_t*)a.q, (const uint8_t*)b.q, out_a, out_b, a.n_out, b.n_out};
    if (a.fmt == W_F32) float_gemm_launch<W_F32>(m, x, a.n_in, n_tok, 1.0f, s);
    else if (a.fmt == W_F16) float_gemm_launch<W_F16>(m, x, a.n_in, n_tok, 1.0f, s);
    else float_gemm_launch<W_BF16>(m, x, a.n_in, n_tok, 1.0f, s);
    return true;
}

void matmul(const WView& w, const float* x, const float* act_scales, const int8_t* act_quants, int n_tok,
            float* out, float out_scale, int exact, hipStream_t s) {
    if (n_tok <= 0 || w.n_out <= 0) return;
    // (fast mode adds each scaled block sum with one rounding: 4 ms of a 174 ms prefill pass)
    if (q8_gemm(w, act_scales, act_quants, n_tok, out, out_scale, s, !exact)) return;
    if (w.fmt == W_Q8_0 || w.fmt == W_NVFP4) {
        GemvP p{};
        p.q = (const uint8_t*)w.q;
        p.s = (const uint8_t*)w.scales;
        p.act_scales = act_scales;
        p.act_quants = act_quants;
        p.out = out;
        p.n_in = w.n_in;
        p.n_out = w.n_out;
        p.x_mode = 0;
        p.n_used = 1;
        p.out_scale = out_scale;
        if (w.fmt == W_Q8_0) launch_gemv<W_Q8_0, false>(p, n_tok, s);
        else launch_gemv<W_NVFP4, false>(p, n_tok, s);
        return;
    }
    if (!exact) {
        if (w.fmt == W_F32 && float_matmul_fast<W_F32>(w, x, n_tok, out, out_scale, s)) return;
        if (w.fmt == W_F16 && float_matmul_fast<W_F16>(w, x, n_tok, out, out_scale, s)) return;
        if (w.fmt == W_BF16 && float_matmul_fast<W_BF16>(w, x, n_tok, out, out_scale, s)) return;
    }
    int64_t total = (int64_t)w.n_out * n_tok;
    dim3 grid((unsigned)((total + 127) / 128)), block(128);
    const uint8_t* wp = (const uint8_t*)w.q;
    if (w.fmt == W_F32)
        hipLaunchKernelGGL(dense_float_k<W_F32>, grid, block, 0, s, wp, x, out, w.n_in, w.n_out, n_tok, out_scale);
    else if (w.fmt == W_F16)
        hipLaunchKernelGGL(dense_float_k<W_F16>, grid, block, 0, s, wp, x, out, w.n_in, w.n_out, n_tok, out_scale);
    else
        hipLaunchKernelGGL(dense_float_k<W_BF16>, grid, block, 0, s, wp, x, out, w.n_in, w.n_out, n_tok,
                           out_scale);
}

static GemvP experts_params(const ExpertsView& w, const int32_t* ids, int n_used, int x_mode,
                            const float* act_scales, const int8_t* act_quants, float* out) {
    GemvP p{};
    p.q = (const uint8_t*)w.q;
    p.s = (const uint8_t*)w.scales;
    p.q_stride = w.q_stride;
    p.s_stride = w.s_stride;
    p.ids = ids;
    p.q_tab = w.q_tab;
    p.s_tab = w.s_tab;
    p.scale2 = w.scale2;
    p.act_scales = act_scales;
    p.act_quants = act_quants;
    p.out = out;
    p.n_in = w.n_in;
    p.n_out = w.n_out;
    p.x_mode = x_mode;
    p.n_used = n_used < 1 ? 1 : n_used;
    p.out_scale = 1.0f;
    return p;
}

void matmul_experts(const ExpertsView& w, const int32_t* ids, int n_picks, int n_used, int x_mode,
                    const float* act_scales, const int8_t* act_quants, float* out, hipStream_t s) {
    if (n_picks <= 0) return;
    GemvP p = experts_params(w, ids, n_used, x_mode, act_scales, act_quants, out);
    if (w.fmt == W_Q8_0) launch_gemv<W_Q8_0, false>(p, n_picks, s);
    else launch_gemv<W_NVFP4, false>(p, n_picks, s);
}

void moe_glu(const ExpertsView& gate, const ExpertsView& up, const int32_t* ids, int n_picks, int n_used,
             int x_mode, const float* act_scales, const int8_t* act_quants, float* out, hipStream_t s) {
    if (n_picks <= 0) return;
    GemvP p = experts_params(gate, ids, n_used, x_mode, act_scales, act_quants, out);
    p.q2 = (const uint8_t*)up.q;
    p.s2 = (const uint8_t*)up.scales;
    p.q2_tab = up.q_tab;
    p.s2_tab = up.s_tab;
    p.scale2_up = up.scale2;
    if (gate.fmt == W_Q8_0) launch_gemv<W_Q8_0, true>(p, n_picks, s);
    else launch_gemv<W_NVFP4, true>(p, n_picks, s);
}

}  // namespace itk
