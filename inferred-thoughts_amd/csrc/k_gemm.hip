// Batched (prefill) matmuls on the int8 matrix cores.
//
// out[t][j] = sum_b (float)isum(t, j, b) * (dw[j][b] * dx[t][b]), b ascending: the per-block
// integer dot of the reference's Q8_0 x Q8_0 product (src/quant/dot.rs), formed by one
// v_mfma_i32_16x16x32_i8 per 32-element block with a zero accumulator, then scaled and added
// in f32 in block order.  The arithmetic and its order are the GEMV kernels' and the CPU
// path's, so results are bit-identical; what changes is that a weight row is read once per
// 128 tokens instead of once per token.
//
// MFMA operand layout (16x16x32, i8): lane l supplies 8 consecutive k of row (l % 16) at
// k = 8 * (l / 16) for both A (weight rows) and B (tokens); it receives D for token l % 16
// and weight rows 4 * (l / 16) + {0,1,2,3}.
#include "it_device.h"
#include "kernels.h"

namespace itk {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
constexpr int GT = 256;    // four waves: four groups of 16 weight rows
constexpr int SLAB = 128;  // k per staging step: four Q8_0 blocks
constexpr int LSTR = SLAB + 8;  // LDS row stride in bytes (padded)

// A block owns 64 weight rows x NT*16 tokens.  Each step stages a 128-wide k slab of both
// operands and their block scales into LDS with coalesced 16-byte loads (the next slab's
// loads are in flight while the current one is multiplied), then every wave runs its 16 rows
// against all token tiles: one MFMA per (block, tile), four scaled adds per lane after it.
template <int NT>
__global__ __launch_bounds__(GT) void q8_gemm_k(const int8_t* __restrict__ wq, const uint16_t* __restrict__ ws,
                                                const int8_t* __restrict__ xq, const float* __restrict__ xs,
                                                float* __restrict__ out, int n_in, int n_out, int n_tok,
                                                float out_scale) {
    constexpr int TOK = NT * 16;
    constexpr int BL = (TOK * 8 + GT - 1) / GT;      // 16-byte loads per thread for the token slab
    constexpr int BS = (TOK * 4 + GT - 1) / GT;      // scale loads per thread for the token slab
    __shared__ __align__(16) int8_t As[2][64 * LSTR];
    __shared__ __align__(16) int8_t Bs[2][TOK * LSTR];
    __shared__ uint16_t Asc[2][64 * 4];
    __shared__ float Bsc[2][TOK * 4];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int m = lane & 15, g = lane >> 4;
    const int row0 = blockIdx.x * 64, tok0 = blockIdx.y * TOK;
    const int nb = n_in >> 5;
    const int nslab = (n_in + SLAB - 1) / SLAB;

    uint4 ra[2], rb[BL];
    uint16_t rsa;
    float rsb[BS];
    auto fetch = [&](int s) {
        const int k0 = s * SLAB;
#pragma unroll
        for (int p = 0; p < 2; p++) {
            const int idx = tid + p * GT, row = idx >> 3, seg = idx & 7;
            const int k = k0 + seg * 16;
            ra[p] = k < n_in ? *(const uint4*)(wq + (int64_t)min(row0 + row, n_out - 1) * n_in + k) : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int p = 0; p < BL; p++) {
            const int idx = tid + p * GT, tok = idx >> 3, seg = idx & 7;
            const int k = k0 + seg * 16;
            rb[p] = (tok < TOK && k < n_in) ? *(const uint4*)(xq + (int64_t)min(tok0 + tok, n_tok - 1) * n_in + k)
                                            : make_uint4(0, 0, 0, 0);
        }
        {
            const int row = tid >> 2, bi = tid & 3, bb = s * 4 + bi;
            rsa = bb < nb ? ws[(int64_t)min(row0 + row, n_out - 1) * nb + bb] : (uint16_t)0;
        }
#pragma unroll
        for (int p = 0; p < BS; p++) {
            const int idx = tid + p * GT, tok = idx >> 2, bi = idx & 3, bb = s * 4 + bi;
            rsb[p] = (tok < TOK && bb < nb) ? xs[(int64_t)min(tok0 + tok, n_tok - 1) * nb + bb] : 0.0f;
        }
    };
    auto stash = [&](int buf) {
#pragma unroll
        for (int p = 0; p < 2; p++) {
            const int idx = tid + p * GT, row = idx >> 3, seg = idx & 7;
            *(uint4*)(As[buf] + row * LSTR + seg * 16) = ra[p];
        }
#pragma unroll
        for (int p = 0; p < BL; p++) {
            const int idx = tid + p * GT, tok = idx >> 3, seg = idx & 7;
            if (tok < TOK) *(uint4*)(Bs[buf] + tok * LSTR + seg * 16) = rb[p];
        }
        Asc[buf][tid] = rsa;
#pragma unroll
        for (int p = 0; p < BS; p++) {
            const int idx = tid + p * GT;
            if (idx < TOK * 4) Bsc[buf][idx] = rsb[p];
        }
    };

    float acc[NT][4];
#pragma unroll
    for (int tt = 0; tt < NT; tt++)
#pragma unroll
        for (int i = 0; i < 4; i++) acc[tt][i] = 0.0f;

    fetch(0);
    stash(0);
    __syncthreads();
    for (int s = 0; s < nslab; s++) {
        const int buf = s & 1;
        if (s + 1 < nslab) fetch(s + 1);
        const int nblk = min(4, nb - s * 4);
        for (int bi = 0; bi < nblk; bi++) {
            const long a = *(const long*)(As[buf] + (wave * 16 + m) * LSTR + bi * 32 + g * 8);
            float dw[4];
#pragma unroll
            for (int i = 0; i < 4; i++) dw[i] = it_f16_to_f32(Asc[buf][(wave * 16 + 4 * g + i) * 4 + bi]);
#pragma unroll
            for (int tt = 0; tt < NT; tt++) {
                const long bv = *(const long*)(Bs[buf] + (tt * 16 + m) * LSTR + bi * 32 + g * 8);
                const float dx = Bsc[buf][(tt * 16 + m) * 4 + bi];
                const v4i z = {0, 0, 0, 0};
                const v4i d = __builtin_amdgcn_mfma_i32_16x16x32_i8(a, bv, z, 0, 0, 0);
#pragma unroll
                for (int i = 0; i < 4; i++) acc[tt][i] += (float)d[i] * (dw[i] * dx);
            }
        }
        if (s + 1 < nslab) stash(buf ^ 1);
        __syncthreads();
    }
#pragma unroll
    for (int tt = 0; tt < NT; tt++) {
        const int t = tok0 + tt * 16 + m;
        if (t >= n_tok) continue;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int j = row0 + wave * 16 + 4 * g + i;
            if (j < n_out) out[(int64_t)t * n_out + j] = out_scale != 1.0f ? acc[tt][i] * out_scale : acc[tt][i];
        }
    }
}

}  // namespace

bool q8_gemm(const WView& w, const float* act_scales, const int8_t* act_quants, int n_tok, float* out, float out_scale,
             hipStream_t s) {
    if (w.fmt != W_Q8_0 || n_tok < 16 || w.n_in % 32 || w.n_in <= 0 || w.n_out <= 0) return false;
    if ((reinterpret_cast<uintptr_t>(w.q) & 15) || (reinterpret_cast<uintptr_t>(act_quants) & 15)) return false;
    const int tiles = (n_tok + 15) / 16;
    const int gx = (w.n_out + 63) / 64;
    const int8_t* wq = (const int8_t*)w.q;
    const uint16_t* ws = (const uint16_t*)w.scales;
#define IT_GEMM(NT)                                                                                                  \
    hipLaunchKernelGGL((q8_gemm_k<NT>), dim3(gx, (tiles + NT - 1) / NT), dim3(GT), 0, s, wq, ws, act_quants, act_scales, \
                       out, w.n_in, w.n_out, n_tok, out_scale)
    if (tiles >= 8) IT_GEMM(8);
    else if (tiles >= 4) IT_GEMM(4);
    else if (tiles >= 2) IT_GEMM(2);
    else IT_GEMM(1);
#undef IT_GEMM
    return true;
}

}  // namespace itk
