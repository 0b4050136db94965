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
#include "it_dot.h"
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
template <int NT, bool FMA = false>
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
                for (int i = 0; i < 4; i++) {
                    if (FMA) acc[tt][i] = fmaf((float)d[i], dw[i] * dx, acc[tt][i]);
                    else acc[tt][i] += (float)d[i] * (dw[i] * dx);
                }
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
             hipStream_t s, bool fma) {
    if (w.fmt != W_Q8_0 || n_tok < 16 || w.n_in % 32 || w.n_in <= 0 || w.n_out <= 0) return false;
    if ((reinterpret_cast<uintptr_t>(w.q) & 15) || (reinterpret_cast<uintptr_t>(act_quants) & 15)) return false;
    const int tiles = (n_tok + 15) / 16;
    const int gx = (w.n_out + 63) / 64;
    const int8_t* wq = (const int8_t*)w.q;
    const uint16_t* ws = (const uint16_t*)w.scales;
#define IT_GEMM(NT)                                                                                                  \
    do {                                                                                                             \
        if (fma) hipLaunchKernelGGL((q8_gemm_k<NT, true>), dim3(gx, (tiles + NT - 1) / NT), dim3(GT), 0, s, wq, ws, act_quants, act_scales, \
                                    out, w.n_in, w.n_out, n_tok, out_scale);                                        \
        else hipLaunchKernelGGL((q8_gemm_k<NT, false>), dim3(gx, (tiles + NT - 1) / NT), dim3(GT), 0, s, wq, ws, act_quants, act_scales, \
                                out, w.n_in, w.n_out, n_tok, out_scale);                                            \
    } while (0)
    // 64 tokens per block at most: four blocks fit a CU (38 KB of LDS, 98 VGPRs) and hide each other's LDS and
    // barrier waits; 128 tokens per block (two blocks per CU) measured 20 % slower despite reading the weights half as often
    // ... unless that leaves fewer than two blocks per CU (a short batch, few rows): then narrower blocks, which re-read
    // the weights (from the cache) but fill the chip (the dense matmuls of an 8-layer model over a 96-token prompt:
    // 1.57 against 2.16 ms); the arithmetic per output is the same for every width
    int nt = tiles >= 4 ? 4 : tiles >= 2 ? 2 : 1;
    while (nt > 1 && (int64_t)gx * ((tiles + nt - 1) / nt) < 512) nt >>= 1;
    if (nt == 4) IT_GEMM(4);
    else if (nt == 2) IT_GEMM(2);
    else IT_GEMM(1);
#undef IT_GEMM
    return true;
}

}  // namespace itk

// =====================================================================================
// Grouped expert matmuls for a batch of (token, pick) pairs.
//
// The per-pair GEMV reads an expert's matrix once per pair.  Here the pairs are first sorted
// into per-expert lists ("expert-sorted token lists": moe_group_k), the lists are cut into
// tiles of up to 16 pairs, and one block multiplies 64 rows of that expert's matrix with the
// tile's 16 activation rows on the int8 matrix cores, so a matrix is read once per tile.
// Per pair and row the arithmetic is the GEMV's: per-block integer dots, scaled and added in
// block order (Q8_0: (float)isum * (dw * dx); NVFP4: (dy * dA) * (float)sa then
// (dy * dB) * (float)sb per 32-element chunk), then the expert's second scale, then silu-mul
// for the gate/up pair.  An NVFP4 chunk holds two 16-element sub-blocks with their own
// scales; each needs its own integer sum, so the chunk takes two MFMAs whose token operand is
// zeroed outside the sub-block.
namespace itk {
namespace {

// One block.  work layout: [0] = number of tiles; tiles as int4 {expert, first slot, pairs, 0};
// order[slot] = pair index.  The order of pairs inside an expert's list depends on the atomics'
// arrival order; it only decides which lane computes which pair, never a value.
// tile_pairs: most pairs of one tile (16 for the int8 kernels, 128 for the f16 kernel).
__global__ __launch_bounds__(1024) void moe_group_k(const int32_t* __restrict__ ids, int n_picks, int n_expert,
                                                    int tile_pairs, int32_t* __restrict__ n_tiles,
                                                    int4* __restrict__ tiles, int32_t* __restrict__ order) {
    __shared__ int cnt[1024], off[1024], toff[1024], cur[1024];
    const int tid = threadIdx.x;
    cnt[tid] = 0;
    __syncthreads();
    // eight picks' ids in flight per thread: the walk is bound by the latency of these loads
    for (int p0 = tid; p0 < n_picks; p0 += 8 * 1024) {
        int e[8];
#pragma unroll
        for (int u = 0; u < 8; u++) e[u] = p0 + u * 1024 < n_picks ? ids[p0 + u * 1024] : -1;
#pragma unroll
        for (int u = 0; u < 8; u++)
            if (e[u] >= 0) atomicAdd(&cnt[e[u]], 1);
    }
    __syncthreads();
    // exclusive prefix sums of the pair counts and of the tile counts, all 1024 slots at once
    const int mine = tid < n_expert ? cnt[tid] : 0;
    const int my_tiles = (mine + tile_pairs - 1) / tile_pairs;
    off[tid] = mine;
    toff[tid] = my_tiles;
    __syncthreads();
    for (int d = 1; d < 1024; d <<= 1) {
        const int a = tid >= d ? off[tid - d] : 0, b = tid >= d ? toff[tid - d] : 0;
        __syncthreads();
        off[tid] += a;
        toff[tid] += b;
        __syncthreads();
    }
    if (tid == 1023) *n_tiles = toff[1023];
    const int my_off = off[tid] - mine, my_toff = toff[tid] - my_tiles;
    cur[tid] = my_off;
    __syncthreads();
    for (int p0 = tid; p0 < n_picks; p0 += 8 * 1024) {
        int e[8];
#pragma unroll
        for (int u = 0; u < 8; u++) e[u] = p0 + u * 1024 < n_picks ? ids[p0 + u * 1024] : -1;
#pragma unroll
        for (int u = 0; u < 8; u++)
            if (e[u] >= 0) order[atomicAdd(&cur[e[u]], 1)] = p0 + u * 1024;
    }
    for (int k = 0; k < my_tiles; k++)
        tiles[my_toff + k] = make_int4(tid, my_off + tile_pairs * k, min(tile_pairs, mine - tile_pairs * k), 0);
}

struct ExpertsGemmP {
    const uint8_t *q, *s, *q2, *s2;
    const uint8_t* const *q_tab, *const *s_tab, *const *q2_tab, *const *s2_tab;  // expert placement tables or null
    int64_t q_stride, s_stride;
    const float *scale2, *scale2_up;
    const float* act_scales;
    const int8_t* act_quants;
    float* out;
    int n_in, n_out, x_mode, n_used;
    const int32_t* n_tiles;
    const int4* tiles;
    const int32_t* order;
};

constexpr int NSTR = 64 + 8;  // LDS row stride of an NVFP4 slab (64 nibble bytes + pad)

template <int FMT, bool GLU>
__global__ __launch_bounds__(GT) void experts_gemm_k(ExpertsGemmP p) {
    constexpr int NM = GLU ? 2 : 1;
    constexpr int ASTR = FMT == W_Q8_0 ? LSTR : NSTR;
    constexpr int SPR = FMT == W_Q8_0 ? 4 : 8;  // scales per row per slab
    __shared__ __align__(16) int8_t As[2][NM][64 * ASTR];
    __shared__ float Asc[2][NM][64 * SPR];
    __shared__ __align__(16) int8_t Bs[2][16 * LSTR];
    __shared__ float Bsc[2][16 * 4];
    __shared__ int xrow_s[16], pair_s[16];
    const int tile = blockIdx.x;
    if (tile >= *p.n_tiles) return;
    const int4 td = p.tiles[tile];
    const int64_t e = td.x;
    const int cnt = td.z;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int m = lane & 15, g = lane >> 4;
    const int row0 = blockIdx.y * 64;
    const int n_in = p.n_in, nb = n_in >> 5;
    const int nslab = n_in / SLAB;
    if (tid < 16) {
        const int pair = p.order[td.y + min(tid, cnt - 1)];
        pair_s[tid] = pair;
        xrow_s[tid] = p.x_mode == 0 ? pair : (p.x_mode == 1 ? pair / p.n_used : 0);
    }
    __syncthreads();
    const uint8_t* wq[2] = {it_expert_at(p.q, p.q_tab, e, p.q_stride), GLU ? it_expert_at(p.q2, p.q2_tab, e, p.q_stride) : nullptr};
    const uint8_t* ws[2] = {it_expert_at(p.s, p.s_tab, e, p.s_stride), GLU ? it_expert_at(p.s2, p.s2_tab, e, p.s_stride) : nullptr};

    uint4 ra[NM][2], rb;
    float rsa[NM][2], rsb;
    rb = make_uint4(0, 0, 0, 0);
    rsb = 0.0f;
#pragma unroll
    for (int mt = 0; mt < NM; mt++)
#pragma unroll
        for (int q = 0; q < 2; q++) {
            ra[mt][q] = rb;
            rsa[mt][q] = 0.0f;
        }
    auto fetch = [&](int s) {
#pragma unroll
        for (int mt = 0; mt < NM; mt++) {
            if (FMT == W_Q8_0) {
#pragma unroll
                for (int q = 0; q < 2; q++) {
                    const int idx = tid + q * GT, row = idx >> 3, seg = idx & 7;
                    ra[mt][q] = *(const uint4*)(wq[mt] + (int64_t)min(row0 + row, p.n_out - 1) * n_in + s * SLAB + seg * 16);
                }
                const int row = tid >> 2, bi = tid & 3;
                rsa[mt][0] = it_f16_to_f32(((const uint16_t*)ws[mt])[(int64_t)min(row0 + row, p.n_out - 1) * nb + s * 4 + bi]);
            } else {
                const int row = tid >> 2, seg = tid & 3;
                ra[mt][0] = *(const uint4*)(wq[mt] + (int64_t)min(row0 + row, p.n_out - 1) * (n_in >> 1) + s * 64 + seg * 16);
#pragma unroll
                for (int q = 0; q < 2; q++) {
                    const int idx = tid + q * GT, r2 = idx >> 3, k = idx & 7;
                    rsa[mt][q] = it_ue4m3_to_f32(ws[mt][(int64_t)min(row0 + r2, p.n_out - 1) * (n_in >> 4) + s * 8 + k]);
                }
            }
        }
        if (tid < 128) {
            const int pr = tid >> 3, seg = tid & 7;
            rb = *(const uint4*)(p.act_quants + (int64_t)xrow_s[pr] * n_in + s * SLAB + seg * 16);
        }
        if (tid < 64) rsb = p.act_scales[(int64_t)xrow_s[tid >> 2] * nb + s * 4 + (tid & 3)];
    };
    auto stash = [&](int buf) {
#pragma unroll
        for (int mt = 0; mt < NM; mt++) {
            if (FMT == W_Q8_0) {
#pragma unroll
                for (int q = 0; q < 2; q++) {
                    const int idx = tid + q * GT, row = idx >> 3, seg = idx & 7;
                    *(uint4*)(As[buf][mt] + row * ASTR + seg * 16) = ra[mt][q];
                }
                Asc[buf][mt][tid] = rsa[mt][0];
            } else {
                const int row = tid >> 2, seg = tid & 3;
                *(uint4*)(As[buf][mt] + row * ASTR + seg * 16) = ra[mt][0];
#pragma unroll
                for (int q = 0; q < 2; q++) Asc[buf][mt][tid + q * GT] = rsa[mt][q];
            }
        }
        if (tid < 128) *(uint4*)(Bs[buf] + (tid >> 3) * LSTR + (tid & 7) * 16) = rb;
        if (tid < 64) Bsc[buf][tid] = rsb;
    };

    float acc[NM][4];
#pragma unroll
    for (int mt = 0; mt < NM; mt++)
#pragma unroll
        for (int i = 0; i < 4; i++) acc[mt][i] = 0.0f;
    const v4i z = {0, 0, 0, 0};

    fetch(0);
    stash(0);
    __syncthreads();
    for (int s = 0; s < nslab; s++) {
        const int buf = s & 1;
        if (s + 1 < nslab) fetch(s + 1);
#pragma unroll
        for (int bi = 0; bi < 4; bi++) {
            const long bv = *(const long*)(Bs[buf] + m * LSTR + bi * 32 + g * 8);
            const float dx = Bsc[buf][m * 4 + bi];
#pragma unroll
            for (int mt = 0; mt < NM; mt++) {
                if (FMT == W_Q8_0) {
                    const long a = *(const long*)(As[buf][mt] + (wave * 16 + m) * ASTR + bi * 32 + g * 8);
                    const v4i d = __builtin_amdgcn_mfma_i32_16x16x32_i8(a, bv, z, 0, 0, 0);
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const float dw = Asc[buf][mt][(wave * 16 + 4 * g + i) * 4 + bi];
                        acc[mt][i] += (float)d[i] * (dw * dx);
                    }
                } else {
                    // lane (m, g): sub-block g / 2 of the chunk, its low (g even) or high nibbles
                    const uint2 nb8 = *(const uint2*)(As[buf][mt] + (wave * 16 + m) * ASTR + bi * 16 + (g >> 1) * 8);
                    const int sh = (g & 1) * 4;
                    const uint32_t lo = fp4x4_to_i8x4((nb8.x >> sh) & 0x0f0f0f0fu), hi = fp4x4_to_i8x4((nb8.y >> sh) & 0x0f0f0f0fu);
                    const long a = (long)(((unsigned long long)hi << 32) | lo);
                    const long bA = g < 2 ? bv : 0l, bB = g < 2 ? 0l : bv;
                    const v4i dA = __builtin_amdgcn_mfma_i32_16x16x32_i8(a, bA, z, 0, 0, 0);
                    const v4i dB = __builtin_amdgcn_mfma_i32_16x16x32_i8(a, bB, z, 0, 0, 0);
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const float sA = Asc[buf][mt][(wave * 16 + 4 * g + i) * 8 + 2 * bi];
                        const float sB = Asc[buf][mt][(wave * 16 + 4 * g + i) * 8 + 2 * bi + 1];
                        acc[mt][i] += (dx * sA) * (float)dA[i];
                        acc[mt][i] += (dx * sB) * (float)dB[i];
                    }
                }
            }
        }
        if (s + 1 < nslab) stash(buf ^ 1);
        __syncthreads();
    }
    if (m < cnt) {
        const int64_t pair = pair_s[m];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int j = row0 + wave * 16 + 4 * g + i;
            if (j >= p.n_out) continue;
            float a0 = acc[0][i];
            if (p.scale2) a0 *= p.scale2[e];
            if (GLU) {
                float a1 = acc[NM - 1][i];
                if (p.scale2_up) a1 *= p.scale2_up[e];
                a0 = it_silu(a0) * a1;
            }
            p.out[pair * p.n_out + j] = a0;
        }
    }
}

}  // namespace

size_t experts_group_work_ints(int n_picks, int n_expert) {
    // sized for the smallest tiles any kernel groups for (eight pairs)
    return 16 + (size_t)(n_expert + n_picks / 8 + 2) * 4 + (size_t)n_picks;
}

bool experts_gemm(const ExpertsView& w, const ExpertsView* up, const int32_t* ids, int n_picks, int n_used, int x_mode,
                  const float* act_scales, const int8_t* act_quants, float* out, int32_t* work, size_t work_ints,
                  bool grouped, hipStream_t s) {
    if (n_picks < 32 || !work || w.n_expert > 1024 || w.n_in % SLAB || (w.fmt != W_Q8_0 && w.fmt != W_NVFP4)) return false;
    if (work_ints < experts_group_work_ints(n_picks, w.n_expert)) return false;
    if ((reinterpret_cast<uintptr_t>(w.q) & 15) || w.q_stride % 16 || (reinterpret_cast<uintptr_t>(act_quants) & 15)) return false;
    if (up && (up->fmt != w.fmt || up->n_in != w.n_in || up->n_out != w.n_out || (reinterpret_cast<uintptr_t>(up->q) & 15)))
        return false;
    const int max_tiles = w.n_expert + n_picks / 16 + 1;
    int32_t* n_tiles = work;
    int4* tiles = (int4*)(work + 16);
    int32_t* order = work + 16 + (size_t)(max_tiles + 1) * 4;
    if (!grouped) hipLaunchKernelGGL(moe_group_k, dim3(1), dim3(1024), 0, s, ids, n_picks, w.n_expert, 16, n_tiles, tiles, order);
    ExpertsGemmP p{};
    p.q = (const uint8_t*)w.q;
    p.s = (const uint8_t*)w.scales;
    p.q2 = up ? (const uint8_t*)up->q : nullptr;
    p.s2 = up ? (const uint8_t*)up->scales : nullptr;
    p.q_stride = w.q_stride;
    p.s_stride = w.s_stride;
    p.q_tab = w.q_tab;
    p.s_tab = w.s_tab;
    p.q2_tab = up ? up->q_tab : nullptr;
    p.s2_tab = up ? up->s_tab : nullptr;
    p.scale2 = w.scale2;
    p.scale2_up = up ? up->scale2 : nullptr;
    p.act_scales = act_scales;
    p.act_quants = act_quants;
    p.out = out;
    p.n_in = w.n_in;
    p.n_out = w.n_out;
    p.x_mode = x_mode;
    p.n_used = n_used < 1 ? 1 : n_used;
    p.n_tiles = n_tiles;
    p.tiles = tiles;
    p.order = order;
    dim3 grid(max_tiles, (w.n_out + 63) / 64);
    if (w.fmt == W_Q8_0) {
        if (up) hipLaunchKernelGGL((experts_gemm_k<W_Q8_0, true>), grid, dim3(GT), 0, s, p);
        else hipLaunchKernelGGL((experts_gemm_k<W_Q8_0, false>), grid, dim3(GT), 0, s, p);
    } else {
        if (up) hipLaunchKernelGGL((experts_gemm_k<W_NVFP4, true>), grid, dim3(GT), 0, s, p);
        else hipLaunchKernelGGL((experts_gemm_k<W_NVFP4, false>), grid, dim3(GT), 0, s, p);
    }
    return true;
}


void moe_group(const int32_t* ids, int n_picks, int n_expert, int tile_pairs, int32_t* n_tiles, int4* tiles,
               int32_t* order, hipStream_t s) {
    hipLaunchKernelGGL(moe_group_k, dim3(1), dim3(1024), 0, s, ids, n_picks, n_expert, tile_pairs, n_tiles, tiles, order);
}

}  // namespace itk
