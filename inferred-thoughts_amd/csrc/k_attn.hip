// GQA attention over the f16 KV slabs.
//
// attend_exact keeps the reference CPU path's order (/root/reference
// src/ops/naive.rs:420-466): score = (serial dot) * scale; softmax with a serial
// sum; the weighted V sum walks positions outermost.  Bit-identical to the CPU.
//
// attend_split is split-K flash decoding: each block owns one kv head (all of its
// query heads share the K/V stream) and one range of positions, keeps an
// online-softmax partial (acc, m, l), and a second kernel merges the partials.
// Up to 16 queries take the f16 matrix-core kernel (attend_decode_k), larger
// batches that the one-pass prefill kernel does not take a position-per-thread
// kernel over 128-position chunks.  Reordered sums: compared against the exact
// path at 1e-3.
#include <algorithm>
#include "it_device.h"
#include "it_reduce.h"
#include "kernels.h"

// Phase stamps for tuning: a build with -DIT_STAMPS records the 100 MHz wall clock of one block's thread 0 at
// the marked points of the few-query kernel; the library build compiles them away.
#ifdef IT_STAMPS
__device__ long long it_attn_stamps[32];
__device__ int it_attn_stamp_split;
#define ATTN_STAMP(i)                                                                                      \
    do {                                                                                                   \
        if ((int)blockIdx.y == it_attn_stamp_split && blockIdx.x == 0 && threadIdx.x == 0) it_attn_stamps[i] = wall_clock64(); \
    } while (0)
#else
#define ATTN_STAMP(i) \
    do {              \
    } while (0)
#endif

namespace itk {

// ------------------------------------------------------------------ exact
__global__ __launch_bounds__(256) void attend_exact_k(AttnArgs a, float* __restrict__ scratch,
                                                      float* __restrict__ out) {
    extern __shared__ float qs[];  // head_dim
    __shared__ float red[8];
    const int hd = a.head_dim;
    const int n_pos_last = a.n_pos_dyn ? *a.n_pos_dyn : a.n_pos;
    const int t = blockIdx.x / a.n_head, h = blockIdx.x % a.n_head;
    const int group = a.n_head / a.n_head_kv;
    const int h_kv = h / group;
    const int n_pos = n_pos_last - a.n_q + 1 + t;
    const int off = h_kv * hd;
    const float* q = a.q + ((int64_t)t * a.n_head + h) * hd;
    float* sc = scratch + (int64_t)blockIdx.x * n_pos_last;
    for (int i = threadIdx.x; i < hd; i += 256) qs[i] = q[i];
    __syncthreads();
    float m = -INFINITY;
    for (int s = threadIdx.x; s < n_pos; s += 256) {
        const uint16_t* key = a.k + (int64_t)s * a.kv_dim + off;
        float dot = 0.0f;
        for (int i = 0; i < hd; i += 8) {
            uint4 kk = *(const uint4*)(key + i);
            uint32_t w[4] = {kk.x, kk.y, kk.z, kk.w};
#pragma unroll
            for (int c = 0; c < 4; c++) {
                dot += qs[i + 2 * c] * it_f16_to_f32((uint16_t)(w[c] & 0xffff));
                dot += qs[i + 2 * c + 1] * it_f16_to_f32((uint16_t)(w[c] >> 16));
            }
        }
        float v = dot * a.scale;
        sc[s] = v;
        m = fmaxf(m, v);
    }
    for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_down(m, o, 64));
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
    __syncthreads();
    m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    for (int s = threadIdx.x; s < n_pos; s += 256) sc[s] = it_expf(sc[s] - m);
    __threadfence_block();
    __syncthreads();
    if (threadIdx.x == 0) {
        float sum = 0.0f;
        for (int s = 0; s < n_pos; s++) sum += sc[s];
        red[4] = sum;
    }
    __syncthreads();
    float sum = red[4];
    for (int i = threadIdx.x; i < hd; i += 256) {
        float acc = 0.0f;
        for (int s = 0; s < n_pos; s++) {
            float w = sc[s] / sum;
            acc += w * it_f16_to_f32(a.v[(int64_t)s * a.kv_dim + off + i]);
        }
        out[((int64_t)t * a.n_head + h) * hd + i] = acc;
    }
}

void attend_exact(const AttnArgs& a, float* scratch, float* out, hipStream_t s) {
    if (a.n_q <= 0) return;
    hipLaunchKernelGGL(attend_exact_k, dim3(a.n_q * a.n_head), dim3(256), a.head_dim * sizeof(float), s, a,
                       scratch, out);
}

// ------------------------------------------------------------------ split-K
constexpr int CHUNK = 128;


// partial layout per (t, head, split): [hd acc][m][l]
template <int G>
__global__ __launch_bounds__(256) void attend_split_k(AttnArgs a, int n_split, float* __restrict__ part) {
    extern __shared__ float lds[];
    const int hd = a.head_dim;
    float* qs = lds;                 // [G][hd]
    float* sc = lds + G * hd;        // [CHUNK][G]
    __shared__ float mrow[G], lrow[G];
    const int n_pos_last = a.n_pos_dyn ? *a.n_pos_dyn : a.n_pos;
    const int t = blockIdx.x / a.n_head_kv, h_kv = blockIdx.x % a.n_head_kv;
    const int split = blockIdx.y;
    const int n_pos = n_pos_last - a.n_q + 1 + t;
    const int s0 = split * CHUNK;
    const int len = min(CHUNK, n_pos - s0);
    const int off = h_kv * hd;
    const int h0 = h_kv * G;
    float* my_part = part + (((int64_t)t * a.n_head + h0) * n_split + split) * (hd + 2);
    const int64_t part_head_stride = (int64_t)n_split * (hd + 2);
    if (len <= 0) {
        // empty chunk: m = -inf, l = 0 marks it for the merge
        if (threadIdx.x < G) {
            float* p = my_part + threadIdx.x * part_head_stride;
            p[hd] = -INFINITY;
            p[hd + 1] = 0.0f;
        }
        return;
    }
    for (int i = threadIdx.x; i < G * hd; i += 256) qs[i] = a.q[((int64_t)t * a.n_head + h0) * hd + i];
    __syncthreads();
    // scores: thread = (position, half of the group)
    {
        const int s = threadIdx.x % CHUNK, half = threadIdx.x / CHUNK;  // 256 threads = 128 x 2
        constexpr int GH = (G + 1) / 2;
        const int g0 = half * GH;
        if (s < len) {
            float acc[GH];
#pragma unroll
            for (int g = 0; g < GH; g++) acc[g] = 0.0f;
            const uint16_t* key = a.k + (int64_t)(s0 + s) * a.kv_dim + off;
            for (int i = 0; i < hd; i += 8) {
                uint4 kk = *(const uint4*)(key + i);
                float kf[8];
                kf[0] = it_f16_to_f32((uint16_t)(kk.x & 0xffff)); kf[1] = it_f16_to_f32((uint16_t)(kk.x >> 16));
                kf[2] = it_f16_to_f32((uint16_t)(kk.y & 0xffff)); kf[3] = it_f16_to_f32((uint16_t)(kk.y >> 16));
                kf[4] = it_f16_to_f32((uint16_t)(kk.z & 0xffff)); kf[5] = it_f16_to_f32((uint16_t)(kk.z >> 16));
                kf[6] = it_f16_to_f32((uint16_t)(kk.w & 0xffff)); kf[7] = it_f16_to_f32((uint16_t)(kk.w >> 16));
#pragma unroll
                for (int g = 0; g < GH; g++) {
                    if (g0 + g < G) {
                        const float4 q0 = *(const float4*)(qs + (g0 + g) * hd + i);
                        const float4 q1 = *(const float4*)(qs + (g0 + g) * hd + i + 4);
                        acc[g] += q0.x * kf[0] + q0.y * kf[1] + q0.z * kf[2] + q0.w * kf[3] + q1.x * kf[4] +
                                  q1.y * kf[5] + q1.z * kf[6] + q1.w * kf[7];
                    }
                }
            }
#pragma unroll
            for (int g = 0; g < GH; g++)
                if (g0 + g < G) sc[s * G + g0 + g] = acc[g] * a.scale;
        }
    }
    __syncthreads();
    // per-head max and exp-sum over the chunk: wave w takes heads w, w+4, ...
    {
        const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
        for (int g = wave; g < G; g += 4) {
            float m = -INFINITY;
            for (int s = lane; s < len; s += 64) m = fmaxf(m, sc[s * G + g]);
            for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
            float l = 0.0f;
            for (int s = lane; s < len; s += 64) {
                float p = __expf(sc[s * G + g] - m);
                sc[s * G + g] = p;
                l += p;
            }
            for (int o = 32; o > 0; o >>= 1) l += __shfl_xor(l, o, 64);
            if (lane == 0) {
                mrow[g] = m;
                lrow[g] = l;
            }
        }
    }
    __syncthreads();
    // weighted values: thread = output dimension
    for (int i = threadIdx.x; i < hd; i += 256) {
        float acc[G];
#pragma unroll
        for (int g = 0; g < G; g++) acc[g] = 0.0f;
        const uint16_t* val = a.v + (int64_t)s0 * a.kv_dim + off + i;
        for (int s = 0; s < len; s++) {
            float v = it_f16_to_f32(val[(int64_t)s * a.kv_dim]);
#pragma unroll
            for (int g = 0; g < G; g++) acc[g] += sc[s * G + g] * v;
        }
#pragma unroll
        for (int g = 0; g < G; g++) my_part[g * part_head_stride + i] = acc[g];
    }
    if (threadIdx.x < G) {
        float* p = my_part + threadIdx.x * part_head_stride;
        p[hd] = mrow[threadIdx.x];
        p[hd + 1] = lrow[threadIdx.x];
    }
}

// ------------------------------------------------------------------ split-K for a few queries (decode)
// Keys per tile of the few-query kernel below.
constexpr int TILE = 64;

// ------------------------------------------------------------------ split-K for a few queries on the f16 matrix cores
// One block per (query, kv head, key range): the live context is cut into n_split equal ranges (a multiple
// of 16 keys), so every block has work whatever the position.  A range is walked in tiles of 64 keys; a tile's K
// (as stored, [key][dim]) and V (transposed on the way in, [dim][key]) are staged in LDS with coalesced 16-byte
// loads, the next tile's loads in flight while the current one is used.
//     S^T = K Q^T   (32 keys x 32 columns per MFMA tile): the G query heads sit in columns 0..G-1 as the high
//                   f16 halves of the scaled query and in columns 8..8+G-1 as the low halves, so one
//                   product carries both and a lane move within its row of 16 lanes adds them;
//     O^T = V^T P^T (32 dims x 32 columns per MFMA tile).
// All four waves form the same scores (they run on different SIMDs, so the repetition costs no time and
// saves every exchange: each wave has the whole P^T in registers and the same running maximum and sum);
// wave w then owns the output dims 32 w .. 32 w + 31 (+128), i.e. a quarter of O^T.  A lane holds, for ITS
// column, 16 of the 32 keys of a score tile and 16 of the 32 dims of an output tile, so the softmax
// bookkeeping stays in the lane (one exchange with lane l ^ 32) and the probabilities go from the score
// accumulators to the next MFMA's B operand without leaving the registers (the k order of an MFMA is free
// as long as both operands agree).  Partial layout as above: [hd acc][m][l] per (t, head, split).
// With PREP the block forms its query heads itself (norm + rotation), and the block whose range holds the
// new position forms that position's key and value rows: they go to the slabs and straight into the tile.
// MFMA operand layout (32x32x16, f16): lane l supplies 8 k values of row (l % 32), k group l / 32, for A and
// for B; it receives D for column l % 32 and rows 8 * (i / 4) + 4 * (l / 32) + i % 4.
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));
constexpr int DVS = TILE + 4;  // row stride of V^T in LDS, in f16 (136 bytes)

IT_DEV float row_ror8(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x128, 0xf, 0xf, true));
}

template <int HD, int G, bool PREP>
__global__ __launch_bounds__(256) void attend_decode_k(AttnArgs a, TilePrepP pr, int n_split, float* __restrict__ part) {
    constexpr int KS = HD + 8;                  // row stride of K and of the query rows in LDS, in f16
    constexpr int NS = HD / 16;                 // k steps of a score tile
    constexpr int ND = HD / 32;                 // output tiles along the head dimension
    constexpr int NDW = (ND + 3) / 4;           // of them per wave
    constexpr int KSEG = TILE * HD / 8 / 256;   // 16-byte pieces of K per thread
    constexpr int UNITS = (TILE / 4) * (HD / 8);  // 4-key x 8-dim pieces of V per tile
    constexpr int VU = (UNITS + 255) / 256;     // per thread
    constexpr int QROWS = 17;                   // high halves of 8 heads, low halves of 8 heads, a row of zeros
    static_assert(G <= 8, "hi and lo halves of the query heads share the 32 columns in two groups of 8");
    extern __shared__ __align__(16) uint16_t dlds[];
    uint16_t* Ks = dlds;                      // [64][KS]
    uint16_t* Vt = dlds + TILE * KS;          // [HD][DVS]
    uint16_t* Qs = Vt + HD * DVS;             // [17][KS]
    const int tid = threadIdx.x, lane = tid & 63, w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int c = lane & 31, g = lane >> 5;
    const int t = blockIdx.x / a.n_head_kv, kvh = blockIdx.x % a.n_head_kv;
    const int split = blockIdx.y;
    ATTN_STAMP(0);
    const int n_pos_last = a.n_pos_dyn ? *a.n_pos_dyn : a.n_pos;
    const int n_pos = n_pos_last - a.n_q + 1 + t;
    const int h0 = kvh * G;
    float* my_part = part + (((int64_t)t * a.n_head + h0) * n_split + split) * (HD + 2);
    const int64_t part_head_stride = (int64_t)n_split * (HD + 2);
    // keys per block: the live context over the blocks, in whole groups of 16
    const int kpb = max(16, ((n_pos + n_split - 1) / n_split + 15) & ~15);
    const int k0 = split * kpb, k1 = min(n_pos, k0 + kpb);
    if (k0 >= k1) {
        if (tid < G) {
            float* p = my_part + tid * part_head_stride;
            p[HD] = -INFINITY;
            p[HD + 1] = 0.0f;
        }
        return;
    }
    ATTN_STAMP(1);
    const int n_kt = (k1 - k0 + TILE - 1) / TILE;
    const uint16_t* kbase = a.k + kvh * HD;
    const uint16_t* vbase = a.v + kvh * HD;

    uint4 rk[KSEG], rv[VU][4];
#pragma unroll
    for (int p = 0; p < KSEG; p++) rk[p] = make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int u = 0; u < VU; u++)
#pragma unroll
        for (int q = 0; q < 4; q++) rv[u][q] = make_uint4(0, 0, 0, 0);
    // rows past the range are not fetched: their K rows keep what the tile held (the scores are masked), their
    // V rows are zero (a masked key's probability is 0, and 0 times a stale NaN would not be)
    auto fetch_k = [&](int kt) __attribute__((always_inline)) {
#pragma unroll
        for (int p = 0; p < KSEG; p++) {
            const int idx = tid + p * 256, key = idx / (HD / 8), seg = idx % (HD / 8);
            const int gk = k0 + kt * TILE + key;
            if (gk < k1) rk[p] = *(const uint4*)(kbase + (int64_t)gk * a.kv_dim + seg * 8);
        }
    };
    auto fetch_v = [&](int kt) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < VU; u++) {
            const int unit = tid + u * 256, ka = unit % (TILE / 4), b = unit / (TILE / 4);
            if (unit < UNITS) {
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const int gk = k0 + kt * TILE + 4 * ka + q;
                    rv[u][q] = gk < k1 ? *(const uint4*)(vbase + (int64_t)gk * a.kv_dim + 8 * b) : make_uint4(0, 0, 0, 0);
                }
            }
        }
    };
    auto stash_k = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int p = 0; p < KSEG; p++) {
            const int idx = tid + p * 256, key = idx / (HD / 8), seg = idx % (HD / 8);
            *(uint4*)(Ks + key * KS + seg * 8) = rk[p];
        }
    };
    auto stash_v = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < VU; u++) {
            const int unit = tid + u * 256, ka = unit % (TILE / 4), b = unit / (TILE / 4);  // 16 key groups across lanes: the transposed writes of a wave hit every bank once
            if (unit >= UNITS) continue;
            const uint32_t x[4][4] = {{rv[u][0].x, rv[u][0].y, rv[u][0].z, rv[u][0].w},
                                      {rv[u][1].x, rv[u][1].y, rv[u][1].z, rv[u][1].w},
                                      {rv[u][2].x, rv[u][2].y, rv[u][2].z, rv[u][2].w},
                                      {rv[u][3].x, rv[u][3].y, rv[u][3].z, rv[u][3].w}};
#pragma unroll
            for (int p = 0; p < 4; p++) {  // dims 8b + 2p (low halves) and 8b + 2p + 1 (high halves) of the four keys
                const uint32_t lo0 = __builtin_amdgcn_perm(x[1][p], x[0][p], 0x05040100u);
                const uint32_t lo1 = __builtin_amdgcn_perm(x[3][p], x[2][p], 0x05040100u);
                const uint32_t hi0 = __builtin_amdgcn_perm(x[1][p], x[0][p], 0x07060302u);
                const uint32_t hi1 = __builtin_amdgcn_perm(x[3][p], x[2][p], 0x07060302u);
                *(uint2*)(Vt + (8 * b + 2 * p) * DVS + 4 * ka) = make_uint2(lo0, lo1);
                *(uint2*)(Vt + (8 * b + 2 * p + 1) * DVS + 4 * ka) = make_uint2(hi0, hi1);
            }
        }
    };

    // The query heads as rows of Q^T's columns in LDS: row h = high f16 halves of head h (scaled), row 8 + h = the
    // low halves, row 16 = zeros (what the columns without a head read).  Their loads go out ahead of the tile's.
    const float qsc = a.scale * 1.4426950408889634f;
    auto put_q = [&](int head, int d4, float4 v) __attribute__((always_inline)) {
        const float x[4] = {v.x * qsc, v.y * qsc, v.z * qsc, v.w * qsc};
        uint16_t hi[4], lo[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const _Float16 h = (_Float16)x[e];
            hi[e] = __builtin_bit_cast(uint16_t, h);
            lo[e] = __builtin_bit_cast(uint16_t, (_Float16)(x[e] - (float)h));
        }
        *(uint2*)(Qs + head * KS + 4 * d4) = make_uint2(hi[0] | ((uint32_t)hi[1] << 16), hi[2] | ((uint32_t)hi[3] << 16));
        *(uint2*)(Qs + (8 + head) * KS + 4 * d4) = make_uint2(lo[0] | ((uint32_t)lo[1] << 16), lo[2] | ((uint32_t)lo[3] << 16));
    };
    // rows no head fills
    for (int i = tid; i < QROWS * (HD / 4); i += 256) {
        const int row = i / (HD / 4), d4 = i % (HD / 4);
        if (row == 16 || (row & 7) >= G) *(uint2*)(Qs + row * KS + 4 * d4) = make_uint2(0, 0);
    }
    float4 qv[(G * HD / 4 + 255) / 256];
    if (!PREP) {
#pragma unroll
        for (int j = 0; j < (G * HD / 4 + 255) / 256; j++) {
            const int i = tid + j * 256;
            qv[j] = i < G * HD / 4 ? ((const float4*)(a.q + ((int64_t)t * a.n_head + h0) * HD))[i] : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    }
    fetch_k(0);
    fetch_v(0);
    ATTN_STAMP(2);
    if (!PREP) {
#pragma unroll
        for (int j = 0; j < (G * HD / 4 + 255) / 256; j++) {
            const int i = tid + j * 256;
            if (i < G * HD / 4) put_q(i / (HD / 4), i % (HD / 4), qv[j]);
        }
    } else {
        constexpr int LPH = HD / 4, HPP = 64 / LPH;  // lanes per head, heads per wave pass
        const int li = lane % LPH;
        for (int g0 = w * HPP; g0 < G; g0 += 4 * HPP) {
            const int gq = g0 + lane / LPH;  // G is a multiple of HPP or smaller than it
            if (gq < G) {
                float4 v = ((const float4*)(pr.qg + (int64_t)(h0 + gq) * 2 * HD))[li];
                v = head_norm_rope<HD>(v, pr.q_norm, pr.eps, pr.rope, pr.n_rot, n_pos - 1, li);
                put_q(gq, li, v);
            }
        }
    }
    // (tile, row) of the new position when this block's range holds it
    const int new_at = PREP && n_pos - 1 >= k0 && n_pos - 1 < k1 ? n_pos - 1 - k0 : -1;

    v16f o[NDW];
#pragma unroll
    for (int dw = 0; dw < NDW; dw++)
#pragma unroll
        for (int i = 0; i < 16; i++) o[dw][i] = 0.0f;
    float m = -INFINITY, l = 0.0f;
    const uint16_t* qcol = Qs + (c < 16 ? c : 16) * KS + 8 * g;  // this lane's column of Q^T

    ATTN_STAMP(3);
    for (int kt = 0; kt < n_kt; kt++) {
        const bool fresh = PREP && new_at >= 0 && new_at / TILE == kt;  // the same for every thread of the block
        stash_k();
        ATTN_STAMP(4);
        __syncthreads();
        ATTN_STAMP(5);
        if (kt + 1 < n_kt) fetch_k(kt + 1);
        if (fresh) {
            constexpr int LPH = HD / 4;
            const int li = lane % LPH, row = new_at % TILE, pos_now = n_pos - 1;
            if (w == 0 && lane < LPH) {
                float4 v = ((const float4*)(pr.kproj + (int64_t)kvh * HD))[li];
                v = head_norm_rope<HD>(v, pr.k_norm, pr.eps, pr.rope, pr.n_rot, pos_now, li);
                uint2 hv;
                hv.x = (uint32_t)it_f32_to_f16(v.x) | ((uint32_t)it_f32_to_f16(v.y) << 16);
                hv.y = (uint32_t)it_f32_to_f16(v.z) | ((uint32_t)it_f32_to_f16(v.w) << 16);
                *(uint2*)(pr.k_slab + (int64_t)pos_now * a.kv_dim + kvh * HD + 4 * li) = hv;
                *(uint2*)(Ks + row * KS + 4 * li) = hv;
            }
            __syncthreads();
        }
        ATTN_STAMP(6);
        v16f sc[2];
#pragma unroll
        for (int kk = 0; kk < 2; kk++)
#pragma unroll
            for (int i = 0; i < 16; i++) sc[kk][i] = 0.0f;
#pragma unroll
        for (int s = 0; s < NS; s++) {
            const h8 qf = *(const h8*)(qcol + 16 * s);
#pragma unroll
            for (int kk = 0; kk < 2; kk++) {
                const h8 kf = *(const h8*)(Ks + (32 * kk + c) * KS + 16 * s + 8 * g);
                sc[kk] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf, qf, sc[kk], 0, 0, 0);
            }
        }
        ATTN_STAMP(7);
        // high + low halves (columns c and c + 8 of the same row of 16 lanes), then the keys past the range
        const int left = k1 - (k0 + kt * TILE);  // live keys of this tile
#pragma unroll
        for (int kk = 0; kk < 2; kk++)
#pragma unroll
            for (int i = 0; i < 16; i++) {
                float v = sc[kk][i];
                v += row_ror8(v);
                const int key = 32 * kk + 8 * (i >> 2) + 4 * g + (i & 3);
                sc[kk][i] = key < left ? v : -INFINITY;
            }
        float mt = -INFINITY;
#pragma unroll
        for (int kk = 0; kk < 2; kk++)
#pragma unroll
            for (int i = 0; i < 16; i++) mt = fmaxf(mt, sc[kk][i]);
        mt = fmaxf(mt, __shfl_xor(mt, 32, 64));
        const float m_new = fmaxf(m, mt);  // finite: the first key of a tile is live
        const float alpha = __builtin_amdgcn_exp2f(m - m_new);
        float psum = 0.0f;
        h8 pf[4];
#pragma unroll
        for (int kk = 0; kk < 2; kk++)
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const float p = __builtin_amdgcn_exp2f(sc[kk][i] - m_new);
                psum += p;
                pf[2 * kk + (i >> 3)][i & 7] = (_Float16)p;
            }
        l = l * alpha + psum;
        m = m_new;
        if (kt > 0) {
#pragma unroll
            for (int dw = 0; dw < NDW; dw++)
#pragma unroll
                for (int i = 0; i < 16; i++) o[dw][i] *= alpha;
        }
        ATTN_STAMP(8);
        // the values arrive while the scores are formed
        stash_v();
        if (fresh) {
            __syncthreads();  // the stale row of the tile is written before the new one
            constexpr int LPH = HD / 4;
            const int li = lane % LPH, row = new_at % TILE, pos_now = n_pos - 1;
            if (w == 1 && lane < LPH) {
                const float4 v = ((const float4*)(pr.vproj + (int64_t)kvh * HD))[li];
                const uint16_t e0 = it_f32_to_f16(v.x), e1 = it_f32_to_f16(v.y), e2 = it_f32_to_f16(v.z), e3 = it_f32_to_f16(v.w);
                uint2 hv;
                hv.x = (uint32_t)e0 | ((uint32_t)e1 << 16);
                hv.y = (uint32_t)e2 | ((uint32_t)e3 << 16);
                *(uint2*)(pr.v_slab + (int64_t)pos_now * a.kv_dim + kvh * HD + 4 * li) = hv;
                Vt[(4 * li + 0) * DVS + row] = e0;
                Vt[(4 * li + 1) * DVS + row] = e1;
                Vt[(4 * li + 2) * DVS + row] = e2;
                Vt[(4 * li + 3) * DVS + row] = e3;
            }
        }
        __syncthreads();
        if (kt + 1 < n_kt) fetch_v(kt + 1);
        ATTN_STAMP(9);
#pragma unroll
        for (int dw = 0; dw < NDW; dw++) {
            const int dt = w + 4 * dw;
            if (dt < ND) {
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const uint16_t* vp = Vt + (32 * dt + c) * DVS + 16 * j + 4 * g;
                    const uint2 v0 = *(const uint2*)vp, v1 = *(const uint2*)(vp + 8);
                    const h8 vf = __builtin_bit_cast(h8, make_uint4(v0.x, v0.y, v1.x, v1.y));
                    o[dw] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf, pf[j], o[dw], 0, 0, 0);
                }
            }
        }
        ATTN_STAMP(10);
        if (kt + 1 < n_kt) __syncthreads();  // the tiles are read: the next ones may land
    }

    l += __shfl_xor(l, 32, 64);
    if (c < G) {
        float* p = my_part + c * part_head_stride;
#pragma unroll
        for (int dw = 0; dw < NDW; dw++) {
            const int dt = w + 4 * dw;
            if (dt < ND) {
#pragma unroll
                for (int i4 = 0; i4 < 4; i4++) {
                    float* q = p + 32 * dt + 8 * i4 + 4 * g;  // 8-byte aligned: the partial stride is even
                    *(float2*)q = make_float2(o[dw][4 * i4], o[dw][4 * i4 + 1]);
                    *(float2*)(q + 2) = make_float2(o[dw][4 * i4 + 2], o[dw][4 * i4 + 3]);
                }
            }
        }
        if (w == 0 && g == 0) {
            p[HD] = m * 0.6931471805599453f;  // the maximum in the natural-log domain, as the merge expects
            p[HD + 1] = l;
        }
    }
    ATTN_STAMP(11);
}

// gate (optional): out *= sigmoid(gate[head * gate_stride + i]) — the attention block's output gate.
// One block per (query, head).  Only the splits that hold positions are visited (n_live of them);
// their weights exp(m_s - m) are formed once, in LDS.
__global__ __launch_bounds__(1024) void attend_merge_k(const float* __restrict__ part, int n_split, int hd,
                                                       float* __restrict__ out, const float* __restrict__ gate,
                                                       int gate_stride, int n_q, int n_head, int chunk, int n_pos_arg,
                                                       const int* n_pos_dyn) {
    // blockDim = 4 * hd: four groups of hd threads, group g sums the splits s = g (mod 4)
    extern __shared__ float wsplit[];  // [n_split] then [4][hd]
    __shared__ float redm[16], redl[16];
    float* accs = wsplit + n_split;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nw = (blockDim.x + 63) >> 6;
    const int t = blockIdx.x / n_head;
    const int n_pos = (n_pos_dyn ? *n_pos_dyn : n_pos_arg) - n_q + 1 + t;
    int n_live = (n_pos + chunk - 1) / chunk;
    if (n_live > n_split) n_live = n_split;
    const float* p = part + (int64_t)blockIdx.x * n_split * (hd + 2);
    float m = -INFINITY;
    for (int s = tid; s < n_live; s += blockDim.x) m = fmaxf(m, p[(int64_t)s * (hd + 2) + hd]);
    for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
    if (lane == 0) redm[wave] = m;
    __syncthreads();
    m = redm[0];
    for (int w = 1; w < nw; w++) m = fmaxf(m, redm[w]);
    float l = 0.0f;
    for (int s = tid; s < n_live; s += blockDim.x) {
        const float ms = p[(int64_t)s * (hd + 2) + hd];
        const float w = ms != -INFINITY ? __expf(ms - m) : 0.0f;
        wsplit[s] = w;
        l += p[(int64_t)s * (hd + 2) + hd + 1] * w;
    }
    for (int o = 32; o > 0; o >>= 1) l += __shfl_xor(l, o, 64);
    if (lane == 0) redl[wave] = l;
    __syncthreads();
    l = 0.0f;
    for (int w = 0; w < nw; w++) l += redl[w];
    const int g = tid / hd, i = tid - g * hd;
    float a0 = 0.0f, a1 = 0.0f;
    int s = g;
    for (; s + 4 < n_live; s += 8) {
        a0 += p[(int64_t)s * (hd + 2) + i] * wsplit[s];
        a1 += p[(int64_t)(s + 4) * (hd + 2) + i] * wsplit[s + 4];
    }
    if (s < n_live) a0 += p[(int64_t)s * (hd + 2) + i] * wsplit[s];
    accs[g * hd + i] = a0 + a1;
    __syncthreads();
    if (g == 0) {
        float r = ((accs[i] + accs[hd + i]) + (accs[2 * hd + i] + accs[3 * hd + i])) / l;
        if (gate) r *= fx_sigmoid(gate[(int64_t)blockIdx.x * gate_stride + i]);
        out[(int64_t)blockIdx.x * hd + i] = r;
    }
}

// The same merge for up to 256 splits, spread over the chip: one block per (query, head, 32 output dims).  A
// thread loads the statistics of split `tid` and, before any of them is needed, its share of the partial
// sums (split group tid / 32, dim tid % 32: every load of the block is in flight at once); the block then
// agrees on the maximum, forms the weights exp(m_s - m) in LDS and adds up.  Splits without keys carry
// m = -inf and l = 0; their sums were never written and are not used.
constexpr int MERGE_MAX_SPLIT = 256;
__global__ __launch_bounds__(256) void attend_merge_wide_k(const float* __restrict__ part, int n_split, int hd,
                                                           float* __restrict__ out, const float* __restrict__ gate,
                                                           int gate_stride) {
    __shared__ float wsplit[MERGE_MAX_SPLIT];
    __shared__ float red[8], accs[8][32];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int sg = tid >> 5, i = tid & 31;
    const int d0 = blockIdx.y * 32;
    const float* p = part + (int64_t)blockIdx.x * n_split * (hd + 2);
    const bool has = tid < n_split;
    const float ms = has ? p[(int64_t)tid * (hd + 2) + hd] : -INFINITY;
    const float ls = has ? p[(int64_t)tid * (hd + 2) + hd + 1] : 0.0f;
    float o[MERGE_MAX_SPLIT / 8];
#pragma unroll
    for (int j = 0; j < MERGE_MAX_SPLIT / 8; j++) {
        const int sp = sg + 8 * j;
        o[j] = sp < n_split ? p[(int64_t)sp * (hd + 2) + d0 + i] : 0.0f;
    }
    float m = ms;
    for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
    if (lane == 0) red[wave] = m;
    __syncthreads();
    m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    const float wgt = ms != -INFINITY ? __expf(ms - m) : 0.0f;
    wsplit[tid] = wgt;
    float l = ls * wgt;
    for (int off = 32; off > 0; off >>= 1) l += __shfl_xor(l, off, 64);
    if (lane == 0) red[4 + wave] = l;
    __syncthreads();
    l = (red[4] + red[5]) + (red[6] + red[7]);
    float a0 = 0.0f, a1 = 0.0f;
#pragma unroll
    for (int j = 0; j < MERGE_MAX_SPLIT / 8; j += 2) {
        const float w0 = wsplit[sg + 8 * j], w1 = wsplit[sg + 8 * j + 8];
        a0 += w0 != 0.0f ? o[j] * w0 : 0.0f;
        a1 += w1 != 0.0f ? o[j + 1] * w1 : 0.0f;
    }
    accs[sg][i] = a0 + a1;
    __syncthreads();
    if (tid < 32) {
        float r = (((accs[0][i] + accs[1][i]) + (accs[2][i] + accs[3][i])) + ((accs[4][i] + accs[5][i]) + (accs[6][i] + accs[7][i]))) / l;
        if (gate) r *= fx_sigmoid(gate[(int64_t)blockIdx.x * gate_stride + d0 + i]);
        out[(int64_t)blockIdx.x * hd + d0 + i] = r;
    }
}

bool attend_split(const AttnArgs& a, int n_split, float* scratch, float* out, hipStream_t s) {
    if (attend_prefill(a, out, s)) return true;
    return attend_split_gated(a, n_split, scratch, out, nullptr, 0, s);
}

// queries at or below this count take the tile kernel (chunk TILE); larger batches the
// position-per-thread kernel (chunk CHUNK)
constexpr int TILE_MAX_Q = 16;
static bool tile_path(int n_q, int head_dim, int G) {
    return n_q <= TILE_MAX_Q && (head_dim == 64 || head_dim == 128 || head_dim == 256) && G <= 8;
}

// blocks per (query, kv head) of the few-query kernel: a tile's worth of keys each, at most this many
constexpr int DECODE_SPLIT_MAX = 256;
int attend_split_count(int n_pos_max, int n_q, int head_dim, int group) {
    if (tile_path(n_q, head_dim, group)) return std::max(1, std::min(DECODE_SPLIT_MAX, (n_pos_max + TILE - 1) / TILE));
    return (n_pos_max + CHUNK - 1) / CHUNK;
}

bool attend_tile_prep_ok(const AttnArgs& a, const TilePrepP& pr) {
    const int G = a.n_head / a.n_head_kv, half = pr.n_rot / 2;
    if (a.n_q != 1 || !tile_path(1, a.head_dim, G) || !a.n_pos_dyn) return false;
    const int lph = a.head_dim / 4, hpp = 64 / lph;
    if (G % hpp && G > hpp) return false;
    // the rotated halves must be whole lanes and a power-of-two number of them, inside the head
    if (pr.n_rot <= 0 || half % 4 || ((half / 4) & (half / 4 - 1)) || pr.n_rot > a.head_dim) return false;
    return a.kv_dim % 4 == 0;
}

static bool attend_split_impl(const AttnArgs& a, const TilePrepP* prep, int n_split, float* scratch, float* out,
                              const float* gate, int gate_stride, hipStream_t s);

bool attend_split_gated(const AttnArgs& a, int n_split, float* scratch, float* out, const float* gate,
                        int gate_stride, hipStream_t s) {
    return attend_split_impl(a, nullptr, n_split, scratch, out, gate, gate_stride, s);
}

bool attend_split_gated_prep(const AttnArgs& a, const TilePrepP& pr, int n_split, float* scratch, float* out,
                             const float* gate, int gate_stride, hipStream_t s) {
    return attend_split_impl(a, &pr, n_split, scratch, out, gate, gate_stride, s);
}

// false: nothing was launched and `out` is untouched (a group size the kernels do not take, or the tile kernel's
// LDS size could not be set); the caller records the error
static bool attend_split_impl(const AttnArgs& a, const TilePrepP* prep, int n_split, float* scratch, float* out,
                              const float* gate, int gate_stride, hipStream_t s) {
    if (a.n_q <= 0) return true;
    const int G = a.n_head / a.n_head_kv;
    dim3 grid(a.n_q * a.n_head_kv, n_split), block(256);
    const bool tile = tile_path(a.n_q, a.head_dim, G);
    if (tile) {
#define IT_TILE(HD, GG)                                                                                          \
    do {                                                                                                         \
        constexpr size_t lds = ((size_t)(TILE + 17) * (HD + 8) + (size_t)HD * DVS) * sizeof(uint16_t); \
        static bool sized[2] = {false, false};                                                                   \
        if (!sized[prep ? 1 : 0]) {                                                                              \
            const void* fn = prep ? (const void*)attend_decode_k<HD, GG, true> : (const void*)attend_decode_k<HD, GG, false>; \
            if (lds > 64 * 1024 && hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) { \
                (void)hipGetLastError();                                                                         \
                return false;                                                                                    \
            }                                                                                                    \
            sized[prep ? 1 : 0] = true;                                                                          \
        }                                                                                                        \
        if (prep) hipLaunchKernelGGL((attend_decode_k<HD, GG, true>), grid, block, lds, s, a, *prep, n_split, scratch); \
        else hipLaunchKernelGGL((attend_decode_k<HD, GG, false>), grid, block, lds, s, a, TilePrepP{}, n_split, scratch); \
    } while (0)
#define IT_TILE_G(HD)                  \
    switch (G) {                       \
        case 1: IT_TILE(HD, 1); break; \
        case 2: IT_TILE(HD, 2); break; \
        case 4: IT_TILE(HD, 4); break; \
        case 8: IT_TILE(HD, 8); break; \
        default: return false;         \
    }
        if (a.head_dim == 64) { IT_TILE_G(64) }
        else if (a.head_dim == 128) { IT_TILE_G(128) }
        else { IT_TILE_G(256) }
#undef IT_TILE_G
#undef IT_TILE
    } else {
        size_t lds = ((size_t)G * a.head_dim + (size_t)CHUNK * G) * sizeof(float);
        switch (G) {
            case 1: hipLaunchKernelGGL(attend_split_k<1>, grid, block, lds, s, a, n_split, scratch); break;
            case 2: hipLaunchKernelGGL(attend_split_k<2>, grid, block, lds, s, a, n_split, scratch); break;
            case 4: hipLaunchKernelGGL(attend_split_k<4>, grid, block, lds, s, a, n_split, scratch); break;
            case 8: hipLaunchKernelGGL(attend_split_k<8>, grid, block, lds, s, a, n_split, scratch); break;
            default: return false;  // the caller takes the exact kernel for other group sizes
        }
    }
    if (tile && n_split <= MERGE_MAX_SPLIT && a.head_dim % 32 == 0) {
        hipLaunchKernelGGL(attend_merge_wide_k, dim3(a.n_q * a.n_head, a.head_dim / 32), dim3(256), 0, s, scratch, n_split,
                           a.head_dim, out, gate, gate_stride);
        return true;
    }
    hipLaunchKernelGGL(attend_merge_k, dim3(a.n_q * a.n_head), dim3(4 * a.head_dim),
                       (size_t)(n_split + 4 * a.head_dim) * sizeof(float), s, scratch, n_split, a.head_dim, out, gate,
                       gate_stride, a.n_q, a.n_head, tile ? 1 : CHUNK, a.n_pos, a.n_pos_dyn);  // the few-query kernel spreads the keys over every split
    return true;
}

}  // namespace itk
