// Causal attention for a batch of queries (prefill) on the f16 matrix cores, one pass over the keys.
//
// Same function as /root/reference src/ops/naive.rs:137-203 (scores, softmax, weighted values per
// head; query i of a batch of n_q sees positions 0 .. n_pos - n_q + i), computed tile by tile with a
// running maximum and sum per query instead of a full score row.  Fast mode only: the sums are not
// in the CPU path's order.
//
// A block owns 128 query rows of one KV head: 128 / G tokens x the G query heads that share the head.
// It walks the keys in tiles of 64; a tile's K (as stored, f16 [key][dim]) and V (transposed on the
// way in, [dim][key]) are staged in LDS once for all 128 rows.  Each wave owns 32 rows and forms
//     S^T = K Q^T   (32 keys x 32 queries per MFMA tile, A = K from LDS, B = Q from registers)
//     O^T = V^T P^T (32 dims x 32 queries per MFMA tile, A = V^T from LDS, B = P from registers)
// so a lane holds, for ITS query (column l % 32), 16 of the 32 keys of a score tile and 16 of the 32
// dims of an output tile: the running maximum, the rescaling and the final division stay inside
// the lane (one exchange with lane l ^ 32), and the probabilities go from the score accumulators
// to the next MFMA's B operand without leaving the registers (the k order of an MFMA is free as
// long as both operands agree: lane group g's eight probabilities of step j are keys
// 16 j + 4 g + {0..3} and 8 more, and V^T is read at those keys).
// The query is scaled by scale * log2(e) and split into an f16 pair (hi + lo, 22 bits kept); K, V
// are f16 in the cache; probabilities are rounded to f16 (relative 2^-11 each, unbiased).
//
// MFMA operand layout (32x32x16, f16): lane l supplies 8 k values of row (l % 32), k group l / 32,
// for A and for B; it receives D for column l % 32 and rows 8 * (i / 4) + 4 * (l / 32) + i % 4.
#include "it_device.h"
#include "kernels.h"

namespace itk {
namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));
constexpr int KT = 64;       // keys per tile
constexpr int VS = KT + 4;   // row stride of V^T in LDS, in f16 (136 bytes)

template <int HD, int G>
__global__ __launch_bounds__(256) void attend_prefill_k(AttnArgs a, float* __restrict__ out) {
    constexpr int QT = 128 / G;                     // tokens per block
    constexpr int KS = HD + 8;                      // row stride of K in LDS, in f16
    constexpr int NS = HD / 16;                     // k steps of a score tile
    constexpr int ND = HD / 32;                     // output tiles along the head dimension
    constexpr int KSEG = KT * HD / 8 / 256;         // 16-byte pieces of K per thread
    constexpr int UNITS = (KT / 4) * (HD / 8);      // 4-key x 8-dim pieces of V per tile
    constexpr int VU = (UNITS + 255) / 256;         // per thread
    extern __shared__ __align__(16) uint16_t lds[];
    uint16_t* Ks = lds;                // [64][KS]
    uint16_t* Vt = lds + KT * KS;      // [HD][VS]
    uint16_t* Ql = Vt + HD * VS;       // [128][KS]: the low halves of the query rows (registers are short)
    const int tid = threadIdx.x, lane = tid & 63, w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 31, g = lane >> 5;
    const int n_qt = (a.n_q + QT - 1) / QT;
    const int qt = n_qt - 1 - (int)blockIdx.x;      // the longest rows first
    const int kvh = blockIdx.y;
    const int row = 32 * w + r;
    const int token = qt * QT + row / G, head = kvh * G + row % G;
    const bool valid = token < a.n_q;
    const int base_pos = a.n_pos - a.n_q;
    const int pos = valid ? base_pos + token : 0x7fffffff;
    const int qdim = a.n_head * HD;

    // this lane's query row, scaled, as an f16 pair
    h8 qh[NS];
    {
        const float qs = a.scale * 1.4426950408889634f;
        const float* qrow = a.q + (int64_t)min(token, a.n_q - 1) * qdim + head * HD + 8 * g;
#pragma unroll
        for (int s = 0; s < NS; s++) {
            const float4 x0 = *(const float4*)(qrow + 16 * s), x1 = *(const float4*)(qrow + 16 * s + 4);
            const float x[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
            h8 lo;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const float v = valid ? x[e] * qs : 0.0f;
                const _Float16 hi = (_Float16)v;
                qh[s][e] = hi;
                lo[e] = (_Float16)(v - (float)hi);
            }
            *(h8*)(Ql + row * KS + 16 * s + 8 * g) = lo;   // read back by this lane only
        }
    }

    const int first_pos = base_pos + qt * QT;                            // smallest position of the block
    const int last_pos = base_pos + min(a.n_q, (qt + 1) * QT) - 1;       // largest
    const int n_kt = last_pos / KT + 1;
    const uint16_t* kbase = a.k + kvh * HD;
    const uint16_t* vbase = a.v + kvh * HD;

    uint4 rk[KSEG], rv[VU][4];
#pragma unroll
    for (int p = 0; p < KSEG; p++) rk[p] = make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int u = 0; u < VU; u++)
#pragma unroll
        for (int c = 0; c < 4; c++) rv[u][c] = make_uint4(0, 0, 0, 0);
    auto fetch = [&](int kt) __attribute__((always_inline)) {
#pragma unroll
        for (int p = 0; p < KSEG; p++) {
            const int idx = tid + p * 256, key = idx / (HD / 8), seg = idx % (HD / 8);
            const int64_t gk = min(kt * KT + key, a.n_pos - 1);
            rk[p] = *(const uint4*)(kbase + gk * a.kv_dim + seg * 8);
        }
#pragma unroll
        for (int u = 0; u < VU; u++) {
            const int unit = tid + u * 256, ka = unit % (KT / 4), b = unit / (KT / 4);   // 16 key groups across lanes: the transposed LDS writes of a wave hit every bank once
            if (unit < UNITS) {
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    const int64_t gk = min(kt * KT + 4 * ka + c, a.n_pos - 1);
                    rv[u][c] = *(const uint4*)(vbase + gk * a.kv_dim + 8 * b);
                }
            }
        }
    };
    auto stash = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int p = 0; p < KSEG; p++) {
            const int idx = tid + p * 256, key = idx / (HD / 8), seg = idx % (HD / 8);
            *(uint4*)(Ks + key * KS + seg * 8) = rk[p];
        }
#pragma unroll
        for (int u = 0; u < VU; u++) {
            const int unit = tid + u * 256, ka = unit % (KT / 4), b = unit / (KT / 4);   // 16 key groups across lanes: the transposed LDS writes of a wave hit every bank once
            if (unit >= UNITS) continue;
            const uint32_t x[4][4] = {{rv[u][0].x, rv[u][0].y, rv[u][0].z, rv[u][0].w},
                                      {rv[u][1].x, rv[u][1].y, rv[u][1].z, rv[u][1].w},
                                      {rv[u][2].x, rv[u][2].y, rv[u][2].z, rv[u][2].w},
                                      {rv[u][3].x, rv[u][3].y, rv[u][3].z, rv[u][3].w}};
#pragma unroll
            for (int p = 0; p < 4; p++) {   // dims 8b + 2p (low halves) and 8b + 2p + 1 (high halves) of the four keys
                const uint32_t lo0 = __builtin_amdgcn_perm(x[1][p], x[0][p], 0x05040100u);
                const uint32_t lo1 = __builtin_amdgcn_perm(x[3][p], x[2][p], 0x05040100u);
                const uint32_t hi0 = __builtin_amdgcn_perm(x[1][p], x[0][p], 0x07060302u);
                const uint32_t hi1 = __builtin_amdgcn_perm(x[3][p], x[2][p], 0x07060302u);
                *(uint2*)(Vt + (8 * b + 2 * p) * VS + 4 * ka) = make_uint2(lo0, lo1);
                *(uint2*)(Vt + (8 * b + 2 * p + 1) * VS + 4 * ka) = make_uint2(hi0, hi1);
            }
        }
    };

    v16f o[ND];
#pragma unroll
    for (int dt = 0; dt < ND; dt++)
#pragma unroll
        for (int i = 0; i < 16; i++) o[dt][i] = 0.0f;
    float m = -INFINITY, l = 0.0f;

    fetch(0);
    for (int kt = 0; kt < n_kt; kt++) {
        stash();
        __syncthreads();
        if (kt + 1 < n_kt) fetch(kt + 1);

        v16f sc[2];
#pragma unroll
        for (int kk = 0; kk < 2; kk++)
#pragma unroll
            for (int i = 0; i < 16; i++) sc[kk][i] = 0.0f;
#pragma unroll
        for (int s = 0; s < NS; s++) {
            const h8 qlo = *(const h8*)(Ql + row * KS + 16 * s + 8 * g);
#pragma unroll
            for (int kk = 0; kk < 2; kk++) {
                const h8 kf = *(const h8*)(Ks + (32 * kk + r) * KS + 16 * s + 8 * g);
                sc[kk] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf, qh[s], sc[kk], 0, 0, 0);
                sc[kk] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf, qlo, sc[kk], 0, 0, 0);
            }
            if ((s & 3) == 3) __builtin_amdgcn_sched_barrier(0);   // a few fragments in flight: registers are short
        }
        if (kt * KT + KT - 1 > first_pos) {   // some row of the block cannot see the whole tile
#pragma unroll
            for (int kk = 0; kk < 2; kk++)
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    const int key = kt * KT + 32 * kk + 8 * (i >> 2) + 4 * g + (i & 3);
                    if (key > pos) sc[kk][i] = -INFINITY;
                }
        }
        float mt = -INFINITY;
#pragma unroll
        for (int kk = 0; kk < 2; kk++)
#pragma unroll
            for (int i = 0; i < 16; i++) mt = fmaxf(mt, sc[kk][i]);
        mt = fmaxf(mt, __shfl_xor(mt, 32, 64));
        const float m_new = fmaxf(m, mt);   // finite from the first tile on: key 0 is visible to every row
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
        if (__any(alpha != 1.0f)) {
#pragma unroll
            for (int dt = 0; dt < ND; dt++)
#pragma unroll
                for (int i = 0; i < 16; i++) o[dt][i] *= alpha;
        }
#pragma unroll
        for (int dt = 0; dt < ND; dt++) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const uint16_t* vp = Vt + (32 * dt + r) * VS + 16 * j + 4 * g;
                const uint2 v0 = *(const uint2*)vp, v1 = *(const uint2*)(vp + 8);
                const h8 vf = __builtin_bit_cast(h8, make_uint4(v0.x, v0.y, v1.x, v1.y));
                o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf, pf[j], o[dt], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        __syncthreads();
    }

    l += __shfl_xor(l, 32, 64);
    if (valid) {
        const float inv = 1.0f / l;
        float* orow = out + (int64_t)token * qdim + head * HD + 4 * g;
#pragma unroll
        for (int dt = 0; dt < ND; dt++)
#pragma unroll
            for (int i4 = 0; i4 < 4; i4++)
                *(float4*)(orow + 32 * dt + 8 * i4) = make_float4(o[dt][4 * i4] * inv, o[dt][4 * i4 + 1] * inv,
                                                                 o[dt][4 * i4 + 2] * inv, o[dt][4 * i4 + 3] * inv);
    }
}

template <int HD, int G>
bool launch_prefill(const AttnArgs& a, float* out, hipStream_t s) {
    constexpr int QT = 128 / G;
    const size_t lds = ((size_t)(KT + 128) * (HD + 8) + (size_t)HD * VS) * sizeof(uint16_t);
    static bool sized = false;
    if (!sized) {
        if (lds > 64 * 1024 &&
            hipFuncSetAttribute((const void*)attend_prefill_k<HD, G>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) {
            (void)hipGetLastError();
            return false;
        }
        sized = true;
    }
    hipLaunchKernelGGL((attend_prefill_k<HD, G>), dim3((a.n_q + QT - 1) / QT, a.n_head_kv), dim3(256), lds, s, a, out);
    return true;
}

template <int HD>
bool launch_prefill_g(const AttnArgs& a, float* out, hipStream_t s) {
    switch (a.n_head / a.n_head_kv) {
        case 1: return launch_prefill<HD, 1>(a, out, s);
        case 2: return launch_prefill<HD, 2>(a, out, s);
        case 4: return launch_prefill<HD, 4>(a, out, s);
        case 8: return launch_prefill<HD, 8>(a, out, s);
        case 16: return launch_prefill<HD, 16>(a, out, s);
        default: return false;
    }
}

}  // namespace

// whether the one-pass kernel takes the shape (then the split kernels' scratch is not needed)
bool attend_prefill_takes(const AttnArgs& a, const float* out) {
    if (a.n_pos_dyn || a.n_q <= 16 || a.n_pos < a.n_q || a.n_head_kv <= 0 || a.n_head % a.n_head_kv) return false;
    if (a.kv_dim % 8 || (reinterpret_cast<uintptr_t>(a.k) & 15) || (reinterpret_cast<uintptr_t>(a.v) & 15) ||
        (reinterpret_cast<uintptr_t>(a.q) & 15) || (reinterpret_cast<uintptr_t>(out) & 15))
        return false;
    const int G = a.n_head / a.n_head_kv;
    if (G != 1 && G != 2 && G != 4 && G != 8 && G != 16) return false;
    return a.head_dim == 64 || a.head_dim == 128 || a.head_dim == 256;
}

// false: not a shape this kernel takes (the caller uses the split kernels)
bool attend_prefill(const AttnArgs& a, float* out, hipStream_t s) {
    if (!attend_prefill_takes(a, out)) return false;
    switch (a.head_dim) {
        case 64: return launch_prefill_g<64>(a, out, s);
        case 128: return launch_prefill_g<128>(a, out, s);
        case 256: return launch_prefill_g<256>(a, out, s);
        default: return false;
    }
}

}  // namespace itk
