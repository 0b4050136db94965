// Gated delta rule over a long batch, in chunks of 64 tokens, with the dense products on fp32 MFMA.
//
// Same recurrence as /root/reference src/ops/naive.rs:86-135 (per token) and :339-350 (batch):
//     S' = g_t S,   d_t = beta_t (v_t - S' k_t),   S = S' + d_t k_t^T,   o_t = S (q_t / sqrt(dk))
// with S = [value row][key].  Within a chunk starting from S0, with c_t = sum_{s<=t} log g_s,
//     S_t = e^{c_t} S0 + sum_{i<=t} e^{c_t - c_i} u_i k_i^T
// and the corrections u_t solve the unit lower-triangular system
//     (I + A) U = diag(beta) (V - diag(e^{c}) K S0^T),   A[t][i] = beta_t e^{c_t - c_i} (k_t . k_i), i < t.
// So per chunk:  U = T R with T = (I + A)^-1,  O = diag(e^{c}) Q S0^T + P U with
// P[t][i] = e^{c_t - c_i} (q_t . k_i) for i <= t,  and  S_C = e^{c_C} S0 + U^T diag(e^{c_C - c_t}) K.
// T and P do not depend on the state: one launch forms them for every (chunk, head) at once;
// a second launch walks the chunks in order, one block per 16 value rows of a head (the rows of
// S are independent), and carries its slice of S in MFMA accumulators from chunk to chunk.
//
// The sums are not in the CPU path's order: fast mode only; results agree to ~1e-5.
#include "it_device.h"
#include "kernels.h"

// Phase stamps for tuning: a build with -DIT_STAMPS records the 100 MHz wall clock of one block's
// first lane of one wave at the marked points of one chunk; the library build compiles them away.
#ifdef IT_STAMPS
__device__ long long it_gdn_stamps[32];
__device__ int it_gdn_stamp_block, it_gdn_stamp_wave, it_gdn_stamp_chunk;
#define GDN_STAMP(i)                                                                                      \
    do {                                                                                                  \
        if ((int)blockIdx.x == it_gdn_stamp_block && w == it_gdn_stamp_wave && c == it_gdn_stamp_chunk && \
            lane == 0)                                                                                    \
            it_gdn_stamps[i] = wall_clock64();                                                            \
    } while (0)
#else
#define GDN_STAMP(i) \
    do {             \
    } while (0)
#endif

namespace itk {

typedef float v4f __attribute__((ext_vector_type(4)));

namespace {
constexpr int GC = 64;                      // tokens per chunk
constexpr int TS = GC + 4;                  // LDS row stride of the 64 x 64 matrices
constexpr int DVS = 16;                     // value rows per block of the scan
constexpr int US = 20;                      // LDS row stride of U and of R: four rows apart are 16 banks apart
// per (chunk, head): T[64][64], P[64][64], e^{c_t}, e^{c_C - c_t}, beta_t, and e^{c_C} in one padded row
constexpr int WS_T = 0, WS_P = GC * GC, WS_GAM = 2 * GC * GC, WS_DEC = WS_GAM + GC, WS_BET = WS_DEC + GC,
              WS_GC = WS_BET + GC, WS_FLOATS = WS_GC + GC;

// D = A(16 x 4) B(4 x 16) + C: lane l gives A[l % 16][l / 16] and B[l / 16][l % 16], and holds
// D[4 * (l / 16) + i][l % 16] in component i.
__device__ __forceinline__ v4f mfma4(float a, float b, v4f c) {
    return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}
}  // namespace

size_t gdn_chunk_work_floats(int n_tokens, int n_v_heads) {
    return (size_t)((n_tokens + GC - 1) / GC) * n_v_heads * WS_FLOATS;
}

// ---------------------------------------------------------------- T and P of every (chunk, head)
template <int DK>
__global__ __launch_bounds__(256) void gdn_chunk_prep_k(DeltaArgs d, float* __restrict__ work, float q_scale) {
    constexpr int LS = DK + 4;
    extern __shared__ __align__(16) float lds[];
    float* Ks = lds;                 // [64][LS]
    float* Qs = Ks + GC * LS;        // [64][LS]
    float* At = Qs;                  // [64][TS]: A transposed, written once the products with Q are done
    float* cum = Qs + GC * LS;       // [64]
    float* bet = cum + GC;           // [64]
    const int tid = threadIdx.x, lane = tid & 63, w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int c = blockIdx.x, h = blockIdx.y, kh = h % d.n_k_heads;
    const int t0 = c * GC;
    const int kper = d.n_k_heads * DK;
    float* ws = work + ((size_t)c * d.n_v_heads + h) * WS_FLOATS;

    if (w == 0) {
        const int t = t0 + lane;
        const bool ok = t < d.n_tokens;
        float lg = 0.0f, beta = 0.0f;
        if (ok) {
            const float a = d.alpha[(int64_t)t * d.n_v_heads + h] + d.dt_bias[h];
            const float softplus = a > 20.0f ? a : fx_logf(1.0f + fx_expf(a));
            lg = softplus * d.ssm_a[h];
            beta = 1.0f / (1.0f + fx_expf(-d.beta[(int64_t)t * d.n_v_heads + h]));
        }
        float x = lg;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const float y = __shfl_up(x, off, 64);
            if (lane >= off) x += y;
        }
        const float xc = __shfl(x, 63, 64);
        cum[lane] = x;
        bet[lane] = beta;
        ws[WS_GAM + lane] = fx_expf(x);
        ws[WS_DEC + lane] = fx_expf(xc - x);
        ws[WS_BET + lane] = beta;
        ws[WS_GC + lane] = fx_expf(xc);
    }
    for (int idx = tid; idx < GC * DK / 4; idx += 256) {
        const int tt = idx / (DK / 4), c4 = idx % (DK / 4);
        float4 kk = make_float4(0.f, 0.f, 0.f, 0.f), qq = kk;
        if (t0 + tt < d.n_tokens) {
            kk = ((const float4*)(d.k + (int64_t)(t0 + tt) * kper + kh * DK))[c4];
            qq = ((const float4*)(d.q + (int64_t)(t0 + tt) * kper + kh * DK))[c4];
        }
        *(float4*)(Ks + tt * LS + 4 * c4) = kk;
        *(float4*)(Qs + tt * LS + 4 * c4) = make_float4(qq.x * q_scale, qq.y * q_scale, qq.z * q_scale, qq.w * q_scale);
    }
    __syncthreads();

    // wave w: token rows 16w..16w+15 against the column tiles at or below the diagonal
    const int m = lane & 15, g = lane >> 4;
    // products first (they read Q), masks after the barrier (A^T takes Q's place)
    v4f accG[4], accQ[4];
#pragma unroll
    for (int ct = 0; ct < 4; ct++) {
        accG[ct] = accQ[ct] = v4f{0.f, 0.f, 0.f, 0.f};
        if (ct <= w) {
            v4f ag = {0.f, 0.f, 0.f, 0.f}, aq = ag;
#pragma unroll 8
            for (int s = 0; s < DK / 4; s++) {
                const float b = Ks[(16 * ct + m) * LS + 4 * s + g];
                ag = mfma4(Ks[(16 * w + m) * LS + 4 * s + g], b, ag);
                aq = mfma4(Qs[(16 * w + m) * LS + 4 * s + g], b, aq);
            }
            accG[ct] = ag;
            accQ[ct] = aq;
        }
    }
    __syncthreads();   // every wave is done reading Q before A takes its place
    float* P = ws + WS_P;
#pragma unroll
    for (int ct = 0; ct < 4; ct++) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int t = 16 * w + 4 * g + i, ii = 16 * ct + m;
            float a = 0.0f, p = 0.0f;
            if (ii <= t) {
                const float ratio = __expf(cum[t] - cum[ii]);
                p = ratio * accQ[ct][i];
                if (ii < t) a = bet[t] * ratio * accG[ct][i];
            }
            At[ii * TS + t] = a;
            P[t * GC + ii] = p;
        }
    }
    __syncthreads();

    // T = (I + A)^-1 by forward substitution, one column per lane: T_t = e_t - sum_{i<t} A[t][i] T_i.
    // Row i, once final, is taken out of every later row at once: 63 - i independent multiply-adds,
    // so the only serial chain is one multiply-add per row.
    if (w == 0) {
        float Tr[GC];
        float* T = ws + WS_T;
#pragma unroll
        for (int t = 0; t < GC; t++) Tr[t] = lane == t ? 1.0f : 0.0f;
#pragma unroll
        for (int i0 = 0; i0 < GC; i0 += 2) {
            // two rows of A^T at a time, fetched together so the LDS latency is paid once per batch
            __builtin_amdgcn_sched_barrier(0);   // keep later batches' loads from being hoisted over this one
            float a[2][GC];
#pragma unroll
            for (int r = 0; r < 2; r++)
#pragma unroll
                for (int t = 0; t < GC; t++)
                    if (t >= i0) a[r][t] = At[(i0 + r) * TS + t];
#pragma unroll
            for (int r = 0; r < 2; r++) {
                const int i = i0 + r;
                T[i * GC + lane] = Tr[i];
#pragma unroll
                for (int t = 0; t < GC; t++)
                    if (t > i) Tr[t] = fmaf(-a[r][t], Tr[i], Tr[t]);
            }
        }
    }
}

// ---------------------------------------------------------------- the walk over the chunks
template <int DK>
__global__ __launch_bounds__(256) void gdn_chunk_scan_k(DeltaArgs d, const float* __restrict__ work,
                                                        float* __restrict__ state, float* __restrict__ out,
                                                        float q_scale) {
    constexpr int LS = DK + 4;
    constexpr int KQV = GC * DK / 4 / 256;   // float4 of K (and of Q) per thread
    constexpr int CT = DK / 64;              // state column tiles per wave
    extern __shared__ __align__(16) float lds[];
    float* Ks = lds;                 // [64][LS]
    float* Qs = Ks + GC * LS;        // [64][LS]
    float* Ts = Qs + GC * LS;        // [64][TS]
    float* Ps = Ts + GC * TS;        // [64][TS]
    float* Ss = Ps + GC * TS;        // [16][LS]
    float* Vs = Ss + DVS * LS;       // [64][16]
    float* Rs = Vs + GC * DVS;       // [64][US]
    float* Us = Rs + GC * US;        // [64][US]
    float* gam = Us + GC * US;       // [64] e^{c_t}
    float* dec = gam + GC;           // [64] e^{c_C - c_t}
    float* bet = dec + GC;           // [64]
    float* gcs = bet + GC;           // [64] e^{c_C}
    const int tid = threadIdx.x, lane = tid & 63, w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int m = lane & 15, g = lane >> 4;
    // blocks are dealt to the 8 XCDs round-robin: the slices of one head take consecutive places on ONE XCD,
    // so a chunk's K, Q, T and P are fetched into one L2 rather than eight
    const int dv = d.head_v_dim;
    const int n_slices = dv / DVS, total = d.n_v_heads * n_slices, per_xcd = (total + 7) / 8;
    const int item = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (item >= total) return;
    const int h = item / n_slices, kh = h % d.n_k_heads, j0 = (item % n_slices) * DVS;
    const int kper = d.n_k_heads * DK, vper = d.n_v_heads * dv;
    const int n_chunks = (d.n_tokens + GC - 1) / GC;
    float* S = state + ((int64_t)h * dv + j0) * DK;

    // this wave's tiles of S: rows 4g+i, columns 16 * (w + 4 * x) + m
    v4f st[CT];
#pragma unroll
    for (int x = 0; x < CT; x++)
#pragma unroll
        for (int i = 0; i < 4; i++) st[x][i] = S[(4 * g + i) * DK + 16 * (w + 4 * x) + m];

    float4 rk[KQV], rq[KQV], rt[4], rp[4], rv, rg;
    rv = rg = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int p = 0; p < 4; p++) rt[p] = rp[p] = rv;
    // the next chunk's operands come in three parts, issued between the stages of the current one, so the
    // load unit is never handed 100 KB at once
    auto fetch_k = [&](int c) __attribute__((always_inline)) {
        const int t0 = c * GC;
#pragma unroll
        for (int p = 0; p < KQV; p++) {
            const int idx = tid + p * 256, tt = idx / (DK / 4), c4 = idx % (DK / 4);
            rk[p] = t0 + tt < d.n_tokens ? ((const float4*)(d.k + (int64_t)(t0 + tt) * kper + kh * DK))[c4]
                                         : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    };
    auto fetch_q = [&](int c) __attribute__((always_inline)) {
        const int t0 = c * GC;
#pragma unroll
        for (int p = 0; p < KQV; p++) {
            const int idx = tid + p * 256, tt = idx / (DK / 4), c4 = idx % (DK / 4);
            rq[p] = t0 + tt < d.n_tokens ? ((const float4*)(d.q + (int64_t)(t0 + tt) * kper + kh * DK))[c4]
                                         : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    };
    auto fetch_rest = [&](int c) __attribute__((always_inline)) {
        const int t0 = c * GC;
        const float* ws = work + ((size_t)c * d.n_v_heads + h) * WS_FLOATS;
#pragma unroll
        for (int p = 0; p < 4; p++) {
            rt[p] = ((const float4*)(ws + WS_T))[tid + p * 256];
            rp[p] = ((const float4*)(ws + WS_P))[tid + p * 256];
        }
        {
            const int tt = tid >> 2, c4 = tid & 3;
            rv = t0 + tt < d.n_tokens ? ((const float4*)(d.v + (int64_t)(t0 + tt) * vper + h * dv + j0))[c4]
                                      : make_float4(0.f, 0.f, 0.f, 0.f);
        }
        if (tid < GC) rg = ((const float4*)(ws + WS_GAM))[tid];   // gam, dec, bet, gcs are contiguous
    };
    auto stash = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int p = 0; p < KQV; p++) {
            const int idx = tid + p * 256, tt = idx / (DK / 4), c4 = idx % (DK / 4);
            *(float4*)(Ks + tt * LS + 4 * c4) = rk[p];
            *(float4*)(Qs + tt * LS + 4 * c4) =
                make_float4(rq[p].x * q_scale, rq[p].y * q_scale, rq[p].z * q_scale, rq[p].w * q_scale);
        }
#pragma unroll
        for (int p = 0; p < 4; p++) {
            const int idx = tid + p * 256, tt = idx >> 4, c4 = idx & 15;
            *(float4*)(Ts + tt * TS + 4 * c4) = rt[p];
            *(float4*)(Ps + tt * TS + 4 * c4) = rp[p];
        }
        ((float4*)Vs)[tid] = rv;
        if (tid < GC) ((float4*)gam)[tid] = rg;
#pragma unroll
        for (int x = 0; x < CT; x++)
#pragma unroll
            for (int i = 0; i < 4; i++) Ss[(4 * g + i) * LS + 16 * (w + 4 * x) + m] = st[x][i];
    };

    fetch_k(0);
    fetch_q(0);
    fetch_rest(0);
    for (int c = 0; c < n_chunks; c++) {
        const int t0 = c * GC;
        GDN_STAMP(0);
        stash();
        GDN_STAMP(1);
        __syncthreads();
        GDN_STAMP(2);
        const bool more = c + 1 < n_chunks;
        if (more) fetch_k(c + 1);
        GDN_STAMP(3);

        // K S0^T and Q S0^T for this wave's 16 tokens
        // operands of four steps are read while the four steps before them are on the matrix unit
        v4f aw = {0.f, 0.f, 0.f, 0.f}, ao = {0.f, 0.f, 0.f, 0.f};
        {
            // (the k order inside a step of 16 is free as long as both operands agree: lane group g takes k = 4 g + j in
            // step j, so that a lane's four values are one 16-byte read, which no two lanes of a pass take from one bank)
            constexpr int NB = DK / 16;
            float4 ka[2], qa[2], sb[2];
            const float* kp = Ks + (16 * w + m) * LS + 4 * g;
            const float* qp = Qs + (16 * w + m) * LS + 4 * g;
            const float* sp = Ss + m * LS + 4 * g;
            ka[0] = *(const float4*)kp; qa[0] = *(const float4*)qp; sb[0] = *(const float4*)sp;
#pragma unroll
            for (int b = 0; b < NB; b++) {
                if (b + 1 < NB) {
                    ka[(b + 1) & 1] = *(const float4*)(kp + 16 * (b + 1));
                    qa[(b + 1) & 1] = *(const float4*)(qp + 16 * (b + 1));
                    sb[(b + 1) & 1] = *(const float4*)(sp + 16 * (b + 1));
                }
                __builtin_amdgcn_sched_barrier(0);   // the reads stay ahead of the products they overlap
                const float4 k4 = ka[b & 1], q4 = qa[b & 1], s4v = sb[b & 1];
                aw = mfma4(k4.x, s4v.x, aw); ao = mfma4(q4.x, s4v.x, ao);
                aw = mfma4(k4.y, s4v.y, aw); ao = mfma4(q4.y, s4v.y, ao);
                aw = mfma4(k4.z, s4v.z, aw); ao = mfma4(q4.z, s4v.z, ao);
                aw = mfma4(k4.w, s4v.w, aw); ao = mfma4(q4.w, s4v.w, ao);
            }
        }
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int t = 16 * w + 4 * g + i;
            Rs[t * US + m] = bet[t] * (Vs[t * DVS + m] - gam[t] * aw[i]);
            ao[i] *= gam[t];
        }
        GDN_STAMP(4);
        __syncthreads();
        GDN_STAMP(5);
        if (more) fetch_q(c + 1);

        // U = T R: rows of T at or left of the diagonal tile
        v4f au = {0.f, 0.f, 0.f, 0.f};
        for (int s4 = 0; s4 <= w; s4++) {
            const float4 t4 = *(const float4*)(Ts + (16 * w + m) * TS + 16 * s4 + 4 * g);
            const float* rp_ = Rs + (16 * s4 + 4 * g) * US + m;
            au = mfma4(t4.x, rp_[0], au);
            au = mfma4(t4.y, rp_[US], au);
            au = mfma4(t4.z, rp_[2 * US], au);
            au = mfma4(t4.w, rp_[3 * US], au);
        }
#pragma unroll
        for (int i = 0; i < 4; i++) Us[(16 * w + 4 * g + i) * US + m] = au[i];
        GDN_STAMP(6);
        __syncthreads();
        GDN_STAMP(7);
        if (more) fetch_rest(c + 1);

        // O = e^{c} Q S0^T + P U
        for (int s4 = 0; s4 <= w; s4++) {
            const float4 p4 = *(const float4*)(Ps + (16 * w + m) * TS + 16 * s4 + 4 * g);
            const float* up_ = Us + (16 * s4 + 4 * g) * US + m;
            ao = mfma4(p4.x, up_[0], ao);
            ao = mfma4(p4.y, up_[US], ao);
            ao = mfma4(p4.z, up_[2 * US], ao);
            ao = mfma4(p4.w, up_[3 * US], ao);
        }
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int t = t0 + 16 * w + 4 * g + i;
            if (t < d.n_tokens) out[(int64_t)t * vper + h * dv + j0 + m] = ao[i];
        }

        GDN_STAMP(8);
        // S = e^{c_C} S0 + U^T diag(e^{c_C - c_t}) K
        const float gc = gcs[0];
#pragma unroll
        for (int x = 0; x < CT; x++)
#pragma unroll
            for (int i = 0; i < 4; i++) st[x][i] *= gc;
        {
            // any order of the 64 tokens will do: lane group g takes tokens 2g apart, which spreads the
            // four groups' reads of K and of U over all 32 banks
            float ua[2][4], kb[2][4][CT];
            auto token = [&](int s) { return 8 * (s >> 1) + 2 * g + (s & 1); };
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int t = token(u);
                ua[0][u] = Us[t * US + m] * dec[t];
#pragma unroll
                for (int x = 0; x < CT; x++) kb[0][u][x] = Ks[t * LS + 16 * (w + 4 * x) + m];
            }
#pragma unroll
            for (int b = 0; b < GC / 16; b++) {
                if (b + 1 < GC / 16) {
#pragma unroll
                    for (int u = 0; u < 4; u++) {
                        const int t = token(4 * (b + 1) + u);
                        ua[(b + 1) & 1][u] = Us[t * US + m] * dec[t];
#pragma unroll
                        for (int x = 0; x < CT; x++) kb[(b + 1) & 1][u][x] = Ks[t * LS + 16 * (w + 4 * x) + m];
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int u = 0; u < 4; u++)
#pragma unroll
                    for (int x = 0; x < CT; x++) st[x] = mfma4(ua[b & 1][u], kb[b & 1][u][x], st[x]);
            }
        }
        GDN_STAMP(9);
        __syncthreads();
        GDN_STAMP(10);
    }
#pragma unroll
    for (int x = 0; x < CT; x++)
#pragma unroll
        for (int i = 0; i < 4; i++) S[(4 * g + i) * DK + 16 * (w + 4 * x) + m] = st[x][i];
}

template <int DK>
static bool launch_chunked(const DeltaArgs& d, float* state, float* out, float* work, float q_scale, hipStream_t s) {
    constexpr int LS = DK + 4;
    const size_t prep_lds = (2 * GC * LS + 2 * GC) * sizeof(float);
    const size_t scan_lds = (2 * GC * LS + 2 * GC * TS + DVS * LS + GC * DVS + 2 * GC * US + 4 * GC) * sizeof(float);
    static bool sized = false;
    if (!sized) {
        if (hipFuncSetAttribute((const void*)gdn_chunk_prep_k<DK>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)prep_lds) != hipSuccess ||
            hipFuncSetAttribute((const void*)gdn_chunk_scan_k<DK>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)scan_lds) != hipSuccess) {
            (void)hipGetLastError();
            return false;
        }
        sized = true;
    }
    const int n_chunks = (d.n_tokens + GC - 1) / GC;
    hipLaunchKernelGGL(gdn_chunk_prep_k<DK>, dim3(n_chunks, d.n_v_heads), dim3(256), prep_lds, s, d, work, q_scale);
    const int items = d.n_v_heads * (d.head_v_dim / DVS);
    hipLaunchKernelGGL(gdn_chunk_scan_k<DK>, dim3((items + 7) / 8 * 8), dim3(256), scan_lds, s, d, work, state, out, q_scale);
    return true;
}

bool delta_rule_chunked(const DeltaArgs& d, float* state, float* out, float* work, size_t work_floats, hipStream_t s) {
    if (!work || d.n_tokens < GC || d.head_v_dim % DVS != 0) return false;
    if (work_floats < gdn_chunk_work_floats(d.n_tokens, d.n_v_heads)) return false;
    const float q_scale = 1.0f / sqrtf((float)d.head_k_dim);
    if (d.head_k_dim == 128) return launch_chunked<128>(d, state, out, work, q_scale, s);
    if (d.head_k_dim == 64) return launch_chunked<64>(d, state, out, work, q_scale, s);
    return false;
}

}  // namespace itk
