// Gated delta rule (GatedDeltaNet's recurrent core).
//
// Follows /root/reference src/ops/naive.rs:86-135 per token and :339-350 over the
// batch; head grouping is modulo (src/ops/mod.rs:404-413).  State is
// [value head][value row][key] f32, key contiguous.
//
// One lane owns one value row: the row's dk floats stay in registers for the
// whole batch, so the three sweeps (decay+predict, correct, read out) run in the
// reference's order with no cross-lane reduction and the result is bit-identical
// to the CPU path.  The 64-row tile moves between HBM and registers through a
// padded LDS tile so both the load and the store are fully coalesced.
#include "it_device.h"
#include "it_reduce.h"
#include "kernels.h"

namespace itk {

template <int DK>
__global__ __launch_bounds__(64) void delta_rule_k(DeltaArgs d, float* __restrict__ state,
                                                   float* __restrict__ out, float q_scale) {
    __shared__ float tile[64 * (DK + 1)];
    __shared__ __align__(16) float kq[2 * DK];
    const int lane = threadIdx.x;
    const int dv = d.head_v_dim;
    const int blocks_per_head = (dv + 63) / 64;
    const int h = blockIdx.x / blocks_per_head, jb = blockIdx.x % blocks_per_head;
    const int kh = h % d.n_k_heads;
    const int j = jb * 64 + lane;
    const bool live = j < dv;
    const int rows_here = min(64, dv - jb * 64);
    float* S = state + ((int64_t)h * dv + (int64_t)jb * 64) * DK;

    // 64 rows x DK floats = 16*DK float4; every load is issued before the first LDS write
    {
        constexpr int V = DK / 4;  // float4 per row
        const float4* S4 = (const float4*)S;
        float4 stage[V];
#pragma unroll
        for (int it = 0; it < V; it++) {
            int idx4 = it * 64 + lane;
            stage[it] = (idx4 < rows_here * V) ? S4[idx4] : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int it = 0; it < V; it++) {
            int idx4 = it * 64 + lane;
            int r = idx4 / V, c = (idx4 - r * V) * 4;
            float* t = tile + r * (DK + 1) + c;
            t[0] = stage[it].x; t[1] = stage[it].y; t[2] = stage[it].z; t[3] = stage[it].w;
        }
    }
    __syncthreads();
    float row[DK];
#pragma unroll
    for (int i = 0; i < DK; i++) row[i] = live ? tile[lane * (DK + 1) + i] : 0.0f;

    const int kper = d.n_k_heads * DK, vper = d.n_v_heads * dv;
    for (int t = 0; t < d.n_tokens; t++) {
        __syncthreads();
        for (int i = lane; i < DK; i += 64) {
            kq[i] = d.k[(int64_t)t * kper + kh * DK + i];
            kq[DK + i] = d.q[(int64_t)t * kper + kh * DK + i];
        }
        __syncthreads();
        float a = d.alpha[(int64_t)t * d.n_v_heads + h] + d.dt_bias[h];
        float softplus = a > 20.0f ? a : it_logf(1.0f + it_expf(a));
        float g = it_expf(softplus * d.ssm_a[h]);
        float beta = 1.0f / (1.0f + it_expf(-d.beta[(int64_t)t * d.n_v_heads + h]));
        float v = live ? d.v[(int64_t)t * vper + h * dv + j] : 0.0f;
        float pred = 0.0f;
        const float4* k4 = (const float4*)kq;
        const float4* q4 = (const float4*)(kq + DK);
#pragma unroll
        for (int i = 0; i < DK; i += 4) {
            float4 kk = k4[i / 4];
            row[i] *= g;     pred += row[i] * kk.x;
            row[i + 1] *= g; pred += row[i + 1] * kk.y;
            row[i + 2] *= g; pred += row[i + 2] * kk.z;
            row[i + 3] *= g; pred += row[i + 3] * kk.w;
        }
        float delta = beta * (v - pred);
        float o = 0.0f;
#pragma unroll
        for (int i = 0; i < DK; i += 4) {
            float4 kk = k4[i / 4], qq = q4[i / 4];
            row[i] += kk.x * delta;     o += row[i] * (qq.x * q_scale);
            row[i + 1] += kk.y * delta; o += row[i + 1] * (qq.y * q_scale);
            row[i + 2] += kk.z * delta; o += row[i + 2] * (qq.z * q_scale);
            row[i + 3] += kk.w * delta; o += row[i + 3] * (qq.w * q_scale);
        }
        if (live) out[(int64_t)t * vper + h * dv + j] = o;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < DK; i++)
        if (live) tile[lane * (DK + 1) + i] = row[i];
    __syncthreads();
    {
        constexpr int V = DK / 4;
        float4* S4 = (float4*)S;
#pragma unroll
        for (int it = 0; it < V; it++) {
            int idx4 = it * 64 + lane;
            int r = idx4 / V, c = (idx4 - r * V) * 4;
            const float* t = tile + r * (DK + 1) + c;
            if (idx4 < rows_here * V) S4[idx4] = make_float4(t[0], t[1], t[2], t[3]);
        }
    }
}

// ------------------------------------------------------------------ fast form over a batch
// 32 value rows per block, 8 lanes per row (DK / 8 keys each): the row's dots are reduced
// with three lane exchanges, so the sums are not in the CPU path's order (fast mode only).
// The gates of every token of the batch are formed once, up front, in LDS.  The batch is
// walked in chunks of 16 tokens: a chunk's k, q and v are staged into LDS with coalesced
// loads while the previous chunk is being applied, so a token step touches only LDS and
// registers and the only block barrier is the one between chunks.
constexpr int GDN_TCH = 16;

template <int DK>
__global__ __launch_bounds__(256) void delta_rule_fast_k(DeltaArgs d, float* __restrict__ state,
                                                         float* __restrict__ out, float q_scale) {
    constexpr int SEG = DK / 8;
    constexpr int V4 = SEG / 4;
    constexpr int KQ4 = GDN_TCH * DK / 4;          // float4 per chunk of k (and of q)
    constexpr int KQL = (KQ4 + 255) / 256;          // per thread
    extern __shared__ __align__(16) float lds[];
    float* gates = lds;                                               // [n_tokens][2]
    float* kbuf = lds + (((size_t)d.n_tokens * 2 + 3) & ~(size_t)3);  // [2][TCH][DK]
    float* qbuf = kbuf + 2 * GDN_TCH * DK;                            // [2][TCH][DK]
    float* vbuf = qbuf + 2 * GDN_TCH * DK;                            // [2][TCH][32]
    const int tid = threadIdx.x, seg = tid & 7, r = tid >> 3;
    const int dv = d.head_v_dim;
    const int bph = dv / 32;
    const int h = blockIdx.x / bph, jb = blockIdx.x % bph, kh = h % d.n_k_heads;
    const int j = jb * 32 + r;
    const int kper = d.n_k_heads * DK, vper = d.n_v_heads * dv;
    for (int t = tid; t < d.n_tokens; t += 256) {
        const float a = d.alpha[(int64_t)t * d.n_v_heads + h] + d.dt_bias[h];
        const float softplus = a > 20.0f ? a : fx_logf(1.0f + fx_expf(a));
        gates[2 * t] = fx_expf(softplus * d.ssm_a[h]);
        gates[2 * t + 1] = fx_sigmoid(d.beta[(int64_t)t * d.n_v_heads + h]);
    }
    float* S = state + ((int64_t)h * dv + j) * DK + seg * SEG;
    float row[SEG];
#pragma unroll
    for (int i = 0; i < V4; i++) {
        const float4 t4 = ((const float4*)S)[i];
        row[4 * i] = t4.x; row[4 * i + 1] = t4.y; row[4 * i + 2] = t4.z; row[4 * i + 3] = t4.w;
    }
    float4 rk[KQL], rq[KQL];
    float rv[2];
    auto fetch = [&](int t0) {
#pragma unroll
        for (int p = 0; p < KQL; p++) {
            const int idx = tid + p * 256, tt = idx / (DK / 4), c4 = idx % (DK / 4);
            const bool ok = idx < KQ4 && t0 + tt < d.n_tokens;
            rk[p] = ok ? ((const float4*)(d.k + (int64_t)(t0 + tt) * kper + kh * DK))[c4] : make_float4(0.f, 0.f, 0.f, 0.f);
            rq[p] = ok ? ((const float4*)(d.q + (int64_t)(t0 + tt) * kper + kh * DK))[c4] : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int p = 0; p < 2; p++) {
            const int idx = tid + p * 256, tt = idx >> 5, rr = idx & 31;
            rv[p] = t0 + tt < d.n_tokens ? d.v[(int64_t)(t0 + tt) * vper + h * dv + jb * 32 + rr] : 0.0f;
        }
    };
    auto stash = [&](int buf) {
#pragma unroll
        for (int p = 0; p < KQL; p++) {
            const int idx = tid + p * 256;
            if (idx < KQ4) {
                ((float4*)(kbuf + buf * GDN_TCH * DK))[idx] = rk[p];
                ((float4*)(qbuf + buf * GDN_TCH * DK))[idx] = rq[p];
            }
        }
#pragma unroll
        for (int p = 0; p < 2; p++) vbuf[buf * GDN_TCH * 32 + tid + p * 256] = rv[p];
    };
    fetch(0);
    stash(0);
    __syncthreads();
    for (int t0 = 0, c = 0; t0 < d.n_tokens; t0 += GDN_TCH, c++) {
        const int buf = c & 1;
        if (t0 + GDN_TCH < d.n_tokens) fetch(t0 + GDN_TCH);
        const int nt = min(GDN_TCH, d.n_tokens - t0);
        for (int tt = 0; tt < nt; tt++) {
            const float4* k4 = (const float4*)(kbuf + (buf * GDN_TCH + tt) * DK + seg * SEG);
            const float4* q4 = (const float4*)(qbuf + (buf * GDN_TCH + tt) * DK + seg * SEG);
            float kk[SEG], qq[SEG];
#pragma unroll
            for (int i = 0; i < V4; i++) {
                const float4 a = k4[i], b = q4[i];
                kk[4 * i] = a.x; kk[4 * i + 1] = a.y; kk[4 * i + 2] = a.z; kk[4 * i + 3] = a.w;
                qq[4 * i] = b.x; qq[4 * i + 1] = b.y; qq[4 * i + 2] = b.z; qq[4 * i + 3] = b.w;
            }
            const float v = vbuf[(buf * GDN_TCH + tt) * 32 + r];
            const float g = gates[2 * (t0 + tt)], beta = gates[2 * (t0 + tt) + 1];
            float pred = 0.0f;
#pragma unroll
            for (int i = 0; i < SEG; i++) {
                row[i] *= g;
                pred += row[i] * kk[i];
            }
            pred = sum8_lanes(pred);
            const float delta = beta * (v - pred);
            float o = 0.0f;
#pragma unroll
            for (int i = 0; i < SEG; i++) {
                row[i] += kk[i] * delta;
                o += row[i] * (qq[i] * q_scale);
            }
            o = sum8_lanes(o);
            if (seg == 0) out[(int64_t)(t0 + tt) * vper + h * dv + j] = o;
        }
        if (t0 + GDN_TCH < d.n_tokens) stash(buf ^ 1);
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < V4; i++)
        ((float4*)S)[i] = make_float4(row[4 * i], row[4 * i + 1], row[4 * i + 2], row[4 * i + 3]);
}

void delta_rule(const DeltaArgs& d, float* state, float* out, int exact, float* work, size_t work_floats, hipStream_t s) {
    if (d.n_tokens <= 0) return;
    if (!exact && delta_rule_chunked(d, state, out, work, work_floats, s)) return;
    float q_scale = 1.0f / sqrtf((float)d.head_k_dim);
    const size_t gate_lds = ((((size_t)d.n_tokens * 2 + 3) & ~(size_t)3) + 4 * GDN_TCH * d.head_k_dim + 2 * GDN_TCH * 32) * sizeof(float);
    if (!exact && d.head_v_dim % 32 == 0 && (d.head_k_dim == 64 || d.head_k_dim == 128) && gate_lds <= 96 * 1024) {
        const int blocks = d.n_v_heads * (d.head_v_dim / 32);
        if (d.head_k_dim == 64) hipLaunchKernelGGL(delta_rule_fast_k<64>, dim3(blocks), dim3(256), gate_lds, s, d, state, out, q_scale);
        else hipLaunchKernelGGL(delta_rule_fast_k<128>, dim3(blocks), dim3(256), gate_lds, s, d, state, out, q_scale);
        return;
    }
    int blocks = d.n_v_heads * ((d.head_v_dim + 63) / 64);
    switch (d.head_k_dim) {
        case 32: hipLaunchKernelGGL(delta_rule_k<32>, dim3(blocks), dim3(64), 0, s, d, state, out, q_scale); break;
        case 64: hipLaunchKernelGGL(delta_rule_k<64>, dim3(blocks), dim3(64), 0, s, d, state, out, q_scale); break;
        case 128: hipLaunchKernelGGL(delta_rule_k<128>, dim3(blocks), dim3(64), 0, s, d, state, out, q_scale); break;
        default: break;  // the caller validates head_k_dim
    }
}

}  // namespace itk
