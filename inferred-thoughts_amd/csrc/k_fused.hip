// Fused single-token kernels.
//
// A decode pass issues ~35 seam ops per layer, each a microsecond-scale kernel, so the
// pass is bound by launch latency rather than HBM.  When a decode pass is captured
// into a graph the backend rewrites runs of seam ops into the kernels below.  Each
// one performs exactly the arithmetic of the ops it replaces, in the same order
// (the `exact` flag keeps the serial f64 norm sums), so results do not change by a bit.
//
//   fused_gemv      [rms_norm] + quantize_q8_0 + up to 4 matmuls on one activation
//                   (+ causal conv + silu on the first output, or += into the output)
//   gdn_core        gather q/k/v + l2_norm(q,k) + delta_rule + rms_norm_heads + silu_mul
//   moe_glu_fused   softmax + top-k + quantize + expert gate/up + shared gate/up + silu_mul
//   moe_down_fused  quantize + expert down + shared down + moe_finish + add_assign
//   attn_prep       gather q/gate + rms_norm_heads(q,k) + rope(q,k) + kv_write(k,v)
//   attn_merge_gate split-K merge + sigmoid_mul
#include "it_device.h"
#include "it_dot.h"
#include "it_reduce.h"
#include "kernels.h"
#include "kernels_fused.h"

namespace itk {

// Q8_0 quantization of `n` floats in LDS (naive.rs:652-675), 8 lanes per 32-block.
__device__ void lds_quantize_q8_0(const float* xf, int n, float* xs, int8_t* xq) {
    const int nb = n >> 5;
    const int tid = threadIdx.x, sub = tid & 7;
    for (int base = 0; base < nb; base += (int)blockDim.x >> 3) {
        int b = base + (tid >> 3);
        bool live = b < nb;
        float4 v = live ? *(const float4*)(xf + b * 32 + sub * 4) : make_float4(0.f, 0.f, 0.f, 0.f);
        float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
        amax = fmaxf(amax, __shfl_xor(amax, 1, 64));
        amax = fmaxf(amax, __shfl_xor(amax, 2, 64));
        amax = fmaxf(amax, __shfl_xor(amax, 4, 64));
        if (live) {
            float d = amax / 127.0f;
            float id = d != 0.0f ? 1.0f / d : 0.0f;
            float r[4] = {roundf(v.x * id), roundf(v.y * id), roundf(v.z * id), roundf(v.w * id)};
            uint32_t packed = 0;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                float c = fminf(fmaxf(r[i], -128.0f), 127.0f);
                int q = (r[i] != r[i]) ? 0 : (int)c;
                packed |= ((uint32_t)(q & 0xff)) << (8 * i);
            }
            *(uint32_t*)(xq + b * 32 + sub * 4) = packed;
            if (sub == 0) xs[b] = it_f16_to_f32(it_f32_to_f16(d));
        }
    }
}

IT_DEV void wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
}

// Terms of `nrows` rows starting at `row0` of one matrix against the LDS activation.
// Two phases so every HBM load of the group is in flight before the first dot: a lane
// owns IPL (row, 32-element unit) items, loads them all, then computes.
template <int IPL>
struct RowRegs {
    uint4 wa[IPL], wb[IPL];
    uint32_t sc[IPL];
};

template <int FMT, int IPL>
__device__ __forceinline__ void load_items(RowRegs<IPL>& rr, const uint8_t* wq, const uint8_t* ws, int n_in, int row0,
                                           int nrows, int lane) {
    const int U = n_in >> 5;
    const int items = nrows * U;
#pragma unroll
    for (int k = 0; k < IPL; k++) {
        int it = k * 64 + lane;
        if (it < items) {
            int r = it / U, u = it - r * U;
            int64_t row = row0 + r;
            if (FMT == W_Q8_0) {
                const uint4* wp = (const uint4*)(wq + row * n_in + u * 32);
                rr.wa[k] = wp[0];
                rr.wb[k] = wp[1];
            } else {
                rr.wa[k] = *(const uint4*)(wq + row * (n_in >> 1) + u * 16);
            }
            rr.sc[k] = ((const uint16_t*)ws)[row * U + u];
        }
    }
}

template <int FMT, int IPL>
__device__ __forceinline__ void compute_items(const RowRegs<IPL>& rr, int n_in, int nrows, const int8_t* xq,
                                              const float* xs, float* terms, int tstride, int lane) {
    const int U = n_in >> 5;
    const int items = nrows * U;
#pragma unroll
    for (int k = 0; k < IPL; k++) {
        int it = k * 64 + lane;
        if (it < items) {
            int r = it / U, u = it - r * U;
            const uint4* ap = (const uint4*)(xq + u * 32);
            uint4 a0 = ap[0], a1 = ap[1];
            float dx = xs[u];
            if (FMT == W_Q8_0) {
                terms[r * tstride + u] = unit_q8_0(rr.wa[k], rr.wb[k], (uint16_t)rr.sc[k], a0, a1, dx);
            } else {
                float tA, tB;
                unit_nvfp4(rr.wa[k], rr.sc[k], a0, a1, dx, &tA, &tB);
                terms[r * tstride + 2 * u] = tA;
                terms[r * tstride + 2 * u + 1] = tB;
            }
        }
    }
}

template <int FMT, int IPL>
__device__ __forceinline__ void wave_row_terms_n(const uint8_t* wq, const uint8_t* ws, int n_in, int row0, int nrows,
                                                 const int8_t* xq, const float* xs, float* terms, int tstride,
                                                 int lane) {
    RowRegs<IPL> rr;
    load_items<FMT, IPL>(rr, wq, ws, n_in, row0, nrows, lane);
    compute_items<FMT, IPL>(rr, n_in, nrows, xq, xs, terms, tstride, lane);
}

// nrows * (n_in / 32) must not exceed 512 (the launchers size rows_per_wave for that)
template <int FMT>
__device__ void wave_row_terms(const uint8_t* wq, const uint8_t* ws, int n_in, int row0, int nrows,
                               const int8_t* xq, const float* xs, float* terms, int tstride, int lane) {
    const int items = nrows * (n_in >> 5);
    if (items <= 64) wave_row_terms_n<FMT, 1>(wq, ws, n_in, row0, nrows, xq, xs, terms, tstride, lane);
    else if (items <= 128) wave_row_terms_n<FMT, 2>(wq, ws, n_in, row0, nrows, xq, xs, terms, tstride, lane);
    else if (items <= 256) wave_row_terms_n<FMT, 4>(wq, ws, n_in, row0, nrows, xq, xs, terms, tstride, lane);
    else wave_row_terms_n<FMT, 8>(wq, ws, n_in, row0, nrows, xq, xs, terms, tstride, lane);
}

// ------------------------------------------------------------------ fused_gemv
// prologue modes: 0 = the activation as is; 1 = rms_norm(x, norm_w); 2 = per-head
// rms_norm of x (weight norm_w[head_dim]) gated by silu(gate): silu(g) * ((x*scale)*w)
// ------------------------------------------------------------------ router in one wave
// softmax over all experts, then n_used rounds of arg-max with ties to the lower id, the
// picked probabilities summed in pick order (src/ops/mod.rs:1191-1216, naive.rs:362-376).
// Called by one wave; probs (LDS, n_expert floats) holds the logits on entry.
__device__ void wave_route(float* probs, int n_expert, int n_used, int exact, int* ids, float* weights, int lane) {
    float m = -INFINITY;
    for (int e = lane; e < n_expert; e += 64) m = fmaxf(m, probs[e]);
    for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
    float part = 0.0f;
    for (int e = lane; e < n_expert; e += 64) {
        float v = it_expf(probs[e] - m);
        probs[e] = v;
        part += v;
    }
    wave_lds_sync();
    float sum;
    if (exact) {
        float acc = 0.0f;
        if (lane == 0)
            for (int e = 0; e < n_expert; e++) acc += probs[e];
        sum = __shfl(acc, 0, 64);
    } else {
        for (int o = 32; o > 0; o >>= 1) part += __shfl_xor(part, o, 64);
        sum = part;
    }
    for (int e = lane; e < n_expert; e += 64) probs[e] = probs[e] / sum;
    wave_lds_sync();
    float picked_p = 0.0f;  // lane r keeps pick r's probability
    int picked_id = -1;
    for (int r = 0; r < n_used; r++) {
        float bv = 0.0f;
        int bi = -1;
        for (int e = lane; e < n_expert; e += 64) {
            float v = probs[e];
            if (v < 0.0f) continue;  // taken (probabilities are never negative)
            if (bi < 0 || v > bv) {
                bv = v;
                bi = e;
            }
        }
        for (int o = 32; o > 0; o >>= 1) {
            float ov = __shfl_xor(bv, o, 64);
            int oi = __shfl_xor(bi, o, 64);
            bool take = oi >= 0 && (bi < 0 || ov > bv || (ov == bv && oi < bi));
            if (take) {
                bv = ov;
                bi = oi;
            }
        }
        if (lane == r) {
            picked_p = bv;
            picked_id = bi;
        }
        if (lane == 0 && bi >= 0) probs[bi] = -1.0f;
        wave_lds_sync();
    }
    // sum in pick order, serial f32
    float s = 0.0f;
    for (int r = 0; r < n_used; r++) s += __shfl(picked_p, r, 64);
    float denom = fmaxf(s, 6.103515625e-5f);
    if (lane < n_used) {
        ids[lane] = picked_id;
        weights[lane] = picked_p / denom;
    }
    wave_lds_sync();
}

constexpr int FG_THREADS = 512;

IT_DEV int mat_index(const FusedGemvP& p, int g) {
    int mi = 0;
#pragma unroll
    for (int k = 1; k < 4; k++)
        if (k < p.n_mats && g >= p.m[k].group0) mi = k;
    return mi;
}

// fold each row's terms in order and apply the matrix's epilogue
IT_DEV void finish_rows(const FusedGemvP& p, const FusedMat& m, int row0, int nrows, const float* terms, int tstride,
                        int nb, int lane) {
    if (lane >= nrows) return;
    const int T = m.fmt == W_NVFP4 ? nb * 2 : nb;
    float acc = fold_terms(terms + lane * tstride, T);
    const int j = row0 + lane;
    if (m.epi == 0) {
        m.out[j] = acc;
    } else if (m.epi == 2) {
        m.out[j] += acc;
    } else if (m.epi == 3) {
        m.out[j] = it_silu(acc);
    } else {
        // causal conv (kernel 4) + silu on channel j, state [channel][3] oldest first
        float* past = p.conv_state + (int64_t)j * 3;
        const float* w = p.conv_w + (int64_t)j * 4;
        float p0 = past[0], p1 = past[1], p2 = past[2];
        float sum = 0.0f;
        sum += p0 * w[0];
        sum += p1 * w[1];
        sum += p2 * w[2];
        sum += acc * w[3];
        m.out[j] = it_silu(sum);
        past[0] = p1;
        past[1] = p2;
        past[2] = acc;
    }
}

__global__ __launch_bounds__(FG_THREADS) void fused_gemv_k(FusedGemvP p) {
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ double red[FG_THREADS / 64 + 1];
    __shared__ float hscale[64];
    const int n_in = p.n_in, nb = n_in >> 5;
    float* xf = (float*)smem;
    float* xs = xf + n_in;
    int8_t* xq = (int8_t*)(xs + ((nb + 3) & ~3));
    float* terms_all = (float*)(xq + n_in);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

    // the first row group's weights start moving before the activation prologue runs
    constexpr int W = FG_THREADS / 64;
    const int R = p.rows_per_wave;
    const int tstride = nb * 2 + 4;
    float* terms = terms_all + (size_t)wave * R * tstride;
    const int g0 = blockIdx.x * W + wave;
    const bool has0 = g0 < p.total_groups;
    const FusedMat& m0 = p.m[has0 ? mat_index(p, g0) : 0];
    const int row00 = has0 ? (g0 - m0.group0) * R : 0;
    const int nrows0 = has0 ? min(R, m0.n_out - row00) : 0;
    RowRegs<8> rr;
    if (has0) {
        if (m0.fmt == W_NVFP4) load_items<W_NVFP4, 8>(rr, m0.q, m0.s, n_in, row00, nrows0, lane);
        else load_items<W_Q8_0, 8>(rr, m0.q, m0.s, n_in, row00, nrows0, lane);
    }

    for (int i = tid; i < n_in; i += FG_THREADS) xf[i] = p.x[i];
    __syncthreads();
    if (p.mode == 1) {
        double sum = block_sumsq<FG_THREADS>(xf, n_in, p.exact, red);
        float mean = (float)(sum / (double)n_in);
        float scale = 1.0f / sqrtf(mean + p.eps);
        for (int i = tid; i < n_in; i += FG_THREADS) xf[i] = xf[i] * scale * p.norm_w[i];
        __syncthreads();
    } else if (p.mode == 2 || p.mode == 3) {
        const int hd = p.head_dim, nh = n_in / hd;  // nh <= 64 (checked on the host)
        if (p.exact) {
            if (tid < nh) {
                double sum = 0.0;
                const float* h = xf + tid * hd;
                for (int i = 0; i < hd; i++) sum += (double)(h[i] * h[i]);
                hscale[tid] = 1.0f / sqrtf((float)(sum / (double)hd) + p.eps);
            }
        } else {
            // 4 lanes per head
            for (int h0 = 0; h0 < nh; h0 += FG_THREADS / 4) {
                int h = h0 + (tid >> 2), sub = tid & 3;
                double part = 0.0;
                if (h < nh)
                    for (int i = sub; i < hd; i += 4) part += (double)(xf[h * hd + i] * xf[h * hd + i]);
                part += __shfl_xor(part, 1, 64);
                part += __shfl_xor(part, 2, 64);
                if (h < nh && sub == 0) hscale[h] = 1.0f / sqrtf((float)(part / (double)hd) + p.eps);
            }
        }
        __syncthreads();
        for (int i = tid; i < n_in; i += FG_THREADS) {
            float core = xf[i] * hscale[i / hd] * p.norm_w[i % hd];
            xf[i] = (p.mode == 2 ? it_silu(p.gate[i]) : p.gate[i]) * core;
        }
        __syncthreads();
    }
    if (blockIdx.x == 0) {
        if (p.x_copy)
            for (int i = tid; i < n_in; i += FG_THREADS) p.x_copy[i] = xf[i];
        if (p.x_copy2)
            for (int i = tid; i < n_in; i += FG_THREADS) p.x_copy2[i] = xf[i];
    }
    lds_quantize_q8_0(xf, n_in, xs, xq);
    __syncthreads();

    if (has0) {
        if (m0.fmt == W_NVFP4) compute_items<W_NVFP4, 8>(rr, n_in, nrows0, xq, xs, terms, tstride, lane);
        else compute_items<W_Q8_0, 8>(rr, n_in, nrows0, xq, xs, terms, tstride, lane);
        wave_lds_sync();
        finish_rows(p, m0, row00, nrows0, terms, tstride, nb, lane);
        wave_lds_sync();
    }
    for (int g = g0 + gridDim.x * W; g < p.total_groups; g += gridDim.x * W) {
        const FusedMat& m = p.m[mat_index(p, g)];
        const int row0 = (g - m.group0) * R;
        const int nrows = min(R, m.n_out - row0);
        if (m.fmt == W_NVFP4) wave_row_terms<W_NVFP4>(m.q, m.s, n_in, row0, nrows, xq, xs, terms, tstride, lane);
        else wave_row_terms<W_Q8_0>(m.q, m.s, n_in, row0, nrows, xq, xs, terms, tstride, lane);
        wave_lds_sync();
        finish_rows(p, m, row0, nrows, terms, tstride, nb, lane);
        wave_lds_sync();
    }
    if (p.route_counter) {
        // The block that finishes last turns the router logits (matrix 0's output) into the
        // token's expert choice, so the next kernel starts with the ids in hand.
        __shared__ int is_last;
        __threadfence();
        __syncthreads();
        if (tid == 0) {
            unsigned prev = atomicAdd(p.route_counter, 1u);
            is_last = prev == gridDim.x - 1;
        }
        __syncthreads();
        if (is_last) {
            __threadfence();
            float* probs = xf;  // n_expert <= n_in (checked on the host)
            for (int i = tid; i < p.n_expert; i += FG_THREADS)
                probs[i] = __hip_atomic_load(p.m[0].out + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __syncthreads();
            if (wave == 0) {
                __shared__ int rids[64];
                __shared__ float rwts[64];
                wave_route(probs, p.n_expert, p.n_used, p.exact, rids, rwts, lane);
                if (lane < p.n_used) {
                    p.route_ids[lane] = rids[lane];
                    p.route_w[lane] = rwts[lane];
                }
                if (lane == 0) *p.route_counter = 0u;
            }
        }
    }
}

void fused_gemv(FusedGemvP p, hipStream_t s) {
    if (fused_gemv_fast(p, s)) return;
    constexpr int W = FG_THREADS / 64;
    int total_rows = 0;
    for (int i = 0; i < p.n_mats; i++) total_rows += p.m[i].n_out;
    const int nb = p.n_in / 32;
    // enough waves to cover HBM latency: aim for ~4096 row groups, at most 512 items per wave pass
    // fewest passes per wave over 256 blocks of W waves, then the fewest rows per pass
    int R = 1;
    {
        int best = 1 << 30;
        for (int r = 1; r <= 16 && r * nb <= 512; r *= 2) {
            int passes = ((total_rows + r - 1) / r + 256 * W - 1) / (256 * W);
            if (passes < best) {
                best = passes;
                R = r;
            }
        }
    }
    auto lds_for = [&](int r) {
        return (size_t)p.n_in * 4 + (size_t)((nb + 3) & ~3) * 4 + p.n_in + (size_t)W * r * (nb * 2 + 4) * 4;
    };
    while (R > 1 && lds_for(R) > 60 * 1024) R /= 2;
    p.rows_per_wave = R;
    int g = 0;
    for (int i = 0; i < p.n_mats; i++) {
        p.m[i].group0 = g;
        g += (p.m[i].n_out + R - 1) / R;
    }
    p.total_groups = g;
    int blocks = (g + W - 1) / W;
    // one block per CU: every block pays the activation prologue, so more blocks than CUs
    // only repeats it (measured: 256 blocks 12 us, 772 blocks 22 us for norm + 12k rows of 2048)
    if (blocks > 256) blocks = 256;
    hipLaunchKernelGGL(fused_gemv_k, dim3(blocks), dim3(FG_THREADS), lds_for(R), s, p);
}

// ------------------------------------------------------------------ gdn rows
// l2-normalised k (first half of kq) and q (second half) of key head `kh`, read from the
// conv output [q | k | v] (naive.rs:254-273).
template <int DK, int THREADS>
__device__ void load_kq_l2(const float* conv, int key_dim, int kh, float eps, int exact, float* kq, double* red) {
    const int tid = threadIdx.x;
    for (int i = tid; i < DK; i += THREADS) {
        kq[i] = conv[key_dim + kh * DK + i];
        kq[DK + i] = conv[kh * DK + i];
    }
    __syncthreads();
    for (int which = 0; which < 2; which++) {
        float* dst = kq + which * DK;
        double sum = block_sumsq<THREADS>(dst, DK, exact, red);
        float scale = 1.0f / fmaxf(sqrtf((float)sum), eps);
        __syncthreads();
        for (int i = tid; i < DK; i += THREADS) dst[i] = dst[i] * scale;
        __syncthreads();
    }
}

// Fast form for a block of 256 threads: thread t < DK holds k[t], thread DK + t holds q[t]; each
// vector's sum of squares is reduced in its own waves, two barriers in all.
// `v` is the thread's element, loaded by the caller (ahead of its other loads: loads return in order).
template <int DK>
__device__ __forceinline__ void l2_kq_fast(float v, float eps, float* kq, double* red) {
    static_assert(DK == 64 || DK == 128, "one or two waves per vector");
    constexpr int WPV = DK / 64;  // waves per vector
    const int tid = threadIdx.x, wave = tid >> 6;
    const bool live = tid < 2 * DK;
    const bool is_q = tid >= DK;
    const int i = is_q ? tid - DK : tid;
    const double part = wave_sum_f64_tail((double)(v * v));
    if ((tid & 63) == 63) red[wave] = part;
    __syncthreads();
    if (live) {
        const int w0 = is_q ? WPV : 0;
        double sum = red[w0];
        if (WPV == 2) sum += red[w0 + 1];
        const float scale = 1.0f / fmaxf(sqrtf((float)sum), eps);
        kq[(is_q ? DK : 0) + i] = v * scale;
    }
    __syncthreads();
}

IT_DEV void gdn_gates(const GdnCoreP& p, int h, float* g, float* beta) {
    float a = p.alpha[h] + p.dt_bias[h];
    float softplus = a > 20.0f ? a : it_logf(1.0f + it_expf(a));
    *g = it_expf(softplus * p.ssm_a[h]);
    *beta = 1.0f / (1.0f + it_expf(-p.beta[h]));
}
// the same on the transcendental unit, for the kernel that reorders its sums anyway
IT_DEV void gdn_gates_fast(const GdnCoreP& p, int h, float* g, float* beta) {
    float a = p.alpha[h] + p.dt_bias[h];
    float softplus = a > 20.0f ? a : fx_logf(1.0f + fx_expf(a));
    *g = fx_expf(softplus * p.ssm_a[h]);
    *beta = fx_sigmoid(p.beta[h]);
}

// Exact form: one lane owns one value row, the three sweeps run in the CPU path's order.
template <int DK>
__global__ __launch_bounds__(64) void gdn_rows_exact_k(GdnCoreP p) {
    __shared__ __align__(16) float kq[2 * DK];
    __shared__ double red[2];
    const int lane = threadIdx.x;
    const int dv = DK;
    const int bph = dv / 64;
    const int h = blockIdx.x / bph, jb = blockIdx.x % bph, kh = h % p.n_k_heads;
    const int key_dim = p.n_k_heads * DK;
    load_kq_l2<DK, 64>(p.conv, key_dim, kh, p.eps, p.exact, kq, red);
    const int j = jb * 64 + lane;
    float* S = p.state + ((int64_t)h * dv + j) * DK;
    float row[DK];
    const float4* S4 = (const float4*)S;
#pragma unroll
    for (int i = 0; i < DK / 4; i++) {
        float4 t = S4[i];
        row[4 * i] = t.x; row[4 * i + 1] = t.y; row[4 * i + 2] = t.z; row[4 * i + 3] = t.w;
    }
    float g, beta;
    gdn_gates(p, h, &g, &beta);
    float v = p.conv[2 * key_dim + h * dv + j];
    const float4* k4 = (const float4*)kq;
    const float4* q4 = (const float4*)(kq + DK);
    float pred = 0.0f;
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
        row[i] += kk.x * delta;     o += row[i] * (qq.x * p.q_scale);
        row[i + 1] += kk.y * delta; o += row[i + 1] * (qq.y * p.q_scale);
        row[i + 2] += kk.z * delta; o += row[i + 2] * (qq.z * p.q_scale);
        row[i + 3] += kk.w * delta; o += row[i + 3] * (qq.w * p.q_scale);
    }
    float4* W4 = (float4*)S;
#pragma unroll
    for (int i = 0; i < DK / 4; i++) W4[i] = make_float4(row[4 * i], row[4 * i + 1], row[4 * i + 2], row[4 * i + 3]);
    p.core[h * dv + j] = o;
}

// Fast form: LPR lanes share a row (each a contiguous DK/LPR slice, so a row is one 512-byte coalesced read), partial
// dots meet through DPP moves.  Reordered sums: 1e-3 class.  LPR = 8 gives 32 rows per block, LPR = 16 gives 16: the
// launcher takes the one that puts a block on every CU (32 value heads of 128 rows: 256 blocks with LPR = 16).
template <int DK, int LPR>
__global__ __launch_bounds__(256) void gdn_rows_fast_k(GdnCoreP p) {
    constexpr int SEG = DK / LPR;
    constexpr int ROWS = 256 / LPR;
    __shared__ __align__(16) float kq[2 * DK];
    __shared__ double red[5];
    const int tid = threadIdx.x, seg = tid % LPR;
    const int dv = DK;
    const int bph = dv / ROWS;
    const int h = blockIdx.x / bph, jb = blockIdx.x % bph, kh = h % p.n_k_heads;
    const int key_dim = p.n_k_heads * DK;
    // key / query element first, then the state rows: both are in flight while k and q are normalized
    const float kqv = tid < 2 * DK ? p.conv[(tid >= DK ? 0 : key_dim) + kh * DK + (tid >= DK ? tid - DK : tid)] : 0.0f;
    const int j = jb * ROWS + tid / LPR;
    float* S = p.state + ((int64_t)h * dv + j) * DK + seg * SEG;
    float4 st[SEG / 4];
#pragma unroll
    for (int i = 0; i < SEG / 4; i++) st[i] = ((const float4*)S)[i];
    l2_kq_fast<DK>(kqv, p.eps, kq, red);
    float row[SEG];
#pragma unroll
    for (int i = 0; i < SEG / 4; i++) {
        row[4 * i] = st[i].x; row[4 * i + 1] = st[i].y; row[4 * i + 2] = st[i].z; row[4 * i + 3] = st[i].w;
    }
    float g, beta;
    gdn_gates_fast(p, h, &g, &beta);
    float v = p.conv[2 * key_dim + h * dv + j];
    const float* kk = kq + seg * SEG;
    const float* qq = kq + DK + seg * SEG;
    float pred = 0.0f;
#pragma unroll
    for (int i = 0; i < SEG; i++) {
        row[i] *= g;
        pred += row[i] * kk[i];
    }
    pred = group_sum<LPR>(pred);
    float delta = beta * (v - pred);
    float o = 0.0f;
#pragma unroll
    for (int i = 0; i < SEG; i++) {
        row[i] += kk[i] * delta;
        o += row[i] * (qq[i] * p.q_scale);
    }
    o = group_sum<LPR>(o);
#pragma unroll
    for (int i = 0; i < SEG / 4; i++)
        ((float4*)S)[i] = make_float4(row[4 * i], row[4 * i + 1], row[4 * i + 2], row[4 * i + 3]);
    if (seg == 0) p.core[h * dv + j] = o;
}

void gdn_core(const GdnCoreP& p, int dk, hipStream_t s) {
    if (p.exact) {
        int blocks = p.n_v_heads * (dk / 64);
        if (dk == 64) hipLaunchKernelGGL(gdn_rows_exact_k<64>, dim3(blocks), dim3(64), 0, s, p);
        else if (dk == 128) hipLaunchKernelGGL(gdn_rows_exact_k<128>, dim3(blocks), dim3(64), 0, s, p);
    } else {
        // sixteen lanes a row while that still leaves at most a block per CU (256 on this chip), eight otherwise
        const bool wide = p.n_v_heads * (dk / 16) <= 256;
        const int blocks = p.n_v_heads * (dk / (wide ? 16 : 32));
        if (dk == 64 && wide) hipLaunchKernelGGL((gdn_rows_fast_k<64, 16>), dim3(blocks), dim3(256), 0, s, p);
        else if (dk == 64) hipLaunchKernelGGL((gdn_rows_fast_k<64, 8>), dim3(blocks), dim3(256), 0, s, p);
        else if (dk == 128 && wide) hipLaunchKernelGGL((gdn_rows_fast_k<128, 16>), dim3(blocks), dim3(256), 0, s, p);
        else if (dk == 128) hipLaunchKernelGGL((gdn_rows_fast_k<128, 8>), dim3(blocks), dim3(256), 0, s, p);
    }
}

// ------------------------------------------------------------------ moe_glu_fused
// grid (row blocks, n_used + 1): y < n_used is routed pick y, y == n_used the shared expert.
__global__ __launch_bounds__(256) void moe_glu_fused_k(MoeGluP p) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int n_in = p.n_in, nb = n_in >> 5;
    float* xf = (float*)smem;
    float* xs = xf + n_in;
    int8_t* xq = (int8_t*)(xs + ((nb + 3) & ~3));
    float* terms_all = (float*)(xq + n_in);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int y = blockIdx.y;
    const bool shared = y == p.n_used;
    const int fmt = shared ? p.sh_fmt : p.fmt;
    const int64_t e = shared ? 0 : p.route_ids[y];
    const uint8_t* gq = shared ? p.sh_gq : p.gq + e * p.q_stride;
    const uint8_t* gs = shared ? p.sh_gs : p.gs + e * p.s_stride;
    const uint8_t* uq = shared ? p.sh_uq : p.uq + e * p.q_stride;
    const uint8_t* us = shared ? p.sh_us : p.us + e * p.s_stride;
    const int n_out = shared ? p.sh_n_out : p.n_out;
    float* out = shared ? p.sh_out : p.out + (int64_t)y * p.n_out;

    const int R = p.rows_per_wave;
    const int tstride = nb * 2 + 4;
    float* tg = terms_all + (size_t)wave * 2 * R * tstride;
    float* tu = tg + (size_t)R * tstride;
    const int T = fmt == W_NVFP4 ? nb * 2 : nb;
    const int groups = (n_out + R - 1) / R;
    // first group's gate and up rows start moving before the activation is quantized
    const int g0 = blockIdx.x * 4 + wave;
    const bool has0 = g0 < groups;
    const int row00 = g0 * R, nrows0 = has0 ? min(R, n_out - row00) : 0;
    RowRegs<4> rg, ru;
    if (has0) {
        if (fmt == W_NVFP4) {
            load_items<W_NVFP4, 4>(rg, gq, gs, n_in, row00, nrows0, lane);
            load_items<W_NVFP4, 4>(ru, uq, us, n_in, row00, nrows0, lane);
        } else {
            load_items<W_Q8_0, 4>(rg, gq, gs, n_in, row00, nrows0, lane);
            load_items<W_Q8_0, 4>(ru, uq, us, n_in, row00, nrows0, lane);
        }
    }
    for (int i = tid; i < n_in; i += 256) xf[i] = p.x[i];
    __syncthreads();
    lds_quantize_q8_0(xf, n_in, xs, xq);
    __syncthreads();
    for (int g = g0; g < groups; g += gridDim.x * 4) {
        const int row0 = g * R, nrows = min(R, n_out - row0);
        if (g != g0) {
            if (fmt == W_NVFP4) {
                load_items<W_NVFP4, 4>(rg, gq, gs, n_in, row0, nrows, lane);
                load_items<W_NVFP4, 4>(ru, uq, us, n_in, row0, nrows, lane);
            } else {
                load_items<W_Q8_0, 4>(rg, gq, gs, n_in, row0, nrows, lane);
                load_items<W_Q8_0, 4>(ru, uq, us, n_in, row0, nrows, lane);
            }
        }
        if (fmt == W_NVFP4) {
            compute_items<W_NVFP4, 4>(rg, n_in, nrows, xq, xs, tg, tstride, lane);
            compute_items<W_NVFP4, 4>(ru, n_in, nrows, xq, xs, tu, tstride, lane);
        } else {
            compute_items<W_Q8_0, 4>(rg, n_in, nrows, xq, xs, tg, tstride, lane);
            compute_items<W_Q8_0, 4>(ru, n_in, nrows, xq, xs, tu, tstride, lane);
        }
        wave_lds_sync();
        if (lane < nrows) {
            float ag = fold_terms(tg + lane * tstride, T);
            float au = fold_terms(tu + lane * tstride, T);
            if (!shared) {
                if (p.gscale2) ag *= p.gscale2[e];
                if (p.uscale2) au *= p.uscale2[e];
            } else {   // a scale of 1 (no scale tensor) leaves the bits as they are
                au *= p.sh_uscale;
                ag *= p.sh_gscale;
            }
            out[row0 + lane] = it_silu(ag) * au;
        }
        wave_lds_sync();
    }
}

void moe_glu_fused(MoeGluP p, hipStream_t s) {
    if (moe_glu_fast(p, s)) return;
    const int nb = p.n_in / 32;
    int R = 4;
    while (R > 1 && R * nb > 256) R /= 2;
    auto lds_for = [&](int r) {
        return (size_t)p.n_in * 4 + (size_t)((nb + 3) & ~3) * 4 + p.n_in + (size_t)4 * 2 * r * (nb * 2 + 4) * 4;
    };
    while (R > 1 && lds_for(R) > 60 * 1024) R /= 2;
    p.rows_per_wave = R;
    int n_out = p.n_out > p.sh_n_out ? p.n_out : p.sh_n_out;
    int gx = (n_out + 4 * R - 1) / (4 * R);  // one row group per wave
    if (gx < 1) gx = 1;
    hipLaunchKernelGGL(moe_glu_fused_k, dim3(gx, p.n_used + 1), dim3(256), lds_for(R), s, p);
}

// ------------------------------------------------------------------ moe_down_fused
// x[j] += sum_e w_e * (down_e[j] . g_e * scale2_e) + (shared_down[j] . g_sh) * sigmoid(logit)
// (src/ops/mod.rs:1134-1171 then add_assign), experts ascending, shared last.
__global__ __launch_bounds__(256) void moe_down_fused_k(MoeDownP p) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int n_in = p.n_in, nb = n_in >> 5;       // expert down: n_in = expert_ff
    const int sh_in = p.sh_n_in, sh_nb = sh_in >> 5;
    const int NU = p.n_used;
    // LDS: per pick quantized activation, then the shared one
    float* xs = (float*)smem;                                     // NU*nb + sh_nb scales
    int8_t* xq = (int8_t*)(xs + ((NU * nb + sh_nb + 3) & ~3));    // NU*n_in + sh_in quants
    float* terms_all = (float*)(xq + ((NU * n_in + sh_in + 15) & ~15));
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    it_count_expert_reads(p.route_ids, NU, p.counts_gate, p.counts_up, p.counts_down, p.tally);
    constexpr int MAXU = 16;  // n_used <= 16 (checked on the host)
    const int R = p.rows_per_wave;  // R * (n_in / 32) <= 64: one item per lane per expert
    const int T = p.fmt == W_NVFP4 ? nb * 2 : nb;
    const int shT = p.sh_fmt == W_NVFP4 ? sh_nb * 2 : sh_nb;
    const int Tmax = (T > shT ? T : shT);
    const int tstride = Tmax + 4;
    // terms[(y * R + r) * tstride + k]
    float* terms = terms_all + (size_t)wave * (NU + 1) * R * tstride;
    const int groups = (p.n_out + R - 1) / R;
    RowRegs<1> rr[MAXU], rsh;
    auto load_all = [&](int row0, int nrows) {
#pragma unroll
        for (int y = 0; y < MAXU; y++) {
            if (y < NU) {
                const int64_t e = p.route_ids[y];
                if (p.fmt == W_NVFP4) load_items<W_NVFP4, 1>(rr[y], p.q + e * p.q_stride, p.s + e * p.s_stride, n_in, row0, nrows, lane);
                else load_items<W_Q8_0, 1>(rr[y], p.q + e * p.q_stride, p.s + e * p.s_stride, n_in, row0, nrows, lane);
            }
        }
        if (p.sh_fmt == W_NVFP4) load_items<W_NVFP4, 1>(rsh, p.sh_q, p.sh_s, sh_in, row0, nrows, lane);
        else load_items<W_Q8_0, 1>(rsh, p.sh_q, p.sh_s, sh_in, row0, nrows, lane);
    };
    const int g0 = blockIdx.x * 4 + wave;
    if (g0 < groups) load_all(g0 * R, min(R, p.n_out - g0 * R));
    const float gate = it_sigmoid(p.logit[0]);
    // stage all NU + 1 intermediates as f32 (the term region is free until the main loop)
    {
        float* all = terms_all;
        const int total = NU * n_in + sh_in;
        for (int i = tid; i < total; i += 256) all[i] = i < NU * n_in ? p.g_all[i] : p.g_shared[i - NU * n_in];
        __syncthreads();
        // one Q8_0 block per 8 lanes; picks and the shared vector are back to back and 32-aligned
        lds_quantize_q8_0(all, total, xs, xq);
        __syncthreads();
    }
    for (int g = g0; g < groups; g += gridDim.x * 4) {
        const int row0 = g * R, nrows = min(R, p.n_out - row0);
        if (g != g0) load_all(row0, nrows);
#pragma unroll
        for (int y = 0; y < MAXU; y++) {
            if (y < NU) {
                float* t = terms + (size_t)y * R * tstride;
                if (p.fmt == W_NVFP4) compute_items<W_NVFP4, 1>(rr[y], n_in, nrows, xq + y * n_in, xs + y * nb, t, tstride, lane);
                else compute_items<W_Q8_0, 1>(rr[y], n_in, nrows, xq + y * n_in, xs + y * nb, t, tstride, lane);
            }
        }
        {
            float* t = terms + (size_t)NU * R * tstride;
            if (p.sh_fmt == W_NVFP4) compute_items<W_NVFP4, 1>(rsh, sh_in, nrows, xq + NU * n_in, xs + NU * nb, t, tstride, lane);
            else compute_items<W_Q8_0, 1>(rsh, sh_in, nrows, xq + NU * n_in, xs + NU * nb, t, tstride, lane);
        }
        wave_lds_sync();
        // lane = (y, r): fold its dot, park it in slot 0 of its own term row
        float dot = 0.0f;
        const int pairs = (NU + 1) * nrows;
        if (lane < pairs) {
            const int y = lane / nrows, r = lane - y * nrows;
            dot = fold_terms(terms + ((size_t)y * R + r) * tstride, y < NU ? T : shT);
            if (y < NU && p.scale2) dot *= p.scale2[p.route_ids[y]];
            if (y == NU) dot *= p.sh_dscale;
        }
        wave_lds_sync();
        if (lane < pairs) {
            const int y = lane / nrows, r = lane - y * nrows;
            terms[((size_t)y * R + r) * tstride] = dot;
        }
        wave_lds_sync();
        if (lane < nrows) {
            float v = 0.0f;
            for (int y = 0; y < NU; y++) v += p.route_w[y] * terms[((size_t)y * R + lane) * tstride];
            v += terms[((size_t)NU * R + lane) * tstride] * gate;
            p.x[row0 + lane] += v;
        }
        wave_lds_sync();
    }
}

void moe_down_fused(MoeDownP p, hipStream_t s) {
    if (!p.exact && moe_down_fast(p, s)) return;
    const int nb = p.n_in / 32, sh_nb = p.sh_n_in / 32;
    const int T = (p.fmt == W_NVFP4 ? nb * 2 : nb), shT = (p.sh_fmt == W_NVFP4 ? sh_nb * 2 : sh_nb);
    const int Tmax = T > shT ? T : shT;
    int R = 4;
    while (R > 1 && (p.n_used + 1) * R > 64) R /= 2;
    while (R > 1 && (R * nb > 64 || R * sh_nb > 64)) R /= 2;
    auto lds_for = [&](int r) {
        size_t terms = (size_t)4 * (p.n_used + 1) * r * (Tmax + 4) * 4;
        size_t stage = (size_t)(p.n_used * p.n_in + p.sh_n_in) * 4;  // f32 staging shares the term region
        return (size_t)((p.n_used * nb + sh_nb + 3) & ~3) * 4 + (size_t)((p.n_used * p.n_in + p.sh_n_in + 15) & ~15) +
               (terms > stage ? terms : stage);
    };
    while (R > 1 && lds_for(R) > 60 * 1024) R /= 2;
    p.rows_per_wave = R;
    int groups = (p.n_out + R - 1) / R;
    int blocks = (groups + 3) / 4;
    if (blocks > 512) blocks = 512;
    hipLaunchKernelGGL(moe_down_fused_k, dim3(blocks), dim3(256), lds_for(R), s, p);
}

// ------------------------------------------------------------------ attention prep
// One block per head: query heads take q out of the interleaved [q | gate] projection,
// rms_norm_heads, rope; key heads the same and write f16 into the K slab at `pos`;
// value heads write f16 into the V slab.
__global__ __launch_bounds__(64) void attn_prep_k(AttnPrepP p) {
    extern __shared__ float hbuf[];
    __shared__ double red[2];
    const int hd = p.head_dim, tid = threadIdx.x;
    const int pos = *p.pos_dyn;
    int b = blockIdx.x;
    if (b >= p.n_head + p.n_head_kv) {  // value head
        const int h = b - p.n_head - p.n_head_kv;
        uint16_t* dst = p.v_slab + (int64_t)pos * p.kv_dim + h * hd;
        for (int i = tid; i < hd; i += 64) dst[i] = it_f32_to_f16(p.v[h * hd + i]);
        return;
    }
    const bool is_q = b < p.n_head;
    const int h = is_q ? b : b - p.n_head;
    const float* src = is_q ? p.qg + (int64_t)h * 2 * hd : p.k + (int64_t)h * hd;
    const float* w = is_q ? p.q_norm : p.k_norm;
    for (int i = tid; i < hd; i += 64) hbuf[i] = src[i];
    __syncthreads();
    double sum = block_sumsq<64>(hbuf, hd, p.exact, red);
    float scale = 1.0f / sqrtf((float)(sum / (double)hd) + p.eps);
    __syncthreads();
    for (int i = tid; i < hd; i += 64) hbuf[i] = hbuf[i] * scale * w[i];
    __syncthreads();
    const int half = p.n_rot / 2;
    for (int i = tid; i < half; i += 64) {
        float2 cs = p.rope[(int64_t)pos * half + i];
        float x0 = hbuf[i], x1 = hbuf[i + half];
        hbuf[i] = x0 * cs.x - x1 * cs.y;
        hbuf[i + half] = x0 * cs.y + x1 * cs.x;
    }
    __syncthreads();
    if (is_q) {
        for (int i = tid; i < hd; i += 64) p.q[h * hd + i] = hbuf[i];
    } else {
        uint16_t* dst = p.k_slab + (int64_t)pos * p.kv_dim + h * hd;
        for (int i = tid; i < hd; i += 64) dst[i] = it_f32_to_f16(hbuf[i]);
    }
}

void attn_prep(const AttnPrepP& p, hipStream_t s) {
    hipLaunchKernelGGL(attn_prep_k, dim3(p.n_head + 2 * p.n_head_kv), dim3(64), p.head_dim * sizeof(float), s, p);
}

}  // namespace itk
