// Device-side router and the routed FFN's tail.
//
// route_topk follows /root/reference src/ops/mod.rs:1191-1216: n_used rounds, each an
// ascending scan that takes a new best only on a strict '>' (ties to the lower id),
// then the picked probabilities summed in pick order and divided by
// max(sum, 6.103515625e-5).  moe_finish follows src/ops/mod.rs:1134-1171.
#include <algorithm>

#include "it_device.h"
#include "kernels.h"

namespace itk {

__global__ __launch_bounds__(256) void route_topk_k(const float* __restrict__ probs, int n_expert, int n_used,
                                                    int32_t* __restrict__ ids, float* __restrict__ weights) {
    extern __shared__ float p[];            // n_expert probabilities
    __shared__ float rv[256];
    __shared__ int ri[256];
    __shared__ int picked[64];
    const int t = blockIdx.x;
    const float* row = probs + (int64_t)t * n_expert;
    for (int e = threadIdx.x; e < n_expert; e += 256) p[e] = row[e];
    __syncthreads();
    for (int r = 0; r < n_used; r++) {
        float bv = 0.0f;
        int bi = -1;
        for (int e = threadIdx.x; e < n_expert; e += 256) {
            bool taken = false;
            for (int k = 0; k < r; k++) taken |= (picked[k] == e);
            if (taken) continue;
            if (bi < 0 || p[e] > bv) {
                bv = p[e];
                bi = e;
            }
        }
        rv[threadIdx.x] = bv;
        ri[threadIdx.x] = bi;
        __syncthreads();
        for (int off = 128; off > 0; off >>= 1) {
            if ((int)threadIdx.x < off) {
                int oi = ri[threadIdx.x + off], mi = ri[threadIdx.x];
                float ov = rv[threadIdx.x + off], mv = rv[threadIdx.x];
                bool take = oi >= 0 && (mi < 0 || ov > mv || (ov == mv && oi < mi));
                if (take) {
                    rv[threadIdx.x] = ov;
                    ri[threadIdx.x] = oi;
                }
            }
            __syncthreads();
        }
        if (threadIdx.x == 0) picked[r] = ri[0];
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        float sum = 0.0f;
        for (int r = 0; r < n_used; r++) sum += p[picked[r]];
        float denom = fmaxf(sum, 6.103515625e-5f);
        for (int r = 0; r < n_used; r++) {
            ids[(int64_t)t * n_used + r] = picked[r];
            weights[(int64_t)t * n_used + r] = p[picked[r]] / denom;
        }
    }
}

// The same rule with one wave per token (up to 1024 experts, 16 picks): a probability is non-negative, so its
// bit pattern orders like its value; a pick is compared as the 64-bit key (probability bits, ~id): the largest key
// is the largest probability and, among equals, the smallest id.  A lane holds the keys of experts lane, lane + 64,
// ...; each round takes the wave's largest key and retires it.  Same picks and weights as route_topk_k, bit for bit.
template <int K>
__global__ __launch_bounds__(256) void route_topk_wave_k(const float* __restrict__ probs, int n_tok, int n_expert, int n_used,
                                                         int32_t* __restrict__ ids, float* __restrict__ weights) {
    const int lane = threadIdx.x & 63;
    const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= n_tok) return;
    const float* row = probs + (int64_t)t * n_expert;
    unsigned long long key[K];
#pragma unroll
    for (int k = 0; k < K; k++) {
        const int e = lane + 64 * k;
        key[k] = e < n_expert ? ((unsigned long long)__float_as_uint(row[e]) << 32) | (0xffffffffu - (unsigned)e) : 0ull;
    }
    float sum = 0.0f;
    float mine = 0.0f;     // lane r keeps pick r's probability
    int mine_id = 0;
    for (int r = 0; r < n_used; r++) {
        unsigned long long m = key[0];
#pragma unroll
        for (int k = 1; k < K; k++) m = key[k] > m ? key[k] : m;
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const unsigned long long other = __shfl_xor(m, o, 64);
            m = other > m ? other : m;
        }
#pragma unroll
        for (int k = 0; k < K; k++)
            if (key[k] == m) key[k] = 0ull;
        const float pv = __uint_as_float((unsigned)(m >> 32));
        sum += pv;                         // pick order, as the CPU path adds them
        if (lane == r) {
            mine = pv;
            mine_id = (int)(0xffffffffu - (unsigned)(m & 0xffffffffu));
        }
    }
    const float denom = fmaxf(sum, 6.103515625e-5f);
    if (lane < n_used) {
        ids[(int64_t)t * n_used + lane] = mine_id;
        weights[(int64_t)t * n_used + lane] = mine / denom;
    }
}

// A block counts its slice of the picks in LDS and adds the bins it touched to the global counters: a few hundred
// global atomics for a prefill batch's tens of thousands of picks.  counts_b: a second tensor read with the same
// picks (the up matrices beside the gate matrices), or null.
constexpr int COUNT_BINS = 2048;
__global__ __launch_bounds__(256) void expert_count_k(const int32_t* __restrict__ ids, int n_picks, int n_expert,
                                                      uint32_t* __restrict__ counts_a, uint32_t* __restrict__ counts_b,
                                                      unsigned long long* __restrict__ tally,
                                                      const uint8_t* __restrict__ tier_a, const uint8_t* __restrict__ tier_b) {
    __shared__ unsigned bins[COUNT_BINS];
    __shared__ unsigned host_reads;
    if (threadIdx.x == 0) host_reads = 0;
    const bool local = n_expert <= COUNT_BINS;
    if (local)
        for (int e = threadIdx.x; e < n_expert; e += 256) bins[e] = 0;
    __syncthreads();
    const int per = (n_picks + gridDim.x - 1) / gridDim.x;
    const int lo = blockIdx.x * per, hi = min(n_picks, lo + per);
    for (int i = lo + threadIdx.x; i < hi; i += 256) {
        const int e = ids[i];
        if (local) {
            atomicAdd(&bins[e], 1u);
        } else {
            atomicAdd(counts_a + e, 1u);
            if (counts_b) atomicAdd(counts_b + e, 1u);
            const unsigned h = (tier_a && tier_a[e] ? 1u : 0u) + (counts_b && tier_b && tier_b[e] ? 1u : 0u);
            if (h) atomicAdd(&host_reads, h);
        }
    }
    __syncthreads();
    if (local)
        for (int e = threadIdx.x; e < n_expert; e += 256) {
            const unsigned c = bins[e];
            if (c) {
                atomicAdd(counts_a + e, c);
                if (counts_b) atomicAdd(counts_b + e, c);
                const unsigned h = (tier_a && tier_a[e] ? c : 0u) + (counts_b && tier_b && tier_b[e] ? c : 0u);
                if (h) atomicAdd(&host_reads, h);
            }
        }
    __syncthreads();
    // tally[0]: reads served from device memory, tally[1]: reads that crossed the bus to the pinned host tier
    if (threadIdx.x == 0) {
        const unsigned long long mine = (unsigned long long)max(hi - lo, 0) * (counts_b ? 2 : 1), h = host_reads;
        if (h) atomicAdd(tally + 1, h);
        if (mine > h) atomicAdd(tally, mine - h);
    }
}

// Placement-table entries of experts that changed tier (a cold expert fetched into a slot, its victim pointed at the
// sentinel): one thread per entry, ordered on the stream between the kernels that read the old and the new placement.
__global__ void expert_patch_k(const ExpertPatch* __restrict__ patches, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const ExpertPatch p = patches[i];
    *p.q_at = p.q;
    *p.s_at = p.s;
    *p.tier_at = (uint8_t)p.tier;
}

void expert_patch(const ExpertPatch* patches, int n, hipStream_t s) {
    if (n <= 0) return;
    hipLaunchKernelGGL(expert_patch_k, dim3((n + 63) / 64), dim3(64), 0, s, patches, n);
}

void expert_count(const int32_t* ids, int n_picks, int n_expert, uint32_t* counts_a, uint32_t* counts_b,
                  unsigned long long* tally, hipStream_t s, const uint8_t* tier_a, const uint8_t* tier_b) {
    if (n_picks <= 0 || !counts_a || !tally) return;
    const int blocks = std::max(1, std::min(64, (n_picks + 1023) / 1024));
    hipLaunchKernelGGL(expert_count_k, dim3(blocks), dim3(256), 0, s, ids, n_picks, n_expert, counts_a, counts_b, tally,
                       tier_a, tier_b);
}

void route_topk(const float* probs, int n_tok, int n_expert, int n_used, int32_t* ids, float* weights,
                hipStream_t s) {
    if (n_tok <= 0) return;
    if (n_used <= 16 && n_used <= n_expert && n_expert <= 1024) {
        const dim3 grid((n_tok + 3) / 4), block(256);
        if (n_expert <= 64) hipLaunchKernelGGL(route_topk_wave_k<1>, grid, block, 0, s, probs, n_tok, n_expert, n_used, ids, weights);
        else if (n_expert <= 256) hipLaunchKernelGGL(route_topk_wave_k<4>, grid, block, 0, s, probs, n_tok, n_expert, n_used, ids, weights);
        else if (n_expert <= 512) hipLaunchKernelGGL(route_topk_wave_k<8>, grid, block, 0, s, probs, n_tok, n_expert, n_used, ids, weights);
        else hipLaunchKernelGGL(route_topk_wave_k<16>, grid, block, 0, s, probs, n_tok, n_expert, n_used, ids, weights);
        return;
    }
    hipLaunchKernelGGL(route_topk_k, dim3(n_tok), dim3(256), n_expert * sizeof(float), s, probs, n_expert, n_used,
                       ids, weights);
}

__global__ void moe_finish_k(float* __restrict__ out, int64_t at, int n, const float* __restrict__ rows,
                             const float* __restrict__ weights, int n_tok, int n_used,
                             const float* __restrict__ shared, const float* __restrict__ logit,
                             int64_t logit_at) {
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (int64_t)n_tok * n) return;
    int64_t t = idx / n;
    int j = (int)(idx - t * n);
    float g = it_sigmoid(logit[logit_at + t]);
    const float* w = weights + t * n_used;
    float v = 0.0f;
    for (int e = 0; e < n_used; e++) v += w[e] * rows[(t * n_used + e) * n + j];
    v += shared[t * n + j] * g;
    out[at + t * n + j] = v;
}

// Four neighbouring outputs per lane with the picks' rows all in flight at once (NU = picks per token, 0 = any):
// the same sum per output, in pick order.
template <int NU, bool FX>
__global__ __launch_bounds__(256) void moe_finish4_k(float* __restrict__ out, int64_t at, int n4,
                                                     const float4* __restrict__ rows, const float* __restrict__ weights,
                                                     int n_tok, int n_used, const float4* __restrict__ shared,
                                                     const float* __restrict__ logit, int64_t logit_at) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (int64_t)n_tok * n4) return;
    const int64_t t = idx / n4;
    const int j = (int)(idx - t * n4);
    const int nu = NU ? NU : n_used;
    const float g = FX ? fx_sigmoid(logit[logit_at + t]) : it_sigmoid(logit[logit_at + t]);
    const float* w = weights + t * nu;
    const float4* r = rows + t * nu * n4 + j;
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if constexpr (NU > 0) {
        float4 rr[NU];
#pragma unroll
        for (int e = 0; e < NU; e++) rr[e] = r[(int64_t)e * n4];
#pragma unroll
        for (int e = 0; e < NU; e++) {
            const float we = w[e];
            v.x += we * rr[e].x; v.y += we * rr[e].y; v.z += we * rr[e].z; v.w += we * rr[e].w;
        }
    } else {
        for (int e = 0; e < nu; e++) {
            const float we = w[e];
            const float4 re = r[(int64_t)e * n4];
            v.x += we * re.x; v.y += we * re.y; v.z += we * re.z; v.w += we * re.w;
        }
    }
    const float4 sh = shared[t * n4 + j];
    v.x += sh.x * g; v.y += sh.y * g; v.z += sh.z * g; v.w += sh.w * g;
    *(float4*)(out + at + t * (int64_t)n4 * 4 + j * 4) = v;
}

void moe_finish(float* out, int64_t at, int n, const float* rows, const float* weights, int n_tok, int n_used,
                const float* shared, const float* logit, int64_t logit_at, int exact, hipStream_t s) {
    int64_t total = (int64_t)n_tok * n;
    if (total <= 0) return;
    auto al = [](const void* p) { return ((uintptr_t)p & 15) == 0; };
    if (n_tok >= 16 && n % 4 == 0 && at % 4 == 0 && al(out) && al(rows) && al(shared)) {
        const int n4 = n / 4;
        const dim3 grid((unsigned)((total / 4 + 255) / 256)), block(256);
#define IT_FIN(NU)                                                                                                      \
    do {                                                                                                                \
        if (exact) hipLaunchKernelGGL((moe_finish4_k<NU, false>), grid, block, 0, s, out, at, n4, (const float4*)rows, weights, \
                                      n_tok, n_used, (const float4*)shared, logit, logit_at);                           \
        else hipLaunchKernelGGL((moe_finish4_k<NU, true>), grid, block, 0, s, out, at, n4, (const float4*)rows, weights, \
                                n_tok, n_used, (const float4*)shared, logit, logit_at);                                 \
    } while (0)
        switch (n_used) {
            case 4: IT_FIN(4); break;
            case 8: IT_FIN(8); break;
            case 10: IT_FIN(10); break;
            default: IT_FIN(0); break;
        }
#undef IT_FIN
        return;
    }
    hipLaunchKernelGGL(moe_finish_k, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, out, at, n, rows,
                       weights, n_tok, n_used, shared, logit, logit_at);
}

}  // namespace itk
