// GQA attention over the f16 KV slabs.
//
// attend_exact keeps the reference CPU path's order (/root/reference
// src/ops/naive.rs:420-466): score = (serial dot) * scale; softmax with a serial
// sum; the weighted V sum walks positions outermost.  Bit-identical to the CPU.
//
// attend_split is split-K flash decoding for long contexts: each block owns one
// kv head (all of its query heads share the K/V stream) and one 128-position
// chunk, keeps an online-softmax partial (acc, m, l), and a second kernel merges
// the partials.  Reordered sums: compared against the exact path at 1e-3.
#include "it_device.h"
#include "kernels.h"

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

int attend_split_count(int n_pos_max) { return (n_pos_max + CHUNK - 1) / CHUNK; }

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

// gate (optional): out *= sigmoid(gate[head * gate_stride + i]) — the attention block's output gate
__global__ void attend_merge_k(const float* __restrict__ part, int n_split, int hd, float* __restrict__ out,
                               const float* __restrict__ gate, int gate_stride) {
    const float* p = part + (int64_t)blockIdx.x * n_split * (hd + 2);
    float m = -INFINITY;
    for (int s = 0; s < n_split; s++) m = fmaxf(m, p[(int64_t)s * (hd + 2) + hd]);
    float l = 0.0f;
    for (int s = 0; s < n_split; s++) {
        float ms = p[(int64_t)s * (hd + 2) + hd];
        if (ms != -INFINITY) l += p[(int64_t)s * (hd + 2) + hd + 1] * __expf(ms - m);
    }
    for (int i = threadIdx.x; i < hd; i += blockDim.x) {
        float acc = 0.0f;
        for (int s = 0; s < n_split; s++) {
            float ms = p[(int64_t)s * (hd + 2) + hd];
            if (ms != -INFINITY) acc += p[(int64_t)s * (hd + 2) + i] * __expf(ms - m);
        }
        float r = acc / l;
        if (gate) r *= it_sigmoid(gate[(int64_t)blockIdx.x * gate_stride + i]);
        out[(int64_t)blockIdx.x * hd + i] = r;
    }
}

void attend_split(const AttnArgs& a, int n_split, float* scratch, float* out, hipStream_t s) {
    attend_split_gated(a, n_split, scratch, out, nullptr, 0, s);
}

void attend_split_gated(const AttnArgs& a, int n_split, float* scratch, float* out, const float* gate,
                        int gate_stride, hipStream_t s) {
    if (a.n_q <= 0) return;
    const int G = a.n_head / a.n_head_kv;
    dim3 grid(a.n_q * a.n_head_kv, n_split), block(256);
    size_t lds = ((size_t)G * a.head_dim + (size_t)CHUNK * G) * sizeof(float);
    switch (G) {
        case 1: hipLaunchKernelGGL(attend_split_k<1>, grid, block, lds, s, a, n_split, scratch); break;
        case 2: hipLaunchKernelGGL(attend_split_k<2>, grid, block, lds, s, a, n_split, scratch); break;
        case 4: hipLaunchKernelGGL(attend_split_k<4>, grid, block, lds, s, a, n_split, scratch); break;
        case 8: hipLaunchKernelGGL(attend_split_k<8>, grid, block, lds, s, a, n_split, scratch); break;
        default: return;  // the caller falls back to the exact kernel for other group sizes
    }
    hipLaunchKernelGGL(attend_merge_k, dim3(a.n_q * a.n_head), dim3(a.head_dim < 256 ? 64 : 256), 0, s, scratch,
                       n_split, a.head_dim, out, gate, gate_stride);
}

}  // namespace itk
