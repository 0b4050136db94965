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
#include "it_reduce.h"
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
// One block per (query, kv head, 64-position tile).  The K and V tiles are staged into LDS
// with coalesced 16-byte loads (every thread has its 2 * HD / 32 loads in flight at once),
// scores are computed with lane = position (wave w takes query heads w, w+4, ...), the
// tile's softmax statistics come from wave reductions, and the weighted values with
// lane = output dimensions (wave w takes positions 16w..16w+15; the four partial sums meet
// in LDS).  Partial layout as above: [hd acc][m][l] per (t, head, split).
constexpr int TILE = 64;

// Per-head rms_norm (weight w) and NeoX rotation at `pos` of one head's HD values, four per lane
// (lane li of the head's HD / 4 lanes holds dims 4 li .. 4 li + 3): what rms_norm_heads + rope_neox do
// for a single token (naive.rs:180-218, 633-650), with the sum of squares reduced across the lanes.
template <int HD>
IT_DEV float4 head_norm_rope(float4 v, const float* __restrict__ w, float eps, const float2* __restrict__ rope,
                             int n_rot, int pos, int li) {
    constexpr int LPH = HD / 4;
    double part = (double)(v.x * v.x);
    part += (double)(v.y * v.y);
    part += (double)(v.z * v.z);
    part += (double)(v.w * v.w);
    part += dpp_f64(part, 0);
    part += dpp_f64(part, 1);
    part += dpp_f64(part, 2);
    part += dpp_f64(part, 3);
    if (LPH >= 32) part += __shfl_xor(part, 16, 64);
    if (LPH >= 64) part += __shfl_xor(part, 32, 64);
    const float scale = 1.0f / sqrtf((float)(part / (double)HD) + eps);
    const float4 ww = ((const float4*)w)[li];
    v.x = v.x * scale * ww.x;
    v.y = v.y * scale * ww.y;
    v.z = v.z * scale * ww.z;
    v.w = v.w * scale * ww.w;
    const int half = n_rot >> 1, hl = half >> 2;  // lanes per rotated half (a power of two)
    float4 o;
    o.x = __shfl_xor(v.x, hl, 64);
    o.y = __shfl_xor(v.y, hl, 64);
    o.z = __shfl_xor(v.z, hl, 64);
    o.w = __shfl_xor(v.w, hl, 64);
    if (li < 2 * hl) {
        const float4* cs = (const float4*)(rope + (int64_t)pos * half + 4 * (li & (hl - 1)));
        const float4 c01 = cs[0], c23 = cs[1];  // (cos, sin) of dims i, i+1 and i+2, i+3
        if (li < hl) {  // x0 = mine, x1 = partner
            v = make_float4(v.x * c01.x - o.x * c01.y, v.y * c01.z - o.y * c01.w, v.z * c23.x - o.z * c23.y,
                            v.w * c23.z - o.w * c23.w);
        } else {        // x0 = partner, x1 = mine
            v = make_float4(o.x * c01.y + v.x * c01.x, o.y * c01.w + v.y * c01.z, o.z * c23.y + v.z * c23.x,
                            o.w * c23.w + v.w * c23.z);
        }
    }
    return v;
}

template <int HD, int G, bool PREP>
__global__ __launch_bounds__(256) void attend_tile_k(AttnArgs a, TilePrepP pr, int n_split, float* __restrict__ part) {
    constexpr int CPR = HD / 8;            // 16-byte chunks per K or V row
    constexpr int KSTR = HD * 2 + 16;      // K row stride in LDS: padded so lanes reading rows do not collide
    constexpr int DPL = HD / 64;           // output dimensions per lane
    constexpr int NLD = TILE * CPR / 256;  // 16-byte loads per thread per tile
    __shared__ __align__(16) unsigned char tiles[TILE * KSTR + TILE * HD * 2];
    unsigned char* ktile = tiles;
    unsigned char* vtile = tiles + TILE * KSTR;
    __shared__ __align__(16) float qs[G * HD];
    __shared__ __align__(16) float sc[TILE * G];
    __shared__ float mrow[G], lrow[G];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n_pos_last = a.n_pos_dyn ? *a.n_pos_dyn : a.n_pos;
    const int t = blockIdx.x / a.n_head_kv, h_kv = blockIdx.x % a.n_head_kv;
    const int split = blockIdx.y;
    const int n_pos = n_pos_last - a.n_q + 1 + t;
    const int s0 = split * TILE;
    const int len = min(TILE, n_pos - s0);
    const int off = h_kv * HD;
    const int h0 = h_kv * G;
    float* my_part = part + (((int64_t)t * a.n_head + h0) * n_split + split) * (HD + 2);
    const int64_t part_head_stride = (int64_t)n_split * (HD + 2);
    if (len <= 0) {
        if (tid < G) {
            float* p = my_part + tid * part_head_stride;
            p[HD] = -INFINITY;
            p[HD + 1] = 0.0f;
        }
        return;
    }
    // With PREP the block forms its query heads itself, and the block whose tile holds the new position
    // forms that position's key and value rows: they go to the slabs and straight into the tile.
    const int new_row = PREP ? (n_pos - 1) - s0 : -1;  // in [0, len) only in the last live tile
    // stage K and V (rows past the context are zero)
    {
        uint4 kr[NLD], vr[NLD];
#pragma unroll
        for (int i = 0; i < NLD; i++) {
            const int idx = tid + i * 256, pos = idx / CPR, c = idx % CPR;
            if (pos < len && pos != new_row) {
                const int64_t g = (int64_t)(s0 + pos) * a.kv_dim + off + c * 8;
                kr[i] = *(const uint4*)(a.k + g);
                vr[i] = *(const uint4*)(a.v + g);
            } else {
                kr[i] = make_uint4(0, 0, 0, 0);
                vr[i] = make_uint4(0, 0, 0, 0);
            }
        }
        if (!PREP) {
            for (int i = tid; i < G * HD / 4; i += 256)
                ((float4*)qs)[i] = ((const float4*)(a.q + ((int64_t)t * a.n_head + h0) * HD))[i];
        } else {
            constexpr int LPH = HD / 4, HPP = 64 / LPH;  // lanes per head, heads per wave pass
            const int li = lane % LPH, pos_now = n_pos - 1;
            for (int g0 = wave * HPP; g0 < G; g0 += 4 * HPP) {
                const int g = g0 + lane / LPH;  // G is a multiple of HPP or smaller than it
                if (g < G) {
                    float4 v = ((const float4*)(pr.qg + (int64_t)(h0 + g) * 2 * HD))[li];
                    v = head_norm_rope<HD>(v, pr.q_norm, pr.eps, pr.rope, pr.n_rot, pos_now, li);
                    ((float4*)(qs + g * HD))[li] = v;
                }
            }
            if (new_row >= 0 && new_row < len) {
                if (wave == 0 && lane < LPH) {
                    float4 v = ((const float4*)(pr.kproj + (int64_t)h_kv * HD))[li];
                    v = head_norm_rope<HD>(v, pr.k_norm, pr.eps, pr.rope, pr.n_rot, pos_now, li);
                    uint2 hv;
                    hv.x = (uint32_t)it_f32_to_f16(v.x) | ((uint32_t)it_f32_to_f16(v.y) << 16);
                    hv.y = (uint32_t)it_f32_to_f16(v.z) | ((uint32_t)it_f32_to_f16(v.w) << 16);
                    *(uint2*)(pr.k_slab + (int64_t)pos_now * a.kv_dim + off + 4 * li) = hv;
                    *(uint2*)(ktile + new_row * KSTR + 8 * li) = hv;
                } else if (wave == 1 && lane < LPH) {
                    const float4 v = ((const float4*)(pr.vproj + (int64_t)h_kv * HD))[li];
                    uint2 hv;
                    hv.x = (uint32_t)it_f32_to_f16(v.x) | ((uint32_t)it_f32_to_f16(v.y) << 16);
                    hv.y = (uint32_t)it_f32_to_f16(v.z) | ((uint32_t)it_f32_to_f16(v.w) << 16);
                    *(uint2*)(pr.v_slab + (int64_t)pos_now * a.kv_dim + off + 4 * li) = hv;
                    *(uint2*)(vtile + new_row * HD * 2 + 8 * li) = hv;
                }
            }
        }
#pragma unroll
        for (int i = 0; i < NLD; i++) {
            const int idx = tid + i * 256, pos = idx / CPR, c = idx % CPR;
            if (pos != new_row) {
                *(uint4*)(ktile + pos * KSTR + c * 16) = kr[i];
                *(uint4*)(vtile + pos * HD * 2 + c * 16) = vr[i];
            }
        }
    }
    __syncthreads();
    // scores and the tile's softmax statistics: lane = position
    for (int g = wave; g < G; g += 4) {
        const unsigned char* krow = ktile + lane * KSTR;
        const float* q = qs + g * HD;
        float acc = 0.0f;
#pragma unroll 4
        for (int i = 0; i < HD; i += 8) {
            const uint4 kk = *(const uint4*)(krow + i * 2);
            const float4 q0 = *(const float4*)(q + i), q1 = *(const float4*)(q + i + 4);
            acc += q0.x * it_f16_to_f32((uint16_t)(kk.x & 0xffff)) + q0.y * it_f16_to_f32((uint16_t)(kk.x >> 16)) +
                   q0.z * it_f16_to_f32((uint16_t)(kk.y & 0xffff)) + q0.w * it_f16_to_f32((uint16_t)(kk.y >> 16)) +
                   q1.x * it_f16_to_f32((uint16_t)(kk.z & 0xffff)) + q1.y * it_f16_to_f32((uint16_t)(kk.z >> 16)) +
                   q1.z * it_f16_to_f32((uint16_t)(kk.w & 0xffff)) + q1.w * it_f16_to_f32((uint16_t)(kk.w >> 16));
        }
        const float sco = lane < len ? acc * a.scale : -INFINITY;
        const float m = group_max<64>(sco);
        const float p = lane < len ? __expf(sco - m) : 0.0f;
        const float l = group_sum_tail<64>(p);
        sc[lane * G + g] = p;
        if (lane == 63) {
            mrow[g] = m;
            lrow[g] = l;
        }
    }
    __syncthreads();
    // weighted values: lane = DPL output dimensions, this wave's quarter of the positions
    float acc[G][DPL];
#pragma unroll
    for (int g = 0; g < G; g++)
#pragma unroll
        for (int d = 0; d < DPL; d++) acc[g][d] = 0.0f;
#pragma unroll 4
    for (int s = wave * (TILE / 4); s < (wave + 1) * (TILE / 4); s++) {
        float v[DPL];
        const unsigned char* vrow = vtile + s * HD * 2 + lane * DPL * 2;
        if (DPL == 4) {
            const uint2 r = *(const uint2*)vrow;
            v[0] = it_f16_to_f32((uint16_t)(r.x & 0xffff));
            v[1 % DPL] = it_f16_to_f32((uint16_t)(r.x >> 16));
            v[2 % DPL] = it_f16_to_f32((uint16_t)(r.y & 0xffff));
            v[3 % DPL] = it_f16_to_f32((uint16_t)(r.y >> 16));
        } else if (DPL == 2) {
            const uint32_t r = *(const uint32_t*)vrow;
            v[0] = it_f16_to_f32((uint16_t)(r & 0xffff));
            v[1 % DPL] = it_f16_to_f32((uint16_t)(r >> 16));
        } else {
            v[0] = it_f16_to_f32(*(const uint16_t*)vrow);
        }
        float p[G];
#pragma unroll
        for (int g = 0; g < G; g++) p[g] = sc[s * G + g];
#pragma unroll
        for (int g = 0; g < G; g++)
#pragma unroll
            for (int d = 0; d < DPL; d++) acc[g][d] += p[g] * v[d];
    }
    __syncthreads();  // the tiles are dead: their space takes the four waves' partial sums
    static_assert(4 * G * HD * 4 <= TILE * KSTR + TILE * HD * 2, "partial sums must fit in the tile space");
    float* red = (float*)tiles;  // [4][G][HD]
#pragma unroll
    for (int g = 0; g < G; g++)
#pragma unroll
        for (int d = 0; d < DPL; d++) red[(wave * G + g) * HD + lane * DPL + d] = acc[g][d];
    __syncthreads();
    for (int i = tid; i < G * HD; i += 256) {
        float sum = 0.0f;
#pragma unroll
        for (int w = 0; w < 4; w++) sum += red[w * G * HD + i];
        my_part[(i / HD) * part_head_stride + (i % HD)] = sum;
    }
    if (tid < G) {
        float* p = my_part + tid * part_head_stride;
        p[HD] = mrow[tid];
        p[HD + 1] = lrow[tid];
    }
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
        if (gate) r *= it_sigmoid(gate[(int64_t)blockIdx.x * gate_stride + i]);
        out[(int64_t)blockIdx.x * hd + i] = r;
    }
}

void attend_split(const AttnArgs& a, int n_split, float* scratch, float* out, hipStream_t s) {
    if (attend_prefill(a, out, s)) return;
    attend_split_gated(a, n_split, scratch, out, nullptr, 0, s);
}

// queries at or below this count take the tile kernel (chunk TILE); larger batches the
// position-per-thread kernel (chunk CHUNK)
constexpr int TILE_MAX_Q = 16;
static bool tile_path(int n_q, int head_dim, int G) {
    return n_q <= TILE_MAX_Q && (head_dim == 64 || head_dim == 128 || head_dim == 256) && G <= 8;
}

int attend_split_count(int n_pos_max, int n_q, int head_dim, int group) {
    const int chunk = tile_path(n_q, head_dim, group) ? TILE : CHUNK;
    return (n_pos_max + chunk - 1) / chunk;
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

static void attend_split_impl(const AttnArgs& a, const TilePrepP* prep, int n_split, float* scratch, float* out,
                              const float* gate, int gate_stride, hipStream_t s);

void attend_split_gated(const AttnArgs& a, int n_split, float* scratch, float* out, const float* gate,
                        int gate_stride, hipStream_t s) {
    attend_split_impl(a, nullptr, n_split, scratch, out, gate, gate_stride, s);
}

void attend_split_gated_prep(const AttnArgs& a, const TilePrepP& pr, int n_split, float* scratch, float* out,
                             const float* gate, int gate_stride, hipStream_t s) {
    attend_split_impl(a, &pr, n_split, scratch, out, gate, gate_stride, s);
}

static void attend_split_impl(const AttnArgs& a, const TilePrepP* prep, int n_split, float* scratch, float* out,
                              const float* gate, int gate_stride, hipStream_t s) {
    if (a.n_q <= 0) return;
    const int G = a.n_head / a.n_head_kv;
    dim3 grid(a.n_q * a.n_head_kv, n_split), block(256);
    const bool tile = tile_path(a.n_q, a.head_dim, G);
    if (tile) {
#define IT_TILE(HD, GG)                                                                                      \
    do {                                                                                                     \
        if (prep) hipLaunchKernelGGL((attend_tile_k<HD, GG, true>), grid, block, 0, s, a, *prep, n_split, scratch); \
        else hipLaunchKernelGGL((attend_tile_k<HD, GG, false>), grid, block, 0, s, a, TilePrepP{}, n_split, scratch); \
    } while (0)
#define IT_TILE_G(HD)                  \
    switch (G) {                       \
        case 1: IT_TILE(HD, 1); break; \
        case 2: IT_TILE(HD, 2); break; \
        case 4: IT_TILE(HD, 4); break; \
        case 8: IT_TILE(HD, 8); break; \
        default: return;               \
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
            default: return;  // the caller falls back to the exact kernel for other group sizes
        }
    }
    hipLaunchKernelGGL(attend_merge_k, dim3(a.n_q * a.n_head), dim3(4 * a.head_dim),
                       (size_t)(n_split + 4 * a.head_dim) * sizeof(float), s, scratch, n_split, a.head_dim, out, gate,
                       gate_stride, a.n_q, a.n_head, tile ? TILE : CHUNK, a.n_pos, a.n_pos_dyn);
}

}  // namespace itk
