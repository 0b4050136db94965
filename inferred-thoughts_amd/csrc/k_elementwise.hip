// Norms, RoPE, softmax, elementwise ops, KV write, conv, activation quantization.
//
// Each kernel keeps the accumulation order of the reference's scalar CPU path
// (/root/reference src/ops/naive.rs) wherever the `exact` flag is set; the fast
// variants reorder only the long f64 sums (tree instead of serial).
#include <cstring>
#include "it_device.h"
#include "kernels.h"
#include "it_reduce.h"

namespace itk {

static inline int blocks_for(int64_t n, int threads) {
    int64_t b = (n + threads - 1) / threads;
    if (b > 65535LL * 16) b = 65535LL * 16;
    if (b < 1) b = 1;
    return (int)b;
}

// naive.rs:139-152: out = x * scale * w, two f32 multiplies left to right.
template <int THREADS>
__global__ __launch_bounds__(THREADS) void rms_norm_k(const float* __restrict__ x, const float* __restrict__ w,
                                                      float eps, float* __restrict__ out, int nd, int exact) {
    extern __shared__ float lds[];
    __shared__ double red[THREADS / 64 + 1];
    const float* row = x + (int64_t)blockIdx.x * nd;
    float* o = out + (int64_t)blockIdx.x * nd;
    for (int i = threadIdx.x; i < nd; i += THREADS) lds[i] = row[i];
    __syncthreads();
    double sum = block_sumsq<THREADS>(lds, nd, exact, red);
    float mean = (float)(sum / (double)nd);
    float scale = 1.0f / sqrtf(mean + eps);
    for (int i = threadIdx.x; i < nd; i += THREADS) o[i] = lds[i] * scale * w[i];
}

// The same rows, four outputs per lane, with the Q8_0 form of every output row written beside it (naive.rs:652-675,
// the arithmetic of quantize_q8_0_k: eight neighbouring lanes hold one 32-element block).  What the next op, a
// product with quantized weights, would otherwise compute in a launch of its own; values and quants are bit for bit
// those of the two separate kernels.  nd a multiple of 32.
template <int THREADS>
__global__ __launch_bounds__(THREADS) void rms_norm_q8_k(const float* __restrict__ x, const float* __restrict__ w,
                                                         float eps, float* __restrict__ out, int nd, int exact,
                                                         float* __restrict__ q_scales, int8_t* __restrict__ q_quants) {
    extern __shared__ float lds[];
    __shared__ double red[THREADS / 64 + 1];
    const float* row = x + (int64_t)blockIdx.x * nd;
    float* o = out + (int64_t)blockIdx.x * nd;
    for (int i = threadIdx.x; i < nd / 4; i += THREADS) ((float4*)lds)[i] = ((const float4*)row)[i];
    __syncthreads();
    double sum = block_sumsq<THREADS>(lds, nd, exact, red);
    float mean = (float)(sum / (double)nd);
    float scale = 1.0f / sqrtf(mean + eps);
    const int64_t blk0 = (int64_t)blockIdx.x * (nd / 32);
    for (int i0 = 0; i0 < nd / 4; i0 += THREADS) {      // uniform trip count: the lane moves below need every lane
        const int i = i0 + threadIdx.x;
        const bool live = i < nd / 4;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (live) {
            const float4 a = ((const float4*)lds)[i], ww = ((const float4*)w)[i];
            v = make_float4(a.x * scale * ww.x, a.y * scale * ww.y, a.z * scale * ww.z, a.w * scale * ww.w);
            ((float4*)o)[i] = v;
        }
        float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
        amax = fmaxf(amax, __shfl_xor(amax, 1, 64));
        amax = fmaxf(amax, __shfl_xor(amax, 2, 64));
        amax = fmaxf(amax, __shfl_xor(amax, 4, 64));
        if (!live) continue;
        const float d = amax / 127.0f;
        const float id = d != 0.0f ? 1.0f / d : 0.0f;
        const float r[4] = {roundf(v.x * id), roundf(v.y * id), roundf(v.z * id), roundf(v.w * id)};
        uint32_t packed = 0;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const float c = fminf(fmaxf(r[k], -128.0f), 127.0f);
            const int q = (r[k] != r[k]) ? 0 : (int)c;
            packed |= ((uint32_t)(q & 0xff)) << (8 * k);
        }
        *(uint32_t*)(q_quants + (int64_t)blockIdx.x * nd + (int64_t)i * 4) = packed;
        if ((i & 7) == 0) q_scales[blk0 + (i >> 3)] = it_f16_to_f32(it_f32_to_f16(d));
    }
}

bool rms_norm_writes_q8(const float* x, const float* w, const float* out, int nd) {
    auto al = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
    return nd % 32 == 0 && al(x) && al(w) && al(out);
}

void rms_norm(const float* x, const float* w, float eps, float* out, int64_t n_rows, int nd, int exact,
              hipStream_t s, float* q_scales, int8_t* q_quants) {
    if (n_rows <= 0) return;
    if (q_scales && q_quants && rms_norm_writes_q8(x, w, out, nd)) {
        hipLaunchKernelGGL(rms_norm_q8_k<256>, dim3((unsigned)n_rows), dim3(256), nd * sizeof(float), s, x, w, eps, out, nd,
                           exact, q_scales, q_quants);
        return;
    }
    hipLaunchKernelGGL(rms_norm_k<256>, dim3((unsigned)n_rows), dim3(256), nd * sizeof(float), s, x, w, eps, out,
                       nd, exact);
}

// naive.rs:154-164 (mode 0) and naive.rs:254-273 (mode 1: l2, eps clamps the norm).
__global__ __launch_bounds__(64) void head_norm_k(float* __restrict__ x, const float* __restrict__ w, int hd,
                                                  float eps, int mode, int exact) {
    extern __shared__ float lds[];
    __shared__ double red[2];
    float* head = x + (int64_t)blockIdx.x * hd;
    for (int i = threadIdx.x; i < hd; i += 64) lds[i] = head[i];
    __syncthreads();
    double sum = block_sumsq<64>(lds, hd, exact, red);
    float scale;
    if (mode == 0) {
        float mean = (float)(sum / (double)hd);
        scale = 1.0f / sqrtf(mean + eps);
        for (int i = threadIdx.x; i < hd; i += 64) head[i] = lds[i] * scale * w[i];
    } else {
        float nrm = sqrtf((float)sum);
        scale = 1.0f / fmaxf(nrm, eps);
        for (int i = threadIdx.x; i < hd; i += 64) head[i] = lds[i] * scale;
    }
}

// The same for many heads when the order of the sum is free: a wave per head, PER neighbouring elements per
// lane held in registers, the f64 partial sums added across the wave by lane moves (no LDS, no barrier).
template <int PER>
__global__ __launch_bounds__(256) void head_norm_wave_k(float* __restrict__ x, const float* __restrict__ w,
                                                        int64_t n_heads, float eps, int mode) {
    constexpr int HD = 64 * PER;
    const int lane = threadIdx.x & 63;
    const int64_t h = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (h >= n_heads) return;
    float* at = x + h * HD + lane * PER;
    float v[PER];
    if constexpr (PER == 4) {
        const float4 t = *(const float4*)at;
        v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
    } else if constexpr (PER == 2) {
        const float2 t = *(const float2*)at;
        v[0] = t.x; v[1] = t.y;
    } else {
        v[0] = at[0];
    }
    double part = 0.0;
#pragma unroll
    for (int e = 0; e < PER; e++) part += (double)(v[e] * v[e]);
    const double sum = __shfl(wave_sum_f64_tail(part), 63, 64);
    float o[PER];
    if (mode == 0) {
        const float mean = (float)(sum / (double)HD);
        const float scale = 1.0f / sqrtf(mean + eps);
#pragma unroll
        for (int e = 0; e < PER; e++) o[e] = v[e] * scale * w[lane * PER + e];
    } else {
        const float nrm = sqrtf((float)sum);
        const float scale = 1.0f / fmaxf(nrm, eps);
#pragma unroll
        for (int e = 0; e < PER; e++) o[e] = v[e] * scale;
    }
    if constexpr (PER == 4) *(float4*)at = make_float4(o[0], o[1], o[2], o[3]);
    else if constexpr (PER == 2) *(float2*)at = make_float2(o[0], o[1]);
    else at[0] = o[0];
}

static bool head_norm_wave(float* x, const float* w, int head_dim, float eps, int64_t n_heads, int mode, hipStream_t s) {
    if (n_heads < 256 || ((uintptr_t)x & 15) != 0) return false;
    const dim3 grid((unsigned)((n_heads + 3) / 4)), block(256);
    switch (head_dim) {
        case 64: hipLaunchKernelGGL(head_norm_wave_k<1>, grid, block, 0, s, x, w, n_heads, eps, mode); return true;
        case 128: hipLaunchKernelGGL(head_norm_wave_k<2>, grid, block, 0, s, x, w, n_heads, eps, mode); return true;
        case 256: hipLaunchKernelGGL(head_norm_wave_k<4>, grid, block, 0, s, x, w, n_heads, eps, mode); return true;
        default: return false;
    }
}

void rms_norm_heads(float* x, const float* w, int head_dim, float eps, int64_t n_heads, int exact,
                    hipStream_t s) {
    if (n_heads <= 0) return;
    if (!exact && head_norm_wave(x, w, head_dim, eps, n_heads, 0, s)) return;
    hipLaunchKernelGGL(head_norm_k, dim3((unsigned)n_heads), dim3(64), head_dim * sizeof(float), s, x, w,
                       head_dim, eps, 0, exact);
}
void l2_norm_heads(float* x, int head_dim, float eps, int64_t n_heads, int exact, hipStream_t s) {
    if (n_heads <= 0) return;
    if (!exact && head_norm_wave(x, nullptr, head_dim, eps, n_heads, 1, s)) return;
    hipLaunchKernelGGL(head_norm_k, dim3((unsigned)n_heads), dim3(64), head_dim * sizeof(float), s, x,
                       (const float*)nullptr, head_dim, eps, 1, exact);
}

// naive.rs:180-218.  The (cos, sin) table is built on the host in f64 and narrowed,
// exactly as the reference builds it; entry [pos][i] = (cos, sin)(pos * theta^(-2i/n_rot)).
__global__ void rope_k(float* __restrict__ x, const float2* __restrict__ table, int half, int64_t total,
                       int pos, const int* __restrict__ pos_dyn, int head_dim, int n_heads) {
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    int p0 = pos_dyn ? *pos_dyn : pos;
    int i = (int)(idx % half);
    int64_t th = idx / half;  // token * n_heads + head
    int64_t t = th / n_heads;
    float2 cs = table[(int64_t)(p0 + t) * half + i];
    float* head = x + th * head_dim;
    float x0 = head[i], x1 = head[i + half];
    head[i] = x0 * cs.x - x1 * cs.y;
    head[i + half] = x0 * cs.y + x1 * cs.x;
}

void rope_neox(float* x, const float2* table, int table_half, int64_t n_tok, int pos, const int* pos_dyn,
               int head_dim, int n_rot, int n_heads, hipStream_t s) {
    int half = n_rot / 2;
    int64_t total = n_tok * n_heads * half;
    if (total <= 0) return;
    (void)table_half;
    hipLaunchKernelGGL(rope_k, dim3(blocks_for(total, 256)), dim3(256), 0, s, x, table, half, total, pos,
                       pos_dyn, head_dim, n_heads);
}

// naive.rs:362-376: max, exp(v - max) with a serial sum, divide.
template <int THREADS>
__global__ __launch_bounds__(THREADS) void softmax_k(float* __restrict__ x, int row, int exact) {
    extern __shared__ float lds[];
    __shared__ float red[THREADS / 64 + 1];
    float* r = x + (int64_t)blockIdx.x * row;
    float m = -INFINITY;
    for (int i = threadIdx.x; i < row; i += THREADS) {
        float v = r[i];
        lds[i] = v;
        m = fmaxf(m, v);
    }
    for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_down(m, off, 64));
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) {
        float mm = red[0];
        for (int w = 1; w < THREADS / 64; w++) mm = fmaxf(mm, red[w]);
        red[THREADS / 64] = mm;
    }
    __syncthreads();
    m = red[THREADS / 64];
    float part = 0.0f;
    for (int i = threadIdx.x; i < row; i += THREADS) {
        float e = it_expf(lds[i] - m);
        lds[i] = e;
        part += e;
    }
    __syncthreads();
    float sum;
    if (exact) {
        if (threadIdx.x == 0) {
            float acc = 0.0f;
            for (int i = 0; i < row; i++) acc += lds[i];
            red[0] = acc;
        }
        __syncthreads();
        sum = red[0];
    } else {
        for (int off = 32; off > 0; off >>= 1) part += __shfl_down(part, off, 64);
        if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = part;
        __syncthreads();
        if (threadIdx.x == 0) {
            float acc = 0.0f;
            for (int w = 0; w < THREADS / 64; w++) acc += red[w];
            red[0] = acc;
        }
        __syncthreads();
        sum = red[0];
    }
    for (int i = threadIdx.x; i < row; i += THREADS) r[i] = lds[i] / sum;
}

void softmax_rows(float* x, int64_t n_rows, int row, int exact, hipStream_t s) {
    if (n_rows <= 0 || row <= 0) return;
    hipLaunchKernelGGL(softmax_k<256>, dim3((unsigned)n_rows), dim3(256), row * sizeof(float), s, x, row, exact);
}

// ------------------------------------------------------------------ elementwise
__global__ void silu_mul_k(float* __restrict__ g, const float* __restrict__ u, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
        float v = g[i];
        g[i] = it_silu(v) * u[i];
    }
}
__global__ void sigmoid_mul_k(float* __restrict__ x, const float* __restrict__ g, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        x[i] *= it_sigmoid(g[i]);
}
__global__ void add_assign_k(float* __restrict__ a, const float* __restrict__ b, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        a[i] += b[i];
}
__global__ void scale_k(float* __restrict__ a, float v, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        a[i] *= v;
}
__global__ void add_scaled_k(float* __restrict__ a, const float* __restrict__ b, float v, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        a[i] += b[i] * v;
}
__global__ void add_scaled_sigmoid_k(float* __restrict__ a, const float* __restrict__ b,
                                     const float* __restrict__ logit, int64_t n) {
    float sg = it_sigmoid(logit[0]);
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        a[i] += b[i] * sg;
}
__global__ void add_scaled_rows_k(float* __restrict__ acc, int64_t n, const float* __restrict__ rows,
                                  const float* __restrict__ scales, int n_scales) {
    for (int64_t j = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; j < n; j += (int64_t)gridDim.x * blockDim.x) {
        float v = 0.0f;
        for (int e = 0; e < n_scales; e++) v += scales[e] * rows[(int64_t)e * n + j];
        acc[j] = v;
    }
}
__global__ void gather_chunks_k(const float* __restrict__ src, int64_t chunk, int64_t stride, int64_t offset,
                                float* __restrict__ out, int64_t out_len) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < out_len;
         i += (int64_t)gridDim.x * blockDim.x) {
        int64_t c = i / chunk, j = i % chunk;
        out[i] = src[c * stride + offset + j];
    }
}
__global__ void scatter_chunks_k(const float* __restrict__ src, int64_t src_len, int64_t chunk, int64_t stride,
                                 int64_t offset, float* __restrict__ dst) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < src_len;
         i += (int64_t)gridDim.x * blockDim.x) {
        int64_t c = i / chunk, j = i % chunk;
        dst[offset + c * stride + j] = src[i];
    }
}
// ops/mod.rs:1421-1425: f32 -> f16 round to nearest even.
__global__ void kv_write_k(uint16_t* __restrict__ slab, int64_t offset, const int* __restrict__ offset_dyn,
                           int64_t offset_mul, const float* __restrict__ src, int64_t n) {
    int64_t off = offset_dyn ? (int64_t)(*offset_dyn) * offset_mul : offset;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        slab[off + i] = it_f32_to_f16(src[i]);
}
// a few host values into device memory with the launch itself: they travel in the argument block, so the stream sees
// one small kernel where a host-to-device copy would put a transfer (and its wait) between two passes
struct PokeInts {
    int v[POKE_MAX];
};
__global__ void poke_ints_k(int* __restrict__ dst, PokeInts v, int n) {
    if ((int)threadIdx.x < n) dst[threadIdx.x] = v.v[threadIdx.x];
}
__global__ void fill_zero_k(uint32_t* p, int64_t n_words) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_words;
         i += (int64_t)gridDim.x * blockDim.x)
        p[i] = 0u;
}

// Four elements per lane for the long batches: the same arithmetic per element, 16-byte accesses.
// FX: the exponential on the transcendental unit (fast mode) instead of the CPU path's libm form
template <bool FX> IT_DEV float silu_of(float v) { return FX ? fx_silu(v) : it_silu(v); }
template <bool FX> IT_DEV float sigmoid_of(float v) { return FX ? fx_sigmoid(v) : it_sigmoid(v); }
template <bool FX>
__global__ void silu_mul4_k(float4* __restrict__ g, const float4* __restrict__ u, int64_t n4) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += (int64_t)gridDim.x * blockDim.x) {
        float4 a = g[i];
        const float4 b = u[i];
        a.x = silu_of<FX>(a.x) * b.x; a.y = silu_of<FX>(a.y) * b.y; a.z = silu_of<FX>(a.z) * b.z; a.w = silu_of<FX>(a.w) * b.w;
        g[i] = a;
    }
}
template <bool FX>
__global__ void sigmoid_mul4_k(float4* __restrict__ x, const float4* __restrict__ g, int64_t n4) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += (int64_t)gridDim.x * blockDim.x) {
        float4 a = x[i];
        const float4 b = g[i];
        a.x *= sigmoid_of<FX>(b.x); a.y *= sigmoid_of<FX>(b.y); a.z *= sigmoid_of<FX>(b.z); a.w *= sigmoid_of<FX>(b.w);
        x[i] = a;
    }
}
__global__ void add_assign4_k(float4* __restrict__ a, const float4* __restrict__ b, int64_t n4) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += (int64_t)gridDim.x * blockDim.x) {
        float4 v = a[i];
        const float4 w = b[i];
        v.x += w.x; v.y += w.y; v.z += w.z; v.w += w.w;
        a[i] = v;
    }
}
// chunk, stride and offset in units of four floats, every index below 2^31
__global__ void gather_chunks4_k(const float4* __restrict__ src, uint32_t chunk4, uint32_t stride4, uint32_t offset4,
                                 float4* __restrict__ out, uint32_t out_len4) {
    for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < out_len4; i += gridDim.x * blockDim.x) {
        const uint32_t c = i / chunk4, j = i - c * chunk4;
        out[i] = src[c * stride4 + offset4 + j];
    }
}
static inline bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }
constexpr int64_t VEC_MIN = 1 << 14;  // below this one pass of scalar lanes is as quick

#define EW_LAUNCH(kern, n, ...)                                                              \
    do {                                                                                     \
        if ((n) > 0) hipLaunchKernelGGL(kern, dim3(blocks_for((n), 256)), dim3(256), 0, s, __VA_ARGS__); \
    } while (0)

void silu_mul(float* gate, const float* up, int64_t n, int exact, hipStream_t s) {
    if (n >= VEC_MIN && n % 4 == 0 && aligned16(gate) && aligned16(up)) {
        if (exact) EW_LAUNCH(silu_mul4_k<false>, n / 4, (float4*)gate, (const float4*)up, n / 4);
        else EW_LAUNCH(silu_mul4_k<true>, n / 4, (float4*)gate, (const float4*)up, n / 4);
    } else
        EW_LAUNCH(silu_mul_k, n, gate, up, n);
}
void sigmoid_mul(float* x, const float* g, int64_t n, int exact, hipStream_t s) {
    if (n >= VEC_MIN && n % 4 == 0 && aligned16(x) && aligned16(g)) {
        if (exact) EW_LAUNCH(sigmoid_mul4_k<false>, n / 4, (float4*)x, (const float4*)g, n / 4);
        else EW_LAUNCH(sigmoid_mul4_k<true>, n / 4, (float4*)x, (const float4*)g, n / 4);
    } else
        EW_LAUNCH(sigmoid_mul_k, n, x, g, n);
}
void add_assign(float* a, const float* b, int64_t n, hipStream_t s) {
    if (n >= VEC_MIN && n % 4 == 0 && aligned16(a) && aligned16(b))
        EW_LAUNCH(add_assign4_k, n / 4, (float4*)a, (const float4*)b, n / 4);
    else
        EW_LAUNCH(add_assign_k, n, a, b, n);
}
void scale(float* a, float v, int64_t n, hipStream_t s) { EW_LAUNCH(scale_k, n, a, v, n); }
void add_scaled(float* a, const float* b, float v, int64_t n, hipStream_t s) {
    EW_LAUNCH(add_scaled_k, n, a, b, v, n);
}
void add_scaled_rows(float* acc, int64_t n, const float* rows, const float* scales, int n_scales,
                     hipStream_t s) {
    EW_LAUNCH(add_scaled_rows_k, n, acc, n, rows, scales, n_scales);
}
void add_scaled_sigmoid(float* acc, const float* b, int64_t n, const float* logit, hipStream_t s) {
    EW_LAUNCH(add_scaled_sigmoid_k, n, acc, b, logit, n);
}
void gather_chunks(const float* src, int64_t chunk, int64_t stride, int64_t offset, float* out,
                   int64_t out_len, hipStream_t s) {
    const int64_t n_chunks = chunk > 0 ? (out_len + chunk - 1) / chunk : 0;
    if (out_len >= VEC_MIN && chunk % 4 == 0 && stride % 4 == 0 && offset % 4 == 0 && out_len % 4 == 0 && offset >= 0 &&
        aligned16(src) && aligned16(out) && (n_chunks * stride + offset) / 4 < (1ll << 31) && out_len / 4 < (1ll << 31)) {
        EW_LAUNCH(gather_chunks4_k, out_len / 4, (const float4*)src, (uint32_t)(chunk / 4), (uint32_t)(stride / 4),
                  (uint32_t)(offset / 4), (float4*)out, (uint32_t)(out_len / 4));
        return;
    }
    EW_LAUNCH(gather_chunks_k, out_len, src, chunk, stride, offset, out, out_len);
}
void scatter_chunks(const float* src, int64_t src_len, int64_t chunk, int64_t stride, int64_t offset,
                    float* dst, hipStream_t s) {
    EW_LAUNCH(scatter_chunks_k, src_len, src, src_len, chunk, stride, offset, dst);
}
void kv_write(uint16_t* slab, int64_t offset, const int* offset_dyn, int64_t offset_mul, const float* src,
              int64_t n, hipStream_t s) {
    EW_LAUNCH(kv_write_k, n, slab, offset, offset_dyn, offset_mul, src, n);
}
bool poke_ints(int* dst, const int* host_values, int n, hipStream_t s) {
    if (n < 1 || n > POKE_MAX) return false;
    PokeInts v;
    std::memcpy(v.v, host_values, (size_t)n * sizeof(int));
    hipLaunchKernelGGL(poke_ints_k, dim3(1), dim3(POKE_MAX), 0, s, dst, v, n);
    return true;
}
void fill_zero(void* p, int64_t bytes, hipStream_t s) {
    int64_t words = bytes / 4;
    EW_LAUNCH(fill_zero_k, words, (uint32_t*)p, words);
}

// ------------------------------------------------------------------ Q8_0 activations
// naive.rs:652-675: per 32: amax, d = amax/127, id = d ? 1/d : 0, q = round-half-away(x*id)
// saturated to i8, scale stored through f16.  Eight lanes share a block.
__global__ void quantize_q8_0_k(const float* __restrict__ x, float* __restrict__ scales,
                                int8_t* __restrict__ quants, int64_t n_blocks) {
    int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t b = gid >> 3;
    int sub = (int)(gid & 7);
    bool live = b < n_blocks;
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (live) v = *(const float4*)(x + b * 32 + sub * 4);
    float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    amax = fmaxf(amax, __shfl_xor(amax, 1, 64));
    amax = fmaxf(amax, __shfl_xor(amax, 2, 64));
    amax = fmaxf(amax, __shfl_xor(amax, 4, 64));
    if (!live) return;
    float d = amax / 127.0f;
    float id = d != 0.0f ? 1.0f / d : 0.0f;
    float r[4] = {roundf(v.x * id), roundf(v.y * id), roundf(v.z * id), roundf(v.w * id)};
    uint32_t packed = 0;
    for (int i = 0; i < 4; i++) {
        float c = fminf(fmaxf(r[i], -128.0f), 127.0f);
        int q = (r[i] != r[i]) ? 0 : (int)c;
        packed |= ((uint32_t)(q & 0xff)) << (8 * i);
    }
    *(uint32_t*)(quants + b * 32 + sub * 4) = packed;
    if (sub == 0) scales[b] = it_f16_to_f32(it_f32_to_f16(d));
}

void quantize_q8_0(const float* x, float* scales, int8_t* quants, int64_t n, hipStream_t s) {
    int64_t n_blocks = n / 32;
    if (n_blocks <= 0) return;
    int64_t threads = n_blocks * 8;
    hipLaunchKernelGGL(quantize_q8_0_k, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, s, x, scales,
                       quants, n_blocks);
}

// ------------------------------------------------------------------ causal conv + silu
// naive.rs:275-315.  One thread per channel and token chunk, the window in registers;
// state is [channel][kernel-1], oldest first.
// Tokens are independent given their window, so the batch is cut into chunks of CONV_TOK tokens
// (grid.y): a thread rebuilds its window from the inputs before its chunk, or from the state for
// the first tokens of the batch.  Only chunk 0 reads the old state, and it is the one that
// writes the new one (the last KEEP inputs), so no block reads what another writes.
constexpr int CONV_TOK = 16;
template <int KEEP>
__global__ void ssm_conv_k(float* __restrict__ state, const float* __restrict__ x, const float* __restrict__ w,
                           int nc, int n_tok, float* __restrict__ out) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= nc) return;
    const int t0 = blockIdx.y * CONV_TOK, t1 = min(n_tok, t0 + CONV_TOK);
    float past[KEEP], wt[KEEP + 1], old[KEEP];
    for (int k = 0; k < KEEP; k++) {
        const int idx = t0 - KEEP + k;
        old[k] = blockIdx.y == 0 ? state[(int64_t)c * KEEP + k] : 0.0f;
        past[k] = idx >= 0 ? x[(int64_t)idx * nc + c] : old[KEEP + idx];
    }
    for (int k = 0; k <= KEEP; k++) wt[k] = w[(int64_t)c * (KEEP + 1) + k];
    for (int t = t0; t < t1; t++) {
        float xv = x[(int64_t)t * nc + c];
        float sum = 0.0f;
        for (int k = 0; k < KEEP; k++) sum += past[k] * wt[k];
        sum += xv * wt[KEEP];
        out[(int64_t)t * nc + c] = it_silu(sum);
        for (int k = 0; k + 1 < KEEP; k++) past[k] = past[k + 1];
        past[KEEP - 1] = xv;
    }
    if (blockIdx.y == 0) {
        for (int k = 0; k < KEEP; k++) {
            const int idx = n_tok - KEEP + k;
            state[(int64_t)c * KEEP + k] = idx >= 0 ? x[(int64_t)idx * nc + c] : old[KEEP + idx];
        }
    }
}

// The same for four neighbouring channels per lane: 16-byte accesses, the chunk's inputs all in flight at once.
template <int KEEP, bool FX>
__global__ __launch_bounds__(128) void ssm_conv4_k(float* __restrict__ state, const float* __restrict__ x,
                                                   const float* __restrict__ w, int nc, int n_tok,
                                                   float* __restrict__ out) {
    const int c = (blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (c >= nc) return;
    const int t0 = blockIdx.y * CONV_TOK, t1 = min(n_tok, t0 + CONV_TOK);
    float past[KEEP][4], wt[KEEP + 1][4];
#pragma unroll
    for (int k = 0; k < KEEP; k++) {
        if (blockIdx.y == 0) {
#pragma unroll
            for (int e = 0; e < 4; e++) past[k][e] = state[(int64_t)(c + e) * KEEP + k];
        } else {
            const float4 v = *(const float4*)(x + (int64_t)(t0 - KEEP + k) * nc + c);
            past[k][0] = v.x; past[k][1] = v.y; past[k][2] = v.z; past[k][3] = v.w;
        }
    }
#pragma unroll
    for (int k = 0; k <= KEEP; k++)
#pragma unroll
        for (int e = 0; e < 4; e++) wt[k][e] = w[(int64_t)(c + e) * (KEEP + 1) + k];
    float4 xin[CONV_TOK];
#pragma unroll
    for (int i = 0; i < CONV_TOK; i++)
        xin[i] = t0 + i < t1 ? *(const float4*)(x + (int64_t)(t0 + i) * nc + c) : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int i = 0; i < CONV_TOK; i++) {
        if (t0 + i >= t1) break;
        const float xv[4] = {xin[i].x, xin[i].y, xin[i].z, xin[i].w};
        float o[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            float sum = 0.0f;
#pragma unroll
            for (int k = 0; k < KEEP; k++) sum += past[k][e] * wt[k][e];
            sum += xv[e] * wt[KEEP][e];
            o[e] = silu_of<FX>(sum);
#pragma unroll
            for (int k = 0; k + 1 < KEEP; k++) past[k][e] = past[k + 1][e];
            past[KEEP - 1][e] = xv[e];
        }
        *(float4*)(out + (int64_t)(t0 + i) * nc + c) = make_float4(o[0], o[1], o[2], o[3]);
    }
    // the batch is longer than the window (the launcher sees to it): the new state is its last KEEP inputs
    if (blockIdx.y == 0) {
#pragma unroll
        for (int k = 0; k < KEEP; k++)
#pragma unroll
            for (int e = 0; e < 4; e++) state[(int64_t)(c + e) * KEEP + k] = x[(int64_t)(n_tok - KEEP + k) * nc + c + e];
    }
}

// The Gated DeltaNet's input path over a batch in one pass over the data (fast mode): the causal conv + silu of
// ssm_conv4_k over the q | k | v channels, each part written straight to its own buffer (the three gather_chunks that
// follow the conv, qwen35.rs:1262-1270) and the q and k heads l2-normalised on the way (head_norm_wave_k's arithmetic:
// f64 sum of the squares, 1 / max(norm, eps)).  A head is 128 channels: the 32 neighbouring lanes of four channels.
template <int KEEP>
__global__ __launch_bounds__(128) void conv_split_l2_k(float* __restrict__ state, const float* __restrict__ x,
                                                       const float* __restrict__ w, int nc, int n_tok,
                                                       float* __restrict__ q_out, float* __restrict__ k_out,
                                                       float* __restrict__ v_out, int kdim, float eps) {
    const int c = (blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (c >= nc) return;
    const int t0 = blockIdx.y * CONV_TOK, t1 = min(n_tok, t0 + CONV_TOK);
    const int vdim = nc - 2 * kdim;
    float past[KEEP][4], wt[KEEP + 1][4];
#pragma unroll
    for (int k = 0; k < KEEP; k++) {
        if (blockIdx.y == 0) {
#pragma unroll
            for (int e = 0; e < 4; e++) past[k][e] = state[(int64_t)(c + e) * KEEP + k];
        } else {
            const float4 v = *(const float4*)(x + (int64_t)(t0 - KEEP + k) * nc + c);
            past[k][0] = v.x; past[k][1] = v.y; past[k][2] = v.z; past[k][3] = v.w;
        }
    }
#pragma unroll
    for (int k = 0; k <= KEEP; k++)
#pragma unroll
        for (int e = 0; e < 4; e++) wt[k][e] = w[(int64_t)(c + e) * (KEEP + 1) + k];
    float4 xin[CONV_TOK];
#pragma unroll
    for (int i = 0; i < CONV_TOK; i++)
        xin[i] = t0 + i < t1 ? *(const float4*)(x + (int64_t)(t0 + i) * nc + c) : make_float4(0.f, 0.f, 0.f, 0.f);
    const bool normed = c < 2 * kdim;   // the same for the 32 lanes of a head
    float* const dst = c < kdim ? q_out + c : (normed ? k_out + (c - kdim) : v_out + (c - 2 * kdim));
    const int dstride = normed ? kdim : vdim;
#pragma unroll
    for (int i = 0; i < CONV_TOK; i++) {
        if (t0 + i >= t1) break;
        const float xv[4] = {xin[i].x, xin[i].y, xin[i].z, xin[i].w};
        float o[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            float sum = 0.0f;
#pragma unroll
            for (int k = 0; k < KEEP; k++) sum += past[k][e] * wt[k][e];
            sum += xv[e] * wt[KEEP][e];
            o[e] = silu_of<true>(sum);
#pragma unroll
            for (int k = 0; k + 1 < KEEP; k++) past[k][e] = past[k + 1][e];
            past[KEEP - 1][e] = xv[e];
        }
        if (normed) {
            double part = 0.0;
#pragma unroll
            for (int e = 0; e < 4; e++) part += (double)(o[e] * o[e]);
#pragma unroll
            for (int m = 1; m < 32; m <<= 1) part += __shfl_xor(part, m, 64);
            const float nrm = sqrtf((float)part);
            const float scale = 1.0f / fmaxf(nrm, eps);
#pragma unroll
            for (int e = 0; e < 4; e++) o[e] = o[e] * scale;
        }
        *(float4*)(dst + (int64_t)(t0 + i) * dstride) = make_float4(o[0], o[1], o[2], o[3]);
    }
    if (blockIdx.y == 0) {
#pragma unroll
        for (int k = 0; k < KEEP; k++)
#pragma unroll
            for (int e = 0; e < 4; e++) state[(int64_t)(c + e) * KEEP + k] = x[(int64_t)(n_tok - KEEP + k) * nc + c + e];
    }
}

bool conv_split_l2(float* state, const float* x, const float* w, int kernel, int nc, int n_tok, float* q_out, float* k_out,
                   float* v_out, int kdim, float eps, hipStream_t s) {
    if (n_tok < 64 || nc % 128 || kdim <= 0 || kdim % 128 || 2 * kdim >= nc || kernel < 2 || kernel > 5) return false;
    if (!aligned16(x) || !aligned16(q_out) || !aligned16(k_out) || !aligned16(v_out)) return false;
    dim3 grid((nc / 4 + 127) / 128, (n_tok + CONV_TOK - 1) / CONV_TOK), block(128);
    switch (kernel) {
        case 2: hipLaunchKernelGGL(conv_split_l2_k<1>, grid, block, 0, s, state, x, w, nc, n_tok, q_out, k_out, v_out, kdim, eps); break;
        case 3: hipLaunchKernelGGL(conv_split_l2_k<2>, grid, block, 0, s, state, x, w, nc, n_tok, q_out, k_out, v_out, kdim, eps); break;
        case 4: hipLaunchKernelGGL(conv_split_l2_k<3>, grid, block, 0, s, state, x, w, nc, n_tok, q_out, k_out, v_out, kdim, eps); break;
        default: hipLaunchKernelGGL(conv_split_l2_k<4>, grid, block, 0, s, state, x, w, nc, n_tok, q_out, k_out, v_out, kdim, eps); break;
    }
    return true;
}

// The Gated DeltaNet's output path over a batch in one pass (fast mode): the per-head rms norm of the delta rule's
// output (head_norm_wave_k<2>), z = silu(z) * normed (silu_mul4_k) and the Q8_0 form of z for the out-projection
// (quantize_q8_0_k), each with the arithmetic of the kernel it replaces.  A wave per head of 128, two elements a lane;
// a Q8_0 block is 16 neighbouring lanes.
__global__ __launch_bounds__(256) void gated_norm_silu_q8_k(const float* __restrict__ core, const float* __restrict__ w,
                                                            float* __restrict__ z, float* __restrict__ scales,
                                                            int8_t* __restrict__ quants, int64_t n_heads, float eps) {
    const int lane = threadIdx.x & 63;
    const int64_t h = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (h >= n_heads) return;
    const int64_t at = h * 128 + lane * 2;
    const float2 v = *(const float2*)(core + at);
    double part = 0.0;
    part += (double)(v.x * v.x);
    part += (double)(v.y * v.y);
    const double sum = __shfl(wave_sum_f64_tail(part), 63, 64);
    const float mean = (float)(sum / 128.0);
    const float scale = 1.0f / sqrtf(mean + eps);
    const float n0 = v.x * scale * w[lane * 2], n1 = v.y * scale * w[lane * 2 + 1];
    const float2 g = *(const float2*)(z + at);
    const float o0 = silu_of<true>(g.x) * n0, o1 = silu_of<true>(g.y) * n1;
    *(float2*)(z + at) = make_float2(o0, o1);
    float amax = fmaxf(fabsf(o0), fabsf(o1));
#pragma unroll
    for (int m = 1; m < 16; m <<= 1) amax = fmaxf(amax, __shfl_xor(amax, m, 64));
    const float d = amax / 127.0f;
    const float id = d != 0.0f ? 1.0f / d : 0.0f;
    const float r[2] = {roundf(o0 * id), roundf(o1 * id)};
    uint32_t packed = 0;
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const float cl = fminf(fmaxf(r[i], -128.0f), 127.0f);
        const int q = (r[i] != r[i]) ? 0 : (int)cl;
        packed |= ((uint32_t)(q & 0xff)) << (8 * i);
    }
    *(uint16_t*)(quants + at) = (uint16_t)packed;
    if ((lane & 15) == 0) scales[at >> 5] = it_f16_to_f32(it_f32_to_f16(d));
}

bool gated_norm_silu_q8(const float* core, const float* w, float* z, float* scales, int8_t* quants, int64_t n_heads, float eps,
                        hipStream_t s) {
    if (n_heads < 256 || ((uintptr_t)core & 7) || ((uintptr_t)z & 7) || ((uintptr_t)quants & 1)) return false;
    hipLaunchKernelGGL(gated_norm_silu_q8_k, dim3((unsigned)((n_heads + 3) / 4)), dim3(256), 0, s, core, w, z, scales, quants, n_heads, eps);
    return true;
}

void ssm_conv(float* state, const float* x, const float* w, int kernel, int nc, int n_tok, float* out, int exact,
              hipStream_t s) {
    if (nc <= 0 || n_tok <= 0) return;
    if (n_tok >= 64 && nc % 4 == 0 && aligned16(x) && aligned16(out) && kernel >= 2 && kernel <= 5) {
        dim3 grid((nc / 4 + 127) / 128, (n_tok + CONV_TOK - 1) / CONV_TOK), block(128);
#define IT_CONV4(KEEP)                                                                                        \
    do {                                                                                                      \
        if (exact) hipLaunchKernelGGL((ssm_conv4_k<KEEP, false>), grid, block, 0, s, state, x, w, nc, n_tok, out); \
        else hipLaunchKernelGGL((ssm_conv4_k<KEEP, true>), grid, block, 0, s, state, x, w, nc, n_tok, out);   \
    } while (0)
        switch (kernel) {
            case 2: IT_CONV4(1); break;
            case 3: IT_CONV4(2); break;
            case 4: IT_CONV4(3); break;
            default: IT_CONV4(4); break;
        }
#undef IT_CONV4
        return;
    }
    dim3 grid((nc + 127) / 128, (n_tok + CONV_TOK - 1) / CONV_TOK), block(128);
    switch (kernel) {
        case 2: hipLaunchKernelGGL(ssm_conv_k<1>, grid, block, 0, s, state, x, w, nc, n_tok, out); break;
        case 3: hipLaunchKernelGGL(ssm_conv_k<2>, grid, block, 0, s, state, x, w, nc, n_tok, out); break;
        case 4: hipLaunchKernelGGL(ssm_conv_k<3>, grid, block, 0, s, state, x, w, nc, n_tok, out); break;
        case 5: hipLaunchKernelGGL(ssm_conv_k<4>, grid, block, 0, s, state, x, w, nc, n_tok, out); break;
        default: break;  // the caller validates `kernel`
    }
}

// ------------------------------------------------------------------ argmax
// First strict maximum (ties to the lower index), /root/reference src/profile.rs:192-213.
__global__ __launch_bounds__(256) void argmax_part_k(const float* __restrict__ x, int64_t n,
                                                     int32_t* __restrict__ pidx, float* __restrict__ pval) {
    __shared__ float sv[256];
    __shared__ int si[256];
    int64_t per = (n + gridDim.x - 1) / gridDim.x;
    int64_t lo = per * blockIdx.x, hi = lo + per < n ? lo + per : n;
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int64_t i = lo + threadIdx.x; i < hi; i += 256) {
        float v = x[i];
        if (v > bv || bi == 0x7fffffff) {
            // strided scan visits ascending indices per thread, so strict > keeps the lowest
            if (bi == 0x7fffffff || v > bv) {
                bv = v;
                bi = (int)i;
            }
        }
    }
    sv[threadIdx.x] = bv;
    si[threadIdx.x] = bi;
    __syncthreads();
    for (int off = 128; off > 0; off >>= 1) {
        if ((int)threadIdx.x < off) {
            float ov = sv[threadIdx.x + off];
            int oi = si[threadIdx.x + off];
            float mv = sv[threadIdx.x];
            int mi = si[threadIdx.x];
            bool take = (oi != 0x7fffffff) && (mi == 0x7fffffff || ov > mv || (ov == mv && oi < mi));
            if (take) {
                sv[threadIdx.x] = ov;
                si[threadIdx.x] = oi;
            }
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        pidx[blockIdx.x] = si[0];
        pval[blockIdx.x] = sv[0];
    }
}
// the first strict maximum among the partial results, found by one wave: every lane ends with the winner
IT_DEV int argmax_of_parts(const int32_t* __restrict__ pidx, const float* __restrict__ pval, int n_part, int lane) {
    float bv = 0.f;
    int bi = 0x7fffffff;
    for (int p = lane; p < n_part; p += 64) {
        const int oi = pidx[p];
        const float ov = pval[p];
        if (oi != 0x7fffffff && (bi == 0x7fffffff || ov > bv || (ov == bv && oi < bi))) {
            bv = ov;
            bi = oi;
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, 64);
        const int oi = __shfl_xor(bi, off, 64);
        if (oi != 0x7fffffff && (bi == 0x7fffffff || ov > bv || (ov == bv && oi < bi))) {
            bv = ov;
            bi = oi;
        }
    }
    return bi == 0x7fffffff ? 0 : bi;
}
__global__ __launch_bounds__(64) void argmax_final_k(const int32_t* __restrict__ pidx, const float* __restrict__ pval, int n_part,
                                                     int32_t* __restrict__ out) {
    const int bi = argmax_of_parts(pidx, pval, n_part, threadIdx.x);
    if (threadIdx.x == 0) out[0] = bi;
}

void argmax(const float* x, int64_t n, int32_t* out, int32_t* scratch_idx, float* scratch_val, hipStream_t s) {
    int parts = 64;
    hipLaunchKernelGGL(argmax_part_k, dim3(parts), dim3(256), 0, s, x, n, scratch_idx, scratch_val);
    hipLaunchKernelGGL(argmax_final_k, dim3(1), dim3(64), 0, s, scratch_idx, scratch_val, parts, out);
}

// ------------------------------------------------------------------ embedding row by device token id
// x[i] = row `*token` of the table, dequantized exactly as the host does (Q8_0: f16 scale
// times the int8 quant; F16/BF16 widened; F32 copied), and the id is filed in `ring`.
__global__ __launch_bounds__(256) void embed_row_k(WView w, const int32_t* __restrict__ token, float* __restrict__ x,
                                                   int32_t* __restrict__ ring, int ring_idx,
                                                   const int* __restrict__ ring_dyn) {
    const int64_t tok = *token;
    if (blockIdx.x == 0 && threadIdx.x == 0 && ring) ring[ring_dyn ? *ring_dyn : ring_idx] = (int32_t)tok;
    const int n_in = w.n_in;
    for (int i = blockIdx.x * 256 + threadIdx.x; i < n_in; i += gridDim.x * 256) {
        float v;
        if (w.fmt == W_Q8_0) {
            const int8_t q = ((const int8_t*)w.q)[tok * n_in + i];
            const uint16_t d = ((const uint16_t*)w.scales)[tok * (n_in >> 5) + (i >> 5)];
            v = it_f16_to_f32(d) * (float)q;
        } else if (w.fmt == W_F16) {
            v = it_f16_to_f32(((const uint16_t*)w.q)[tok * n_in + i]);
        } else if (w.fmt == W_BF16) {
            v = it_bf16_to_f32(((const uint16_t*)w.q)[tok * n_in + i]);
        } else {
            v = ((const float*)w.q)[tok * n_in + i];
        }
        x[i] = v;
    }
}

// The last step of the arg-max and the embedding of its result in one launch: every block's first wave picks the
// winner among the partial results (the same in every block), block 0 files it, and the blocks share the row.
__global__ __launch_bounds__(256) void argmax_embed_k(const int32_t* __restrict__ pidx, const float* __restrict__ pval, int n_part,
                                                      int32_t* __restrict__ out, WView w, float* __restrict__ x,
                                                      int32_t* __restrict__ ring, int ring_idx, const int* __restrict__ ring_dyn) {
    __shared__ int winner;
    if (threadIdx.x < 64) {
        const int bi = argmax_of_parts(pidx, pval, n_part, threadIdx.x);
        if (threadIdx.x == 0) {
            winner = bi;
            if (blockIdx.x == 0) {
                out[0] = bi;
                if (ring) ring[ring_dyn ? *ring_dyn : ring_idx] = bi;
            }
        }
    }
    __syncthreads();
    const int64_t tok = winner;
    const int n_in = w.n_in;
    for (int i = blockIdx.x * 256 + threadIdx.x; i < n_in; i += gridDim.x * 256) {
        float v;
        if (w.fmt == W_Q8_0) {
            const int8_t q = ((const int8_t*)w.q)[tok * n_in + i];
            const uint16_t d = ((const uint16_t*)w.scales)[tok * (n_in >> 5) + (i >> 5)];
            v = it_f16_to_f32(d) * (float)q;
        } else if (w.fmt == W_F16) {
            v = it_f16_to_f32(((const uint16_t*)w.q)[tok * n_in + i]);
        } else if (w.fmt == W_BF16) {
            v = it_bf16_to_f32(((const uint16_t*)w.q)[tok * n_in + i]);
        } else {
            v = ((const float*)w.q)[tok * n_in + i];
        }
        x[i] = v;
    }
}

void argmax_embed(const float* logits, int64_t n, int32_t* out, int32_t* scratch_idx, float* scratch_val, const WView& w,
                  float* x, int32_t* ring, int ring_idx, const int* ring_dyn, hipStream_t s) {
    const int parts = 64;
    hipLaunchKernelGGL(argmax_part_k, dim3(parts), dim3(256), 0, s, logits, n, scratch_idx, scratch_val);
    int blocks = (w.n_in + 255) / 256;
    if (blocks > 64) blocks = 64;
    hipLaunchKernelGGL(argmax_embed_k, dim3(blocks), dim3(256), 0, s, scratch_idx, scratch_val, parts, out, w, x, ring, ring_idx,
                       ring_dyn);
}

void embed_row(const WView& w, const int32_t* token, float* x, int32_t* ring, int ring_idx, const int* ring_dyn,
               hipStream_t s) {
    int blocks = (w.n_in + 255) / 256;
    if (blocks > 64) blocks = 64;
    hipLaunchKernelGGL(embed_row_k, dim3(blocks), dim3(256), 0, s, w, token, x, ring, ring_idx, ring_dyn);
}

}  // namespace itk
