// Device pieces shared by the single-token kernels of the fast mode (k_fast.hip) and the layer chain (k_chain.hip):
// 16-byte weight chunks owned by lanes, the matching activation chunks, the per-chunk integer dots, the Q8_0
// quantization of a quad held in registers, and the block-wide router (softmax + top-k of the logits).
//
// A "chunk" is 16 bytes of a repacked weight row: 16 Q8_0 quants (half a block) or 32 NVFP4 nibbles (two
// sub-blocks).  A row of `cpr` chunks is spread over L = min(64, cpr) lanes, CPL = cpr / L chunks each.
#pragma once
#include "it_device.h"
#include "it_dot.h"
#include "it_reduce.h"
#include "kernels.h"

namespace itk {
namespace fastk {

template <int FMT, int CPL> struct XChunks {
    uint4 a[CPL], b[CPL];  // b: second half of an NVFP4 chunk's 32 activations
    float d[CPL];
};
template <int CPL> struct WChunks {
    uint4 w[CPL];
    uint32_t sc[CPL];
};

// activation chunks of lane `sub` from the quantized activation in LDS
template <int FMT, int CPL, int L>
IT_DEV void load_x(XChunks<FMT, CPL>& x, const int8_t* xq, const float* xs, int sub) {
#pragma unroll
    for (int k = 0; k < CPL; k++) {
        const int c = k * L + sub;
        if (FMT == W_Q8_0) {
            x.a[k] = *(const uint4*)(xq + c * 16);
            x.d[k] = xs[c >> 1];
        } else {
            x.a[k] = *(const uint4*)(xq + c * 32);
            x.b[k] = *(const uint4*)(xq + c * 32 + 16);
            x.d[k] = xs[c];
        }
    }
}

template <int FMT, int CPL, int L>
IT_DEV void load_w(WChunks<CPL>& t, const uint8_t* q, const uint8_t* s, int n_in, int64_t row, int sub, bool live) {
    if (!live) {
#pragma unroll
        for (int k = 0; k < CPL; k++) {
            t.w[k] = make_uint4(0, 0, 0, 0);
            t.sc[k] = 0;
        }
        return;
    }
    const uint8_t* rp = q + row * (FMT == W_Q8_0 ? n_in : n_in >> 1);
    const uint16_t* sp = (const uint16_t*)s + row * (n_in >> 5);
#pragma unroll
    for (int k = 0; k < CPL; k++) {
        const int c = k * L + sub;
        {   // read once per token: no reason to keep it in the caches
            typedef unsigned v4u __attribute__((ext_vector_type(4)));
            const v4u nt = __builtin_nontemporal_load((const v4u*)(rp + c * 16));
            t.w[k] = make_uint4(nt.x, nt.y, nt.z, nt.w);
        }
        t.sc[k] = FMT == W_Q8_0 ? sp[c >> 1] : sp[c];
    }
}

template <int FMT, int CPL>
IT_DEV float dot_chunks(const WChunks<CPL>& t, const XChunks<FMT, CPL>& x) {
    float acc = 0.0f;
#pragma unroll
    for (int k = 0; k < CPL; k++) {
        if (FMT == W_Q8_0) {
            int s = 0;
            s = dot4(t.w[k].x, x.a[k].x, s);
            s = dot4(t.w[k].y, x.a[k].y, s);
            s = dot4(t.w[k].z, x.a[k].z, s);
            s = dot4(t.w[k].w, x.a[k].w, s);
            acc += (float)s * (it_f16_to_f32((uint16_t)t.sc[k]) * x.d[k]);
        } else {
            float tA, tB;
            unit_nvfp4(t.w[k], t.sc[k], x.a[k], x.b[k], x.d[k], &tA, &tB);
            acc += tA;
            acc += tB;
        }
    }
    return acc;
}

// the row's dot, complete in the LAST lane of its L-lane group
template <int L> IT_DEV float reduce_lanes(float v) { return group_sum_tail<L>(v); }

// ------------------------------------------------------------------ activation prologue
// Q8_0 block quantization (naive.rs:652-675) of the quad a thread holds; the 8 threads of a
// 32-block are neighbours in a wave.  Dead threads pass zeros and write nothing.
IT_DEV void quant_quad(float4 v, bool live, int qi, int8_t* xq, float* xs) {
    float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    amax = group_max<8>(amax);
    if (!live) return;
    const float d = amax / 127.0f;
    const float id = d != 0.0f ? 1.0f / d : 0.0f;
    const float r[4] = {roundf(v.x * id), roundf(v.y * id), roundf(v.z * id), roundf(v.w * id)};
    uint32_t packed = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const float c = fminf(fmaxf(r[i], -128.0f), 127.0f);
        const int q = (r[i] != r[i]) ? 0 : (int)c;
        packed |= ((uint32_t)(q & 0xff)) << (8 * i);
    }
    *(uint32_t*)(xq + qi * 4) = packed;
    if ((qi & 7) == 0) xs[qi >> 3] = it_f16_to_f32(it_f32_to_f16(d));
}

IT_DEV double quad_sumsq(float4 v) {
    double s = (double)(v.x * v.x);
    s += (double)(v.y * v.y);
    s += (double)(v.z * v.z);
    s += (double)(v.w * v.w);
    return s;
}

// ------------------------------------------------------------------ router in a block
// softmax over n_expert logits, the n_used largest by (probability descending, id ascending),
// weights = picked probabilities over their sum in pick order (src/ops/mod.rs:1191-1216,
// naive.rs:362-376).  Every thread of the block calls this.  After it returns, ids[r] and
// wts[r] (LDS, 16 entries, zero past n_used) hold pick r and its probability; the return
// value is the weights' denominator, the same in every thread.
// n_expert <= 4 * THREADS, n_used <= 16.
//
// Selection is two-level, with every LDS loop of fixed length so its reads pipeline.  (a) Each
// thread ranks its values among the 64 * K of its wave: only wave ranks < n_used can be in the
// global top n_used, and they go to cand[wave][rank].  (b) The NW * 16 candidate slots are
// ranked against each other.//
// Probabilities are non-negative, so their bit patterns order like the values; a pick is
// compared as the 64-bit key (probability bits, ~id): larger key = earlier pick, keys are
// unique, and an empty slot is key 0.
template <int THREADS> struct RouteLds {
    float redf[2 * (THREADS / 64)];
    __attribute__((aligned(16))) unsigned long long keys[4 * THREADS];
    __attribute__((aligned(16))) unsigned long long cand[(THREADS / 64) * 16];
};

IT_DEV unsigned long long route_key(float p, int e) {
    return ((unsigned long long)__float_as_uint(p) << 32) | (unsigned long long)(~(unsigned)e);
}

// ranks this thread's key among the 64 keys of its wave and files the top n_used (n_expert <= THREADS)
IT_DEV void wave_rank_one(const unsigned long long* wave_keys, unsigned long long key, int n_used,
                          unsigned long long* cand) {
    int rank = 0;
    const ulonglong2* p2 = (const ulonglong2*)wave_keys;
#pragma unroll
    for (int j2 = 0; j2 < 32; j2++) {
        const ulonglong2 q = p2[j2];
        rank += q.x > key ? 1 : 0;
        rank += q.y > key ? 1 : 0;
    }
    if (key != 0ull && rank < n_used) cand[rank] = key;
}

// the same with up to four keys per thread (n_expert > THREADS): kept out of line and rolled,
// so the common kernel does not carry its registers
template <int THREADS>
__device__ __attribute__((noinline)) void wave_rank_many(const unsigned long long* keys, unsigned long long key0,
                                                         unsigned long long key1, unsigned long long key2,
                                                         unsigned long long key3, int K, int n_used,
                                                         unsigned long long* cand) {
    const unsigned long long key[4] = {key0, key1, key2, key3};
    int rank[4] = {0, 0, 0, 0};
    for (int k2 = 0; k2 < K; k2++) {
        const unsigned long long* wk = keys + k2 * THREADS + (threadIdx.x & ~63);
#pragma unroll 1
        for (int j = 0; j < 64; j++) {
            const unsigned long long q = wk[j];
#pragma unroll
            for (int k = 0; k < 4; k++) rank[k] += q > key[k] ? 1 : 0;
        }
    }
#pragma unroll
    for (int k = 0; k < 4; k++)
        if (k < K && key[k] != 0ull && rank[k] < n_used) cand[rank[k]] = key[k];
}

// this thread's logits (up to four experts, THREADS apart): fetched ahead of the activation prologue so that the
// two loads share one trip to memory
template <int THREADS>
__device__ __forceinline__ void route_fetch(const float* logits, int n_expert, float l[4]) {
    const int K = (n_expert + THREADS - 1) / THREADS;
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const int e = threadIdx.x + k * THREADS;
        l[k] = (k < K && e < n_expert) ? logits[e] : -INFINITY;
    }
}

template <int THREADS>
__device__ __forceinline__ float block_route(const float l[4], int n_expert, int n_used, RouteLds<THREADS>& sh, int* ids, float* wts) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    constexpr int NW = THREADS / 64;
    const int K = (n_expert + THREADS - 1) / THREADS;  // experts per thread that can be live
    float m = -INFINITY;
#pragma unroll
    for (int k = 0; k < 4; k++) m = fmaxf(m, l[k]);
    if (tid < NW * 16) sh.cand[tid] = 0ull;  // slots a wave does not fill stay empty
    if (tid < 16) wts[tid] = 0.0f;
    m = group_max_tail<64>(m);
    if (lane == 63) sh.redf[wave] = m;
    __syncthreads();
    m = sh.redf[0];
#pragma unroll
    for (int i = 1; i < NW; i++) m = fmaxf(m, sh.redf[i]);
    float v[4];
    float part = 0.0f;
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const int e = tid + k * THREADS;
        v[k] = (k < K && e < n_expert) ? fx_expf(l[k] - m) : 0.0f;
        part += v[k];
    }
    part = group_sum_tail<64>(part);
    if (lane == 63) sh.redf[NW + wave] = part;
    __syncthreads();
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < NW; i++) sum += sh.redf[NW + i];
    unsigned long long key[4];
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const int e = tid + k * THREADS;
        v[k] = v[k] / sum;
        key[k] = (k < K && e < n_expert) ? route_key(v[k], e) : 0ull;
        if (k < K) sh.keys[e] = key[k];
    }
    __syncthreads();
    if (K == 1) wave_rank_one(sh.keys + (tid & ~63), key[0], n_used, sh.cand + wave * 16);
    else wave_rank_many<THREADS>(sh.keys, key[0], key[1], key[2], key[3], K, n_used, sh.cand + wave * 16);
    __syncthreads();
    {
        // four threads per candidate slot, a quarter of the slots each
        const int c = tid >> 2, part = tid & 3;
        const unsigned long long me = sh.cand[c];
        int cnt = 0;
#pragma unroll
        for (int c2 = 0; c2 < NW * 2; c2++) {
            const ulonglong2 q = ((const ulonglong2*)sh.cand)[c2 * 4 + part];  // the four threads of a slot read neighbouring 16-byte pieces: no bank is hit twice
            cnt += q.x > me ? 1 : 0;
            cnt += q.y > me ? 1 : 0;
        }
        cnt += __shfl_xor(cnt, 1, 64);
        cnt += __shfl_xor(cnt, 2, 64);
        if (part == 0 && me != 0ull && cnt < n_used) {
            ids[cnt] = (int)~(unsigned)(me & 0xffffffffull);
            wts[cnt] = __uint_as_float((unsigned)(me >> 32));
        }
    }
    __syncthreads();
    float s = 0.0f;
#pragma unroll
    for (int r4 = 0; r4 < 4; r4++) {
        const float4 w = ((const float4*)wts)[r4];
        s += w.x;
        s += w.y;
        s += w.z;
        s += w.w;
    }
    return fmaxf(s, 6.103515625e-5f);
}

}  // namespace fastk
}  // namespace itk
