// Single-token kernels of the fast mode (reductions in wave order, not the CPU path's).
//
// The order-preserving kernels spend most of their time getting per-block terms into one
// lane's hands.  Here every lane owns a fixed set of 16-byte weight chunks of a row, keeps
// the matching activation chunks in registers for the whole kernel, and rows are reduced
// with cross-lane shuffles; a wave has four chunk loads per lane in flight and fetches its
// next row group while it reduces the current one.  The integer dots and the per-block
// scale products are the ones the reference forms (src/quant/dot.rs); only the order in
// which the per-block terms are added differs, so results agree to rounding, not by bit.
//
// A "chunk" is 16 bytes of a repacked weight row: 16 Q8_0 quants (half a block) or 32
// NVFP4 nibbles (two sub-blocks).  A row of `cpr` chunks is spread over L = min(64, cpr)
// lanes, CPL = cpr / L chunks each, so a wave covers P = 64 / L rows per step.
#include "it_device.h"
#include "it_dot.h"
#include "it_reduce.h"
#include "kernels.h"
#include "kernels_fused.h"
#include "it_fast.h"

// Phase stamps for tuning: a build with -DIT_STAMPS records the 100 MHz wall clock of one block's
// thread 0 at the marked points; the library build compiles them away.
#ifdef IT_STAMPS
__device__ long long it_stamps[32];
__device__ int it_stamp_block;
#define IT_STAMP(i)                                                                        \
    do {                                                                                   \
        if ((int)blockIdx.x == it_stamp_block && threadIdx.x == 0) it_stamps[i] = wall_clock64(); \
    } while (0)
#else
#define IT_STAMP(i) \
    do {            \
    } while (0)
#endif

namespace itk {
using namespace fastk;
namespace {

constexpr int FT = 512, FW = FT / 64;  // threads and waves of the GEMV blocks

// ------------------------------------------------------------------ chunk geometry
struct Geo {
    int cpl = 0, l = 0;
    bool ok = false;
};
inline Geo geo_of(int fmt, int n_in) {
    Geo g;
    const int per = fmt == W_Q8_0 ? 16 : fmt == W_NVFP4 ? 32 : 0;
    if (!per || n_in <= 0 || n_in % 32) return g;
    const int cpr = n_in / per;
    if (cpr & (cpr - 1)) return g;
    if (cpr >= 64) {
        g.l = 64;
        g.cpl = cpr / 64;
        g.ok = g.cpl <= 4;
    } else {
        g.l = cpr;
        g.cpl = 1;
        g.ok = cpr >= 8;
    }
    return g;
}

// The activation of a fused GEMV, from global f32 to quantized LDS, held in registers in
// between: thread t owns floats [4t, 4t+4) and [4(t+THREADS), ...).  n_in <= 8 * THREADS.
//   mode 0: as is; 1: rms_norm(x, norm_w) (naive.rs:633-650); 2: per-head rms_norm gated by
//   silu(gate) (head_dim / 4 a power of two <= 64, so a head sits inside one wave).
// Ends with a block barrier; xq / xs are then complete.
template <int THREADS>
__device__ __forceinline__ void stage_activation(const float* x, int n_in, int mode, const float* norm_w, const float* gate, int head_dim,
                                 float eps, float* copy1, float* copy2, int8_t* xq, float* xs, double* red,
                                 float* xf = nullptr) {
    const int tid = threadIdx.x;
    const int nq = n_in >> 2;
    float4 v[2];
    bool live[2];
#pragma unroll
    for (int k = 0; k < 2; k++) {
        const int qi = tid + k * THREADS;
        live[k] = qi < nq;
        v[k] = live[k] ? ((const float4*)x)[qi] : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    if (mode == 1) {
        float4 w[2];
#pragma unroll
        for (int k = 0; k < 2; k++)
            w[k] = live[k] ? ((const float4*)norm_w)[tid + k * THREADS] : make_float4(0.f, 0.f, 0.f, 0.f);
        double part = wave_sum_f64_tail(quad_sumsq(v[0]) + quad_sumsq(v[1]));
        if ((tid & 63) == 63) red[tid >> 6] = part;
        __syncthreads();
        double sum = 0.0;
#pragma unroll
        for (int i = 0; i < THREADS / 64; i++) sum += red[i];
        const float mean = (float)(sum / (double)n_in);
        const float scale = 1.0f / sqrtf(mean + eps);
#pragma unroll
        for (int k = 0; k < 2; k++) {
            v[k].x = v[k].x * scale * w[k].x;
            v[k].y = v[k].y * scale * w[k].y;
            v[k].z = v[k].z * scale * w[k].z;
            v[k].w = v[k].w * scale * w[k].w;
        }
    } else if (mode == 2 || mode == 3) {
        const int lh = head_dim >> 2;  // lanes per head
#pragma unroll
        for (int k = 0; k < 2; k++) {
            const int qi = tid + k * THREADS;
            double part = quad_sumsq(v[k]);
            for (int o = lh >> 1; o > 0; o >>= 1) part += __shfl_xor(part, o, 64);
            if (live[k]) {
                const float hs = 1.0f / sqrtf((float)(part / (double)head_dim) + eps);
                const float4 w = ((const float4*)norm_w)[qi & (lh - 1)];
                const float4 g = ((const float4*)gate)[qi];
                // mode 3: the producer already stored silu(gate)
                v[k].x = (mode == 2 ? fx_silu(g.x) : g.x) * (v[k].x * hs * w.x);
                v[k].y = (mode == 2 ? fx_silu(g.y) : g.y) * (v[k].y * hs * w.y);
                v[k].z = (mode == 2 ? fx_silu(g.z) : g.z) * (v[k].z * hs * w.z);
                v[k].w = (mode == 2 ? fx_silu(g.w) : g.w) * (v[k].w * hs * w.w);
            }
        }
    }
#pragma unroll
    for (int k = 0; k < 2; k++) {
        const int qi = tid + k * THREADS;
        if (live[k]) {
            if (copy1) ((float4*)copy1)[qi] = v[k];
            if (copy2) ((float4*)copy2)[qi] = v[k];
            if (xf) ((float4*)xf)[qi] = v[k];   // the f32 activation in LDS, for unquantized matrices
        }
        quant_quad(v[k], live[k], qi, xq, xs);
    }
    __syncthreads();
}

// ------------------------------------------------------------------ fused_gemv, fast
IT_DEV int fast_mat_index(const FusedGemvP& p, int g) {
    int mi = 0;
#pragma unroll
    for (int k = 1; k < 4; k++)
        if (k < p.n_mats && g >= p.m[k].group0) mi = k;
    return mi;
}

// row fr of the unquantized matrices (they follow the n_mats quantized ones in p.m): its matrix and its row there
// (an index, not a pointer: the address of a kernel argument would move the whole argument block to scratch memory)
IT_DEV int frow_locate(const FusedGemvP& p, int fr, int* j) {
    int k = p.n_mats;
    while (k + 1 < p.n_mats + p.n_fmats && fr >= p.m[k].n_out) {
        fr -= p.m[k].n_out;
        k++;
    }
    *j = fr;
    return k;
}
// issues the loads of an F32 row's chunks (16 bytes per lane per 256 weights); false when the row is not F32
constexpr int FC = 8;
// (with the row shared by `split` waves, wave `part` of them takes the part-th contiguous run of its chunks)
IT_DEV bool frow_fetch(const FusedGemvP& p, int fr, int n_in, int lane, float4 fw[FC], int split, int part) {
    int j;
    const FusedMat& m = p.m[frow_locate(p, fr, &j)];
    if (m.fmt != W_F32) return false;
    const float* row = (const float*)m.q + (int64_t)j * n_in;
    const int per = (n_in / 256) / split;   // the row's chunks are dealt to the waves that share it in contiguous runs
#pragma unroll
    for (int c = 0; c < FC; c++)
        if (c * 256 < n_in && c / per == part) fw[c] = *(const float4*)(row + c * 256 + lane * 4);
    return true;
}
// The order every kernel sums an F32 row of up to 2,048 weights in (the layer chain, which deals a row's chunks to
// its waves differently, follows the same order and gets the same bits): a chunk of 256 weights is one multiply-add chain per lane from zero
// and a lane reduction; the up to eight chunk sums are added as a balanced tree, absent chunks counting as zero.
IT_DEV float frow_tree(const float pc[FC]) { return ((pc[0] + pc[1]) + (pc[2] + pc[3])) + ((pc[4] + pc[5]) + (pc[6] + pc[7])); }
IT_DEV float frow_chunk(const float4 w, const float4 xv) { return fmaf(w.x, xv.x, fmaf(w.y, xv.y, fmaf(w.z, xv.z, fmaf(w.w, xv.w, 0.0f)))); }

// ONE: one step per group (a matrix of few rows spreads over more blocks, i.e. more CUs pull its weights)
// FM: the launch has unquantized matrices as well (a kernel of its own, so that the registers their rows are held in
// are not charged to the launches without them)
template <int FMT, int CPL, int L, bool ONE = false, bool FM = false>
__global__ __launch_bounds__(FT) void fused_gemv_fast_k(FusedGemvP p) {
    constexpr int P = 64 / L;
    constexpr int RB = ONE || CPL >= 4 ? 1 : 4 / CPL;  // steps per group: four chunk loads per lane in flight
    constexpr int RG = RB * P;
    __shared__ __align__(16) int8_t xq[FT * 8];
    __shared__ float xs[FT * 8 / 32];
    __shared__ double red[FW];
    __shared__ __align__(16) float xf[FT * 8];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int sub = lane % L, rsub = lane / L;
    const int n_in = p.n_in;
    const int gstride = gridDim.x * FW;
    int g = blockIdx.x * FW + wave;

    WChunks<CPL> t[RB];
    // the value an accumulating row adds to (epi 2) is fetched with the weights, not after the dot
    float ep[RB];
    int mi = 0, row0 = 0;
    auto fetch = [&](int gg) {
        mi = fast_mat_index(p, gg);
        const FusedMat& m = p.m[mi];
        row0 = (gg - m.group0) * RG;
#pragma unroll
        for (int r = 0; r < RB; r++) {
            const int row = row0 + r * P + rsub;
            load_w<FMT, CPL, L>(t[r], m.q, m.s, n_in, row, sub, row < m.n_out);
            if (sub == L - 1 && row < m.n_out && m.epi == 2) ep[r] = m.out[row];
        }
    };
    // the first group's weights start moving before the activation prologue runs
    if (g < p.total_groups) fetch(g);
    const bool f32_regs = FM && n_in % 256 == 0 && n_in <= FC * 256;
    float4 fw[FM ? FC : 1];
    bool f_loaded = false;
    const int fsplit = FM ? p.fsplit : 1;                       // 1, 2 or 4 waves a row; more than 1 only with f32_regs
    const int fpart = wave % fsplit, frows_blk = FW / fsplit;  // rows a block takes per trip
    if constexpr (FM) {
        const int fr0 = blockIdx.x * frows_blk + wave / fsplit;
        if (f32_regs && fr0 < p.total_frows) f_loaded = frow_fetch(p, fr0, n_in, lane, fw, fsplit, fpart);
    }

    const bool first = blockIdx.x == 0;
    stage_activation<FT>(p.x, n_in, p.mode, p.norm_w, p.gate, p.head_dim, p.eps, first ? p.x_copy : nullptr,
                         first ? p.x_copy2 : nullptr, xq, xs, red, FM ? xf : nullptr);
    XChunks<FMT, CPL> x;
    load_x<FMT, CPL, L>(x, xq, xs, sub);

    while (g < p.total_groups) {
        float acc[RB];
#pragma unroll
        for (int r = 0; r < RB; r++) acc[r] = dot_chunks<FMT, CPL>(t[r], x);
        const int cmi = mi, crow0 = row0;
        float cp[RB];
#pragma unroll
        for (int r = 0; r < RB; r++) cp[r] = ep[r];
        g += gstride;
        if (g < p.total_groups) fetch(g);
#pragma unroll
        for (int r = 0; r < RB; r++) acc[r] = reduce_lanes<L>(acc[r]);
        if (sub == L - 1) {
            const FusedMat& m = p.m[cmi];
#pragma unroll
            for (int r = 0; r < RB; r++) {
                const int j = crow0 + r * P + rsub;
                if (j >= m.n_out) continue;
                const float a = acc[r];
                if (m.epi == 0) {
                    m.out[j] = a;
                } else if (m.epi == 2) {
                    m.out[j] = cp[r] + a;
                } else if (m.epi == 3) {
                    m.out[j] = fx_silu(a);
                } else {
                    // causal conv (kernel 4) + silu on channel j, state [channel][3] oldest first
                    float* past = p.conv_state + (int64_t)j * 3;
                    const float4 w = *(const float4*)(p.conv_w + (int64_t)j * 4);
                    const float p0 = past[0], p1 = past[1], p2 = past[2];
                    float sum = 0.0f;
                    sum += p0 * w.x;
                    sum += p1 * w.y;
                    sum += p2 * w.z;
                    sum += a * w.w;
                    m.out[j] = fx_silu(sum);
                    past[0] = p1;
                    past[1] = p2;
                    past[2] = a;
                }
            }
        }
    }

    // unquantized matrices (the router and ssm alpha / beta of real files are F32): one wave per row, the row sum
    // split over the lanes.  An F32 row of up to 2,048 weights is held in registers: all of its loads are in flight
    // at once, the first row's since before the prologue and the next row's while this one is reduced.
    if constexpr (!FM) return;
    const int fstride = gridDim.x * frows_blk;
    // every wave of a block makes the same number of trips (the partial sums of a shared row meet behind a barrier)
    for (int base = blockIdx.x * frows_blk; base < p.total_frows; base += fstride) {
        const int fr = base + wave / fsplit;
        const bool live = fr < p.total_frows;
        float* outp = nullptr;
        float acc = 0.0f;
        bool chunked = false;
        if (live) {
            int j;
            const FusedMat& m = p.m[frow_locate(p, fr, &j)];
            outp = m.out + j;
            if (f32_regs && m.fmt == W_F32) {
                if (!f_loaded) frow_fetch(p, fr, n_in, lane, fw, fsplit, fpart);
                f_loaded = false;
                float4 cur[FC];
#pragma unroll
                for (int c = 0; c < FC; c++) cur[c] = fw[c];
                const int nxt = fr + fstride;
                if (nxt < p.total_frows) f_loaded = frow_fetch(p, nxt, n_in, lane, fw, fsplit, fpart);
                float pc[FC];
                const int per = (n_in / 256) / fsplit;
#pragma unroll
                for (int c = 0; c < FC; c++) {
                    pc[c] = 0.0f;
                    if (c * 256 >= n_in || c / per != fpart) continue;
                    pc[c] = reduce_lanes<64>(frow_chunk(cur[c], *(const float4*)(xf + c * 256 + lane * 4)));
                }
                acc = frow_tree(pc);
                chunked = true;
            } else if (fpart == 0) {   // other element types and row lengths: one wave walks the row
                const int esz = m.fmt == W_F32 ? 4 : 2;
                const uint8_t* row = m.q + (int64_t)j * n_in * esz;
                for (int i = lane * 4; i < n_in; i += 256) {
                    float4 wv;
                    if (m.fmt == W_F32) {
                        wv = *(const float4*)(row + (int64_t)i * 4);
                    } else {
                        const uint2 h = *(const uint2*)(row + (int64_t)i * 2);
                        wv = m.fmt == W_F16 ? make_float4(it_f16_to_f32(h.x & 0xffffu), it_f16_to_f32(h.x >> 16), it_f16_to_f32(h.y & 0xffffu), it_f16_to_f32(h.y >> 16))
                                            : make_float4(it_bf16_to_f32(h.x & 0xffffu), it_bf16_to_f32(h.x >> 16), it_bf16_to_f32(h.y & 0xffffu), it_bf16_to_f32(h.y >> 16));
                    }
                    const float4 xv = *(const float4*)(xf + i);
                    acc = fmaf(wv.x, xv.x, fmaf(wv.y, xv.y, fmaf(wv.z, xv.z, fmaf(wv.w, xv.w, acc))));
                }
            }
        }
        if (!chunked) acc = reduce_lanes<64>(acc);   // (the chunked form is reduced chunk by chunk: its sum is in lane 63 already)
        if (fsplit == 1) {
            if (live && lane == 63) *outp = acc;
        } else {
            float* fsum = (float*)red;   // the prologue is done with it; FW doubles hold FW floats
            if (lane == 63) fsum[wave] = acc;
            __syncthreads();
            if (live && fpart == 0 && lane == 63)
                *outp = fsplit == 2 ? fsum[wave] + fsum[wave + 1] : (fsum[wave] + fsum[wave + 1]) + (fsum[wave + 2] + fsum[wave + 3]);
            __syncthreads();
        }
    }
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
inline bool float_fmt(int f) { return f == W_F32 || f == W_F16 || f == W_BF16; }

}  // namespace

// checks p and fills the launch fields (matrix order, groups); false: not a case for the fast kernel
static bool fused_gemv_fast_prepare(FusedGemvP& p, Geo* geo, int* fmt_out, int* blocks_out) {
    if (p.exact || p.route_counter || p.n_mats < 1) return false;
    // quantized matrices first, unquantized ones behind them
    FusedMat qm[4], fm[4];
    int nq = 0, nf = 0;
    for (int i = 0; i < p.n_mats; i++) {
        if (float_fmt(p.m[i].fmt)) fm[nf++] = p.m[i];
        else qm[nq++] = p.m[i];
    }
    for (int i = 0; i < nq; i++) p.m[i] = qm[i];
    for (int i = 0; i < nf; i++) p.m[nq + i] = fm[i];
    p.n_mats = nq;
    p.n_fmats = nf;
    p.total_frows = 0;
    for (int i = 0; i < nf; i++) {
        if (fm[i].epi != 0 || !aligned16(fm[i].q) || p.n_in % 4) return false;
        p.total_frows += fm[i].n_out;
    }
    const int fmt = nq ? p.m[0].fmt : (int)W_Q8_0;
    if (fmt != W_Q8_0 && fmt != W_NVFP4) return false;
    for (int i = 1; i < nq; i++)
        if (p.m[i].fmt != fmt) return false;
    const Geo g = geo_of(fmt, p.n_in);
    if (!g.ok || p.n_in > FT * 8 || p.n_in % 32) return false;
    if (!aligned16(p.x) || !aligned16(p.x_copy) || !aligned16(p.x_copy2)) return false;
    if (p.mode == 1 && !aligned16(p.norm_w)) return false;
    if (p.mode == 2 || p.mode == 3) {
        const int lh = p.head_dim / 4;
        if (p.head_dim % 4 || lh < 1 || lh > 64 || (lh & (lh - 1)) || p.n_in % p.head_dim) return false;
        if (!aligned16(p.norm_w) || !aligned16(p.gate)) return false;
    }
    for (int i = 0; i < nq; i++) {
        if (!aligned16(p.m[i].q) || (reinterpret_cast<uintptr_t>(p.m[i].s) & 1)) return false;
        if (p.m[i].epi == 1 && !aligned16(p.conv_w)) return false;
    }
    const int P = 64 / g.l;
    int RB = g.cpl >= 4 ? 1 : 4 / g.cpl, RG = RB * P;
    int groups = 0;
    auto count_groups = [&]() {
        groups = 0;
        for (int i = 0; i < nq; i++) {
            p.m[i].group0 = groups;
            groups += (p.m[i].n_out + RG - 1) / RG;
        }
    };
    count_groups();
    // few rows (the router's 513): one step per group, so that twice or four times as many CUs pull the weights
    if (RB > 1 && (groups + FW - 1) / FW < 128) {
        RB = 1;
        RG = P;
        count_groups();
    }
    p.total_groups = groups;
    p.rows_per_wave = RG;
    // a launch of unquantized rows only (the F32 router of a real file: 513 rows of 8 KB) would sit on 65 CUs with a
    // wave per row; two waves a row use 129 (431 against 427 tok/s for the model with such a router; four waves a
    // row, 257 CUs, give the gain back to the barrier: 426)
    p.fsplit = 1;
    if (nq == 0 && p.n_in % 256 == 0 && p.n_in <= FC * 256) {
        bool all_f32 = true;
        for (int i = 0; i < nf; i++) all_f32 = all_f32 && fm[i].fmt == W_F32;
        const int chunks = p.n_in / 256;
        while (all_f32 && p.fsplit < 2 && chunks % (2 * p.fsplit) == 0 && (p.total_frows * p.fsplit + FW - 1) / FW < 200) p.fsplit *= 2;
    }
    int blocks = (max(groups, p.total_frows * p.fsplit) + FW - 1) / FW;
    // Whole multiples of the CU count, so that every CU carries the same number of blocks: four per CU for a matrix
    // that loops (the LM head), two per CU for one that would need between two and four (the GDN in-projection's 772
    // blocks, three on some CUs and four on others, ran 0.03 ms per token slower than 512 that loop once or twice;
    // 256, 384, 448, 576, 640 and 768 all measured slower than 512).
    static const int cus = [] {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n < 1) n = 256;
        return n;
    }();
    if (blocks > 4 * cus) blocks = 4 * cus;
    else if (blocks > 2 * cus) blocks = 2 * cus;
    if (blocks < 1) blocks = 1;
    *geo = g;
    *fmt_out = fmt;
    *blocks_out = blocks;
    return true;
}

bool fused_gemv_fast_takes(const FusedGemvP& p) {
    FusedGemvP q = p;
    Geo g;
    int fmt, blocks;
    return fused_gemv_fast_prepare(q, &g, &fmt, &blocks);
}

bool fused_gemv_fast(FusedGemvP p, hipStream_t s) {
    Geo g;
    int fmt, blocks;
    if (!fused_gemv_fast_prepare(p, &g, &fmt, &blocks)) return false;
    const bool one = p.rows_per_wave == 64 / g.l && g.cpl < 4;
    const bool fm = p.n_fmats > 0;
#define IT_LAUNCH(F, C, LL)                                                                                            \
    do {                                                                                                               \
        if (one && fm) hipLaunchKernelGGL((fused_gemv_fast_k<F, C, LL, true, true>), dim3(blocks), dim3(FT), 0, s, p);  \
        else if (one) hipLaunchKernelGGL((fused_gemv_fast_k<F, C, LL, true, false>), dim3(blocks), dim3(FT), 0, s, p);  \
        else if (fm) hipLaunchKernelGGL((fused_gemv_fast_k<F, C, LL, false, true>), dim3(blocks), dim3(FT), 0, s, p);   \
        else hipLaunchKernelGGL((fused_gemv_fast_k<F, C, LL, false, false>), dim3(blocks), dim3(FT), 0, s, p);          \
    } while (0)
    if (fmt == W_Q8_0) {
        if (g.l == 64 && g.cpl == 1) IT_LAUNCH(W_Q8_0, 1, 64);
        else if (g.l == 64 && g.cpl == 2) IT_LAUNCH(W_Q8_0, 2, 64);
        else if (g.l == 64) IT_LAUNCH(W_Q8_0, 4, 64);
        else if (g.l == 32) IT_LAUNCH(W_Q8_0, 1, 32);
        else if (g.l == 16) IT_LAUNCH(W_Q8_0, 1, 16);
        else IT_LAUNCH(W_Q8_0, 1, 8);
    } else {
        if (g.l == 64 && g.cpl == 1) IT_LAUNCH(W_NVFP4, 1, 64);
        else if (g.l == 64 && g.cpl == 2) IT_LAUNCH(W_NVFP4, 2, 64);
        else if (g.l == 64) IT_LAUNCH(W_NVFP4, 4, 64);
        else if (g.l == 32) IT_LAUNCH(W_NVFP4, 1, 32);
        else if (g.l == 16) IT_LAUNCH(W_NVFP4, 1, 16);
        else IT_LAUNCH(W_NVFP4, 1, 8);
    }
#undef IT_LAUNCH
    return true;
}

namespace {

// ------------------------------------------------------------------ moe_glu, fast
// Jobs: n_used * ge routed groups (pick-major), then gs shared-expert groups.  A group is
// RB steps of P (gate row, up row) pairs; out[row] = silu(gate.x * sg) * (up.x * su).
struct GluGeo {
    int e_cpl, e_l, e_groups, e_rg;
    int s_cpl, s_l, s_groups, s_rg;
};

template <int FMT, int CPL, int L>
IT_DEV void glu_job(const uint8_t* gq, const uint8_t* gs, const uint8_t* uq, const uint8_t* us, int n_in, int n_out,
                    int row0, float sg, float su, const int8_t* xq, const float* xs, float* out, int lane,
                    WChunks<CPL>* tg, WChunks<CPL>* tu, bool loaded) {
    constexpr int P = 64 / L;
    constexpr int RB = CPL >= 2 ? 1 : 2;
    const int sub = lane % L, rsub = lane / L;
    if (!loaded) {
#pragma unroll
        for (int r = 0; r < RB; r++) {
            const int row = row0 + r * P + rsub;
            load_w<FMT, CPL, L>(tg[r], gq, gs, n_in, row, sub, row < n_out);
            load_w<FMT, CPL, L>(tu[r], uq, us, n_in, row, sub, row < n_out);
        }
    }
    XChunks<FMT, CPL> x;
    load_x<FMT, CPL, L>(x, xq, xs, sub);
#pragma unroll
    for (int r = 0; r < RB; r++) {
        float ag = reduce_lanes<L>(dot_chunks<FMT, CPL>(tg[r], x));
        float au = reduce_lanes<L>(dot_chunks<FMT, CPL>(tu[r], x));
        const int row = row0 + r * P + rsub;
        if (sub == L - 1 && row < n_out) {
            ag *= sg;
            au *= su;
            out[row] = fx_silu(ag) * au;
        }
    }
}

template <int EF, int ECPL, int EL, int SF, int SCPL, int SL>
__global__ __launch_bounds__(FT) void moe_glu_fast_k(MoeGluP p, GluGeo gg) {
    {   // a short batch: grid row t is token t
        const int64_t t = blockIdx.y;
        p.x += t * p.n_in;
        p.out += t * p.n_used * p.n_out;
        p.sh_out += t * p.sh_n_out;
        if (p.logits) {
            p.logits += t * p.n_expert;
            p.route_ids_out += t * p.n_used;
            p.route_w_out += t * p.n_used;
        } else {
            p.route_ids += t * p.n_used;
        }
    }
    __shared__ __align__(16) int8_t xq[FT * 8];
    __shared__ float xs[FT * 8 / 32];
    __shared__ double red[FW];
    __shared__ RouteLds<FT> route_sh;
    __shared__ int ids[16];
    __shared__ __align__(16) float wts[16];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n_in = p.n_in;
    const int routed_groups = p.n_used * gg.e_groups;
    const int total = routed_groups + gg.s_groups;
    // job j belongs to block j % gridDim.x, wave j / gridDim.x: with a grid of whole multiples of the CU count every CU
    // carries the same number of jobs (to within one)
    const int gstride = gridDim.x * FW;
    int g = blockIdx.x + wave * gridDim.x;

    // a wave whose first job is a shared-expert group knows its rows before the router has run
    WChunks<SCPL> sg[2], su[2];
    const bool pre = g >= routed_groups && g < total;
    if (pre) {
        constexpr int P = 64 / SL, RB = SCPL >= 2 ? 1 : 2;
        const int row0 = (g - routed_groups) * gg.s_rg;
#pragma unroll
        for (int r = 0; r < RB; r++) {
            const int row = row0 + r * P + lane / SL;
            load_w<SF, SCPL, SL>(sg[r], p.sh_gq, p.sh_gs, n_in, row, lane % SL, row < p.sh_n_out);
            load_w<SF, SCPL, SL>(su[r], p.sh_uq, p.sh_us, n_in, row, lane % SL, row < p.sh_n_out);
        }
    }

    float logit[4];
    if (p.logits) route_fetch<FT>(p.logits, p.n_expert, logit);
    stage_activation<FT>(p.x, n_in, 0, nullptr, nullptr, 0, 0.0f, nullptr, nullptr, xq, xs, red);
    if (p.logits) {
        const float denom = block_route<FT>(logit, p.n_expert, p.n_used, route_sh, ids, wts);
        if (blockIdx.x == 0 && tid < p.n_used) {
            p.route_ids_out[tid] = ids[tid];
            p.route_w_out[tid] = wts[tid] / denom;
        }
    } else {
        if (tid < p.n_used) ids[tid] = p.route_ids[tid];
        __syncthreads();
    }
    bool loaded = pre;
    for (; g < total; g += gstride) {
        if (g < routed_groups) {
            const int y = g / gg.e_groups, row0 = (g - y * gg.e_groups) * gg.e_rg;
            const int64_t e = ids[y];
            const float scg = p.gscale2 ? p.gscale2[e] : 1.0f, scu = p.uscale2 ? p.uscale2[e] : 1.0f;
            WChunks<ECPL> tg[2], tu[2];
            glu_job<EF, ECPL, EL>(p.gq + e * p.q_stride, p.gs + e * p.s_stride, p.uq + e * p.q_stride,
                                  p.us + e * p.s_stride, n_in, p.n_out, row0, scg, scu, xq, xs,
                                  p.out + (int64_t)y * p.n_out, lane, tg, tu, false);
        } else {
            const int row0 = (g - routed_groups) * gg.s_rg;
            glu_job<SF, SCPL, SL>(p.sh_gq, p.sh_gs, p.sh_uq, p.sh_us, n_in, p.sh_n_out, row0, p.sh_gscale, p.sh_uscale, xq, xs,
                                  p.sh_out, lane, sg, su, loaded);
        }
        loaded = false;
    }
}

}  // namespace

bool moe_glu_fast(MoeGluP p, hipStream_t s, bool dry_run) {
    if (p.exact) return false;
    const Geo ge = geo_of(p.fmt, p.n_in), gs = geo_of(p.sh_fmt, p.n_in);
    if (!ge.ok || !gs.ok || p.n_in > FT * 8 || p.n_used > 16 || p.n_used < 1) return false;
    if (p.logits && (p.n_expert > FT * 4 || p.n_expert < p.n_used || !p.route_ids_out || !p.route_w_out)) return false;
    if (!p.logits && !p.route_ids) return false;
    if (!aligned16(p.x) || !aligned16(p.gq) || !aligned16(p.uq) || !aligned16(p.sh_gq) || !aligned16(p.sh_uq)) return false;
    if (p.q_stride % 16 || p.s_stride % 2) return false;
    GluGeo gg{};
    gg.e_cpl = ge.cpl;
    gg.e_l = ge.l;
    gg.e_rg = (ge.cpl >= 2 ? 1 : 2) * (64 / ge.l);
    gg.e_groups = (p.n_out + gg.e_rg - 1) / gg.e_rg;
    gg.s_cpl = gs.cpl;
    gg.s_l = gs.l;
    gg.s_rg = (gs.cpl >= 2 ? 1 : 2) * (64 / gs.l);
    gg.s_groups = (p.sh_n_out + gg.s_rg - 1) / gg.s_rg;
    const int total = p.n_used * gg.e_groups + gg.s_groups;
    int blocks = (total + FW - 1) / FW;
    if (blocks > 1024) blocks = 1024;
    if (blocks < 1) blocks = 1;
    const int n_tok = p.n_tok > 1 ? p.n_tok : 1;
    // a grid between one and two blocks per CU leaves some CUs with twice the jobs of others (352 blocks on 256 CUs for
    // the 35B shape): two per CU everywhere, jobs dealt round the blocks, is 1 % of the token faster
    {
        int dev = 0, cus = 0;
        static const int n_cu = (hipGetDevice(&dev) == hipSuccess &&
                                 hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && cus > 0) ? cus : 256;
        if (blocks > n_cu && blocks < 2 * n_cu) blocks = 2 * n_cu;
        // a short batch: about four blocks per CU in all (every block repeats its token's prologue and route, so a
        // token's jobs go to fewer blocks, which loop over them)
        if (n_tok > 1) blocks = std::max(32, std::min(blocks, 4 * n_cu / n_tok));
    }
    // the geometry of both formats follows from n_in: (CPL, L) for Q8_0 and for NVFP4
#define IT_LAUNCH(EF, EC, EL, SF, SC, SL) \
    hipLaunchKernelGGL((moe_glu_fast_k<EF, EC, EL, SF, SC, SL>), dim3(blocks, n_tok), dim3(FT), 0, s, p, gg)
#define IT_BY_FMT(QC, QL, NC, NL)                                                                       \
    do {                                                                                                \
        if (p.fmt == W_Q8_0 && p.sh_fmt == W_Q8_0) IT_LAUNCH(W_Q8_0, QC, QL, W_Q8_0, QC, QL);           \
        else if (p.fmt == W_NVFP4 && p.sh_fmt == W_Q8_0) IT_LAUNCH(W_NVFP4, NC, NL, W_Q8_0, QC, QL);    \
        else if (p.fmt == W_NVFP4 && p.sh_fmt == W_NVFP4) IT_LAUNCH(W_NVFP4, NC, NL, W_NVFP4, NC, NL);  \
        else IT_LAUNCH(W_Q8_0, QC, QL, W_NVFP4, NC, NL);                                                \
    } while (0)
    if (p.n_in != 256 && p.n_in != 512 && p.n_in != 1024 && p.n_in != 2048 && p.n_in != 4096) return false;
    if (dry_run) return true;
    switch (p.n_in) {
        case 256: IT_BY_FMT(1, 16, 1, 8); break;
        case 512: IT_BY_FMT(1, 32, 1, 16); break;
        case 1024: IT_BY_FMT(1, 64, 1, 32); break;
        case 2048: IT_BY_FMT(2, 64, 1, 64); break;
        case 4096: IT_BY_FMT(4, 64, 2, 64); break;
        default: return false;
    }
#undef IT_BY_FMT
#undef IT_LAUNCH
    return true;
}

namespace {

// ------------------------------------------------------------------ moe_down, fast
// x[j] += sum_y w_y * scale2_y * (down_y[j] . g_y) + sigmoid(logit) * (shared_down[j] . g_sh)
// Loads are issued in the order they can be consumed: the small intermediates first (they are quantized while the
// weights are still on their way), then every weight chunk of the wave and the residual it will add to.
constexpr int DT = 512, DW = DT / 64;
constexpr int MAXU = 16, QUARTU = MAXU / 4;

// A wave step covers P = 64 / L output rows.  Four waves share a row group: wave q of the four takes the picks
// y = q, q + 4, ..., the last of them the shared expert as well, and the four partial sums meet in LDS in a fixed
// order.  Eight waves a block (two row groups): the block-wide quantization of the intermediates is three quads a
// thread, and two waves a SIMD cover each other's waits.
template <int EF, int ECPL, int L, int SF, int SCPL>
__global__ __launch_bounds__(DT) void moe_down_fast_k(MoeDownP p) {
    {   // a short batch: grid row t is token t
        const int64_t t = blockIdx.y;
        p.g_all += t * p.n_used * p.n_in;
        p.g_shared += t * p.sh_n_in;
        p.route_ids += t * p.n_used;
        p.route_w += t * p.n_used;
        p.logit += t;
        p.x += t * p.n_out;
        if (p.y) p.y += t * p.n_out;
    }
    extern __shared__ __align__(16) unsigned char smem[];
    constexpr int P = 64 / L;
    const int n_in = p.n_in, sh_in = p.sh_n_in, NU = p.n_used;
    const int total = NU * n_in + sh_in;  // floats staged: picks back to back, then the shared vector
    int8_t* xq = (int8_t*)smem;
    float* xs = (float*)(smem + ((total + 15) & ~15));
    __shared__ float coef[MAXU];
    __shared__ float partial[DW / 4][3][64];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int quarter = wave & 3, group = wave >> 2;
    const int sub = lane % L, rsub = lane / L;
    const int row = (blockIdx.x * (DW / 4) + group) * P + rsub;
    const bool live = row < p.n_out;
    IT_STAMP(0);
    it_count_expert_reads(p.route_ids, NU, p.counts_gate, p.counts_up, p.counts_down, p.tally);

    // the intermediates: up to three quads per thread (12 floats) cover 6144 floats per block
    const int nq = total >> 2, nq_routed = (NU * n_in) >> 2;
    constexpr int QR = 3;
    float4 v[QR];
#pragma unroll
    for (int k = 0; k < QR; k++) {
        const int qi = k * DT + tid;
        v[k] = qi >= nq ? make_float4(0.f, 0.f, 0.f, 0.f)
                        : qi < nq_routed ? ((const float4*)p.g_all)[qi] : ((const float4*)p.g_shared)[qi - nq_routed];
    }
    // this wave's picks: y = 4 * k + quarter
    WChunks<ECPL> t[QUARTU];
    WChunks<SCPL> tsh;
#pragma unroll
    for (int k = 0; k < QUARTU; k++) {
        const int y = 4 * k + quarter;
        if (y < NU) {
            const int64_t e = p.route_ids[y];
            load_w<EF, ECPL, L>(t[k], p.q + e * p.q_stride, p.s + e * p.s_stride, n_in, row, sub, live);
        }
    }
    if (quarter == 3) load_w<SF, SCPL, L>(tsh, p.sh_q, p.sh_s, sh_in, row, sub, live);
    const float x_old = (!quarter && sub == L - 1 && live && !p.y) ? p.x[row] : 0.0f;
    if (tid < NU) coef[tid] = p.route_w[tid] * (p.scale2 ? p.scale2[p.route_ids[tid]] : 1.0f);
    const float gate = fx_sigmoid(p.logit[0]) * p.sh_dscale;
    IT_STAMP(1);

#pragma unroll
    for (int k = 0; k < QR; k++) quant_quad(v[k], k * DT + tid < nq, k * DT + tid, xq, xs);
    IT_STAMP(2);
    __syncthreads();
    IT_STAMP(3);

    float acc = 0.0f;
#pragma unroll
    for (int k = 0; k < QUARTU; k++) {
        const int y = 4 * k + quarter;
        if (y < NU) {
            XChunks<EF, ECPL> x;
            load_x<EF, ECPL, L>(x, xq + y * n_in, xs + y * (n_in >> 5), sub);
            acc += coef[y] * dot_chunks<EF, ECPL>(t[k], x);
        }
    }
    if (quarter == 3) {
        XChunks<SF, SCPL> x;
        load_x<SF, SCPL, L>(x, xq + NU * n_in, xs + NU * (n_in >> 5), sub);
        acc += gate * dot_chunks<SF, SCPL>(tsh, x);
    }
    IT_STAMP(4);
    acc = reduce_lanes<L>(acc);
    if (quarter) partial[group][quarter - 1][lane] = acc;
    __syncthreads();
    IT_STAMP(5);
    if (!quarter && sub == L - 1 && live) {
        const float sum = (acc + partial[group][0][lane]) + (partial[group][1][lane] + partial[group][2][lane]);
        if (p.y) p.y[row] = sum;
        else p.x[row] = x_old + sum;
    }
    IT_STAMP(6);
}

}  // namespace

bool moe_down_fast(MoeDownP p, hipStream_t s, bool dry_run) {
    const Geo ge = geo_of(p.fmt, p.n_in);
    if (!ge.ok || ge.cpl != 1 || p.n_used > MAXU || p.n_used < 1) return false;
    const int L = ge.l;
    // the shared expert's row is spread over the same L lanes
    const int per_s = p.sh_fmt == W_Q8_0 ? 16 : p.sh_fmt == W_NVFP4 ? 32 : 0;
    if (!per_s || p.sh_n_in % 32 || p.n_in % 32) return false;
    const int cpr_s = p.sh_n_in / per_s;
    if (cpr_s % L) return false;
    const int scpl = cpr_s / L;
    if (scpl != 1 && scpl != 2) return false;
    if (!aligned16(p.g_all) || !aligned16(p.g_shared) || !aligned16(p.q) || !aligned16(p.sh_q) || p.q_stride % 16 ||
        p.s_stride % 2)
        return false;
    const int total = p.n_used * p.n_in + p.sh_n_in;
    const size_t lds = (size_t)((total + 15) & ~15) + (size_t)(total / 32) * 4;
    if (lds > 60 * 1024 || total > 3 * DT * 4) return false;
    const int P = 64 / L;
    const int blocks = (p.n_out + (DW / 4) * P - 1) / ((DW / 4) * P);
#define IT_LAUNCH(EF, LL, SF, SC) hipLaunchKernelGGL((moe_down_fast_k<EF, 1, LL, SF, SC>), dim3(blocks, p.n_tok > 1 ? p.n_tok : 1), dim3(DT), lds, s, p)
#define IT_BY_L(EF, SF, SC)                      \
    do {                                         \
        if (L == 64) IT_LAUNCH(EF, 64, SF, SC);  \
        else if (L == 32) IT_LAUNCH(EF, 32, SF, SC); \
        else if (L == 16) IT_LAUNCH(EF, 16, SF, SC); \
        else IT_LAUNCH(EF, 8, SF, SC);           \
    } while (0)
    const bool fmts = (p.fmt == W_NVFP4 && (p.sh_fmt == W_Q8_0 || p.sh_fmt == W_NVFP4)) || (p.fmt == W_Q8_0 && p.sh_fmt == W_Q8_0);
    if (!fmts) return false;
    if (dry_run) return true;
    if (p.fmt == W_NVFP4 && p.sh_fmt == W_Q8_0) {
        if (scpl == 1) IT_BY_L(W_NVFP4, W_Q8_0, 1);
        else IT_BY_L(W_NVFP4, W_Q8_0, 2);
    } else if (p.fmt == W_Q8_0 && p.sh_fmt == W_Q8_0) {
        if (scpl == 1) IT_BY_L(W_Q8_0, W_Q8_0, 1);
        else IT_BY_L(W_Q8_0, W_Q8_0, 2);
    } else if (p.fmt == W_NVFP4 && p.sh_fmt == W_NVFP4) {
        if (scpl == 1) IT_BY_L(W_NVFP4, W_NVFP4, 1);
        else IT_BY_L(W_NVFP4, W_NVFP4, 2);
    } else {
        return false;
    }
#undef IT_BY_L
#undef IT_LAUNCH
    return true;
}

}  // namespace itk
