// =====================================================================================
// NVFP4 expert matmuls on the f16 matrix cores for FEW pairs per expert (fast mode).
//
// The 128-pair tiles of k_gemm_f16.hip pay for themselves from a few dozen pairs per expert on.  A batch
// of 32 .. 1,000 tokens over 512 experts leaves 1 .. 20 pairs per expert: there the work is the expansion
// of every touched expert's nibbles to f16, once, and its stream from HBM; the products are nearly free.
// This kernel keeps the arithmetic of the wide kernel (weights exact in f16 with the sub-block scale folded
// in, activations as an f16 hi + lo pair, f32 accumulation over the whole k range, the row's power of two
// and the expert's scale in the epilogue) on tiles of 16 pairs, MFMA 16x16x32:
//
//  * no LDS in the main loop: a wave is on its own.  Lane l supplies weight row l % 16 and the k group l / 16 of
//    the A operand straight from the nibble bytes it loads from global memory: two 128-bit loads per 256-wide
//    k chunk, units kg and kg + 4, so that the four lanes of a row fetch its whole 128-byte line at once
//    (with one load per 128-wide chunk every line was fetched in two halves, far apart in time: 10 % slower);
//  * the activations of the 16 pairs are stored by acts_split_perm_k in the order the MFMA steps consume
//    them, so a lane's B operands of a chunk are sixteen 128-bit loads (from L2: a batch's activations are a
//    few MB).  They stay in registers while the wave walks its row groups, so every B load feeds
//    `groups` MFMAs;
//  * a wave owns up to 8 groups of 16 rows of ONE matrix and carries their f32 sums in registers across the k
//    chunks; for the gate/up pair two waves of a block take the gate rows and two the same rows of up, whose
//    sums cross to the gate waves through LDS at the end (the only barrier).
//
// MFMA 16x16x32 f16 operands: lane l holds A[l % 16][8 (l / 16) .. + 8], B[8 (l / 16) .. + 8][l % 16] and
// receives D[4 (l / 16) + i][l % 16], i = 0..3.  The k order inside a step is free as long as A and B agree:
// step n of a lane's 32-wide unit takes the elements the n-th dword of the 16 nibble bytes holds (low nibbles:
// elements 16 (n / 2) + 4 (n % 2) + {0..3}; high nibbles: the same + 8).
#include <algorithm>

#include "it_device.h"
#include "it_dot.h"
#include "kernels.h"

namespace itk {
namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));
constexpr int SK_PAIRS = 16;   // pairs per tile
constexpr int SK_KC = 256;     // k per chunk: two 32-wide units per k group, 128 bytes of nibbles per row
constexpr int SK_G = 8;        // row groups per wave at most
constexpr int SK_AHEAD = 1;    // steps of weights in flight per wave

// Rows of f16 hi / lo in MFMA step order and the row's power of two, from Q8_0 quants and scales (the values of
// acts_split_f16_k; inside every 32-element unit, element j moves to 8 n + 4 (j / 8 % 2) + j % 4 with
// n = 2 (j / 16) + (j / 4) % 2).
__global__ __launch_bounds__(256) void acts_split_perm_k(const int8_t* __restrict__ q, const float* __restrict__ sc,
                                                          int n_in, uint16_t* __restrict__ xh, uint16_t* __restrict__ xl,
                                                          float* __restrict__ rscale) {
    __shared__ float part[4];
    const int row = blockIdx.x, tid = threadIdx.x, nb = n_in >> 5;
    float mx = 0.0f;
    for (int b = tid; b < nb; b += 256) mx = fmaxf(mx, fabsf(sc[(int64_t)row * nb + b]));
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
    if ((tid & 63) == 0) part[tid >> 6] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(part[0], part[1]), fmaxf(part[2], part[3])) * 127.0f;
    int ex = 0;
    if (mx > 0.0f) (void)frexpf(mx, &ex);                     // mx = m * 2^ex, m in [0.5, 1)
    ex = max(-100, min(100, ex));
    const float down = ldexpf(1.0f, -ex);
    if (tid == 0) rscale[row] = ldexpf(1.0f, ex);
    for (int i = tid; i < n_in / 4; i += 256) {
        const uint32_t qq = ((const uint32_t*)(q + (int64_t)row * n_in))[i];
        const float d = sc[(int64_t)row * nb + (i >> 3)] * down;
        uint16_t h[4], l[4];
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const float x = (float)(int8_t)(qq >> (8 * k)) * d;
            const _Float16 hi = (_Float16)x;
            const _Float16 lo = (_Float16)(x - (float)hi);
            h[k] = __builtin_bit_cast(uint16_t, hi);
            l[k] = __builtin_bit_cast(uint16_t, lo);
        }
        const int j0 = 4 * (i & 7);                            // first of this thread's four elements inside the unit
        const int n = 2 * (j0 >> 4) + ((j0 >> 2) & 1);
        const int64_t at = (int64_t)row * n_in + 32 * (i >> 3) + 8 * n + 4 * ((j0 >> 3) & 1);
        *(uint2*)(xh + at) = make_uint2(h[0] | ((uint32_t)h[1] << 16), h[2] | ((uint32_t)h[3] << 16));
        *(uint2*)(xl + at) = make_uint2(l[0] | ((uint32_t)l[1] << 16), l[2] | ((uint32_t)l[3] << 16));
    }
}

struct RawW {
    uint4 nib[2];     // units kg and kg + 4 of the chunk: a row's whole 128-byte line is read by its four lanes at once
    uint32_t sc[2];
};

// fragment n (8 weights as f16, sub-block scale folded in) of a lane's 16 nibble bytes
IT_DEV h8 expand_frag(const uint4 nib, const uint32_t rsc, int n) {
    // an e4m3 code moved into an f16's exponent and mantissa fields is the scale times 2^-8 (subnormal codes included);
    // the magnitudes carry 2^7 and the halving back; code 0x7f (not a number) counts as zero, as in the CPU path
    const uint32_t em = (n < 2 ? rsc : rsc >> 8) & 0x7fu;
    const _Float16 sv = __builtin_bit_cast(_Float16, (uint16_t)(em == 0x7fu ? 0u : em << 7));
    const h2 sc = h2{sv, sv};
    const uint32_t wd = n == 0 ? nib.x : n == 1 ? nib.y : n == 2 ? nib.z : nib.w;
    h2 a0, a1, a2, a3;
    fp4x4_to_f16x4(wd & 0x0f0f0f0fu, sc, &a0, &a1);
    fp4x4_to_f16x4((wd >> 4) & 0x0f0f0f0fu, sc, &a2, &a3);
    return h8{a0[0], a0[1], a1[0], a1[1], a2[0], a2[1], a3[0], a3[1]};
}

// GLU: waves 0 and 1 take the gate matrix, waves 2 and 3 the up matrix of the same rows (a wave streams ONE matrix, so
// its sums and operands fit the registers of four to five waves per SIMD); the up waves pass their sums through LDS.
template <bool GLU>
__global__ __launch_bounds__(256) void experts_f16s_k(ExpertsF16P p, int gpw) {
    __shared__ float4 handoff[GLU ? 2 * SK_G * 64 : 1];
    const int tile = blockIdx.x;
    if (tile >= *p.n_tiles) return;
    const int4 td = p.tiles[tile];
    const int64_t e = td.x;
    const int cnt = td.z;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r16 = lane & 15, kg = lane >> 4;
    const int n_in = p.n_in, n_chunk = n_in / SK_KC;
    const int z = GLU ? wave >> 1 : 0;                 // which matrix
    const int wslot = GLU ? wave & 1 : wave;           // which share of the block's row groups
    constexpr int WPB = GLU ? 2 : 4;                   // shares per block
    // this wave's row groups: rows g0 * 16 .. of the matrix, `mine` of them (none: the wave only keeps the barrier)
    const int g0 = (blockIdx.y * WPB + wslot) * gpw;
    const int mine = max(0, min(gpw, (p.n_out + 15) / 16 - g0));
    const int pair = p.order[td.y + min(r16, cnt - 1)];
    const int xrow = p.x_mode == 0 ? pair : (p.x_mode == 1 ? pair / p.n_used : 0);
    const uint16_t* bh = p.xh + (int64_t)xrow * n_in + 32 * kg;
    const uint16_t* bl = p.xl + (int64_t)xrow * n_in + 32 * kg;
    const uint8_t* wq = z ? it_expert_at(p.q2, p.q2_tab, e, p.q_stride) : it_expert_at(p.q, p.q_tab, e, p.q_stride);
    const uint8_t* ws = z ? it_expert_at(p.s2, p.s2_tab, e, p.s_stride) : it_expert_at(p.s, p.s_tab, e, p.s_stride);

    v4f acc[SK_G];
#pragma unroll
    for (int g = 0; g < SK_G; g++) acc[g] = v4f{0.0f, 0.0f, 0.0f, 0.0f};

    if (mine > 0) {
        // A step is one row group of one chunk: chunk st / mine, group st % mine.  Its weights are loaded SK_AHEAD
        // steps ahead.  (Measured on 512 experts x 10 pairs: two to eight steps ahead, or the next chunk's B operands
        // loaded early, cost a wave per SIMD in registers and were 5 - 25 % slower; the weight stream alone, without
        // the products, takes two thirds of the kernel's time.)
        const int n_steps = n_chunk * mine;
        auto load_step = [&](int st) __attribute__((always_inline)) -> RawW {
            RawW o;
            const int c = st / mine, g = st - c * mine;
            const int64_t row = min((g0 + g) * 16 + r16, p.n_out - 1);
            const int u = 8 * c + kg;
#pragma unroll
            for (int h = 0; h < 2; h++) {
                o.nib[h] = *(const uint4*)(wq + row * (n_in >> 1) + (u + 4 * h) * 16);
                o.sc[h] = *(const uint16_t*)(ws + row * (n_in >> 4) + (u + 4 * h) * 2);
            }
            return o;
        };
        RawW q[SK_AHEAD];
#pragma unroll
        for (int d = 0; d < SK_AHEAD; d++) q[d] = load_step(min(d, n_steps - 1));
        uint4 nh[8], nl[8];
        auto load_b = [&](int c) __attribute__((always_inline)) {
#pragma unroll
            for (int n = 0; n < 8; n++) {
                nh[n] = *(const uint4*)(bh + c * SK_KC + 128 * (n >> 2) + 8 * (n & 3));
                nl[n] = *(const uint4*)(bl + c * SK_KC + 128 * (n >> 2) + 8 * (n & 3));
            }
        };
        load_b(0);
        int st = 0;
        for (int c = 0; c < n_chunk; c++) {
            h8 fh[8], fl[8];
            if (c > 0) load_b(c);
#pragma unroll
            for (int n = 0; n < 8; n++) {
                fh[n] = __builtin_bit_cast(h8, nh[n]);
                fl[n] = __builtin_bit_cast(h8, nl[n]);
            }
            // the groups of a chunk, unrolled so that the sums are indexed by constants
#pragma unroll
            for (int g = 0; g < SK_G; g++) {
                if (g < mine) {
                    const RawW cur = q[0];
                    const RawW nx = load_step(min(st + SK_AHEAD, n_steps - 1));
#pragma unroll
                    for (int d = 0; d + 1 < SK_AHEAD; d++) q[d] = q[d + 1];
                    q[SK_AHEAD - 1] = nx;
#pragma unroll
                    for (int n = 0; n < 8; n++) {
                        const h8 a = expand_frag(cur.nib[n >> 2], cur.sc[n >> 2], n & 3);
                        acc[g] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, fh[n], acc[g], 0, 0, 0);
                        acc[g] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, fl[n], acc[g], 0, 0, 0);
                    }
                    st++;
                }
            }
        }
    }
    if (GLU) {
        if (z == 1) {
#pragma unroll
            for (int g = 0; g < SK_G; g++)
                handoff[(wslot * SK_G + g) * 64 + lane] = make_float4(acc[g][0], acc[g][1], acc[g][2], acc[g][3]);
        }
        __syncthreads();
        if (z == 1) return;
    }
    if (r16 >= cnt) return;
    const float rsc = p.rscale[xrow];
    const float e2a = p.scale2 ? p.scale2[e] : 1.0f;
    const float e2b = GLU ? (p.scale2_up ? p.scale2_up[e] : 1.0f) : e2a;
#pragma unroll
    for (int g = 0; g < SK_G; g++) {
        if (g >= mine) break;
        const int row = (g0 + g) * 16 + 4 * kg;
        if (row >= p.n_out) continue;
        float o[4];
        if (GLU) {
            const float4 up = handoff[(wslot * SK_G + g) * 64 + lane];
            const float u4[4] = {up.x, up.y, up.z, up.w};
#pragma unroll
            for (int i = 0; i < 4; i++) o[i] = fx_silu(acc[g][i] * rsc * e2a) * (u4[i] * rsc * e2b);
        } else {
#pragma unroll
            for (int i = 0; i < 4; i++) o[i] = acc[g][i] * rsc * e2a;
        }
        *(float4*)(p.out + (int64_t)pair * p.n_out + row) = make_float4(o[0], o[1], o[2], o[3]);
    }
}


// The same products with the k range split over the waves of a block.  Above, a wave walks one 128-byte column of its
// rows chunk after chunk, so every DRAM page is opened once per chunk and the stream stops at 3.5 TB/s.  Here the KW
// waves of a row set take one 256-wide chunk EACH (n_in = 256 KW, KW = 1, 2, 4 or 8) and walk the same row groups
// together: the block reads whole rows at a time, a wave's B operands are loaded once for the whole kernel, and both
// matrices of the gate/up pair share them.  The price is a reduction of the KW partial sums of every 16 x 16 tile
// through LDS: a batch of four tiles per wave (two row groups of gate and up, or four of one matrix), one barrier per
// batch, two LDS buffers in turn.
template <bool GLU, int KW>
__global__ __launch_bounds__(512) void experts_f16k_k(ExpertsF16P p, int batches_per_block) {
    constexpr int NM = GLU ? 2 : 1;
    constexpr int GB = 4 / NM;        // row groups per batch
    constexpr int RS = 8 / KW;        // row sets per block
    __shared__ float4 red[2][8][4][64];   // [buffer][wave][tile of the batch][lane]
    const int tile = blockIdx.x;
    if (tile >= *p.n_tiles) return;
    const int4 td = p.tiles[tile];
    const int64_t e = td.x;
    const int cnt = td.z;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int kw = wave % KW, rs = wave / KW;
    const int r16 = lane & 15, kg = lane >> 4;
    const int n_in = p.n_in, n_groups = (p.n_out + 15) / 16;
    const int pair = p.order[td.y + min(r16, cnt - 1)];
    const int xrow = p.x_mode == 0 ? pair : (p.x_mode == 1 ? pair / p.n_used : 0);
    const uint8_t* wq[2] = {it_expert_at(p.q, p.q_tab, e, p.q_stride), GLU ? it_expert_at(p.q2, p.q2_tab, e, p.q_stride) : nullptr};
    const uint8_t* ws[2] = {it_expert_at(p.s, p.s_tab, e, p.s_stride), GLU ? it_expert_at(p.s2, p.s2_tab, e, p.s_stride) : nullptr};

    // step st = batch i, group slot j, matrix z of this wave: i = st / 4, (j, z) = st % 4
    const int n_steps = batches_per_block * 4;
    auto group_of = [&](int st) { return ((blockIdx.y * batches_per_block + st / 4) * RS + rs) * GB + (st % 4) / NM; };
    // (the matrix z is passed as a constant of the unrolled code: a pointer picked by a run-time index stops being a
    // global pointer for the compiler, and its loads become flat loads that every wait has to drain)
    auto load_step = [&](int st, int z) __attribute__((always_inline)) -> RawW {
        RawW o;
        const int64_t row = min(group_of(st) * 16 + r16, p.n_out - 1);
        // units 2 kg and 2 kg + 1 of the chunk: the four lanes of a row read its 128-byte line between them, and a
        // lane's four scale bytes are one load (two-byte loads, eight bytes per row, cost a quarter of the stream's time)
        const int u = 8 * kw + 2 * kg;
        o.nib[0] = *(const uint4*)(wq[z] + row * (n_in >> 1) + u * 16);
        o.nib[1] = *(const uint4*)(wq[z] + row * (n_in >> 1) + u * 16 + 16);
        o.sc[0] = *(const uint32_t*)(ws[z] + row * (n_in >> 4) + u * 2);   // unit 2 kg in the low half, 2 kg + 1 above
        o.sc[1] = 0;
        return o;
    };
    // Four register sets, one per step of a batch: step t computes from set t while the load of step t + 3 goes
    // straight into set (t + 3) % 4.  No set is ever copied (a copy of a load's destination waits for the load) and
    // the load is unconditional (past the end it repeats the last step), so the compiler's wait before a step counts
    // exactly the loads issued after the ones it needs.
    constexpr int QD = GLU ? 2 : 4;
    RawW q[QD];
    q[0] = load_step(0, 0);
    if (QD == 4) {
        q[1] = load_step(1, GLU ? 1 : 0);
        q[2] = load_step(2, 0);
    }
    // this wave's B operands: chunk kw of the tile's 16 pairs, for the whole kernel
    h8 fh[8], fl[8];
    {
        const uint16_t* bh = p.xh + (int64_t)xrow * n_in + kw * SK_KC + 64 * kg;
        const uint16_t* bl = p.xl + (int64_t)xrow * n_in + kw * SK_KC + 64 * kg;
#pragma unroll
        for (int n = 0; n < 8; n++) {
            fh[n] = __builtin_bit_cast(h8, *(const uint4*)(bh + 8 * n));
            fl[n] = __builtin_bit_cast(h8, *(const uint4*)(bl + 8 * n));
        }
    }
    const float rsc = p.rscale[xrow];
    const float e2a = p.scale2 ? p.scale2[e] : 1.0f;
    const float e2b = GLU ? (p.scale2_up ? p.scale2_up[e] : 1.0f) : e2a;

    for (int i = 0; i < batches_per_block; i++) {
        const int buf = i & 1;
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const int st = 4 * i + t;
            q[(t + QD - 1) % QD] = load_step(min(st + QD - 1, n_steps - 1), GLU ? (t + QD - 1) & 1 : 0);
            __builtin_amdgcn_sched_barrier(0);   // the loads stay ahead of the step they overlap
            v4f acc = v4f{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int n = 0; n < 8; n++) {
                const h8 a = expand_frag(q[t % QD].nib[n >> 2], n < 4 ? q[t % QD].sc[0] : q[t % QD].sc[0] >> 16, n & 3);
                acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, fh[n], acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, fl[n], acc, 0, 0, 0);
            }
            red[buf][wave][t][lane] = make_float4(acc[0], acc[1], acc[2], acc[3]);
        }
        __syncthreads();
        // group slot j of the batch is finished by the wave kw == j % KW of its row set: the KW partial sums of its
        // tile (of both tiles for the gate/up pair), the epilogue and the store
#pragma unroll
        for (int j = 0; j < GB; j++) {
            if (j % KW != kw) continue;
            const int g = group_of(4 * i + j * NM);
            const int row = g * 16 + 4 * kg;
            if (g >= n_groups || row >= p.n_out || r16 >= cnt) continue;
            float sum[NM][4];
#pragma unroll
            for (int z = 0; z < NM; z++) {
                sum[z][0] = sum[z][1] = sum[z][2] = sum[z][3] = 0.0f;
#pragma unroll
                for (int k = 0; k < KW; k++) {
                    const float4 v = red[buf][rs * KW + k][j * NM + z][lane];
                    sum[z][0] += v.x; sum[z][1] += v.y; sum[z][2] += v.z; sum[z][3] += v.w;
                }
            }
            float o[4];
#pragma unroll
            for (int q = 0; q < 4; q++) {
                if (GLU) o[q] = fx_silu(sum[0][q] * rsc * e2a) * (sum[NM - 1][q] * rsc * e2b);
                else o[q] = sum[0][q] * rsc * e2a;
            }
            *(float4*)(p.out + (int64_t)pair * p.n_out + row) = make_float4(o[0], o[1], o[2], o[3]);
        }
    }
}

}  // namespace

bool experts_f16s_takes(const ExpertsView& w, const ExpertsView* up, int n_picks, const int8_t* act_quants, const float* out) {
    if (n_picks < 32 || w.n_expert > 1024 || w.fmt != W_NVFP4 || w.n_in % SK_KC || w.n_out % 4) return false;
    if ((reinterpret_cast<uintptr_t>(w.q) & 15) || w.q_stride % 16 || w.s_stride % 2 || (reinterpret_cast<uintptr_t>(w.scales) & 1) ||
        (reinterpret_cast<uintptr_t>(act_quants) & 3) || (reinterpret_cast<uintptr_t>(out) & 15))
        return false;
    if (up && (up->fmt != w.fmt || up->n_in != w.n_in || up->n_out != w.n_out || (reinterpret_cast<uintptr_t>(up->q) & 15) ||
               (reinterpret_cast<uintptr_t>(up->scales) & 1) || up->q_stride != w.q_stride || up->s_stride != w.s_stride))
        return false;
    return true;
}

bool experts_gemm_f16s(const ExpertsView& w, const ExpertsView* up, const int32_t* ids, int n_picks, int n_used,
                       int x_mode, const float* act_scales, const int8_t* act_quants, float* out, int32_t* work,
                       size_t work_ints, void* fwork, size_t fwork_bytes, bool grouped, hipStream_t s) {
    if (!work || !fwork || !experts_f16s_takes(w, up, n_picks, act_quants, out)) return false;
    if (n_used < 1) n_used = 1;
    const int x_rows = x_mode == 0 ? n_picks : (x_mode == 1 ? (n_picks + n_used - 1) / n_used : 1);
    if (work_ints < experts_group_work_ints(n_picks, w.n_expert) || fwork_bytes < experts_f16_work_bytes(x_rows, w.n_in)) return false;
    // the layout of the int8 tile kernel's grouping (tiles of 16 pairs): either may reuse the other's
    const int max_tiles = w.n_expert + n_picks / SK_PAIRS + 1;
    int32_t* n_tiles = work;
    int4* tiles = (int4*)(work + 16);
    int32_t* order = work + 16 + (size_t)(max_tiles + 1) * 4;
    if (!grouped) moe_group(ids, n_picks, w.n_expert, SK_PAIRS, n_tiles, tiles, order, s);
    uint16_t* xh = (uint16_t*)fwork;
    uint16_t* xl = xh + (size_t)x_rows * w.n_in;
    float* rscale = (float*)(xl + (size_t)x_rows * w.n_in);
    hipLaunchKernelGGL(acts_split_perm_k, dim3(x_rows), dim3(256), 0, s, act_quants, act_scales, w.n_in, xh, xl, rscale);
    ExpertsF16P p{};
    p.q = (const uint8_t*)w.q;
    p.s = (const uint8_t*)w.scales;
    p.q2 = up ? (const uint8_t*)up->q : nullptr;
    p.s2 = up ? (const uint8_t*)up->scales : nullptr;
    p.q_stride = w.q_stride;
    p.s_stride = w.s_stride;
    p.q_tab = w.q_tab;
    p.s_tab = w.s_tab;
    p.q2_tab = up ? up->q_tab : nullptr;
    p.s2_tab = up ? up->s_tab : nullptr;
    p.scale2 = w.scale2;
    p.scale2_up = up ? up->scale2 : nullptr;
    p.xh = xh;
    p.xl = xl;
    p.rscale = rscale;
    p.out = out;
    p.n_in = w.n_in;
    p.n_out = w.n_out;
    p.x_mode = x_mode;
    p.n_used = n_used;
    p.n_tiles = n_tiles;
    p.tiles = tiles;
    p.order = order;
    const int groups = (w.n_out + 15) / 16;
    const int likely_tiles = std::min(n_picks, w.n_expert) + n_picks / SK_PAIRS;
    const int n_chunk = w.n_in / SK_KC;
    if (n_chunk == 1 || n_chunk == 2 || n_chunk == 4 || n_chunk == 8) {
        // k split over the waves: a batch is 4 / NM row groups per row set, 8 / n_chunk row sets per block; 8 batches
        // per block while that leaves about 1,024 blocks (16 or 32 batches measured 10 % slower, 4 the same)
        const int per_batch = (up ? 2 : 4) * (8 / n_chunk);
        const int batches = (groups + per_batch - 1) / per_batch;
        int bpb = std::min(batches, 8);
        while (bpb > 1 && (int64_t)likely_tiles * ((batches + bpb - 1) / bpb) < 1024) bpb >>= 1;
        const dim3 grid(std::min(n_picks, max_tiles), (batches + bpb - 1) / bpb);
#define IT_F16K(G, K) hipLaunchKernelGGL((experts_f16k_k<G, K>), grid, dim3(512), 0, s, p, bpb)
        if (up) {
            if (n_chunk == 8) IT_F16K(true, 8); else if (n_chunk == 4) IT_F16K(true, 4); else if (n_chunk == 2) IT_F16K(true, 2); else IT_F16K(true, 1);
        } else {
            if (n_chunk == 8) IT_F16K(false, 8); else if (n_chunk == 4) IT_F16K(false, 4); else if (n_chunk == 2) IT_F16K(false, 2); else IT_F16K(false, 1);
        }
#undef IT_F16K
        return true;
    }
    // other row lengths: every wave walks the whole k range of its own rows
    int gpw = SK_G;
    const int wpb = up ? 2 : 4;   // shares of a block's row groups (the gate/up pair puts two waves on each)
    while (gpw > 1 && (int64_t)likely_tiles * ((groups + wpb * gpw - 1) / (wpb * gpw)) < 2048) gpw >>= 1;
    const dim3 grid(std::min(n_picks, max_tiles), (groups + wpb * gpw - 1) / (wpb * gpw));
    if (up) hipLaunchKernelGGL(experts_f16s_k<true>, grid, dim3(256), 0, s, p, gpw);
    else hipLaunchKernelGGL(experts_f16s_k<false>, grid, dim3(256), 0, s, p, gpw);
    return true;
}

}  // namespace itk
