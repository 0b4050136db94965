// =====================================================================================
// Expert matmuls for a small batch (fast mode): a few (token, pick) pairs per expert.
//
// Between one token and a few hundred, a batch touches most experts with one to a dozen pairs each.
// One GEMV per pair (k_matmul.hip) reads an expert's weights once per pair; the matrix-core tiles
// (k_gemm.hip, k_gemm_f16.hip) multiply 16 or 32 token slots of which one or two are live.  Here
// the pairs are sorted by expert (moe_group_k, tiles of up to 8 or 16 pairs) and a block streams a
// group of weight rows of ONE expert exactly once, 128 bits per lane, coalesced: a lane
// expands its 32 weights to int8 in registers (E2M1 through byte permutes; Q8_0 as stored) and
// runs the integer dots of naive.rs:691-734 against every pair of the tile, whose Q8_0
// activations sit in LDS.  The per-block terms are the CPU path's; they are summed per lane and
// then across the lanes of a row, so what differs from the CPU result is the f32 summation
// order only.
//
// Lanes: a row of n_in elements has U = n_in / 32 units of 32 elements (NVFP4: 16 nibble bytes
// and two scale bytes; Q8_0: 32 quants and one f16 scale).  L = min(U, 64) lanes share a row,
// 64 / L rows are in flight per wave instruction, and with U > 64 a lane walks units L apart.
// LDS holds the tile's activations split in two planes of 16-byte pieces (first and second half
// of every unit) so that the 64 lanes of a read touch 64 consecutive pieces, the scales, and
// the block's outputs, which leave as full rows at the end.
#include <algorithm>

#include "it_device.h"
#include "it_dot.h"
#include "it_reduce.h"
#include "kernels.h"

namespace itk {
namespace {

struct ExpertRowsP {
    const uint8_t *q, *s, *q2, *s2;
    const uint8_t* const *q_tab, *const *s_tab, *const *q2_tab, *const *s2_tab;  // expert placement tables or null
    int64_t q_stride, s_stride;
    const float *scale2, *scale2_up;
    const float* act_scales;
    const int8_t* act_quants;
    float* out;
    int n_in, n_out, x_mode, n_used, n_pairs, rows_per_block;
    float out_scale;
    const int32_t* n_tiles;   // null: one matrix, tile t holds pairs 8 t .. 8 t + 7 in order
    const int4* tiles;
    const int32_t* order;
};

// the 32 weights of one unit as eight dwords of int8 and the float scale(s) of the unit
template <int FMT>
struct Unit {
    uint32_t w[8];
    float dA, dB;   // NVFP4: the two sub-block scales; Q8_0: dA only
};
template <int FMT>
struct Raw {
    uint4 a, b;     // NVFP4: a only
    uint32_t sc;
};

template <int FMT>
IT_DEV Raw<FMT> load_raw(const uint8_t* wq, const uint8_t* ws, int64_t row, int n_in, int U, int u) {
    Raw<FMT> r;
    if (FMT == W_NVFP4) {
        r.a = *(const uint4*)(wq + row * (n_in >> 1) + u * 16);
        r.b = make_uint4(0, 0, 0, 0);
    } else {
        const uint4* wp = (const uint4*)(wq + row * n_in + u * 32);
        r.a = wp[0];
        r.b = wp[1];
    }
    r.sc = ((const uint16_t*)ws)[row * U + u];
    return r;
}

template <int FMT>
IT_DEV Unit<FMT> expand(const Raw<FMT>& r) {
    Unit<FMT> o;
    if (FMT == W_NVFP4) {
        // the element order of unit_nvfp4: low nibbles of bytes 0..7, then their high nibbles, per sub-block
        o.w[0] = fp4x4_to_i8x4(r.a.x & 0x0f0f0f0fu);
        o.w[1] = fp4x4_to_i8x4(r.a.y & 0x0f0f0f0fu);
        o.w[2] = fp4x4_to_i8x4((r.a.x >> 4) & 0x0f0f0f0fu);
        o.w[3] = fp4x4_to_i8x4((r.a.y >> 4) & 0x0f0f0f0fu);
        o.w[4] = fp4x4_to_i8x4(r.a.z & 0x0f0f0f0fu);
        o.w[5] = fp4x4_to_i8x4(r.a.w & 0x0f0f0f0fu);
        o.w[6] = fp4x4_to_i8x4((r.a.z >> 4) & 0x0f0f0f0fu);
        o.w[7] = fp4x4_to_i8x4((r.a.w >> 4) & 0x0f0f0f0fu);
        o.dA = it_ue4m3_to_f32(r.sc & 0xffu);
        o.dB = it_ue4m3_to_f32((r.sc >> 8) & 0xffu);
    } else {
        o.w[0] = r.a.x; o.w[1] = r.a.y; o.w[2] = r.a.z; o.w[3] = r.a.w;
        o.w[4] = r.b.x; o.w[5] = r.b.y; o.w[6] = r.b.z; o.w[7] = r.b.w;
        o.dA = it_f16_to_f32((uint16_t)r.sc);
        o.dB = 0.0f;
    }
    return o;
}

// one unit against one pair's activation block (a0: elements 0..15, a1: 16..31) with scale dx, added to acc
template <int FMT>
IT_DEV float unit_term(const Unit<FMT>& w, const uint4 a0, const uint4 a1, float dx, float acc) {
    int sa = 0, sb = 0;
    sa = dot4(w.w[0], a0.x, sa); sa = dot4(w.w[1], a0.y, sa); sa = dot4(w.w[2], a0.z, sa); sa = dot4(w.w[3], a0.w, sa);
    sb = dot4(w.w[4], a1.x, sb); sb = dot4(w.w[5], a1.y, sb); sb = dot4(w.w[6], a1.z, sb); sb = dot4(w.w[7], a1.w, sb);
    if (FMT == W_NVFP4) return fmaf((float)sa, dx * w.dA, fmaf((float)sb, dx * w.dB, acc));
    return fmaf((float)(sa + sb), w.dA * dx, acc);
}

template <int FMT, bool GLU, int L, int RP>
__global__ __launch_bounds__(256) void expert_rows_k(ExpertRowsP p) {
    extern __shared__ __align__(16) uint8_t lds_raw[];
    __shared__ int pair_s[RP], xrow_s[RP];
    const int tile = blockIdx.y;
    int64_t e = 0;
    int first = tile * RP, cnt;
    if (p.n_tiles) {
        if (tile >= *p.n_tiles) return;
        const int4 td = p.tiles[tile];
        e = td.x;
        first = td.y;
        cnt = td.z;
    } else {
        cnt = min(RP, p.n_pairs - first);
        if (cnt <= 0) return;
    }
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n_in = p.n_in, U = n_in >> 5, RB = p.rows_per_block;
    constexpr int RPI = 64 / L;          // rows per wave instruction
    const int sub = lane / L, ul = lane % L;
    const int upl = U / L;               // units per lane and row
    const uint8_t* wq = it_expert_at(p.q, p.q_tab, e, p.q_stride);
    const uint8_t* ws = it_expert_at(p.s, p.s_tab, e, p.s_stride);
    const uint8_t* wq2 = GLU ? it_expert_at(p.q2, p.q2_tab, e, p.q_stride) : nullptr;
    const uint8_t* ws2 = GLU ? it_expert_at(p.s2, p.s2_tab, e, p.s_stride) : nullptr;
    const int row_lo = blockIdx.x * RB, row_hi = min(row_lo + RB, p.n_out);
    // rows row_lo + RPI * (wave + 4 i) + sub; a row past the end repeats the last one and is not stored.
    // A step is one unit of one row: steps i * upl .. i * upl + upl - 1 walk row i's units L apart.
    const int n_iter = (row_hi - row_lo + 4 * RPI - 1) / (4 * RPI);
    const int n_steps = n_iter * upl;
    auto row_of = [&](int i) { return row_lo + RPI * (wave + 4 * i) + sub; };
    struct Both { Raw<FMT> a, b; };
    auto load_step = [&](int st) __attribute__((always_inline)) -> Both {
        Both o;
        const int i = st / upl, u = ul + (st - i * upl) * L;
        const int64_t r = min(row_of(i), p.n_out - 1);
        o.a = load_raw<FMT>(wq, ws, r, n_in, U, u);
        if (GLU) o.b = load_raw<FMT>(wq2, ws2, r, n_in, U, u);
        return o;
    };
    // the first step's weights are on their way while the activations are staged
    Both q0 = load_step(0), q1 = q0;

    uint8_t* xq = lds_raw;                                   // [RP][2][U][16]
    float* xs = (float*)(lds_raw + (size_t)RP * n_in);        // [RP][U]
    float* outs = xs + (size_t)RP * U;                        // [GLU ? 2 : 1][RP][RB]: the row sums
    float* outs2 = outs + (size_t)RP * RB;
    if (tid < RP) {
        const int slot = first + min(tid, cnt - 1);
        const int pair = p.order ? p.order[slot] : slot;
        pair_s[tid] = pair;
        xrow_s[tid] = p.x_mode == 0 ? pair : (p.x_mode == 1 ? pair / p.n_used : 0);
    }
    __syncthreads();
    {
        const int pieces = n_in >> 4;   // 16-byte pieces per row
        for (int i = tid; i < cnt * pieces; i += 256) {
            const int pp = i / pieces, j = i - pp * pieces;
            const uint4 v = *(const uint4*)(p.act_quants + (int64_t)xrow_s[pp] * n_in + j * 16);
            *(uint4*)(xq + (size_t)pp * n_in + (size_t)(j & 1) * (n_in >> 1) + (j >> 1) * 16) = v;
        }
        for (int i = tid; i < cnt * U; i += 256) {
            const int pp = i / U, j = i - pp * U;
            xs[pp * U + j] = p.act_scales[(int64_t)xrow_s[pp] * U + j];
        }
    }
    __syncthreads();

    float acc[RP], acc2[RP];
    auto step = [&](int st, const Both& raw) __attribute__((always_inline)) {
        const int i = st / upl, j = st - i * upl, u = ul + j * L;
        if (j == 0) {
#pragma unroll
            for (int pp = 0; pp < RP; pp++) acc[pp] = acc2[pp] = 0.0f;
        }
        const Unit<FMT> w = expand<FMT>(raw.a);
        Unit<FMT> w2;
        if (GLU) w2 = expand<FMT>(raw.b);
#pragma unroll
        for (int pp = 0; pp < RP; pp++) {
            if (pp < cnt) {
                const uint4 a0 = *(const uint4*)(xq + (size_t)pp * n_in + u * 16);
                const uint4 a1 = *(const uint4*)(xq + (size_t)pp * n_in + (n_in >> 1) + u * 16);
                const float dx = xs[pp * U + u];
                acc[pp] = unit_term<FMT>(w, a0, a1, dx, acc[pp]);
                if (GLU) acc2[pp] = unit_term<FMT>(w2, a0, a1, dx, acc2[pp]);
            }
        }
        if (j == upl - 1) {
            const int row = row_of(i);
            const bool keep = ul == L - 1 && row < row_hi;
#pragma unroll
            for (int pp = 0; pp < RP; pp++) {
                if (pp < cnt) {
                    const float g = group_sum_tail<L>(acc[pp]);
                    if (keep) outs[pp * RB + (row - row_lo)] = g;
                    if (GLU) {
                        const float uu = group_sum_tail<L>(acc2[pp]);
                        if (keep) outs2[pp * RB + (row - row_lo)] = uu;
                    }
                }
            }
        }
    };
    // Two register sets in turn: while a step computes from one, the next step's load goes straight into the other.
    // No set is copied (a copy of a load's destination waits for the load), the load is unconditional (past the end it
    // repeats the last step) and pinned ahead of the step it overlaps, so the wait before a step counts exactly the
    // loads issued after the ones it needs.
    for (int st = 0; st < n_steps; st += 2) {
        q1 = load_step(min(st + 1, n_steps - 1));
        __builtin_amdgcn_sched_barrier(0);
        step(st, q0);
        q0 = load_step(min(st + 2, n_steps - 1));
        __builtin_amdgcn_sched_barrier(0);
        if (st + 1 < n_steps) step(st + 1, q1);
    }
    __syncthreads();
    const float e2a = p.scale2 ? p.scale2[e] : 1.0f;
    const float e2b = GLU ? (p.scale2_up ? p.scale2_up[e] : 1.0f) : 1.0f;
    const int nr = row_hi - row_lo;
    for (int i = tid; i < cnt * nr; i += 256) {
        const int pp = i / nr, r = i - pp * nr;
        float v = outs[pp * RB + r] * e2a;
        if (GLU) v = fx_silu(v) * (outs2[pp * RB + r] * e2b);
        else if (p.out_scale != 1.0f) v *= p.out_scale;
        p.out[(int64_t)pair_s[pp] * p.n_out + row_lo + r] = v;
    }
}

template <int FMT, bool GLU, int RP>
bool launch_rows(const ExpertRowsP& p, int max_tiles, hipStream_t s) {
    const int U = p.n_in >> 5;
    const int L = U >= 64 ? 64 : U;
    const int gx = (p.n_out + p.rows_per_block - 1) / p.rows_per_block;
    const size_t lds = (size_t)RP * p.n_in + (size_t)RP * U * 4 + (size_t)(GLU ? 2 : 1) * RP * p.rows_per_block * 4;
    if (lds > 64 * 1024) return false;   // more than a launch gets without asking: the caller takes another kernel
    const dim3 grid(gx, max_tiles), block(256);
    switch (L) {
        case 64: hipLaunchKernelGGL((expert_rows_k<FMT, GLU, 64, RP>), grid, block, lds, s, p); return true;
        case 32: hipLaunchKernelGGL((expert_rows_k<FMT, GLU, 32, RP>), grid, block, lds, s, p); return true;
        case 16: hipLaunchKernelGGL((expert_rows_k<FMT, GLU, 16, RP>), grid, block, lds, s, p); return true;
        case 8: hipLaunchKernelGGL((expert_rows_k<FMT, GLU, 8, RP>), grid, block, lds, s, p); return true;
        default: return false;
    }
}

}  // namespace

// pairs per tile: 16 once the experts hold four pairs and more on average (and the activations fit LDS), else 8
int expert_rows_tile(int n_picks, int n_expert, int n_in) {
    return (int64_t)n_picks >= 4 * (int64_t)n_expert && n_in <= 2048 ? 16 : 8;
}

bool expert_rows_takes(const ExpertsView& w, const ExpertsView* up, const int8_t* act_quants) {
    if (w.fmt != W_Q8_0 && w.fmt != W_NVFP4) return false;
    const int U = w.n_in >> 5;
    if (w.n_in % 32 || U < 8 || (U < 64 && (U & (U - 1))) || (U > 64 && U % 64) || w.n_in > 4096 || w.n_expert > 1024)
        return false;
    auto al = [](const void* q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
    if (!al(w.q) || w.q_stride % 16 || w.s_stride % 2 || (reinterpret_cast<uintptr_t>(w.scales) & 1) || !al(act_quants))
        return false;
    if (up && (up->fmt != w.fmt || up->n_in != w.n_in || up->n_out != w.n_out || !al(up->q) ||
               (reinterpret_cast<uintptr_t>(up->scales) & 1) || up->q_stride != w.q_stride || up->s_stride != w.s_stride))
        return false;
    return true;
}

bool expert_rows(const ExpertsView& w, const ExpertsView* up, const int32_t* ids, int n_picks, int n_used, int x_mode,
                 const float* act_scales, const int8_t* act_quants, float* out, float out_scale, int32_t* work,
                 size_t work_ints, bool grouped, hipStream_t s) {
    if (n_picks <= 0 || !expert_rows_takes(w, up, act_quants)) return false;
    ExpertRowsP p{};
    const int RP = ids ? expert_rows_tile(n_picks, w.n_expert, w.n_in) : (n_picks >= 64 && w.n_in <= 2048 ? 16 : 8);
    int max_tiles;
    if (ids) {
        if (!work || work_ints < experts_group_work_ints(n_picks, w.n_expert)) return false;
        max_tiles = std::min(n_picks, w.n_expert + n_picks / RP + 1);
        const int layout_tiles = w.n_expert + n_picks / RP + 1;
        int32_t* n_tiles = work;
        int4* tiles = (int4*)(work + 16);
        int32_t* order = work + 16 + (size_t)(layout_tiles + 1) * 4;
        if (!grouped) moe_group(ids, n_picks, w.n_expert, RP, n_tiles, tiles, order, s);
        p.n_tiles = n_tiles;
        p.tiles = tiles;
        p.order = order;
    } else {
        max_tiles = (n_picks + RP - 1) / RP;
    }
    p.q = (const uint8_t*)w.q;
    p.s = (const uint8_t*)w.scales;
    p.q2 = up ? (const uint8_t*)up->q : nullptr;
    p.s2 = up ? (const uint8_t*)up->scales : nullptr;
    p.q_stride = ids ? w.q_stride : 0;
    p.s_stride = ids ? w.s_stride : 0;
    p.q_tab = ids ? w.q_tab : nullptr;
    p.s_tab = ids ? w.s_tab : nullptr;
    p.q2_tab = ids && up ? up->q_tab : nullptr;
    p.s2_tab = ids && up ? up->s_tab : nullptr;
    p.scale2 = w.scale2;
    p.scale2_up = up ? up->scale2 : nullptr;
    p.act_scales = act_scales;
    p.act_quants = act_quants;
    p.out = out;
    p.n_in = w.n_in;
    p.n_out = w.n_out;
    p.x_mode = x_mode;
    p.n_used = n_used < 1 ? 1 : n_used;
    p.n_pairs = n_picks;
    p.out_scale = out_scale;
    // rows per block: a multiple of the rows four waves hold in flight; about 2048 blocks when the batch allows it
    const int U = w.n_in >> 5, rpi = 64 / (U >= 64 ? 64 : U), step = 4 * rpi;
    int rb = w.n_out;
    const int likely_tiles = ids ? std::min(n_picks, w.n_expert) + n_picks / RP : max_tiles;
    while (rb > 4 * step && (int64_t)likely_tiles * ((w.n_out + rb - 1) / rb) < 2048) rb = (rb / 2 + step - 1) / step * step;
    rb = std::max(step, std::min(rb, 256));
    const bool glu = up != nullptr;
    // the block's LDS (the tile's activations and scales, then its outputs) stays within what a launch gets unasked
    auto lds_of = [&](int rows) { return (size_t)RP * w.n_in + (size_t)RP * U * 4 + (size_t)(glu ? 2 : 1) * RP * rows * 4; };
    while (rb > step && lds_of(rb) > 64 * 1024) rb -= step;
    p.rows_per_block = rb;
#define IT_ROWS(F, G, R) launch_rows<F, G, R>(p, max_tiles, s)
    if (w.fmt == W_Q8_0) {
        if (RP == 16) return glu ? IT_ROWS(W_Q8_0, true, 16) : IT_ROWS(W_Q8_0, false, 16);
        return glu ? IT_ROWS(W_Q8_0, true, 8) : IT_ROWS(W_Q8_0, false, 8);
    }
    if (RP == 16) return glu ? IT_ROWS(W_NVFP4, true, 16) : IT_ROWS(W_NVFP4, false, 16);
    return glu ? IT_ROWS(W_NVFP4, true, 8) : IT_ROWS(W_NVFP4, false, 8);
#undef IT_ROWS
}

}  // namespace itk
