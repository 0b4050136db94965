// =====================================================================================
// NVFP4 expert matmuls on the f16 matrix cores (fast mode).
//
// An NVFP4 weight is (doubled e2m1 value) x (halved e4m3 sub-block scale): at most six significant
// bits, so it is EXACT in f16, and so is every product with an f16 activation in the f32
// accumulator.  The Q8_0 activation x = q * dx is divided by a power of two that brings its row
// into [-1, 1] and split into two f16 numbers (x = hi + lo, 22 bits kept); the power of two comes
// back in the epilogue.  With the scales inside the operands the whole k range accumulates in the
// MFMA accumulator: no per-block scaling on the vector ALU, which bounds the int8 kernels above.
// What differs from the CPU path is the f32 summation order and the 2^-22 of the split.
//
// A block owns one tile of up to 128 (token, pick) pairs of one expert and 128 rows of the
// gate AND up matrices (GLU) or 256 rows of one matrix, with eight waves.  A wave owns two sets of
// 32 rows (gate and up rows of the same index, or two row groups) and half of the token tiles
// (waves 0-3 the first one or two groups of 32 pairs, waves 4-7 the next), so a token fragment
// read from LDS feeds four MFMAs (two sets, hi and lo) and the f32 sums of a wave stay within the
// registers that two waves per SIMD leave.  Weight nibbles go through LDS as full 128-byte lines to
// the owning lane's registers (a lane owns 16 contiguous bytes of a row per 64-wide k slab: the
// k order inside an MFMA is free once the scales are folded in) and are expanded there: a byte
// permute yields the f16 high bytes of four magnitudes, the sign bit is or-ed in, two more
// permutes interleave zero low bytes, and v_pk_mul_f16 applies the sub-block scale (the scale code's bits moved
// into an f16's fields are the scale times 2^-8; the magnitudes are stored times 2^7, which also takes the halving).
//
// MFMA operand layout (32x32x16, f16): lane l supplies 8 k values of row (l % 32), k group
// l / 32, for both A (weight rows) and B (tokens); it receives D for token l % 32 and weight
// rows 8 * (i / 4) + 4 * (l / 32) + i % 4, i = 0..15.
#include "it_device.h"
#include "it_dot.h"
#include "kernels.h"

// Phase stamps for tuning: a build with -DIT_STAMPS records the 100 MHz wall clock of one block's first
// lane at the marked points of five consecutive k slabs; the library build compiles them away.
#ifdef IT_STAMPS
__device__ long long it_gemm_stamps[32];
__device__ int it_gemm_stamp_tile, it_gemm_stamp_slab, it_gemm_stamp_glu;
// (five consecutive slabs of one block, six stamps each)
#define GEMM_STAMP(i)                                                                                                  \
    do {                                                                                                               \
        if ((int)blockIdx.x == it_gemm_stamp_tile && (GLU ? 1 : 0) == it_gemm_stamp_glu && s >= it_gemm_stamp_slab && \
            s < it_gemm_stamp_slab + 5 && tid == 0)                                                                    \
            it_gemm_stamps[6 * (s - it_gemm_stamp_slab) + (i)] = wall_clock64();                                       \
    } while (0)
#else
#define GEMM_STAMP(i) \
    do {              \
    } while (0)
#endif

namespace itk {
namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));
constexpr int FK = 64;          // k per slab
constexpr int FBS = FK + 4;     // LDS row stride of a token slab, in f16 (136 bytes: no bank is hit twice by 16 lanes)
constexpr int FPAIRS = 128;     // pairs per tile
constexpr int FSUPER = 256;     // k per weight staging step (one 128-byte line of nibbles per row)
constexpr int FWS = 128 + 16;   // LDS row stride of a weight segment, in bytes

// rows of f16 hi / lo and the row's power of two, from Q8_0 quants and scales
__global__ __launch_bounds__(256) void acts_split_f16_k(const int8_t* __restrict__ q, const float* __restrict__ sc,
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
        ((uint2*)(xh + (int64_t)row * n_in))[i] = make_uint2(h[0] | ((uint32_t)h[1] << 16), h[2] | ((uint32_t)h[3] << 16));
        ((uint2*)(xl + (int64_t)row * n_in))[i] = make_uint2(l[0] | ((uint32_t)l[1] << 16), l[2] | ((uint32_t)l[3] << 16));
    }
}


template <bool GLU, int T>
__device__ __forceinline__ void experts_f16_body(const ExpertsF16P& p, const int4 td, const int row_block, uint16_t* Bh, uint16_t* Bl,
                                                 uint8_t* Wn, uint8_t* Wsc, const int* xrow_s, const int* pair_s) {
    const int64_t e = td.x;
    const int cnt = td.z;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave8 = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave = wave8 & 3;      // which 32 (GLU) or 64 rows of the block
    const int th = wave8 >> 2;       // which half of the tile's token groups: T groups each
    const int r = lane & 31, kg = lane >> 5;
    const int n_in = p.n_in, nslab = n_in / FK;
    // the two row sets of this wave
    const int rows_per_block = GLU ? 128 : 256;
    const int rb0 = row_block * rows_per_block + (GLU ? 32 : 64) * wave;
    const int rbase[2] = {rb0, GLU ? rb0 : rb0 + 32};
    const uint8_t* wq0 = it_expert_at(p.q, p.q_tab, e, p.q_stride);
    const uint8_t* ws0 = it_expert_at(p.s, p.s_tab, e, p.s_stride);
    const uint8_t* wq[2] = {wq0, GLU ? it_expert_at(p.q2, p.q2_tab, e, p.q_stride) : wq0};
    const uint8_t* ws[2] = {ws0, GLU ? it_expert_at(p.s2, p.s2_tab, e, p.s_stride) : ws0};
    // this wave's row segments in the block's weight buffer: GLU [set][wave][row], else [wave][set][row]
    const int myseg[2] = {GLU ? 32 * wave + r : 64 * wave + r, GLU ? 128 + 32 * wave + r : 64 * wave + 32 + r};
    // the segments this thread loads (four rows, one 16-byte piece of each row's 128 nibble bytes) and, for the
    // first 256 threads, the segment whose 16 scale bytes it loads
    const int piece = tid & 7;
    const uint8_t* wload[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int seg = (tid >> 3) + 64 * i;
        const int z = GLU ? seg >> 7 : 0;
        const int64_t row = min(row_block * rows_per_block + (GLU ? seg & 127 : seg), p.n_out - 1);
        // (picked by a conditional, not by an index into the array: a pointer that went through an indexed array is a
        // generic pointer to the compiler, and loads through it are flat loads that every LDS wait has to drain)
        wload[i] = (z ? wq[1] : wq[0]) + row * (n_in >> 1) + piece * 16;
    }
    const uint8_t* sload;
    {
        const int st = tid & 255;
        const int z = GLU ? st >> 7 : 0;
        const int64_t row = min(row_block * rows_per_block + (GLU ? st & 127 : st), p.n_out - 1);
        sload = (z ? ws[1] : ws[0]) + row * (n_in >> 4);
    }

    // Software pipeline.  Weights come in super-slabs of 256 k: every thread loads full 128-byte lines of
    // eight rows (coalesced) one super-slab ahead and parks them in the other LDS weight buffer; a lane
    // then reads its own 16 nibble bytes and 2 scale bytes of the NEXT 64-wide slab and expands them to
    // f16 fragments one at a time between the MFMA groups of the current slab.  Tokens run one slab
    // ahead through registers into the other LDS token buffer.  Inside a slab the token fragments of the
    // next MFMA group are read from LDS while the current group is on the matrix unit.  Loads and LDS
    // stores are dealt out between the MFMA groups one or two at a time (loads over the first groups,
    // the stores of what they brought over the later ones), and the slab's one barrier stands in front
    // of its last group.
    const int n_super = n_in / FSUPER;
    uint4 rw[4], rsw;
    uint4 rbh[T], rbl[T];   // 64 * T tokens x 8 segments of 16 bytes = 512 * T segments per array
    rsw = make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int i = 0; i < 4; i++) rw[i] = rsw;
    // the token rows this thread stages: fixed for the whole k loop
    const uint16_t* xhp[T];
    const uint16_t* xlp[T];
#pragma unroll
    for (int u = 0; u < T; u++) {
        const int idx = tid + u * 512, tok = idx >> 3, seg = idx & 7;
        const int64_t at = (int64_t)xrow_s[tok] * n_in + seg * 8;
        xhp[u] = p.xh + at;
        xlp[u] = p.xl + at;
    }
    auto fetch_w = [&](int S) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 4; i++) rw[i] = *(const uint4*)(wload[i] + S * (FSUPER / 2));
        rsw = *(const uint4*)(sload + S * (FSUPER / 16));
    };
    // The same loads one at a time, to be issued between MFMA groups: a burst of 16-byte loads from all four
    // waves backs up the load unit (about 200 cycles an instruction) and the matrix unit idles behind it.
    // q < 2 T: piece q of the next slab's tokens; then the five loads of the next super-slab.
    constexpr int N_LOADS = 2 * T + 5, LPG = (N_LOADS + 4 * T - 1) / (4 * T);
    auto fetch_one = [&](int q, int s_next, int S_next, bool x_on, bool w_on) __attribute__((always_inline)) {
        if (q < 2 * T) {
            if (x_on) {
                if (q & 1) rbl[q >> 1] = *(const uint4*)(xlp[q >> 1] + s_next * FK);
                else rbh[q >> 1] = *(const uint4*)(xhp[q >> 1] + s_next * FK);
            }
        } else if (q < N_LOADS && w_on) {
            const int i = q - 2 * T;
            if (i < 4) rw[i] = *(const uint4*)(wload[i] + S_next * (FSUPER / 2));
            else rsw = *(const uint4*)(sload + S_next * (FSUPER / 16));
        }
    };
    auto stash_w = [&](int b) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 4; i++) *(uint4*)(Wn + (b * 256 + (tid >> 3) + 64 * i) * FWS + piece * 16) = rw[i];
        if (tid < 256) *(uint4*)(Wsc + (b * 256 + tid) * 16) = rsw;
    };
    auto fetch_x = [&](int s) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < T; u++) {
            rbh[u] = *(const uint4*)(xhp[u] + s * FK);
            rbl[u] = *(const uint4*)(xlp[u] + s * FK);
        }
    };
    auto stash_x = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < T; u++) {
            const int idx = tid + u * 512, tok = idx >> 3, seg = idx & 7;
            uint16_t* dh = Bh + (buf * FPAIRS + tok) * FBS + seg * 8;
            uint16_t* dl = Bl + (buf * FPAIRS + tok) * FBS + seg * 8;
            *(uint2*)dh = make_uint2(rbh[u].x, rbh[u].y);
            *(uint2*)(dh + 4) = make_uint2(rbh[u].z, rbh[u].w);
            *(uint2*)dl = make_uint2(rbl[u].x, rbl[u].y);
            *(uint2*)(dl + 4) = make_uint2(rbl[u].z, rbl[u].w);
        }
    };
    // The same stores one at a time, to go between the MFMA groups of the slab's second half: issued together at the
    // slab's end, the stores of all eight waves are a burst that the LDS works off while no wave has a product to issue,
    // and every wave's first read of the next slab queues behind it (measured with the stores, or the barrier behind
    // them, taken out: a third of the kernel's time).
    // (one address register per staged row: buffer, hi / lo half and part are constant offsets from it; Bl lies
    // 2 * FPAIRS * FBS behind Bh)
    uint16_t* xdst[T];
#pragma unroll
    for (int u = 0; u < T; u++) {
        const int idx = tid + u * 512;
        xdst[u] = Bh + (idx >> 3) * FBS + (idx & 7) * 8;
    }
    auto stash_x_part = [&](int buf, int i) __attribute__((always_inline)) {   // i < 4 T
        const int u = i >> 2, part = i & 3;
        uint16_t* d = xdst[u] + buf * FPAIRS * FBS + (part < 2 ? 0 : 2 * FPAIRS * FBS) + 4 * (part & 1);
        const uint4 v = part < 2 ? rbh[u] : rbl[u];
        *(uint2*)d = (part & 1) ? make_uint2(v.z, v.w) : make_uint2(v.x, v.y);
    };
    auto stash_w_part = [&](int b, int i) __attribute__((always_inline)) {   // i < 5
        // (the register set picked by conditionals: indexed by a value the compiler does not fold early enough, the
        // array would live in scratch memory)
        const uint4 v = i == 0 ? rw[0] : i == 1 ? rw[1] : i == 2 ? rw[2] : rw[3];
        if (i < 4) *(uint4*)(Wn + (b * 256 + (tid >> 3) + 64 * i) * FWS + piece * 16) = v;
        else if (tid < 256) *(uint4*)(Wsc + (b * 256 + tid) * 16) = rsw;
    };
    // this lane's nibbles and scales of slab j of the super-slab in weight buffer b
    uint4 ra[2];
    uint32_t rs[2];
    auto read_nib = [&](int b, int j) __attribute__((always_inline)) {
#pragma unroll
        for (int z = 0; z < 2; z++) {
            ra[z] = *(const uint4*)(Wn + (b * 256 + myseg[z]) * FWS + 32 * j + 16 * kg);
            rs[z] = *(const uint16_t*)(Wsc + (b * 256 + myseg[z]) * 16 + 4 * j + 2 * kg);
        }
    };
    // fragment n of set z from ra / rs
    auto expand = [&](int z, int n) __attribute__((always_inline)) -> h8 {
        // An e4m3 code shifted into an f16's exponent and mantissa fields IS the scale times 2^-8, subnormal codes
        // included (4 exponent bits with bias 7 against 5 with bias 15; f16 subnormals are computed with, not flushed):
        // no conversion arithmetic.  The magnitudes carry the 2^7 back; code 0x7f (not a number) counts as zero, as
        // in the CPU path.
        const uint32_t em = (n < 2 ? rs[z] : rs[z] >> 8) & 0x7fu;
        const _Float16 sv = __builtin_bit_cast(_Float16, (uint16_t)(em == 0x7fu ? 0u : em << 7));
        const h2 sc = h2{sv, sv};
        const uint32_t wd = n == 0 ? ra[z].x : n == 1 ? ra[z].y : n == 2 ? ra[z].z : ra[z].w;
        h2 a0, a1, a2, a3;
        fp4x4_to_f16x4(wd & 0x0f0f0f0fu, sc, &a0, &a1);          // low nibbles: elements i
        fp4x4_to_f16x4((wd >> 4) & 0x0f0f0f0fu, sc, &a2, &a3);   // high nibbles: elements 8 + i
        return h8{a0[0], a0[1], a1[0], a1[1], a2[0], a2[1], a3[0], a3[1]};
    };
    struct Tok { h8 h, l; };
    auto read_tok = [&](int buf, int n, int tt) __attribute__((always_inline)) -> Tok {
        // bytes 16 * kg + 4 * n .. + 3 of the row's slab: sub-block 2 * kg + n / 2, elements 4 * (n % 2) + {0..3}
        // from the low nibbles and 8 more from the high ones
        const int k0 = 32 * kg + 16 * (n >> 1) + 4 * (n & 1);
        const uint16_t* bh = Bh + (buf * FPAIRS + 32 * (T * th + tt) + r) * FBS + k0;
        const uint16_t* bl = Bl + (buf * FPAIRS + 32 * (T * th + tt) + r) * FBS + k0;
        const uint2 h0 = *(const uint2*)bh, h1 = *(const uint2*)(bh + 8);
        const uint2 l0 = *(const uint2*)bl, l1 = *(const uint2*)(bl + 8);
        return Tok{__builtin_bit_cast(h8, make_uint4(h0.x, h0.y, h1.x, h1.y)),
                   __builtin_bit_cast(h8, make_uint4(l0.x, l0.y, l1.x, l1.y))};
    };

    const bool live_half = __builtin_amdgcn_readfirstlane(32 * T * th < cnt ? 1 : 0) != 0;
    v16f acc[2][T];
#pragma unroll
    for (int z = 0; z < 2; z++)
#pragma unroll
        for (int tt = 0; tt < T; tt++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[z][tt][i] = 0.0f;

    fetch_w(0);
    fetch_x(0);
    stash_w(0);
    stash_x(0);
    __syncthreads();
    h8 af[2][2][4];   // [slab parity][set][fragment]
    read_nib(0, 0);
#pragma unroll
    for (int z = 0; z < 2; z++)
#pragma unroll
        for (int n = 0; n < 4; n++) af[0][z][n] = expand(z, n);
    if (live_half) read_nib(0, 1);   // (a row has at least one super-slab: slab 1 is there)
    Tok first = read_tok(0, 0, 0);
    // One super-slab (four slabs) per trip so that every register array is indexed by a constant.
    // The slab's barrier stands IN FRONT of its last MFMA group, whose operands are in registers by then: behind it every
    // wave asks for the first token fragment and the nibbles of what comes next and then still has that group to issue,
    // so the wait for the slowest wave and the LDS round trip of the first read run under products instead of between
    // two slabs.  Everything that the barrier orders is ahead of it: the last read of this slab's token buffer, the
    // stores of the next slab's tokens and of the next super-slab's weights.
    for (int S = 0; S < n_super; S++) {
        const int wb = S & 1;
        const bool more_w = S + 1 < n_super;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int par = j & 1;
            const int s = 4 * S + j;
            const bool more = j < 3 || more_w;
            const bool more2 = j < 2 || more_w;
            GEMM_STAMP(0);
            GEMM_STAMP(1);
            Tok cur = first;
#pragma unroll
            for (int n = 0; n < 4; n++) {
                // one fragment pair of the next slab between the MFMA groups of this one
                if (more && live_half) {   // a wave set without pairs expands nothing: its SIMD belongs to the wave that has them
#pragma unroll
                    for (int z = 0; z < 2; z++) af[par ^ 1][z][n] = expand(z, n);
                }
#pragma unroll
                for (int tt = 0; tt < T; tt++) {
                    Tok nxt = cur;
                    const int g1 = n * T + tt + 1;
                    if (g1 < 4 * T) nxt = read_tok(par, g1 / T, g1 % T);
#pragma unroll
                    for (int q = (g1 - 1) * LPG; q < g1 * LPG; q++) fetch_one(q, s + 1, S + 1, more, j == 0 && more_w);
                    // the next super-slab's weights (loaded a slab ago) over this slab's first groups, the next slab's
                    // tokens (asked for in this slab's first groups) over the groups of its second half but the last
                    if (j == 1 && more_w) {
                        constexpr int WPG = T == 1 ? 2 : 1;
#pragma unroll
                        for (int i = (g1 - 1) * WPG; i < g1 * WPG; i++)
                            if (i < 5) stash_w_part(wb ^ 1, i);
                    }
                    if (more && g1 > 2 * T && g1 < 4 * T) {
                        constexpr int PPG = (4 * T + 2 * T - 2) / (2 * T - 1);
#pragma unroll
                        for (int i = (g1 - 2 * T - 1) * PPG; i < (g1 - 2 * T) * PPG; i++)
                            if (i < 4 * T) stash_x_part(par ^ 1, i);
                    }
                    if (g1 == 4 * T) {
                        GEMM_STAMP(2);
                        __syncthreads();
                        GEMM_STAMP(3);
                        if (more) first = read_tok(par ^ 1, 0, 0);
                        // (the nibbles of the slab after next: this slab's expansions are done)
                        if (more2 && live_half) read_nib(j < 2 ? wb : wb ^ 1, (j + 2) & 3);
                    }
                    __builtin_amdgcn_sched_barrier(0);   // the reads stay ahead of the products they overlap
                    if (live_half) {   // a wave set whose token groups lie past the tile's pairs only helps with the staging
#pragma unroll
                        for (int z = 0; z < 2; z++) {
                            acc[z][tt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[par][z][n], cur.h, acc[z][tt], 0, 0, 0);
                            acc[z][tt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[par][z][n], cur.l, acc[z][tt], 0, 0, 0);
                        }
                    }
                    cur = nxt;
                }
            }
            GEMM_STAMP(4);
            GEMM_STAMP(5);
        }
    }

    const float e2a = p.scale2 ? p.scale2[e] : 1.0f;
    const float e2b = GLU ? (p.scale2_up ? p.scale2_up[e] : 1.0f) : e2a;
#pragma unroll
    for (int tt = 0; tt < T; tt++) {
        const int slot = 32 * (T * th + tt) + r;
        if (slot >= cnt) continue;
        const int64_t pair = pair_s[slot];
        const float rsc = p.rscale[xrow_s[slot]];
#pragma unroll
        for (int i4 = 0; i4 < 4; i4++) {
            if (GLU) {
                const int row = rbase[0] + 8 * i4 + 4 * kg;
                if (row >= p.n_out) continue;
                float o[4];
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const float g = acc[0][tt][4 * i4 + i] * rsc * e2a, u = acc[1][tt][4 * i4 + i] * rsc * e2b;
                    o[i] = fx_silu(g) * u;
                }
                *(float4*)(p.out + pair * p.n_out + row) = make_float4(o[0], o[1], o[2], o[3]);
            } else {
#pragma unroll
                for (int z = 0; z < 2; z++) {
                    const int row = rbase[z] + 8 * i4 + 4 * kg;
                    if (row >= p.n_out) continue;
                    *(float4*)(p.out + pair * p.n_out + row) =
                        make_float4(acc[z][tt][4 * i4] * rsc * e2a, acc[z][tt][4 * i4 + 1] * rsc * e2a,
                                    acc[z][tt][4 * i4 + 2] * rsc * e2a, acc[z][tt][4 * i4 + 3] * rsc * e2a);
                }
            }
        }
    }
}

template <bool GLU>
__global__ __launch_bounds__(512) void experts_f16_k(ExpertsF16P p) {
    extern __shared__ __align__(16) uint16_t flds[];
    uint16_t* Bh = flds;                          // [2][128][FBS]
    uint16_t* Bl = flds + 2 * FPAIRS * FBS;       // [2][128][FBS]
    uint8_t* Wn = (uint8_t*)(flds + 4 * FPAIRS * FBS);   // [2][256][FWS]: nibble bytes of 256 row segments x 256 k
    uint8_t* Wsc = Wn + 2 * 256 * FWS;             // [2][256][16]: their scale bytes
    __shared__ int xrow_s[FPAIRS], pair_s[FPAIRS];
    // Blocks go to the 8 XCDs in turn.  The row blocks of one tile read the same token rows (k slab by k slab, each
    // row block once: far more bytes than the weights): they take consecutive places on ONE XCD, so that they run
    // side by side and all but the first find the rows in that XCD's L2.
    const int n_rb = (p.n_out + (GLU ? 128 : 256) - 1) / (GLU ? 128 : 256);
    const int lin = blockIdx.x;
    const int tile = 8 * (lin / (8 * n_rb)) + (lin & 7), row_block = (lin >> 3) % n_rb;
    if (tile >= *p.n_tiles) return;
    const int4 td = p.tiles[tile];
    const int cnt = td.z;
    if (threadIdx.x < FPAIRS) {
        const int pair = p.order[td.y + min((int)threadIdx.x, cnt - 1)];
        pair_s[threadIdx.x] = pair;
        xrow_s[threadIdx.x] = p.x_mode == 0 ? pair : (p.x_mode == 1 ? pair / p.n_used : 0);
    }
    __syncthreads();
    // waves 0..3 take the first T token groups of the tile, waves 4..7 the next T
    if (cnt <= 64) experts_f16_body<GLU, 1>(p, td, row_block, Bh, Bl, Wn, Wsc, xrow_s, pair_s);
    else experts_f16_body<GLU, 2>(p, td, row_block, Bh, Bl, Wn, Wsc, xrow_s, pair_s);
}

}  // namespace

size_t experts_f16_work_ints(int n_picks, int n_expert) {
    return 16 + (size_t)(n_expert + n_picks / FPAIRS + 2) * 4 + (size_t)n_picks;
}
size_t experts_f16_work_bytes(int x_rows, int n_in) {
    return (size_t)x_rows * n_in * 4 + (((size_t)x_rows * 4 + 255) & ~(size_t)255);
}

bool experts_f16_takes(const ExpertsView& w, const ExpertsView* up, int n_picks, const int8_t* act_quants, const float* out) {
    if (n_picks < 32 || w.n_expert > 1024 || w.fmt != W_NVFP4 || w.n_in % FSUPER || w.n_out % 4) return false;
    if ((reinterpret_cast<uintptr_t>(w.q) & 15) || w.q_stride % 16 || w.s_stride % 16 || (reinterpret_cast<uintptr_t>(w.scales) & 15) ||
        (reinterpret_cast<uintptr_t>(act_quants) & 3) || (reinterpret_cast<uintptr_t>(out) & 15))
        return false;
    if (up && (up->fmt != w.fmt || up->n_in != w.n_in || up->n_out != w.n_out || (reinterpret_cast<uintptr_t>(up->q) & 15) ||
               (reinterpret_cast<uintptr_t>(up->scales) & 15) || up->q_stride != w.q_stride || up->s_stride != w.s_stride))
        return false;
    static int sized = 0;   // 0 unknown, 1 yes, -1 the LDS size was refused
    if (!sized) {
        const size_t lds = (size_t)4 * FPAIRS * FBS * sizeof(uint16_t) + (size_t)2 * 256 * (FWS + 16);
        sized = hipFuncSetAttribute((const void*)experts_f16_k<true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) == hipSuccess &&
                        hipFuncSetAttribute((const void*)experts_f16_k<false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) == hipSuccess
                    ? 1 : -1;
        if (sized < 0) (void)hipGetLastError();
    }
    return sized > 0;
}

bool experts_gemm_f16(const ExpertsView& w, const ExpertsView* up, const int32_t* ids, int n_picks, int n_used,
                      int x_mode, const float* act_scales, const int8_t* act_quants, float* out, int32_t* work,
                      size_t work_ints, void* fwork, size_t fwork_bytes, bool grouped, hipStream_t s) {
    if (!work || !fwork || !experts_f16_takes(w, up, n_picks, act_quants, out)) return false;
    if (n_used < 1) n_used = 1;
    const int x_rows = x_mode == 0 ? n_picks : (x_mode == 1 ? (n_picks + n_used - 1) / n_used : 1);
    if (work_ints < experts_f16_work_ints(n_picks, w.n_expert) || fwork_bytes < experts_f16_work_bytes(x_rows, w.n_in)) return false;
    const size_t lds = (size_t)4 * FPAIRS * FBS * sizeof(uint16_t) + (size_t)2 * 256 * (FWS + 16);
    const int max_tiles = w.n_expert + n_picks / FPAIRS + 1;
    int32_t* n_tiles = work;
    int4* tiles = (int4*)(work + 16);
    int32_t* order = work + 16 + (size_t)(max_tiles + 1) * 4;
    if (!grouped) moe_group(ids, n_picks, w.n_expert, FPAIRS, n_tiles, tiles, order, s);
    uint16_t* xh = (uint16_t*)fwork;
    uint16_t* xl = xh + (size_t)x_rows * w.n_in;
    float* rscale = (float*)(xl + (size_t)x_rows * w.n_in);
    hipLaunchKernelGGL(acts_split_f16_k, dim3(x_rows), dim3(256), 0, s, act_quants, act_scales, w.n_in, xh, xl, rscale);
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
    const int tiles8 = (max_tiles + 7) / 8 * 8;   // (the kernel deals tiles to the XCDs in groups of eight)
    if (up) hipLaunchKernelGGL(experts_f16_k<true>, dim3(tiles8 * ((w.n_out + 127) / 128)), dim3(512), lds, s, p);
    else hipLaunchKernelGGL(experts_f16_k<false>, dim3(tiles8 * ((w.n_out + 255) / 256)), dim3(512), lds, s, p);
    return true;
}

}  // namespace itk

#ifdef IT_STAMPS
// tuning builds only: the stamps of the selected block, then the next selection
extern "C" int it_hip_debug_gemm_stamps(long long* out, int block, int slab, int glu) {
    if (hipDeviceSynchronize() != hipSuccess) return -1;
    if (hipMemcpyFromSymbol(out, HIP_SYMBOL(it_gemm_stamps), 32 * 8) != hipSuccess) return -1;
    if (hipMemcpyToSymbol(HIP_SYMBOL(it_gemm_stamp_tile), &block, 4) != hipSuccess ||
        hipMemcpyToSymbol(HIP_SYMBOL(it_gemm_stamp_slab), &slab, 4) != hipSuccess ||
        hipMemcpyToSymbol(HIP_SYMBOL(it_gemm_stamp_glu), &glu, 4) != hipSuccess)
        return -1;
    return 0;
}
#endif
