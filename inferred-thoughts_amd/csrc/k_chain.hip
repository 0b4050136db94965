// A run of decode layers as one persistent kernel (fast mode).
//
// The per-layer chain of a single-token pass is six launches, each needing the whole output vector of the one
// before (/root/reference src/model/qwen35.rs:1232-1328 the Gated DeltaNet mixer, :1587-1700 the routed FFN), and
// a dependent launch costs about as much as the few megabytes it streams.  Here the six become stages of one
// kernel with one block on every compute unit.  A stage's weight rows are fixed per block and wave, so their
// loads are issued a stage ahead and sit in registers when the stage's input arrives.  The input arrives as
// 8-byte words {payload, epoch} that the producing blocks store to uncached device memory and the consuming
// threads poll until the epoch is the current layer's: one trip through memory, no flag, no fence, nothing to
// clear between uses (an epoch is never reused).  The reference meets the same problem by capturing its decode
// sequence into one graph (src/ops/cuda/mod.rs:600-647); a graph of dependent kernels still pays every boundary.
//
// Stages of a layer (the arithmetic per element is the per-stage fast kernels', k_fast.hip / k_fused.hip):
//   A  rms_norm + Q8_0 quantization of x; rows of wqkv (+ causal conv, silu), wz (+ silu), alpha, beta
//   B  l2 norm of q, k; the delta rule on 16 state rows per block; the read-out times silu(z) and the head-norm
//      weight, with the block's share of the head's sum of squares beside it
//   C  head-norm scale, quantization, rows of ssm_out, residual
//   D  rms_norm + quantization; router rows, the shared expert's gate logit, its gate / up rows
//   E  top-10 of the logits in every block (ranked on the logits; the softmax of the ten follows under the rows'
//      flight); 160 blocks take one 32-element block of one pick's gate / up rows each and publish it quantized, the
//      other 96 touch those rows' lines for the blocks of their XCD; the down rows are issued behind the publication
//   F  down rows of the ten picks and of the shared expert, combine, residual
// An attention layer's mixer (src/model/qwen35.rs:1141-1223) is five stages of its own in front of its FFN's D, E, F:
//   the in-projection (rms_norm + Q8_0 + wq / wk / wv rows), published like stage A's outputs;
//   head norm + rotation of the queries and of the new key, the new cache rows, and the attention of eight query heads
//   over one of 128 ranges of the context per block, on the f16 matrix cores with exact operands (queries and
//   probabilities as f16 pairs, f32 sums), with the range's K / V rows in flight
//   before the queries are waited for; the merge of the ranges with the sigmoid gate, 16 dims a block; the
//   out-projection + residual.  The middle three are a function of their own (attn_core).
// (The older form stays for contexts beyond what that attention is good for, and as a measurement switch: the
// in-projection as the LAST stage of the chain before the layer, the out-projection as the FIRST stage of the chain
// behind it, the matrix-core attention kernels between the two chains.)
// A chain holds up to 56 layers, a whole token of the model this is written for; their parameters travel in the
// kernel's argument block.
//
// Three things place the loads and the polls (each measured with the stage stamps below):
//   * loads return in issue order per wave, so a poll or a publication waits for everything its wave has in flight:
//     few-word inputs (stages B and F) are gathered by waves that issue their own rows only afterwards;
//   * a compute unit pulls 25-30 GB/s whatever it asks for: rows are issued where the stage before leaves the pipe idle;
//   * two waves share a SIMD's vector ALU, so instructions count double: NVFP4 rows go through the hardware's
//     fp4 -> f16 conversion and v_dot2_f32_f16 (half the instructions of the permute + v_dot4 form, same bits).
//
// Every wait is bounded: a poll that runs out of tries sets the abort word, every other wait sees it and the
// grid drains.  The grid must be resident at once (one block per compute unit), which the launcher checks.
#include <cstddef>
#include <cstring>
#define IT_CHAIN_DEVICE_POINTERS
#include "it_fast.h"
#include "kernels_fused.h"

namespace itk {
using namespace fastk;
namespace {

typedef unsigned long long u64;
typedef unsigned v2u __attribute__((ext_vector_type(2)));
typedef unsigned v4u __attribute__((ext_vector_type(4)));

constexpr int CT = 512, CW = CT / 64, NB = CHAIN_BLOCKS;
constexpr int D = 2048, NK = 16, NV = 32, DK = 128, KDIM = NK * DK, VDIM = NV * DK, CDIM = 2 * KDIM + VDIM;
constexpr int NE = 512, NU = 10, FF = 512;
constexpr int EB = NU * FF / 32;   // blocks that take a 32-element block of a pick's intermediates in stage E
static_assert(D == 4 * CT && VDIM == 8 * CT && NE == CT && D == 8 * NB && CDIM == 32 * NB && VDIM == 16 * NB && NV * 8 == NB,
              "the stage geometry below is written for these shapes");

// hand-off regions, in 8-byte words (every start is even: pairs of words are polled with 16-byte loads)
constexpr int RX = 0;                      // D: the residual stream into a layer
constexpr int RA = RX + D;                 // [q | k | v] after conv + silu, silu(z), alpha, beta
constexpr int RA_Z = RA + CDIM, RA_AL = RA_Z + VDIM, RA_BE = RA_AL + NV;
constexpr int RB = RA_BE + NV;             // VDIM gated read-outs, then NB partial sums of squares
constexpr int RB_SS = RB + VDIM;
constexpr int RC = RB_SS + NB;             // D: the residual stream after the mixer
constexpr int RD = RC + D;                 // NE router logits, the shared expert's gate logit
constexpr int RS = RD + NE + 2;            // FF shared-expert intermediates
constexpr int RE = RS + FF;                // NU * FF / 4 packed Q8_0 quads of the routed intermediates, then their scales
constexpr int RE_SC = RE + NU * FF / 4;
constexpr int R_END = RE_SC + EB;
static_assert(R_END <= (int)CHAIN_LL_STAGE_WORDS, "hand-off space");
// An attention mixer's hand-offs reuse the Gated DeltaNet mixer's regions (a layer has one or the other): the
// in-projection's [query + gate of every head | key | value] where the conv output goes, the gated attention output
// where the read-outs go.  The partial results of the key ranges have a space of their own behind the stages'.
constexpr int NH = 16, NKV = 2, HD = 256, AG = NH / NKV, AS = CHAIN_ATTN_SPLITS;
constexpr int RQ = RA, RK = RQ + NH * 2 * HD, RV = RK + NKV * HD, RT = RB;
constexpr int RP = (int)CHAIN_LL_STAGE_WORDS, PW = HD + 2;   // per (query head, key range): HD sums, the maximum, the weight
constexpr int TK = 64;            // keys of a range that are in LDS at a time
constexpr int KSTR = HD + 8;      // f16 row stride of the K and V tiles (528 bytes)
constexpr int PSTR = TK + 8;      // f16 row stride of the probabilities (144 bytes)
// dynamic LDS of an attention mixer's middle: K tile, V tile, the eight scaled queries as f16 pairs (16 rows), the tile's
// scores (f32), the probabilities as f16 pairs (16 rows + 16 of zeros: the unused columns of the matrix-core product),
// the heads' rescaling factors, the merge's partial sums, a wave's results on their way to its stores
constexpr int ATTN_LDS = 2 * TK * KSTR * 2 + 16 * KSTR * 2 + AG * TK * 4 + 32 * PSTR * 2 + AG * 4 + (8 + 8 * 4 * 5) * 4 + AG * HD * 4;
static_assert(RV + NKV * HD <= RB && NH * HD <= VDIM && NB == NKV * AS && CW == AG && NB == NH * 16 && NH * 2 * HD == 32 * NB &&
              NKV * HD == 2 * NB && NH * HD == 8 * CT && HD == 4 * 64 && (PW % 2) == 0 && (RP % 2) == 0, "attention stage shapes");
static_assert(!(RA & 1) && !(RA_Z & 1) && !(RB & 1) && !(RB_SS & 1) && !(RC & 1) && !(RD & 1) && !(RS & 1) && !(RE & 1) && !(RE_SC & 1), "");

// Stage stamps for tuning: a build with -DIT_CHAIN_STAMPS adds up, per stamp point, the 100 MHz wall clock that block
// 0's first thread spent since its previous point; the library build compiles them away.
#ifdef IT_CHAIN_STAMPS
__device__ long long it_chain_stamps[24];
__device__ long long it_attn_core_stamps[8];   // inside an attention mixer's middle, the same clock
#define CH_STAMP(i)                                          \
    do {                                                     \
        if (b0 == 0 && tid0 == 0) {                          \
            const long long now = wall_clock64();            \
            it_chain_stamps[i] += now - tprev;               \
            tprev = now;                                     \
        }                                                    \
    } while (0)
// per wave of block 0, inside stage E: the time since the wave's previous point (point 0 restarts the clock)
__device__ long long it_chain_wave_stamps[8][8];
#define CH_WSTAMP(i)                                                     \
    do {                                                                 \
        if (b0 == 0 && (tid0 & 63) == 0) {                               \
            const long long now = wall_clock64();                        \
            if (i) it_chain_wave_stamps[tid0 >> 6][i] += now - wprev;    \
            wprev = now;                                                 \
        }                                                                \
    } while (0)
#else
#define CH_STAMP(i) \
    do {            \
    } while (0)
#define CH_WSTAMP(i) \
    do {             \
    } while (0)
#endif

#ifndef IT_CHAIN_FP4_HW
#define IT_CHAIN_FP4_HW 1         // NVFP4 rows of stages D and E through the hardware's fp4 / fp8 conversions (1) or through v_perm_b32 + v_dot4 (0)
#endif
// Where the prefetches sit (tuning switches; the defaults are what measured best).
#ifndef IT_CHAIN_F_POLLERS
#define IT_CHAIN_F_POLLERS 1     // stage F's input gathered by waves 4..7 alone (1) or by every thread (0)
#endif
#ifndef IT_CHAIN_B_POLLERS
#define IT_CHAIN_B_POLLERS 1     // stage B's input gathered by waves 5..7 alone (1) or by the first 274 threads (0)
#endif
#ifndef IT_CHAIN_TOUCH
#define IT_CHAIN_TOUCH 1          // stage E's rows touched by the blocks that have none of their own
#endif
#ifndef IT_CHAIN_FLOADS_EARLY
#define IT_CHAIN_FLOADS_EARLY 0   // stage F's down rows: 1 ahead of stage E's barrier and publication, 0 behind them
#endif
#ifndef IT_CHAIN_WC_AT
#define IT_CHAIN_WC_AT 0      // out-projection row: 0 at the head of stage B, 1 after stage A's input has arrived, 2 after stage A's dots, 3 after stage B's input has arrived
#endif
#ifndef IT_CHAIN_D_AT
#define IT_CHAIN_D_AT 1       // stage D's rows: 0 at the head of stage C, 1 after stage B's input has arrived
#endif
#ifndef IT_CHAIN_A_AT
#define IT_CHAIN_A_AT 0x070   // next in-projection, a hex digit of fetch_a parts per site: after D's input | at the head of stage F | after F's input
#endif

struct Ctl {
    unsigned* abort_flag;
    int spin_limit;
};

IT_DEV void ll_put(u64* p, uint32_t bits, unsigned e) {
    // (the hand-off space is device memory: said so, the store is a global one wherever the pointer came from)
    __hip_atomic_store((__attribute__((address_space(1))) u64*)p, ((u64)e << 32) | (u64)bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}
IT_DEV void ll_putf(u64* p, float v, unsigned e) { ll_put(p, __float_as_uint(v), e); }
// two neighbouring words (16-byte aligned) in one store; a reader takes a pair only when both stamps are there.
// (A store of more than 8 bytes reads its data registers up to two wait states after it issues, and the compiler does
// not see a store inside an asm statement: without the s_nop it may refill those registers for the next store at once,
// and the first store then carries the second one's values.)
IT_DEV void ll_put2f(u64* p, float v0, float v1, unsigned e) {
    const v4u w = {__float_as_uint(v0), e, __float_as_uint(v1), e};
    asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1\n\ts_nop 1" ::"v"(p), "v"(w) : "memory");
}

// true when the wait must stop: the tries are used up (this thread raises the abort word) or another wait gave up
#ifndef IT_CHAIN_SLEEP
#define IT_CHAIN_SLEEP 0
#endif
IT_DEV bool ll_give_up(int& spins, const Ctl& c) {
    if (IT_CHAIN_SLEEP > 0) __builtin_amdgcn_s_sleep(IT_CHAIN_SLEEP);
    if (++spins > c.spin_limit) {
        *(volatile unsigned*)c.abort_flag = 1u;
        return true;
    }
    return (spins & 63) == 0 && *(volatile unsigned*)c.abort_flag != 0u;
}

// Polls.  A load and its wait are ONE asm statement: the compiler does not know that the destination of an asm
// load is not ready, so nothing may be schedulable between the two.
// a short sleep ahead of a wait's first poll: a poll issued the moment the wave arrives nearly always fails, and every
// failed poll is traffic that the words it waits for queue behind
#ifndef IT_CHAIN_FIRST_SLEEP
#define IT_CHAIN_FIRST_SLEEP 8
#endif
IT_DEV bool ll_wait1(const u64* p, unsigned e, const Ctl& c, uint32_t* out) {
    int spins = 0;
    if (IT_CHAIN_FIRST_SLEEP > 0) __builtin_amdgcn_s_sleep(IT_CHAIN_FIRST_SLEEP);
    for (;;) {
        v2u w;
        asm volatile("global_load_dwordx2 %0, %1, off sc0 sc1\n\ts_waitcnt vmcnt(0)" : "=&v"(w) : "v"(p) : "memory");
        if (w.y == e) {
            *out = w.x;
            return true;
        }
        if (ll_give_up(spins, c)) return false;
    }
}
// K pairs of words at a[k] (16-byte aligned); out[2k], out[2k+1] = their payloads.  A pair that is complete is
// latched; its load is simply repeated while the others are still awaited.
template <int K>
IT_DEV bool ll_wait_pairs(const u64* const (&a)[K], unsigned e, const Ctl& c, uint32_t (&out)[2 * K]) {
    static_assert(K == 1 || K == 2 || K == 4, "");
    int spins = 0;
    unsigned done = 0;
    if (IT_CHAIN_FIRST_SLEEP > 0) __builtin_amdgcn_s_sleep(IT_CHAIN_FIRST_SLEEP);
    for (;;) {
        v4u w[K];
        if constexpr (K == 4)
            asm volatile("global_load_dwordx4 %0, %4, off sc0 sc1\n\tglobal_load_dwordx4 %1, %5, off sc0 sc1\n\t"
                         "global_load_dwordx4 %2, %6, off sc0 sc1\n\tglobal_load_dwordx4 %3, %7, off sc0 sc1\n\ts_waitcnt vmcnt(0)"
                         : "=&v"(w[0]), "=&v"(w[1]), "=&v"(w[2]), "=&v"(w[3]) : "v"(a[0]), "v"(a[1]), "v"(a[2]), "v"(a[3]) : "memory");
        else if constexpr (K == 2)
            asm volatile("global_load_dwordx4 %0, %2, off sc0 sc1\n\tglobal_load_dwordx4 %1, %3, off sc0 sc1\n\ts_waitcnt vmcnt(0)"
                         : "=&v"(w[0]), "=&v"(w[1]) : "v"(a[0]), "v"(a[1]) : "memory");
        else
            asm volatile("global_load_dwordx4 %0, %1, off sc0 sc1\n\ts_waitcnt vmcnt(0)" : "=&v"(w[0]) : "v"(a[0]) : "memory");
#pragma unroll
        for (int k = 0; k < K; k++) {
            if (!(done & (1u << k)) && w[k].y == e && w[k].w == e) {
                out[2 * k] = w[k].x;
                out[2 * k + 1] = w[k].z;
                done |= 1u << k;
            }
        }
        if (done == (1u << K) - 1u) return true;
        if (ll_give_up(spins, c)) return false;
    }
}

// the four floats [4 * qi, 4 * qi + 4) of a region
IT_DEV bool ll_wait_quad(const u64* region, int qi, unsigned e, const Ctl& c, float4* v) {
    const u64* const a[2] = {region + 4 * qi, region + 4 * qi + 2};
    uint32_t o[4];
    if (!ll_wait_pairs<2>(a, e, c, o)) return false;
    *v = make_float4(__uint_as_float(o[0]), __uint_as_float(o[1]), __uint_as_float(o[2]), __uint_as_float(o[3]));
    return true;
}

// The chunks of lane `sub` of one weight row, as load_w of the per-stage kernels, with the lane's part of the address
// an unsigned 32-bit offset from the row's (wave-uniform or per-lane) base: the loads then take their base from scalar
// registers and one vector register of offset, instead of a 64-bit vector address each.
template <int FMT, int CPL, int L>
IT_DEV void load_row(WChunks<CPL>& t, const uint8_t* q, const uint8_t* s, int n_in, int64_t row, int sub, bool live) {
    if (!live) {
#pragma unroll
        for (int k = 0; k < CPL; k++) {
            t.w[k] = make_uint4(0, 0, 0, 0);
            t.sc[k] = 0;
        }
        return;
    }
    const uint8_t* rp = q + row * (FMT == W_Q8_0 ? n_in : n_in >> 1);
    const uint8_t* sp = s + row * (n_in >> 5) * 2;
    const uint32_t sub16 = (uint32_t)sub * 16u;
#pragma unroll
    for (int k = 0; k < CPL; k++) {
        typedef unsigned v4 __attribute__((ext_vector_type(4)));
        const v4 nt = __builtin_nontemporal_load((const v4*)(rp + (sub16 + (uint32_t)(k * L * 16))));
        t.w[k] = make_uint4(nt.x, nt.y, nt.z, nt.w);
        const uint32_t c = (uint32_t)(k * L) + (uint32_t)sub;
        t.sc[k] = *(const uint16_t*)(sp + (FMT == W_Q8_0 ? (c >> 1) * 2u : c * 2u));
    }
}

// ---- stage weights held in registers
// In-projection: a wave takes four wqkv rows, two wz rows and (wave 0 of the first 64 blocks) one alpha / beta row.
// The epilogue of row k runs in lane k, which also holds the row's conv window and taps.
struct AW {
    WChunks<2> t[7];
    float4 taps;
    float past[3];
    float4 ab;   // unquantized alpha / beta (RF): this wave's four floats a lane of the block's row
};
// What the registers held is no longer wanted: without this the values of a layer before stay live, as far as the
// compiler can tell, through every stage of a layer that loads only a part of them.
IT_DEV void forget(AW& a) {
#pragma unroll
    for (int k = 0; k < 7; k++)
#pragma unroll
        for (int c = 0; c < 2; c++) {
            a.t[k].w[c] = make_uint4(0, 0, 0, 0);
            a.t[k].sc[c] = 0;
        }
    a.taps = make_float4(0.f, 0.f, 0.f, 0.f);
    a.past[0] = a.past[1] = a.past[2] = 0.0f;
    a.ab = make_float4(0.f, 0.f, 0.f, 0.f);
}
IT_DEV int a_row(int k, int b, int wave) {   // row k of the wave in its own matrix
    return k < 4 ? b + NB * (wave + CW * k) : k < 6 ? b + NB * (wave + CW * (k - 4)) : b < NV ? b : b - NV;
}
// An unquantized (F32) row of 2,048 weights is summed in the order the per-stage kernels use (fused_gemv_fast_k's
// frow_chunk / frow_tree), so that these sums come out the same, to the bit, either way: a chunk of 256 weights is one
// multiply-add chain per lane from zero and a lane reduction, and the eight chunk sums are added as a balanced tree.
IT_DEV float f32_chunk(const float4 w, const float4 xv) { return fmaf(w.x, xv.x, fmaf(w.y, xv.y, fmaf(w.z, xv.z, fmaf(w.w, xv.w, 0.0f)))); }
IT_DEV float f32_tree(const float* pc) { return ((pc[0] + pc[1]) + (pc[2] + pc[3])) + ((pc[4] + pc[5]) + (pc[6] + pc[7])); }
// `parts` picks what is fetched: bit 0 the first two wqkv rows and the conv windows, bit 1 the other two wqkv rows,
// bit 2 the two wz rows and the alpha / beta row.  (A block's 105 KB can be issued in pieces at up to three sites of the
// layer before, IT_CHAIN_A_AT: loads return in the order they were issued, and a poll behind a large fetch waits for
// all of it.  All at the head of stage F measured best once that stage's input was gathered by waves that issue
// theirs behind the gather.)
template <int RF, class M>   // M: a ChainMixer, wherever it lives
IT_DEV void fetch_a(const M& m, AW& a, int b, int wave, int lane, int parts = 7) {
    if (parts & 1) {
#pragma unroll
        for (int k = 0; k < 2; k++) load_row<W_Q8_0, 2, 64>(a.t[k], m.qkv_q, m.qkv_s, D, a_row(k, b, wave), lane, true);
        if (lane < 4) {
            const int64_t row = b + NB * (wave + CW * lane);
            a.taps = *(const float4*)(m.conv_w + row * 4);
            a.past[0] = m.conv_state[row * 3];
            a.past[1] = m.conv_state[row * 3 + 1];
            a.past[2] = m.conv_state[row * 3 + 2];
        }
    }
    if (parts & 2) {
#pragma unroll
        for (int k = 2; k < 4; k++) load_row<W_Q8_0, 2, 64>(a.t[k], m.qkv_q, m.qkv_s, D, a_row(k, b, wave), lane, true);
    }
    if (parts & 4) {
#pragma unroll
        for (int k = 4; k < 6; k++) load_row<W_Q8_0, 2, 64>(a.t[k], m.z_q, m.z_s, D, a_row(k, b, wave), lane, true);
        if (RF) {
            // an F32 row of 2,048 floats is shared by the block's eight waves, 256 floats each (a row in one wave would
            // be 32 registers a lane); the partial dots meet in LDS
            a.ab = make_float4(0.f, 0.f, 0.f, 0.f);
            if (b < 2 * NV) a.ab = ((const float4*)((const float*)(b < NV ? m.a_q : m.b_q) + (int64_t)a_row(6, b, wave) * D))[wave * 64 + lane];
        } else {
            const bool extra = wave == 0 && b < 2 * NV;
            load_row<W_Q8_0, 2, 64>(a.t[6], b < NV ? m.a_q : m.b_q, b < NV ? m.a_s : m.b_s, D, a_row(6, b, wave), lane, extra);
        }
    }
}

// The tail stage's rows (the in-projection of the attention layer behind the chain): 36 a block, row r of the flat list
// [wq 8192 | wk 512 | wv 512] on block r % 256; a wave takes four wq rows, waves 0..3 one more (wk: 0, 1; wv: 2, 3).
template <class T>   // ChainTail or ChainAttn: the same three matrices
IT_DEV void fetch_tail(const T& t, AW& a, int b, int wave, int lane) {
#pragma unroll
    for (int k = 0; k < 4; k++) load_row<W_Q8_0, 2, 64>(a.t[k], t.q_q, t.q_s, D, b + NB * (wave + CW * k), lane, true);
    const bool kk = wave < 2;
    load_row<W_Q8_0, 2, 64>(a.t[4], kk ? t.k_q : t.v_q, kk ? t.k_s : t.v_s, D, b + NB * (wave & 1), lane, wave < 4);
}

// An NVFP4 chunk against the activation through gfx950's own conversions: v_cvt_scalef32_pk_f16_fp4 turns one byte (two
// e2m1 nibbles) into two f16 and v_dot2_f32_f16 multiplies them with two f16 activations, 2 instructions for 2 elements
// where nibbles -> int8 through v_perm_b32 + v_dot4 takes 7 for 4.  The activations are the Q8_0 quants as f16 (exact),
// paired as the nibbles of a byte are (element j with element 8 + j of a 16-element sub-block); every product and sum is
// a multiple of 0.5 below 2^24, so the f32 accumulation is exact and the result is the integer path's, bit for bit.
// The sub-block scales come from v_cvt_pk_f32_fp8 (OCP e4m3; the format's ue4m3 is half of that, and the e2m1 values
// here are half of the integer path's doubled ones: the two factors of 2 cancel; code 0x7f is 0 as in it_ue4m3_to_f32).
#if IT_CHAIN_FP4_HW
typedef _Float16 h2v __attribute__((ext_vector_type(2)));
typedef float f2v __attribute__((ext_vector_type(2)));
struct XN {
    uint32_t p[16];   // sub-block A: pairs (j, 8 + j) j = 0..7, then sub-block B
    float d;
};
IT_DEV uint32_t pair_h(uint32_t lo, uint32_t hi, int j) {
    const h2v v = {(_Float16)(int)(int8_t)(lo >> (8 * j)), (_Float16)(int)(int8_t)(hi >> (8 * j))};
    return __builtin_bit_cast(uint32_t, v);
}
IT_DEV void load_xn(XN& x, const int8_t* xq, const float* xs, int lane) {
    XChunks<W_NVFP4, 1> t;
    load_x<W_NVFP4, 1, 64>(t, xq, xs, lane);
#pragma unroll
    for (int j = 0; j < 4; j++) {
        x.p[j] = pair_h(t.a[0].x, t.a[0].z, j);
        x.p[4 + j] = pair_h(t.a[0].y, t.a[0].w, j);
        x.p[8 + j] = pair_h(t.b[0].x, t.b[0].z, j);
        x.p[12 + j] = pair_h(t.b[0].y, t.b[0].w, j);
    }
    x.d = t.d[0];
}
#define IT_FP4_STEP(acc, word, sel, pi) \
    acc = __builtin_amdgcn_fdot2(__builtin_amdgcn_cvt_scalef32_pk_f16_fp4(word, 1.0f, sel), __builtin_bit_cast(h2v, x.p[pi]), acc, false)
IT_DEV float dot_xn(const WChunks<1>& t, const XN& x) {
    const uint4 w = t.w[0];
    float sa = 0.0f, sb = 0.0f;
    IT_FP4_STEP(sa, w.x, 0, 0); IT_FP4_STEP(sa, w.x, 1, 1); IT_FP4_STEP(sa, w.x, 2, 2); IT_FP4_STEP(sa, w.x, 3, 3);
    IT_FP4_STEP(sa, w.y, 0, 4); IT_FP4_STEP(sa, w.y, 1, 5); IT_FP4_STEP(sa, w.y, 2, 6); IT_FP4_STEP(sa, w.y, 3, 7);
    IT_FP4_STEP(sb, w.z, 0, 8); IT_FP4_STEP(sb, w.z, 1, 9); IT_FP4_STEP(sb, w.z, 2, 10); IT_FP4_STEP(sb, w.z, 3, 11);
    IT_FP4_STEP(sb, w.w, 0, 12); IT_FP4_STEP(sb, w.w, 1, 13); IT_FP4_STEP(sb, w.w, 2, 14); IT_FP4_STEP(sb, w.w, 3, 15);
    const uint32_t sc = t.sc[0] & 0x7f7fu;
    const f2v s2 = __builtin_amdgcn_cvt_pk_f32_fp8((int)sc, false);
    const float dA = (sc & 0x7fu) == 0x7fu ? 0.0f : s2.x, dB = (sc >> 8) == 0x7fu ? 0.0f : s2.y;
    float acc = 0.0f;
    acc += (x.d * dA) * sa;
    acc += (x.d * dB) * sb;
    return acc;
}
#else
typedef XChunks<W_NVFP4, 1> XN;
IT_DEV void load_xn(XN& x, const int8_t* xq, const float* xs, int lane) { load_x<W_NVFP4, 1, 64>(x, xq, xs, lane); }
IT_DEV float dot_xn(const WChunks<1>& t, const XN& x) { return dot_chunks<W_NVFP4, 1>(t, x); }
#endif

// a float's bits as an unsigned that orders like the value (negative below positive), and back
IT_DEV uint32_t logit_order(float v) {
    const uint32_t u = __float_as_uint(v);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
IT_DEV float logit_of_order(uint32_t o) { return __uint_as_float((o & 0x80000000u) ? (o & 0x7fffffffu) : ~o); }

// rms_norm (naive.rs:633-650) of the 2,048 floats the block's threads hold as quads, then Q8_0 (naive.rs:652-675)
// into xq / xs.  Two barriers; returns false after the first when the block has to stop.
IT_DEV void norm_quant_finish(float4 v, float4 w, float eps, double sum, int8_t* xq, float* xs, int tid, float* xf = nullptr) {
    const float mean = (float)(sum / (double)D);
    const float scale = 1.0f / sqrtf(mean + eps);
    v.x = v.x * scale * w.x;
    v.y = v.y * scale * w.y;
    v.z = v.z * scale * w.z;
    v.w = v.w * scale * w.w;
    if (xf) ((float4*)xf)[tid] = v;   // the normed vector itself, for rows of unquantized matrices
    quant_quad(v, true, tid, xq, xs);
    __syncthreads();
}
IT_DEV bool norm_quant(float4 v, float4 w, float eps, int8_t* xq, float* xs, double* red, const int* dead, int tid, float* xf = nullptr) {
    const double part = wave_sum_f64_tail(quad_sumsq(v));
    if ((tid & 63) == 63) red[tid >> 6] = part;
    __syncthreads();
    if (*dead) return false;
    double sum = 0.0;
#pragma unroll
    for (int i = 0; i < CW; i++) sum += red[i];
    norm_quant_finish(v, w, eps, sum, xq, xs, tid, xf);
    return true;
}

// ---- the middle of an attention mixer: this block's key range against eight query heads, then the merge of the ranges
// with the sigmoid gate.  A function of its own (never inlined): its registers are allotted apart from the stages
// around it, which have none to spare.  Its LDS is the launch's dynamic allocation.  Every thread runs through every
// barrier whatever its waits return; false: one of this thread's waits gave up (the results are void).
//
// Key ranges.  Block b: KV head b % 2, range b / 2 of 128 equal ranges of the live context (the last range that holds
// keys holds the new position, whose key and value rows this block forms and writes to the cache).  Wave w: query head
// w of the KV head's eight.  The range's rows are in flight before the queries are waited for; scores and weighted
// values on the f16 matrix cores (layouts at the loop), softmax bookkeeping a wave per head; a range is a few dozen
// keys at the contexts this path is measured at, longer ones walk tiles of 64 keys.
// Merge.  Block b: 16 dims of query head b / 16; thread t: range t / 4, four of the 16 dims.
extern __shared__ __align__(16) uint8_t chain_dyn_lds[];   // ATTN_LDS bytes when a layer of the chain is an attention mixer
typedef __attribute__((address_space(1))) uint16_t g_u16;
struct AttnCoreP {   // what of a ChainAttn the function reads
    it_gptr<const float> q_norm, k_norm;
    it_gptr<const float2> rope;
    it_gptr<uint16_t> k_slab, v_slab;
    it_gptr<const int> n_pos;
    it_gptr<const uint8_t> o_q, o_s;   // the out-projection
    float eps_head, scale;
    int n_rot;
};
struct AttnCoreR {
    float dot;   // this wave's out-projection row against the gated attention output (in lane 63)
    int ok;      // 0: one of this thread's waits gave up
};
// (the arguments one by one, so that they travel in registers: a struct by value goes through the stack)
__attribute__((noinline)) __device__ AttnCoreR attn_core(it_gptr<const float> q_norm, it_gptr<const float> k_norm, it_gptr<const float2> rope,
                                                         it_gptr<uint16_t> k_slab, it_gptr<uint16_t> v_slab, it_gptr<const int> n_pos_p,
                                                         it_gptr<const uint8_t> o_q, it_gptr<const uint8_t> o_s, float eps_head, float scale,
                                                         int n_rot, it_gptr<u64> ll_g, unsigned e, it_gptr<unsigned> abort_g, int spin_limit, int tid,
                                                         int b) {
    u64* const ll = (u64*)ll_g;   // (polled through explicit global loads, stored to as global: see ll_put)
    unsigned* const abort_flag = (unsigned*)abort_g;
    const AttnCoreP at{q_norm, k_norm, rope, k_slab, v_slab, n_pos_p, o_q, o_s, eps_head, scale, n_rot};
    const Ctl ctl{abort_flag, spin_limit};
#ifdef IT_CHAIN_STAMPS
    long long ac_prev = wall_clock64();
#define AC_STAMP(i)                                      \
    do {                                                 \
        if (b == 0 && tid == 0) {                        \
            const long long now = wall_clock64();        \
            it_attn_core_stamps[i] += now - ac_prev;     \
            ac_prev = now;                               \
        }                                                \
    } while (0)
#else
#define AC_STAMP(i) \
    do {            \
    } while (0)
#endif
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    uint16_t* const Ks = (uint16_t*)chain_dyn_lds;
    uint16_t* const Vs = Ks + TK * KSTR;
    uint16_t* const Q16 = Vs + TK * KSTR;            // [16][KSTR]: rows 0..7 the high f16 halves of the scaled queries, 8..15 the low halves
    float* const Sf = (float*)(Q16 + 16 * KSTR);     // [8][TK] the tile's scores
    uint16_t* const P16 = (uint16_t*)(Sf + AG * TK);  // [32][PSTR]: rows 0..7 high halves of the probabilities, 8..15 low halves, 16..31 zeros
    float* const Af = (float*)(P16 + 32 * PSTR);      // [8] what a head's sums so far are scaled by
    float* const sm = Af + AG;           // 8 wave maxima
    float* const ws = sm + 8;            // 8 waves x 4 dim groups x (4 sums + the weight)
    float* const Ot = ws + 8 * 4 * 5;    // [8 waves][8 heads][32 dims]: a wave's weighted sums on their way to its stores
    bool ok = true;
    const int n_pos = *at.n_pos;
    const int kpb = max(1, (n_pos + AS - 1) / AS);
    {
        const int kvh = b & 1, split = b >> 1;
        const int k0 = split * kpb, k1 = min(n_pos, k0 + kpb), pos_new = n_pos - 1;
        const int nk = k1 - k0;                                   // keys of the range (none: nothing to do, nothing published)
        const int new_at = (pos_new >= k0 && pos_new < k1) ? pos_new - k0 : -1;   // the new position's place in the range
        const int n_old = new_at >= 0 ? nk - 1 : nk;              // ... the others are in the cache already
        const g_u16* kb = (const g_u16*)at.k_slab + (int64_t)k0 * (NKV * HD) + kvh * HD;
        const g_u16* vb = (const g_u16*)at.v_slab + (int64_t)k0 * (NKV * HD) + kvh * HD;
        typedef __attribute__((address_space(1))) v4u g_v4u;
        auto ld16 = [](const g_u16* q) {
            const v4u t = *(const g_v4u*)q;
            return make_uint4(t.x, t.y, t.z, t.w);
        };
        uint4 rk[4], rv[4];
        auto fetch_kv = [&](int t0) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int idx = tid + i * CT, key = t0 + (idx >> 5), seg = idx & 31;
                const bool live = key < n_old;
                rk[i] = live ? ld16(kb + (int64_t)key * (NKV * HD) + seg * 8) : make_uint4(0, 0, 0, 0);
                rv[i] = live ? ld16(vb + (int64_t)key * (NKV * HD) + seg * 8) : make_uint4(0, 0, 0, 0);
            }
        };
        auto stash_kv = [&](int t0) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int idx = tid + i * CT, key = idx >> 5, seg = idx & 31;
                if (t0 + key == new_at) continue;   // the new position's rows come from the waves that form them
                *(uint4*)(Ks + key * KSTR + seg * 8) = rk[i];
                *(uint4*)(Vs + key * KSTR + seg * 8) = rv[i];
            }
        };
        uint2 fresh = make_uint2(0, 0);   // wave 0: the new key row's four f16 of this lane; wave 1: the new value row's
        if (nk > 0) {
            fetch_kv(0);
            for (int i = tid; i < 16 * PSTR / 2; i += CT) ((uint32_t*)(P16 + 16 * PSTR))[i] = 0u;
            // (the two waves that form the new position's key and value rows ask for them together with their query:
            // one round trip, not two; every other block's merge waits for this block's results)
            float4 qv, nv = make_float4(0.f, 0.f, 0.f, 0.f);
            const u64* const qreg = ll + RQ + (kvh * AG + wave) * 2 * HD;
            const bool forms_row = new_at >= 0 && wave < 2;
            if (forms_row) {
                const u64* const nreg = ll + (wave == 0 ? RK : RV) + kvh * HD;
                const u64* const a4[4] = {qreg + 4 * lane, qreg + 4 * lane + 2, nreg + 4 * lane, nreg + 4 * lane + 2};
                uint32_t o8[8];
                ok = ll_wait_pairs<4>(a4, e, ctl, o8);
                qv = make_float4(__uint_as_float(o8[0]), __uint_as_float(o8[1]), __uint_as_float(o8[2]), __uint_as_float(o8[3]));
                nv = make_float4(__uint_as_float(o8[4]), __uint_as_float(o8[5]), __uint_as_float(o8[6]), __uint_as_float(o8[7]));
            } else {
                ok = ll_wait_quad(qreg, lane, e, ctl, &qv);
            }
            if (ok) {
                qv = head_norm_rope<HD>(qv, at.q_norm, at.eps_head, at.rope, at.n_rot, pos_new, lane);
                // scaled for a base-2 softmax and split into an f16 pair (22 bits): the matrix cores take both halves
                const float qsc = at.scale * 1.4426950408889634f;
                const float x[4] = {qv.x * qsc, qv.y * qsc, qv.z * qsc, qv.w * qsc};
                uint16_t hi[4], lo[4];
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const _Float16 h = (_Float16)x[i];
                    hi[i] = __builtin_bit_cast(uint16_t, h);
                    lo[i] = __builtin_bit_cast(uint16_t, (_Float16)(x[i] - (float)h));
                }
                *(uint2*)(Q16 + wave * KSTR + 4 * lane) = make_uint2(hi[0] | ((uint32_t)hi[1] << 16), hi[2] | ((uint32_t)hi[3] << 16));
                *(uint2*)(Q16 + (8 + wave) * KSTR + 4 * lane) = make_uint2(lo[0] | ((uint32_t)lo[1] << 16), lo[2] | ((uint32_t)lo[3] << 16));
            }
            if (ok && forms_row) {
                {   // the new position's key (norm + rotation) or value row: to the cache, and kept for the tile
                    if (wave == 0) nv = head_norm_rope<HD>(nv, at.k_norm, at.eps_head, at.rope, at.n_rot, pos_new, lane);
                    fresh.x = (uint32_t)it_f32_to_f16(nv.x) | ((uint32_t)it_f32_to_f16(nv.y) << 16);
                    fresh.y = (uint32_t)it_f32_to_f16(nv.z) | ((uint32_t)it_f32_to_f16(nv.w) << 16);
                    typedef __attribute__((address_space(1))) v2u g_v2u;
                    *(g_v2u*)((g_u16*)(wave == 0 ? at.k_slab : at.v_slab) + (int64_t)pos_new * (NKV * HD) + kvh * HD + 4 * lane) = v2u{fresh.x, fresh.y};
                }
            }
        }
        AC_STAMP(0);   // rows issued, queries (and the new key / value) gathered and prepared
        __syncthreads();
        AC_STAMP(1);
        if (nk > 0) {
            // Scores and weighted values on the f16 matrix cores, exact in their operands: K and V rows are f16 as
            // stored, queries and probabilities go in as f16 pairs (the low halves in columns of their own, added
            // afterwards), sums in f32.
            //   S = K Q^T   v_mfma_f32_16x16x32_f16, 16 keys x (8 heads' high halves | 8 heads' low halves), waves 0..3 one
            //               tile of 16 keys each, eight steps of 32 dims; lane l supplies 8 dims of key / column l % 16
            //               at dims 8 * (l / 16) and receives column l % 16, keys 4 * (l / 16) + {0..3}
            //   O^T = V^T P^T  v_mfma_f32_32x32x16_f16, wave w the 32 dims 32 w .., columns as above (+ 16 of zeros), a step
            //               per 16 keys; lane l supplies 8 keys of dim / column l % 32 at keys 8 * (l / 32) (the V^T
            //               operand two bytes at a time from the [key][dim] tile) and receives column l % 32, dims
            //               8 * (i / 4) + 4 * (l / 32) + i % 4
            // The softmax between them runs a wave a head, a lane a key, with the scores and the probabilities in LDS.
            typedef _Float16 h8 __attribute__((ext_vector_type(8)));
            typedef float v4f __attribute__((ext_vector_type(4)));
            typedef float v16f __attribute__((ext_vector_type(16)));
            auto ror8 = [](float v) {   // the value of the lane eight further on in its row of 16
                return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x128, 0xf, 0xf, true));
            };
            float m_run = -INFINITY, l_run = 0.0f;
            v16f o;
#pragma unroll
            for (int i = 0; i < 16; i++) o[i] = 0.0f;
            const int c16 = lane & 15, g4 = lane >> 4, c32 = lane & 31, g2 = lane >> 5;
            for (int t0 = 0; t0 < nk; t0 += TK) {
                if (t0) __syncthreads();   // every wave is done with the tile before
                stash_kv(t0);
                if (new_at >= t0 && new_at < t0 + TK && wave < 2) *(uint2*)((wave == 0 ? Ks : Vs) + (new_at - t0) * KSTR + 4 * lane) = fresh;
                __syncthreads();
                if (t0 + TK < nk) fetch_kv(t0 + TK);
                const int nt = min(TK, nk - t0);
                // (rows behind the tile's last key are zeros: the staging wrote all 64)
                if (wave < 4 && 16 * wave < nt) {
                    v4f sacc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int st = 0; st < HD / 32; st++) {
                        const h8 ka = *(const h8*)(Ks + (16 * wave + c16) * KSTR + 32 * st + 8 * g4);
                        const h8 qb = *(const h8*)(Q16 + c16 * KSTR + 32 * st + 8 * g4);
                        sacc = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka, qb, sacc, 0, 0, 0);
                    }
#pragma unroll
                    for (int i = 0; i < 4; i++) sacc[i] += ror8(sacc[i]);   // high + low halves
                    if (c16 < AG) *(float4*)(Sf + c16 * TK + 16 * wave + 4 * g4) = make_float4(sacc[0], sacc[1], sacc[2], sacc[3]);
                }
                __syncthreads();
                {
                    const float sc = lane < nt ? Sf[wave * TK + lane] : -INFINITY;
                    const float m_new = fmaxf(m_run, group_max<64>(sc));   // finite: the tile has a key
                    const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
                    const float pr = __builtin_amdgcn_exp2f(sc - m_new);
                    const _Float16 ph = (_Float16)pr;
                    P16[wave * PSTR + lane] = __builtin_bit_cast(uint16_t, ph);
                    P16[(8 + wave) * PSTR + lane] = __builtin_bit_cast(uint16_t, (_Float16)(pr - (float)ph));
                    if (lane == 0) Af[wave] = alpha;
                    l_run = l_run * alpha + group_sum<64>(pr);
                    m_run = m_new;
                }
                __syncthreads();
                {
                    const float al = Af[c32 & 7];
#pragma unroll
                    for (int i = 0; i < 16; i++) o[i] *= al;
                    for (int ks = 0; ks < (nt + 15) / 16; ks++) {
                        const uint16_t* vp = Vs + (16 * ks + 8 * g2) * KSTR + 32 * wave + c32;
                        uint32_t a[4];
#pragma unroll
                        for (int q = 0; q < 4; q++) a[q] = (uint32_t)vp[(2 * q) * KSTR] | ((uint32_t)vp[(2 * q + 1) * KSTR] << 16);
                        const h8 va = __builtin_bit_cast(h8, make_uint4(a[0], a[1], a[2], a[3]));
                        const h8 pb = *(const h8*)(P16 + c32 * PSTR + 16 * ks + 8 * g2);
                        o = __builtin_amdgcn_mfma_f32_32x32x16_f16(va, pb, o, 0, 0, 0);
                    }
                }
            }
            AC_STAMP(2);   // the range's keys done
#pragma unroll
            for (int i = 0; i < 16; i++) o[i] += ror8(o[i]);   // high + low halves of the probabilities
            // The wave's 8 heads x 32 dims sit in 16 of its lanes, 16 values each; stored from there they would be eight
            // stores of a quarter-full wave.  Through a piece of LDS of the wave's own (no barrier: a wave's LDS
            // operations complete in order) every lane gets four dims of one head: two full stores.
            {
                float* const Ow = Ot + wave * (AG * 32);   // [8 heads][32 dims]
                if (c32 < AG) {
#pragma unroll
                    for (int q = 0; q < 4; q++) *(float4*)(Ow + c32 * 32 + 8 * q + 4 * g2) = make_float4(o[4 * q], o[4 * q + 1], o[4 * q + 2], o[4 * q + 3]);
                }
                const int hd8 = lane >> 3, d4 = lane & 7;
                const float4 ov = *(const float4*)(Ow + hd8 * 32 + 4 * d4);
                u64* part = ll + RP + (int64_t)((kvh * AG + hd8) * AS + split) * PW + 32 * wave + 4 * d4;
                ll_put2f(part, ov.x, ov.y, e);
                ll_put2f(part + 2, ov.z, ov.w, e);
            }
            if (lane == 0) {   // wave = head for the softmax's sums
                u64* part = ll + RP + (int64_t)((kvh * AG + wave) * AS + split) * PW;
                ll_putf(part + HD, m_run, e);
                ll_putf(part + HD + 1, l_run, e);
            }
        }
    }
    AC_STAMP(3);   // partial results published
    {
        const int h = b >> 4, dc = b & 15;
        const int n_live = (n_pos + kpb - 1) / kpb;   // ranges that hold keys
        const int sp = tid >> 2, q4 = tid & 3;
        float m_s = -INFINITY, l_s = 0.0f;
        float4 o_s = make_float4(0.f, 0.f, 0.f, 0.f);
        // (the gate of this thread's dim, the head's second half of wq's output: published a stage ago; asked for ahead of
        // the ranges' results, whose wait hides the round trip)
        uint32_t gw = 0;
        if (tid < 16 && !ll_wait1(ll + RQ + h * 2 * HD + HD + dc * 16 + tid, e, ctl, &gw)) ok = false;
        if (sp < n_live) {
            const u64* base = ll + RP + (int64_t)(h * AS + sp) * PW;
            const u64* const a4[4] = {base + dc * 16 + q4 * 4, base + dc * 16 + q4 * 4 + 2, base + HD, base + HD};
            uint32_t w8[8];
            if (ll_wait_pairs<4>(a4, e, ctl, w8)) {
                o_s = make_float4(__uint_as_float(w8[0]), __uint_as_float(w8[1]), __uint_as_float(w8[2]), __uint_as_float(w8[3]));
                m_s = __uint_as_float(w8[4]);
                l_s = __uint_as_float(w8[5]);
            } else {
                ok = false;
            }
        }
        AC_STAMP(4);   // the ranges' results gathered
        const float mx = group_max<64>(m_s);
        if (lane == 0) sm[wave] = mx;
        __syncthreads();
        float big = sm[0];
#pragma unroll
        for (int w = 1; w < CW; w++) big = fmaxf(big, sm[w]);
        const float wgt = m_s != -INFINITY ? __builtin_amdgcn_exp2f(m_s - big) : 0.0f;
        float vals[5] = {wgt * o_s.x, wgt * o_s.y, wgt * o_s.z, wgt * o_s.w, wgt * l_s};
#pragma unroll
        for (int i = 0; i < 5; i++) {
            vals[i] += __shfl_xor(vals[i], 4, 64);
            vals[i] += __shfl_xor(vals[i], 8, 64);
            vals[i] += __shfl_xor(vals[i], 16, 64);
            vals[i] += __shfl_xor(vals[i], 32, 64);
        }
        if (lane < 4) {
#pragma unroll
            for (int i = 0; i < 5; i++) ws[(wave * 4 + lane) * 5 + i] = vals[i];
        }
        __syncthreads();
        if (tid < 16) {
            const int q = tid >> 2, i = tid & 3;
            float osum = 0.0f, lsum = 0.0f;
#pragma unroll
            for (int w = 0; w < CW; w++) {
                osum += ws[(w * 4 + q) * 5 + i];
                lsum += ws[(w * 4 + q) * 5 + 4];
            }
            ll_putf(ll + RT + h * HD + dc * 16 + tid, osum / lsum * fx_sigmoid(__uint_as_float(gw)), e);
        }
    }
    AC_STAMP(5);   // merged and published
    // out-projection (quantize + matmul, qwen35.rs:1216-1223): the gated output of every head, Q8_0 (in the K tile's
    // place: the barriers of the merge are behind every read of it), this wave's row
    float dot;
    {
        const int my_row = b * CW + wave;
        WChunks<4> wo;
        load_row<W_Q8_0, 4, 64>(wo, at.o_q, at.o_s, VDIM, my_row, lane, true);
        int8_t* const oq = (int8_t*)chain_dyn_lds;
        float* const os = (float*)(chain_dyn_lds + NH * HD);
        const u64* const a4[4] = {ll + RT + 4 * tid, ll + RT + 4 * tid + 2, ll + RT + 4 * (tid + CT), ll + RT + 4 * (tid + CT) + 2};
        uint32_t o8[8];
        if (!ll_wait_pairs<4>(a4, e, ctl, o8)) ok = false;
        AC_STAMP(6);   // the gated output gathered
        quant_quad(make_float4(__uint_as_float(o8[0]), __uint_as_float(o8[1]), __uint_as_float(o8[2]), __uint_as_float(o8[3])), true, tid, oq, os);
        quant_quad(make_float4(__uint_as_float(o8[4]), __uint_as_float(o8[5]), __uint_as_float(o8[6]), __uint_as_float(o8[7])), true, tid + CT, oq, os);
        __syncthreads();
        XChunks<W_Q8_0, 4> x;
        load_x<W_Q8_0, 4, 64>(x, oq, os, lane);
        dot = reduce_lanes<64>(dot_chunks<W_Q8_0, 4>(wo, x));
    }
    AC_STAMP(7);
    return AttnCoreR{dot, ok ? 1 : 0};
}

template <int SF, int RF, int NL>
__global__ __launch_bounds__(CT) void layer_chain_k(ChainPT<NL> p) {
    __shared__ __align__(16) int8_t xq[NU * FF + FF];   // the stage's quantized activation (largest: the down stage's)
    __shared__ __align__(16) float xs[(NU * FF + FF) / 32];
    __shared__ double red[CW];
    __shared__ __align__(16) float kq[2 * DK];
    __shared__ __align__(16) float ssq[NB];
    __shared__ float sm[64];
    __shared__ __align__(16) float inter[32];
    __shared__ RouteLds<CT> route_sh;
    __shared__ int ids[16];
    __shared__ __align__(16) float wts[16];
    __shared__ float coef[16];
    __shared__ int dead;
    __shared__ float fpart[2 * CW];   // partial dots of rows shared by the waves (RF)
    float* const xf = RF ? (float*)route_sh.keys : nullptr;   // the normed f32 vector of stages A and D (the route's keys come later)
    const int tid0 = threadIdx.x, b0 = blockIdx.x;
    const Ctl ctl{p.abort_flag, p.spin_limit};
    const unsigned e0 = *(const volatile unsigned*)p.epoch;
    if (tid0 == 0) dead = 0;
    // lane 63 of a wave owns one row of the residual stream: row 8 * block + wave
    float x_row = (tid0 & 63) == 63 ? p.x[b0 * CW + (tid0 >> 6)] : 0.0f;
    AW aw;
    if (p.layer[0].has_mixer == 1) fetch_a<RF>(p.layer[0].m, aw, b0, __builtin_amdgcn_readfirstlane(tid0 >> 6), tid0 & 63);
    if (p.layer[0].has_mixer == 3) fetch_tail(p.layer[0].a, aw, b0, __builtin_amdgcn_readfirstlane(tid0 >> 6), tid0 & 63);
    __syncthreads();

#ifdef IT_CHAIN_STAMPS
    long long tprev = wall_clock64(), wprev = tprev;
#endif
    for (int l = 0; l < p.n_layers; l++) {
        // The thread's coordinates pass through an empty asm statement once per layer.  Everything addressed from them
        // (hand-off words, weight rows, LDS slots) is then computed where it is used, a few integer operations, instead
        // of being hoisted out of the layer loop as loop invariants and held in a hundred registers across it.
        int tid = tid0, b = b0;
        asm volatile("" : "+v"(tid), "+s"(b));
        int lane = tid & 63;
        int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        int my_row = b * CW + wave;
        // (again before the FFN's stages: what they address is computed there, not held across the mixer's)
#define CHAIN_RECOORD()                                        \
        do {                                                   \
            tid = tid0;                                        \
            b = b0;                                            \
            asm volatile("" : "+v"(tid), "+s"(b));             \
            lane = tid & 63;                                   \
            wave = __builtin_amdgcn_readfirstlane(tid >> 6);   \
            my_row = b * CW + wave;                            \
        } while (0)
        const auto& L = p.layer[l];
        const auto& m = L.m;
        const auto& f = L.f;
        const unsigned e = e0 + 1 + (unsigned)l;
        const bool mixer = L.has_mixer != 0;   // the FFN's input comes from a mixer stage of this kernel

        // Stage D's rows.  Waves 0, 1: router rows b and NB + b; waves 2, 3: gate and up rows 2 b and 2 b + 1 of the
        // shared expert; wave 4 of the last block: the shared expert's gate-logit row.  Issued at the head of the stage
        // before D (small loads issued at the head of a stage are back before its input is).
        WChunks<2> d0, d1;
        WChunks<1> n0, n1;
        const int sh_row = 2 * b + (wave - 2);
        float4 rf0, rf1, lf;   // RF: this wave's quarter of an unquantized router row (two float4 a lane), its eighth of the gate-logit row
        auto fetch_d = [&]() {
            const bool r = wave < 2, sh = wave == 2 || wave == 3, lg = wave == 4 && b == NB - 1;
            if (RF) {
                // unquantized router and gate-logit rows: row b in waves 0..3, row NB + b in waves 4..7, 512 floats a wave;
                // the gate-logit row in the last block, 256 floats a wave; the partial dots meet in LDS
                const float4* row = (const float4*)((const float*)f.r_q + (int64_t)(b + NB * (wave >> 2)) * D) + (wave & 3) * 128;
                rf0 = row[lane];
                rf1 = row[64 + lane];
                lf = b == NB - 1 ? ((const float4*)f.l_q)[wave * 64 + lane] : make_float4(0.f, 0.f, 0.f, 0.f);
                if (SF == W_Q8_0) {
                    load_row<W_Q8_0, 2, 64>(d0, f.sg_q, f.sg_s, D, sh_row, lane, sh);
                    load_row<W_Q8_0, 2, 64>(d1, f.su_q, f.su_s, D, sh_row, lane, sh);
                } else {
                    load_row<W_NVFP4, 1, 64>(n0, f.sg_q, f.sg_s, D, sh_row, lane, sh);
                    load_row<W_NVFP4, 1, 64>(n1, f.su_q, f.su_s, D, sh_row, lane, sh);
                }
            } else if (SF == W_Q8_0) {
                load_row<W_Q8_0, 2, 64>(d0, r ? f.r_q : sh ? f.sg_q : f.l_q, r ? f.r_s : sh ? f.sg_s : f.l_s, D,
                                      r ? b + NB * wave : sh ? sh_row : 0, lane, r || sh || lg);
                load_row<W_Q8_0, 2, 64>(d1, f.su_q, f.su_s, D, sh_row, lane, sh);
            } else {
                load_row<W_Q8_0, 2, 64>(d0, r ? f.r_q : f.l_q, r ? f.r_s : f.l_s, D, r ? b + NB * wave : 0, lane, r || lg);
                load_row<W_NVFP4, 1, 64>(n0, f.sg_q, f.sg_s, D, sh_row, lane, sh);
                load_row<W_NVFP4, 1, 64>(n1, f.su_q, f.su_s, D, sh_row, lane, sh);
            }
        };
        if (!mixer) fetch_d();

        if (L.has_mixer == 2) {
            // ---------------------------------------------------------------- the attention block's out-projection + residual
            // (quantize + matmul + add_assign, qwen35.rs:1216-1223; the input is in ordinary memory: the merge kernel wrote it)
            WChunks<4> wo;
            load_row<W_Q8_0, 4, 64>(wo, m.o_q, m.o_s, VDIM, my_row, lane, true);
            fetch_d();
#pragma unroll
            for (int k = 0; k < 2; k++) quant_quad(((const float4*)m.attn)[tid + k * CT], true, tid + k * CT, xq, xs);
            __syncthreads();
            XChunks<W_Q8_0, 4> x;
            load_x<W_Q8_0, 4, 64>(x, xq, xs, lane);
            const float acc = reduce_lanes<64>(dot_chunks<W_Q8_0, 4>(wo, x));
            if (lane == 63) {
                x_row += acc;
                ll_putf(p.ll + RC + my_row, x_row, e);
            }
        }
        if (L.has_mixer == 3) {
            // ---------------------------------------------------------------- a whole attention mixer
            // (qwen35.rs:1141-1223: rms_norm, wq / wk / wv, head norms, rotation, cache rows, attention, sigmoid gate,
            // out-projection + residual.)  Three exchanges more than a Gated DeltaNet mixer's: the in-projection's
            // outputs, the key ranges' partial results, the gated output.
            const auto& at = L.a;
            {
                const float4 nw = ((const float4*)at.norm_w)[tid];
                float4 v;
                bool ok = true;
                if (l == 0) v = ((const float4*)p.x)[tid];
                else ok = ll_wait_quad(p.ll + RX, tid, e, ctl, &v);
                if (!ok) dead = 1;
                CH_STAMP(16);
                if (!norm_quant(v, nw, at.eps, xq, xs, red, &dead, tid)) break;
                XChunks<W_Q8_0, 2> x;
                load_x<W_Q8_0, 2, 64>(x, xq, xs, lane);
                float mine = 0.0f;
#pragma unroll
                for (int k = 0; k < 5; k++) {
                    const float acc = reduce_lanes<64>(dot_chunks<W_Q8_0, 2>(aw.t[k], x));
                    const float r = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, acc), 63));
                    mine = lane == k ? r : mine;
                }
                if (lane < 4) ll_putf(p.ll + RQ + b + NB * (wave + CW * lane), mine, e);
                else if (lane == 4 && wave < 2) ll_putf(p.ll + RK + b + NB * wave, mine, e);
                else if (lane == 4 && wave < 4) ll_putf(p.ll + RV + b + NB * (wave - 2), mine, e);
            }
            CH_STAMP(17);
            // ---------------------------------------------------------------- attention over the context, merge, sigmoid gate
            // (a function of its own: its registers are allotted apart from the stages around it, which have none to spare)
            forget(aw);
            const AttnCoreR r = attn_core(at.q_norm, at.k_norm, at.rope, at.k_slab, at.v_slab, at.n_pos, m.o_q, m.o_s, at.eps_head, at.scale, at.n_rot,
                                          (it_gptr<u64>)p.ll, e, (it_gptr<unsigned>)p.abort_flag, p.spin_limit, tid, b);
            CH_STAMP(18);
            fetch_d();
            if (!r.ok) dead = 1;
            if (lane == 63) {   // + residual
                x_row += r.dot;
                ll_putf(p.ll + RC + my_row, x_row, e);
            }
            __syncthreads();
            if (dead) break;
        }
        if (L.has_mixer == 1) {
            // ---------------------------------------------------------------- loads known from the start of the layer
            const int h = b >> 3, j0 = (b & 7) * 16, kh = h % NK;
            float* S = m.state + ((int64_t)(h * DK + j0 + (tid >> 5)) * DK + (tid & 31) * 4);
            const float4 st = *(const float4*)S;
            const float4 nw = ((const float4*)m.norm_w)[tid];
            const float ssm_a = m.ssm_a[h], dt_bias = m.dt_bias[h];
            const float head_w = m.head_norm_w[j0 + (tid >> 5)];

            WChunks<4> wc;   // the out-projection's row of this wave
            // ---------------------------------------------------------------- A: in-projection
            {
                float4 v;
                bool ok = true;
                if (l == 0) v = ((const float4*)p.x)[tid];
                else ok = ll_wait_quad(p.ll + RX, tid, e, ctl, &v);
                if (!ok) dead = 1;
                if (!norm_quant(v, nw, m.eps_norm, xq, xs, red, &dead, tid, xf)) break;
                if (IT_CHAIN_WC_AT == 1) load_row<W_Q8_0, 4, 64>(wc, m.o_q, m.o_s, VDIM, my_row, lane, true);
                CH_STAMP(0);
                XChunks<W_Q8_0, 2> x;
                load_x<W_Q8_0, 2, 64>(x, xq, xs, lane);
                float acc[7];
#pragma unroll
                for (int k = 0; k < 7; k++) acc[k] = (RF && k == 6) ? 0.0f : reduce_lanes<64>(dot_chunks<W_Q8_0, 2>(aw.t[k], x));
                if (IT_CHAIN_WC_AT == 2) load_row<W_Q8_0, 4, 64>(wc, m.o_q, m.o_s, VDIM, my_row, lane, true);
                // row k's dot goes from lane 63 to lane k, which finishes the row
                float mine = 0.0f;
#pragma unroll
                for (int k = 0; k < 7; k++) {
                    const float v = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, acc[k]), 63));
                    mine = lane == k ? v : mine;
                }
                if (lane < 4) {
                    // causal conv (kernel 4) + silu on channel `row`, state [channel][3] oldest first
                    const int64_t row = b + NB * (wave + CW * lane);
                    float sum = 0.0f;
                    sum += aw.past[0] * aw.taps.x;
                    sum += aw.past[1] * aw.taps.y;
                    sum += aw.past[2] * aw.taps.z;
                    sum += mine * aw.taps.w;
                    ll_putf(p.ll + RA + row, fx_silu(sum), e);
                    float* past = m.conv_state + row * 3;
                    past[0] = aw.past[1];
                    past[1] = aw.past[2];
                    past[2] = mine;
                } else if (lane < 6) {
                    ll_putf(p.ll + RA_Z + b + NB * (wave + CW * (lane - 4)), fx_silu(mine), e);
                } else if (!RF && lane == 6 && wave == 0 && b < 2 * NV) {
                    ll_putf(p.ll + RA_AL + b, mine, e);
                }
                if (RF) {
                    // the unquantized alpha / beta row of blocks 0..63 against the normed f32 vector: every wave its 256 floats
                    const float4 xa = ((const float4*)xf)[wave * 64 + lane];
                    const float part = reduce_lanes<64>(f32_chunk(aw.ab, xa));
                    if (lane == 63) fpart[wave] = part;
                    __syncthreads();
                    if (tid == 0 && b < 2 * NV) ll_putf(p.ll + RA_AL + b, f32_tree(fpart), e);
                }
            }
            // ---------------------------------------------------------------- B: delta rule
            CH_STAMP(1);
            // (the out-projection's row goes out first: small loads issued at the head of a stage are back before its input is)
#if IT_CHAIN_B_POLLERS
            // Waves 5..7 gather the stage's 290 words and issue their out-projection row only afterwards; waves 0..4 issue
            // theirs now and poll nothing: a poll returns behind everything its own wave has in flight.
            if (wave < 5) load_row<W_Q8_0, 4, 64>(wc, m.o_q, m.o_s, VDIM, my_row, lane, true);
            float k_scale, q_scale;
            {
                bool ok = true;
                if (wave >= 5) {
                    const int pt = tid - 5 * 64;
                    if (pt < DK) {   // wave 5: the key head's k as 64 pairs, wave 6: its q
                        const int i2 = (pt & 63) * 2;
                        const u64* const a1[1] = {p.ll + (pt < 64 ? RA + KDIM : RA) + kh * DK + i2};
                        uint32_t o[2];
                        ok = ll_wait_pairs<1>(a1, e, ctl, o);
                        const float x0 = __uint_as_float(o[0]), x1 = __uint_as_float(o[1]);
                        *(float2*)(kq + (pt < 64 ? 0 : DK) + i2) = make_float2(x0, x1);
                        // l2 norm: the vector's sum of squares in its own wave (f64 sums of f32 squares: exact, so the
                        // order of the terms does not matter)
                        const double part = wave_sum_f64_tail((double)(x0 * x0) + (double)(x1 * x1));
                        if (lane == 63) red[wave - 5] = part;
                    } else if (pt < DK + 16) {   // 8 pairs of v, 8 pairs of z
                        const int i2 = ((pt - DK) & 7) * 2, j = h * DK + j0 + i2;
                        const bool zz = pt >= DK + 8;
                        const u64* const a1[1] = {p.ll + (zz ? RA_Z : RA + 2 * KDIM) + j};
                        uint32_t o[2];
                        ok = ll_wait_pairs<1>(a1, e, ctl, o);
                        sm[(zz ? 16 : 0) + i2] = __uint_as_float(o[0]);
                        sm[(zz ? 16 : 0) + i2 + 1] = __uint_as_float(o[1]);
                    } else if (pt < DK + 18) {
                        uint32_t w0 = 0;
                        ok = ll_wait1(p.ll + (pt == DK + 16 ? RA_AL : RA_BE) + h, e, ctl, &w0);
                        sm[32 + pt - (DK + 16)] = __uint_as_float(w0);
                    }
                    load_row<W_Q8_0, 4, 64>(wc, m.o_q, m.o_s, VDIM, my_row, lane, true);
                }
                if (!ok) dead = 1;
                __syncthreads();
                if (dead) break;
                CH_STAMP(2);
                if (IT_CHAIN_D_AT) fetch_d();
                k_scale = 1.0f / fmaxf(sqrtf((float)red[0]), m.eps_l2);
                q_scale = 1.0f / fmaxf(sqrtf((float)red[1]), m.eps_l2);
#else
            if (!IT_CHAIN_WC_AT) load_row<W_Q8_0, 4, 64>(wc, m.o_q, m.o_s, VDIM, my_row, lane, true);
            const float k_scale = 1.0f, q_scale = 1.0f;
            {
                uint32_t w0 = 0, w1 = 0;
                bool ok = true;
                if (tid < 2 * DK) {
                    ok = ll_wait1(p.ll + (tid < DK ? RA + KDIM + kh * DK + tid : RA + kh * DK + (tid - DK)), e, ctl, &w0);
                } else if (tid < 2 * DK + 16) {
                    const int j = h * DK + j0 + (tid - 2 * DK);
                    ok = ll_wait1(p.ll + RA + 2 * KDIM + j, e, ctl, &w0) && ll_wait1(p.ll + RA_Z + j, e, ctl, &w1);
                    sm[tid - 2 * DK] = __uint_as_float(w0);
                    sm[16 + tid - 2 * DK] = __uint_as_float(w1);
                } else if (tid < 2 * DK + 18) {
                    ok = ll_wait1(p.ll + (tid == 2 * DK + 16 ? RA_AL : RA_BE) + h, e, ctl, &w0);
                    sm[32 + tid - (2 * DK + 16)] = __uint_as_float(w0);
                }
                if (!ok) dead = 1;
                // l2 norm of k (threads 0..127) and q (128..255): each vector's sum of squares in its own two waves
                const float kqv = tid < 2 * DK ? __uint_as_float(w0) : 0.0f;
                const double part = wave_sum_f64_tail((double)(kqv * kqv));
                if (lane == 63) red[wave] = part;
                __syncthreads();
                if (dead) break;
                CH_STAMP(2);
                if (IT_CHAIN_D_AT) fetch_d();
                if (IT_CHAIN_WC_AT == 3) load_row<W_Q8_0, 4, 64>(wc, m.o_q, m.o_s, VDIM, my_row, lane, true);
                if (tid < 2 * DK) {
                    const int w2 = tid < DK ? 0 : 2;
                    const double sum = red[w2] + red[w2 + 1];
                    kq[tid] = kqv * (1.0f / fmaxf(sqrtf((float)sum), m.eps_l2));
                }
                __syncthreads();
#endif
                const float a = sm[32] + dt_bias;
                const float softplus = a > 20.0f ? a : fx_logf(1.0f + fx_expf(a));
                const float g = fx_expf(softplus * ssm_a);
                const float beta = fx_sigmoid(sm[33]);
                const int j = tid >> 5, seg = tid & 31;
                const float4 kk = *(const float4*)(kq + seg * 4), qq = *(const float4*)(kq + DK + seg * 4);
                float row[4] = {st.x, st.y, st.z, st.w};
                const float kv[4] = {kk.x * k_scale, kk.y * k_scale, kk.z * k_scale, kk.w * k_scale};
                const float qv[4] = {qq.x * q_scale, qq.y * q_scale, qq.z * q_scale, qq.w * q_scale};
                float pred = 0.0f;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    row[i] *= g;
                    pred += row[i] * kv[i];
                }
                pred = group_sum<32>(pred);
                const float delta = beta * (sm[j] - pred);
                float o = 0.0f;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    row[i] += kv[i] * delta;
                    o += row[i] * (qv[i] * m.q_scale);
                }
                o = group_sum<32>(o);
                *(float4*)S = make_float4(row[0], row[1], row[2], row[3]);
                if (seg == 0) {
                    // silu(z) * (o * hs * w) with the head's scale hs applied by the reader, which sums the squares
                    ll_putf(p.ll + RB + h * DK + j0 + j, sm[16 + j] * (o * head_w), e);
                    sm[40 + j] = o * o;
                }
                __syncthreads();
                if (tid == 0) {
                    float s = 0.0f;
#pragma unroll
                    for (int i = 0; i < 16; i++) s += sm[40 + i];
                    ll_putf(p.ll + RB_SS + b, s, e);
                }
            }
            // ---------------------------------------------------------------- C: out-projection + residual
            CH_STAMP(3);
            if (!IT_CHAIN_D_AT) fetch_d();
            {
                const u64* const a4[4] = {p.ll + RB + 4 * tid, p.ll + RB + 4 * tid + 2, p.ll + RB + 4 * (tid + CT), p.ll + RB + 4 * (tid + CT) + 2};
                uint32_t o[8];
                bool ok = ll_wait_pairs<4>(a4, e, ctl, o);
                if (tid < NB / 2) {
                    const u64* const a1[1] = {p.ll + RB_SS + 2 * tid};
                    uint32_t s2[2];
                    ok = ok && ll_wait_pairs<1>(a1, e, ctl, s2);
                    ssq[2 * tid] = __uint_as_float(s2[0]);
                    ssq[2 * tid + 1] = __uint_as_float(s2[1]);
                }
                if (!ok) dead = 1;
                __syncthreads();
                if (dead) break;
                CH_STAMP(4);
#pragma unroll
                for (int k = 0; k < 2; k++) {
                    const int qi = tid + k * CT, head = qi >> 5;
                    const float4 s0 = *(const float4*)(ssq + head * 8), s1 = *(const float4*)(ssq + head * 8 + 4);
                    const double sum = (double)s0.x + (double)s0.y + (double)s0.z + (double)s0.w + (double)s1.x + (double)s1.y +
                                       (double)s1.z + (double)s1.w;
                    const float hs = 1.0f / sqrtf((float)(sum / (double)DK) + m.eps_head);
                    const float4 v = make_float4(__uint_as_float(o[4 * k]) * hs, __uint_as_float(o[4 * k + 1]) * hs,
                                                 __uint_as_float(o[4 * k + 2]) * hs, __uint_as_float(o[4 * k + 3]) * hs);
                    quant_quad(v, true, qi, xq, xs);
                }
                __syncthreads();
                XChunks<W_Q8_0, 4> x;
                load_x<W_Q8_0, 4, 64>(x, xq, xs, lane);
                const float acc = reduce_lanes<64>(dot_chunks<W_Q8_0, 4>(wc, x));
                if (lane == 63) {
                    x_row += acc;
                    ll_putf(p.ll + RC + my_row, x_row, e);
                }
            }
        }

        // -------------------------------------------------------------------- D: router, shared gate logit, shared gate / up
        CH_STAMP(5);
        XN xn;
        {
            const float4 nw = ((const float4*)f.norm_w)[tid];
            float4 v;
            bool ok = true;
            if (mixer) ok = ll_wait_quad(p.ll + RC, tid, e, ctl, &v);
            else if (l == 0) v = ((const float4*)p.x)[tid];
            else ok = ll_wait_quad(p.ll + RX, tid, e, ctl, &v);
            if (!ok) dead = 1;
            if (!norm_quant(v, nw, f.eps, xq, xs, red, &dead, tid, xf)) break;
            if (l + 1 < p.n_layers && p.layer[l + 1].has_mixer == 1 && ((IT_CHAIN_A_AT >> 8) & 15))
                fetch_a<RF>(p.layer[l + 1].m, aw, b, wave, lane, (IT_CHAIN_A_AT >> 8) & 15);
            CH_STAMP(6);
            XChunks<W_Q8_0, 2> x;
            load_x<W_Q8_0, 2, 64>(x, xq, xs, lane);
            load_xn(xn, xq, xs, lane);
            if (RF) {
                const float4 xa = ((const float4*)xf)[(wave & 3) * 128 + lane], xb = ((const float4*)xf)[(wave & 3) * 128 + 64 + lane];
                const float pr = reduce_lanes<64>(f32_chunk(rf0, xa)) + reduce_lanes<64>(f32_chunk(rf1, xb));
                const float4 xl = ((const float4*)xf)[wave * 64 + lane];
                const float pl = reduce_lanes<64>(f32_chunk(lf, xl));
                if (lane == 63) {
                    fpart[wave] = pr;
                    fpart[CW + wave] = pl;
                }
            } else if (wave < 2 || (wave == 4 && b == NB - 1)) {
                const float a = reduce_lanes<64>(dot_chunks<W_Q8_0, 2>(d0, x));
                if (lane == 63) ll_putf(p.ll + RD + (wave < 2 ? b + NB * wave : NE), a, e);
            }
            if (wave == 2 || wave == 3) {
                float ag, au;
                if (SF == W_Q8_0) {
                    ag = reduce_lanes<64>(dot_chunks<W_Q8_0, 2>(d0, x));
                    au = reduce_lanes<64>(dot_chunks<W_Q8_0, 2>(d1, x));
                } else {
                    ag = reduce_lanes<64>(dot_xn(n0, xn));
                    au = reduce_lanes<64>(dot_xn(n1, xn));
                }
                if (lane == 63) {
                    ag *= f.sh_gscale;
                    au *= f.sh_uscale;
                    ll_putf(p.ll + RS + sh_row, fx_silu(ag) * au, e);
                }
            }
            if (RF) {
                __syncthreads();
                if (tid < 2) ll_putf(p.ll + RD + b + NB * tid, (fpart[4 * tid] + fpart[4 * tid + 1]) + (fpart[4 * tid + 2] + fpart[4 * tid + 3]), e);
                if (tid == 64 && b == NB - 1) ll_putf(p.ll + RD + NE, f32_tree(fpart + CW), e);
            }
        }

        // -------------------------------------------------------------------- E: route, routed gate / up
        CH_STAMP(7);
        CHAIN_RECOORD();
        WChunks<1> fd[3];
        WChunks<1> fsh;   // the shared expert's down row: lanes 32..63 (Q8_0) or 32..47 (NVFP4) beside the last two picks
        {
            // The route (softmax over the 512 logits, the 10 largest, src/ops/mod.rs:1191-1216), in the order that lets
            // the picks' rows start moving first: the picks are ranked on the logits themselves (the softmax keeps their
            // order), and the probabilities of the ten are formed afterwards, under the rows' flight.
            uint32_t w0 = 0;
            bool ok = ll_wait1(p.ll + RD + tid, e, ctl, &w0);
            const float my_logit = __uint_as_float(w0);
            const u64 my_key = ((u64)logit_order(my_logit) << 32) | (u64)(~(unsigned)tid);   // larger = earlier pick, unique
            route_sh.keys[tid] = my_key;
            if (tid < (CT / 64) * 16) route_sh.cand[tid] = 0ull;
            if (tid == 0) {
                ok = ok && ll_wait1(p.ll + RD + NE, e, ctl, &w0);
                sm[34] = __uint_as_float(w0);
            }
            if (!ok) dead = 1;
            __syncthreads();
            if (dead) break;
            CH_STAMP(8);
            CH_WSTAMP(0);
            // (a) a key's rank among the 64 of its wave: only wave ranks below 10 can be among the 10 of the block
            wave_rank_one(route_sh.keys + (tid & ~63), my_key, NU, route_sh.cand + wave * 16);
            __syncthreads();
            {   // (b) the 128 candidate slots against each other: four threads a slot, a quarter of the slots each
                const int c = tid >> 2, part = tid & 3;
                const u64 me = route_sh.cand[c];
                int cnt = 0;
#pragma unroll
                for (int c2 = 0; c2 < (CT / 64) * 2; c2++) {
                    const ulonglong2 q = ((const ulonglong2*)route_sh.cand)[c2 * 4 + part];
                    cnt += q.x > me ? 1 : 0;
                    cnt += q.y > me ? 1 : 0;
                }
                cnt += __shfl_xor(cnt, 1, 64);
                cnt += __shfl_xor(cnt, 2, 64);
                if (part == 0 && me != 0ull && cnt < NU) {
                    ids[cnt] = (int)~(unsigned)(me & 0xffffffffull);
                    wts[cnt] = logit_of_order((uint32_t)(me >> 32));   // the pick's logit; its probability follows below
                }
            }
            __syncthreads();
            CH_STAMP(9);
            CH_WSTAMP(1);
            const float my_dscale = (tid < NU && f.dscale2) ? f.dscale2[ids[tid]] : 1.0f;   // issued ahead of the rows below
            // Rows pulled towards the caches ahead of the loads that use them.  A wave's 16-byte-a-lane load asks for eight
            // 128-byte lines; one 4-byte load with every lane on a line of its own asks for 64, so a few such loads put a
            // whole stage's rows in flight at once, from compute units that have nothing else to fetch.
            // The blocks without routed rows (160..255) touch the gate / up rows of the 20 blocks that share their XCD
            // (blocks are dealt to the eight XCDs in turn, each XCD has its own L2): 9 loads a block served.
            uint32_t touched = 0;
            if (IT_CHAIN_TOUCH) {
                if (b >= EB) {
                    const int x = b & 7;
                    for (int wi = ((b - EB) >> 3) * CW + wave; wi < 20 * 9; wi += 12 * CW) {
                        const int tb = x + 8 * (wi / 9), part = wi % 9;
                        const int64_t ex = ids[tb >> 4];
                        const int r0 = (tb & 15) * 32;
                        const uint8_t* a;
                        if (part < 8) {   // eight rows of 1,024 bytes: gate (parts 0..3) or up (4..7)
                            const uint8_t* q = (part < 4 ? f.eg_q : f.eu_q) + ex * f.gu_q_stride;
                            a = q + (int64_t)(r0 + (part & 3) * 8 + (lane >> 3)) * (D / 2) + (lane & 7) * 128;
                        } else {          // the scales of the 32 gate rows (lanes 0..31) and of the 32 up rows
                            const uint8_t* sc = (lane < 32 ? f.eg_s : f.eu_s) + ex * f.gu_s_stride;
                            a = sc + (int64_t)(r0 + (lane & 31)) * (D / 16);
                        }
                        touched += *(const volatile uint32_t*)a;
                    }
                }
            }
            // the picks' rows: this block's 32 gate and 32 up rows
            WChunks<1> tg[4], tu[4];
            float scg = 1.0f, scu = 1.0f;
            if (b < EB) {
                const int y = b >> 4, sb = b & 15;
                const int64_t ex = ids[y];
                const uint8_t *gq = f.eg_q + ex * f.gu_q_stride, *gs = f.eg_s + ex * f.gu_s_stride;
                const uint8_t *uq = f.eu_q + ex * f.gu_q_stride, *us = f.eu_s + ex * f.gu_s_stride;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int j = sb * 32 + wave * 4 + i;
                    load_row<W_NVFP4, 1, 64>(tg[i], gq, gs, D, j, lane, true);
                    load_row<W_NVFP4, 1, 64>(tu[i], uq, us, D, j, lane, true);
                }
                if (f.gscale2) scg = f.gscale2[ex];
                if (f.uscale2) scu = f.uscale2[ex];
                CH_STAMP(13);
                CH_WSTAMP(2);
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    float ag = reduce_lanes<64>(dot_xn(tg[i], xn));
                    float au = reduce_lanes<64>(dot_xn(tu[i], xn));
                    if (lane == 63) {
                        ag *= scg;
                        au *= scu;
                        inter[wave * 4 + i] = fx_silu(ag) * au;
                    }
                    if (i == 0) CH_WSTAMP(3);
                }
            }
            CH_STAMP(14);
            CH_WSTAMP(4);
#if IT_CHAIN_FLOADS_EARLY
            // the down rows of this wave's output row, for stage F: issued behind the publication, they land while the intermediates travel
            // (four picks a step over 16 lanes each, the shared row beside the last two picks)
#pragma unroll
            for (int s = 0; s < 3; s++) {
                const int y = s * 4 + (lane >> 4);
                const bool routed = y < NU;
                const int64_t ex = routed ? ids[y] : 0;
                load_row<W_NVFP4, 1, 16>(fd[s], f.ed_q + ex * f.d_q_stride, f.ed_s + ex * f.d_s_stride, FF, my_row, lane & 15, routed);
            }
            if (SF == W_Q8_0) load_row<W_Q8_0, 1, 32>(fsh, f.sd_q, f.sd_s, FF, my_row, lane & 31, lane >= 32);
            else load_row<W_NVFP4, 1, 16>(fsh, f.sd_q, f.sd_s, FF, my_row, lane & 15, lane >= 32 && lane < 48);
#endif
            // the softmax's sum: exp(logit - largest logit) over the 512, by wave and then over the waves in order
            {
                const float part = group_sum_tail<64>(fx_expf(my_logit - wts[0]));
                if (lane == 63) route_sh.redf[wave] = part;
            }
            CH_STAMP(15);
            CH_WSTAMP(5);
            __syncthreads();
            CH_WSTAMP(6);
            if (b < EB) {
                if (tid < 8) {
                    // Q8_0 of the block's 32 intermediates (naive.rs:652-675), published as four quants a word
                    const float4 v = *(const float4*)(inter + tid * 4);
                    float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
                    amax = group_max<8>(amax);
                    const float d = amax / 127.0f;
                    const float id = d != 0.0f ? 1.0f / d : 0.0f;
                    const float r[4] = {roundf(v.x * id), roundf(v.y * id), roundf(v.z * id), roundf(v.w * id)};
                    uint32_t packed = 0;
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const float cl = fminf(fmaxf(r[i], -128.0f), 127.0f);
                        const int q = (r[i] != r[i]) ? 0 : (int)cl;
                        packed |= ((uint32_t)(q & 0xff)) << (8 * i);
                    }
                    ll_put(p.ll + RE + b * 8 + tid, packed, e);
                    if (tid == 0) ll_putf(p.ll + RE_SC + b, it_f16_to_f32(it_f32_to_f16(d)), e);
                }
            }
#if !IT_CHAIN_FLOADS_EARLY
            // the down rows of this wave's output row, for stage F: issued behind the publication, they land while the intermediates travel
            // (four picks a step over 16 lanes each, the shared row beside the last two picks)
#pragma unroll
            for (int s = 0; s < 3; s++) {
                const int y = s * 4 + (lane >> 4);
                const bool routed = y < NU;
                const int64_t ex = routed ? ids[y] : 0;
                load_row<W_NVFP4, 1, 16>(fd[s], f.ed_q + ex * f.d_q_stride, f.ed_s + ex * f.d_s_stride, FF, my_row, lane & 15, routed);
            }
            if (SF == W_Q8_0) load_row<W_Q8_0, 1, 32>(fsh, f.sd_q, f.sd_s, FF, my_row, lane & 31, lane >= 32);
            else load_row<W_NVFP4, 1, 16>(fsh, f.sd_q, f.sd_s, FF, my_row, lane & 15, lane >= 32 && lane < 48);
#endif
            // the picks' weights for stage F (probability over the sum of the ten, naive.rs:362-376), and what the seam
            // shows of the route (block 0): lane r of the first wave has pick r
            if (wave == 0) {
                float sum = 0.0f;
#pragma unroll
                for (int i = 0; i < CT / 64; i++) sum += route_sh.redf[i];
                const float prob = lane < NU ? fx_expf(wts[lane] - wts[0]) / sum : 0.0f;
                float denom = 0.0f;
#pragma unroll
                for (int r = 0; r < 16; r++)
                    denom += __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, prob), r));
                denom = fmaxf(denom, 6.103515625e-5f);
                if (lane < NU) {
                    const int ex = ids[lane];
                    const float w = prob / denom;
                    coef[lane] = w * my_dscale;
                    if (b == 0) {
                        f.route_ids[lane] = ex;
                        f.route_w[lane] = w;
                        if (f.counts_gate) atomicAdd(f.counts_gate + ex, 1u);
                        if (f.counts_up) atomicAdd(f.counts_up + ex, 1u);
                        if (f.counts_down) atomicAdd(f.counts_down + ex, 1u);
                    }
                }
                if (b == 0 && lane == 0 && p.tally)
                    atomicAdd(p.tally, (unsigned long long)((f.counts_gate ? 1 : 0) + (f.counts_up ? 1 : 0) + (f.counts_down ? 1 : 0)) * NU);
            }
            asm volatile("" ::"v"(touched));
        }
        // the next layer's in-projection rows start moving now: one stage ahead of their use
        CH_STAMP(10);
        const bool next_mixer = l + 1 < p.n_layers && p.layer[l + 1].has_mixer == 1;
        // (the waves that gather stage F's input issue theirs behind that gather: a poll returns behind everything its
        // own wave has in flight)
        auto fetch_next = [&]() {
            if (l + 1 == p.n_layers && p.has_tail) fetch_tail(p.tail, aw, b, wave, lane);
            if (l + 1 < p.n_layers && p.layer[l + 1].has_mixer == 3) fetch_tail(p.layer[l + 1].a, aw, b, wave, lane);
            if (next_mixer && ((IT_CHAIN_A_AT >> 4) & 15)) fetch_a<RF>(p.layer[l + 1].m, aw, b, wave, lane, (IT_CHAIN_A_AT >> 4) & 15);
        };
        if (!IT_CHAIN_F_POLLERS || wave < 4) fetch_next();

        // -------------------------------------------------------------------- F: down, combine, residual
        {
            uint32_t* dst = (uint32_t*)xq;
            // word i < 1,280 is quad i of the routed quants; the rest are the 160 block scales
            auto place = [&](int i, uint32_t v) {
                if (i < NU * FF / 4) dst[i] = v;
                else xs[i - NU * FF / 4] = __uint_as_float(v);
            };
            bool ok = true;
#if IT_CHAIN_F_POLLERS
            // Waves 4..7 gather: the 720 pairs of words of the routed intermediates (quants, then scales) and, waves 4 and
            // 5, the shared ones as quads (whole waves: the quantization's lane exchange needs its eight neighbours).
            if (wave >= 4) {
                const int pt = tid - 4 * 64, q = pt - 128;
                constexpr int PAIRS = (NU * FF / 4 + EB) / 2;
                const int p2 = wave < 6 ? -1 : 512 + q, p3 = (wave >= 6 && 640 + q < PAIRS) ? 640 + q : -1;
                const u64* const a4[4] = {p.ll + RE + 2 * pt, p.ll + RE + 2 * (pt + 256),
                                          wave < 6 ? p.ll + RS + 4 * pt : p.ll + RE + 2 * p2,
                                          wave < 6 ? p.ll + RS + 4 * pt + 2 : p.ll + RE + 2 * (p3 >= 0 ? p3 : pt)};
                uint32_t o[8];
                ok = ll_wait_pairs<4>(a4, e, ctl, o);
                place(2 * pt, o[0]);
                place(2 * pt + 1, o[1]);
                place(2 * (pt + 256), o[2]);
                place(2 * (pt + 256) + 1, o[3]);
                if (wave < 6) {
                    const float4 v = make_float4(__uint_as_float(o[4]), __uint_as_float(o[5]), __uint_as_float(o[6]), __uint_as_float(o[7]));
                    quant_quad(v, true, pt, xq + NU * FF, xs + EB);
                } else {
                    place(2 * p2, o[4]);
                    place(2 * p2 + 1, o[5]);
                    if (p3 >= 0) {
                        place(2 * p3, o[6]);
                        place(2 * p3 + 1, o[7]);
                    }
                }
                fetch_next();
            }
#else
            // 1,440 words of quantized routed intermediates (pairs tid and tid + 512), the shared ones as quads
            const int pr1 = tid + CT;
            const bool two = pr1 < (NU * FF / 4 + EB) / 2, sq = tid < FF / 4;
            const u64* const a4[4] = {p.ll + RE + 2 * tid, two ? p.ll + RE + 2 * pr1 : p.ll + RE + 2 * tid,
                                      sq ? p.ll + RS + 4 * tid : p.ll + RE + 2 * tid, sq ? p.ll + RS + 4 * tid + 2 : p.ll + RE + 2 * tid};
            uint32_t o[8];
            ok = ll_wait_pairs<4>(a4, e, ctl, o);
            place(2 * tid, o[0]);
            place(2 * tid + 1, o[1]);
            if (two) {
                place(2 * pr1, o[2]);
                place(2 * pr1 + 1, o[3]);
            }
            if (tid < 2 * 64) {   // whole waves: the quantization's lane exchange needs its eight neighbours
                const float4 v = make_float4(__uint_as_float(o[4]), __uint_as_float(o[5]), __uint_as_float(o[6]), __uint_as_float(o[7]));
                quant_quad(v, true, tid, xq + NU * FF, xs + EB);
            }
#endif
            if (!ok) dead = 1;
            __syncthreads();
            if (dead) break;
            CH_STAMP(11);
            if (next_mixer && (IT_CHAIN_A_AT & 15)) fetch_a<RF>(p.layer[l + 1].m, aw, b, wave, lane, IT_CHAIN_A_AT & 15);
            float acc = 0.0f;
            const int c = lane & 15;
#pragma unroll
            for (int s = 0; s < 3; s++) {
                const int y = s * 4 + (lane >> 4);
                if (y < NU) {
                    const uint4 xa = *(const uint4*)(xq + y * FF + c * 32), xb = *(const uint4*)(xq + y * FF + c * 32 + 16);
                    float tA, tB;
                    unit_nvfp4(fd[s].w[0], fd[s].sc[0], xa, xb, xs[y * (FF / 32) + c], &tA, &tB);
                    float t = 0.0f;
                    t += tA;
                    t += tB;
                    acc += coef[y] * t;
                }
            }
            if (lane >= 32) {
                const float gate = fx_sigmoid(sm[34]) * f.sh_dscale;
                const WChunks<1>& ws = fsh;
                if (SF == W_Q8_0) {
                    const int c2 = lane - 32;
                    const uint4 xa = *(const uint4*)(xq + NU * FF + c2 * 16);
                    int s = 0;
                    s = dot4(ws.w[0].x, xa.x, s);
                    s = dot4(ws.w[0].y, xa.y, s);
                    s = dot4(ws.w[0].z, xa.z, s);
                    s = dot4(ws.w[0].w, xa.w, s);
                    acc += gate * ((float)s * (it_f16_to_f32((uint16_t)ws.sc[0]) * xs[EB + (c2 >> 1)]));
                } else if (lane < 48) {
                    const uint4 xa = *(const uint4*)(xq + NU * FF + c * 32), xb = *(const uint4*)(xq + NU * FF + c * 32 + 16);
                    float tA, tB;
                    unit_nvfp4(ws.w[0], ws.sc[0], xa, xb, xs[EB + c], &tA, &tB);
                    float t = 0.0f;
                    t += tA;
                    t += tB;
                    acc += gate * t;
                }
            }
            acc = reduce_lanes<64>(acc);
            if (lane == 63) {
                x_row += acc;
                ll_putf(p.ll + RX + my_row, x_row, e + 1);
                p.x[my_row] = x_row;
            }
        }
        CH_STAMP(12);
    }
    // -------------------------------------------------------------------- tail: the next attention layer's in-projection
    if (p.has_tail) {
        __syncthreads();
        if (!dead) {
            int tid = tid0, b = b0;
            asm volatile("" : "+v"(tid), "+s"(b));
            const int lane = tid & 63;
            const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
            const ChainTail& t = p.tail;
            const unsigned e = e0 + 1u + (unsigned)p.n_layers;
            const float4 nw = ((const float4*)t.norm_w)[tid];
            float4 v;
            if (!ll_wait_quad(p.ll + RX, tid, e, ctl, &v)) dead = 1;
            if (norm_quant(v, nw, t.eps, xq, xs, red, &dead, tid)) {
                XChunks<W_Q8_0, 2> x;
                load_x<W_Q8_0, 2, 64>(x, xq, xs, lane);
                float mine = 0.0f;
#pragma unroll
                for (int k = 0; k < 5; k++) {
                    const float acc = reduce_lanes<64>(dot_chunks<W_Q8_0, 2>(aw.t[k], x));
                    const float r = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, acc), 63));
                    mine = lane == k ? r : mine;
                }
                if (lane < 4) t.out_q[b + NB * (wave + CW * lane)] = mine;
                else if (lane == 4 && wave < 2) t.out_k[b + NB * wave] = mine;
                else if (lane == 4 && wave < 4) t.out_v[b + NB * (wave - 2)] = mine;
            }
        }
    }
    if (b0 == 0 && tid0 == 0) *p.epoch = e0 + 1u + (unsigned)p.n_layers;
}

}  // namespace

bool layer_chain_fits() {
    static const bool fits = [] {
        int dev = 0, cus = 0, occ = 0;
        if (hipGetDevice(&dev) != hipSuccess) return false;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < NB) return false;
        const void* fns[8] = {(const void*)layer_chain_k<W_Q8_0, 0, CHAIN_MAX_LAYERS>,    (const void*)layer_chain_k<W_NVFP4, 0, CHAIN_MAX_LAYERS>,
                              (const void*)layer_chain_k<W_Q8_0, 1, CHAIN_MAX_LAYERS>,    (const void*)layer_chain_k<W_NVFP4, 1, CHAIN_MAX_LAYERS>,
                              (const void*)layer_chain_k<W_Q8_0, 0, CHAIN_SHORT_LAYERS>,  (const void*)layer_chain_k<W_NVFP4, 0, CHAIN_SHORT_LAYERS>,
                              (const void*)layer_chain_k<W_Q8_0, 1, CHAIN_SHORT_LAYERS>,  (const void*)layer_chain_k<W_NVFP4, 1, CHAIN_SHORT_LAYERS>};
        // (with the LDS an attention mixer's stages take: every instance is launched with it when a layer is one)
        for (const void* fn : fns)
            if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, ATTN_LDS) != hipSuccess ||
                hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, fn, CT, ATTN_LDS) != hipSuccess || occ < 1)
                return false;
        return true;
    }();
    return fits;
}

template <int NL>
static void launch_chain(const ChainPT<NL>& p, size_t lds, hipStream_t s) {
    if (p.sh_fmt == W_Q8_0 && !p.rf) hipLaunchKernelGGL((layer_chain_k<W_Q8_0, 0, NL>), dim3(NB), dim3(CT), lds, s, p);
    else if (!p.rf) hipLaunchKernelGGL((layer_chain_k<W_NVFP4, 0, NL>), dim3(NB), dim3(CT), lds, s, p);
    else if (p.sh_fmt == W_Q8_0) hipLaunchKernelGGL((layer_chain_k<W_Q8_0, 1, NL>), dim3(NB), dim3(CT), lds, s, p);
    else hipLaunchKernelGGL((layer_chain_k<W_NVFP4, 1, NL>), dim3(NB), dim3(CT), lds, s, p);
}

bool layer_chain(const ChainP& p, hipStream_t s) {
    if (p.n_layers < 1 || p.n_layers > CHAIN_MAX_LAYERS || !p.ll || !p.epoch || !p.abort_flag || !p.x) return false;
    if (p.sh_fmt != W_Q8_0 && p.sh_fmt != W_NVFP4) return false;
    // every pointer a stage dereferences, by the kind of the layer's mixer (an attention out-projection only as layer 0)
    auto all = [](std::initializer_list<const void*> ptrs) {
        for (const void* q : ptrs)
            if (!q) return false;
        return true;
    };
    bool has_attn = false;
    for (int l = 0; l < p.n_layers; l++) {
        const ChainMixer& m = p.layer[l].m;
        const ChainFfn& f = p.layer[l].f;
        const int kind = p.layer[l].has_mixer;
        if (kind < 0 || kind > 3 || (kind == 2 && l != 0)) return false;
        const ChainAttn& a = p.layer[l].a;
        if (kind == 3 && (!all({a.norm_w, a.q_q, a.q_s, a.k_q, a.k_s, a.v_q, a.v_s, a.q_norm, a.k_norm, a.rope, a.k_slab, a.v_slab, a.n_pos,
                                m.o_q, m.o_s}) || a.n_rot <= 0 || a.n_rot > HD || (a.n_rot / 2) % 4 || ((a.n_rot / 8) & (a.n_rot / 8 - 1))))
            return false;
        has_attn = has_attn || kind == 3;
        if (kind == 1 && !p.rf && !all({m.a_s, m.b_s})) return false;
        if (!p.rf && !all({f.r_s, f.l_s})) return false;
        if (kind == 1 && !all({m.norm_w, m.qkv_q, m.qkv_s, m.z_q, m.z_s, m.a_q, m.b_q, m.conv_state, m.conv_w, m.ssm_a,
                               m.dt_bias, m.state, m.head_norm_w, m.o_q, m.o_s}))
            return false;
        if (kind == 2 && !all({m.o_q, m.o_s, m.attn})) return false;
        if (!all({f.norm_w, f.r_q, f.l_q, f.sg_q, f.sg_s, f.su_q, f.su_s, f.sd_q, f.sd_s, f.eg_q, f.eg_s, f.eu_q, f.eu_s,
                  f.ed_q, f.ed_s, f.route_ids, f.route_w}))
            return false;
    }
    if (p.has_tail && !all({p.tail.norm_w, p.tail.q_q, p.tail.q_s, p.tail.k_q, p.tail.k_s, p.tail.v_q, p.tail.v_s, p.tail.out_q,
                            p.tail.out_k, p.tail.out_v}))
        return false;
    if (!layer_chain_fits()) return false;
    const size_t lds = has_attn ? ATTN_LDS : 0;
    if (p.n_layers <= CHAIN_SHORT_LAYERS) {   // the same kernel with room for four layers in its argument block
        ChainPT<CHAIN_SHORT_LAYERS> q;
        std::memcpy((void*)&q, (const void*)&p, offsetof(ChainP, layer) + (size_t)p.n_layers * sizeof(ChainLayer));
        launch_chain(q, lds, s);
    } else {
        launch_chain(p, lds, s);
    }
    return true;
}

}  // namespace itk

#ifdef IT_CHAIN_STAMPS
// tuning builds only: the stage sums (24) and the attention middle's (8), then zeroed
namespace itk {
bool chain_stamps_take(long long* out) {
    long long zero[32] = {0};
    if (hipDeviceSynchronize() != hipSuccess) return false;
    if (hipMemcpyFromSymbol(out, HIP_SYMBOL(it_chain_stamps), 24 * 8) != hipSuccess) return false;
    if (hipMemcpyFromSymbol(out + 24, HIP_SYMBOL(it_attn_core_stamps), 8 * 8) != hipSuccess) return false;
    return hipMemcpyToSymbol(HIP_SYMBOL(it_chain_stamps), zero, 24 * 8) == hipSuccess &&
           hipMemcpyToSymbol(HIP_SYMBOL(it_attn_core_stamps), zero, 8 * 8) == hipSuccess;
}
}  // namespace itk
extern "C" int it_hip_debug_chain_stamps(long long* out) { return itk::chain_stamps_take(out) ? 0 : -1; }
#endif
