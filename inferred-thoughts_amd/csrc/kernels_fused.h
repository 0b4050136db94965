// Argument structs and launchers of the fused single-token kernels (k_fused.hip).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace itk {

struct FusedMat {
    const uint8_t* q;
    const uint8_t* s;
    float* out;
    int n_out, fmt;
    int epi;     // 0 store, 1 causal conv (kernel 4) + silu, 2 accumulate into out, 3 store silu (fast kernels only)
    int group0;  // filled by the launcher
};
struct FusedGemvP {
    const float* x;       // [n_in] f32
    const float* norm_w;  // rms_norm weight (mode 1: [n_in]; mode 2: [head_dim])
    const float* gate;    // mode 2: silu gate, [n_in]; mode 3 (fast kernels only): the same gate, already silu'd
    float* x_copy;        // optional: the activation after the prologue, f32, written by block 0
    float* x_copy2;       // optional second copy (a whole-row gather of it)
    float eps;
    int n_in, mode, head_dim, exact, n_mats, rows_per_wave, total_groups;
    FusedMat m[4];
    // fast kernels only: the launcher moves unquantized (F32 / F16 / BF16) matrices behind the quantized ones;
    // m[n_mats .. n_mats + n_fmats) are those, total_frows rows in all (epi 0 only)
    int n_fmats, total_frows;
    int fsplit;   // waves that share one unquantized row (1 or 2; the kernel also takes 4): a launch of few such rows and nothing else spreads over more CUs
    float* conv_state;    // epi 1
    const float* conv_w;
    // optional: matrix 0 is the router; the last block to finish picks the experts
    unsigned* route_counter;  // zero between launches
    int n_expert, n_used;
    int32_t* route_ids;
    float* route_w;
};
void fused_gemv(FusedGemvP p, hipStream_t s);
// whether the fast kernel takes p (formats, shapes, alignment); unquantized matrices are taken by the fast kernel only
bool fused_gemv_fast_takes(const FusedGemvP& p);

struct GdnCoreP {
    const float* conv;  // [q | k | v] after conv + silu
    const float *alpha, *beta, *ssm_a, *dt_bias;
    float* state;       // [n_v_heads][dv][dk]
    float* core;        // out: delta-rule read-out, [n_v_heads * dv]
    int n_k_heads, n_v_heads, exact;
    float eps, q_scale;
};
void gdn_core(const GdnCoreP& p, int dk, hipStream_t s);

struct MoeGluP {
    const float* x;        // normed activation, f32 [n_in]
    const uint8_t *gq, *gs, *uq, *us;
    const float *gscale2, *uscale2;
    int64_t q_stride, s_stride;
    int fmt, n_in, n_out, n_expert, n_used, exact, rows_per_wave;
    const uint8_t *sh_gq, *sh_gs, *sh_uq, *sh_us;
    int sh_fmt, sh_n_out;
    // the shared expert's per-tensor second scales (ffn_gate_shexp.scale, ffn_up_shexp.scale of an NVFP4 file;
    // src/model/qwen35.rs:1669-1676: up is scaled, then gate, then silu(gate) * up); 1 when the file has none
    float sh_gscale, sh_uscale;
    float* out;            // [n_used][n_out]
    float* sh_out;         // [sh_n_out]
    const int32_t* route_ids;  // [n_used], chosen by the router kernel (when logits is null)
    // fast mode: the router logits; every block ranks them itself and block 0 publishes the
    // picks and their weights for the down kernel
    const float* logits;
    int32_t* route_ids_out;
    float* route_w_out;
    // fast mode, a short batch: token t of n_tok is grid row t, every per-token operand above (x, logits, the picks, out,
    // sh_out) t vectors further on.  0 or 1: one token.
    int n_tok;
};
void moe_glu_fused(MoeGluP p, hipStream_t s);

struct MoeDownP {
    const float* g_all;     // [n_used][n_in]
    const float* g_shared;  // [sh_n_in]
    const uint8_t *q, *s;
    const float* scale2;
    int64_t q_stride, s_stride;
    int fmt, n_in, n_out, n_used, rows_per_wave, exact;
    const uint8_t *sh_q, *sh_s;
    int sh_fmt, sh_n_in;
    float sh_dscale;        // ffn_down_shexp.scale (qwen35.rs:1680-1682: applied to the product, before the gate); 1 when absent
    const int32_t* route_ids;
    const float* route_w;
    const float* logit;     // shared expert gate logit
    float* x;               // residual stream, accumulated into
    // expert read counters (optional): the gate, up and down tensors' per-expert counts and the tally of reads
    // served from device memory; block 0 adds this token's picks
    uint32_t *counts_gate, *counts_up, *counts_down;
    unsigned long long* tally;
    // fast mode, a short batch (see MoeGluP::n_tok); `y` set: the sums are stored there instead of added to x
    // (moe_finish without the add_assign behind it)
    int n_tok;
    float* y;
};
void moe_down_fused(MoeDownP p, hipStream_t s);

struct AttnPrepP {
    const float *qg, *k, *v;     // wq output [n_head][2*head_dim], k and v projections
    const float *q_norm, *k_norm;
    const float2* rope;
    const int* pos_dyn;
    float* q;                     // out [n_head*head_dim]
    uint16_t *k_slab, *v_slab;
    int n_head, n_head_kv, head_dim, n_rot, kv_dim, exact;
    float eps;
};
void attn_prep(const AttnPrepP& p, hipStream_t s);

// Fast-mode forms (reductions in wave order).  Each returns false without launching when
// the shapes, formats or alignments fall outside what it handles; the caller then uses the
// order-preserving kernel.
bool fused_gemv_fast(FusedGemvP p, hipStream_t s);
// (dry_run: only say whether the shape is taken)
bool moe_glu_fast(MoeGluP p, hipStream_t s, bool dry_run = false);
bool moe_down_fast(MoeDownP p, hipStream_t s, bool dry_run = false);

// ------------------------------------------------------------------ layer chain (k_chain.hip, fast mode)
// A run of decode layers as ONE persistent kernel, one block per compute unit: the six dependent launches of a
// Gated DeltaNet layer (in-projection + conv, delta rule, out-projection, router + shared expert gate/up, routed
// gate/up, down + combine) become six stages inside the kernel.  Between stages every block publishes its outputs
// as 8-byte {value, epoch} words in uncached device memory and picks up its inputs by polling for the epoch; the
// weights of a stage are in the block's registers before its inputs arrive.
// Shapes are fixed (hidden 2048; 16 key / 32 value heads of 128; 512 NVFP4 experts, top 10, 512 rows; a shared
// expert of 512 rows in Q8_0 or NVFP4; Q8_0 dense matrices); anything else stays on the per-stage launches.
// Pointers inside the chain's structs are device-memory pointers, and on the device they are declared as such: a
// pointer of unknown kind that reaches a function which is not inlined is a generic one there, whose loads are FLAT
// loads (which every wait for LDS has to drain).  Same size and layout on the host.
#if defined(__HIP_DEVICE_COMPILE__) && defined(IT_CHAIN_DEVICE_POINTERS)   // (set by the file that holds the kernel; host code elsewhere fills plain pointers)
template <class T> using it_gptr = T __attribute__((address_space(1)))*;
#else
template <class T> using it_gptr = T*;
#endif
struct ChainMixer {
    it_gptr<const float> norm_w;
    it_gptr<const uint8_t> qkv_q, qkv_s, z_q, z_s, a_q, a_s, b_q, b_s;
    it_gptr<float> conv_state;
    it_gptr<const float> conv_w;
    it_gptr<const float> ssm_a, dt_bias;
    it_gptr<float> state;
    it_gptr<const float> head_norm_w;
    it_gptr<const uint8_t> o_q, o_s;
    float eps_norm, eps_l2, eps_head, q_scale;
    it_gptr<const float> attn;   // has_mixer == 2 only: the attention block's gated output [4096], the out-projection's input
};
struct ChainFfn {
    it_gptr<const float> norm_w;
    it_gptr<const uint8_t> r_q, r_s, l_q, l_s;   // router rows, and the shared expert's gate-logit row
    it_gptr<const uint8_t> sg_q, sg_s, su_q, su_s;   // shared expert gate / up
    it_gptr<const uint8_t> sd_q, sd_s;                 // shared expert down
    it_gptr<const uint8_t> eg_q, eg_s, eu_q, eu_s, ed_q, ed_s;   // routed experts
    it_gptr<const float> gscale2, uscale2, dscale2;
    int64_t gu_q_stride, gu_s_stride, d_q_stride, d_s_stride;
    float sh_gscale, sh_uscale, sh_dscale, eps;
    it_gptr<int32_t> route_ids;     // seam outputs: this layer's picks and their weights
    it_gptr<float> route_w;
    it_gptr<uint32_t> counts_gate, counts_up, counts_down;   // expert read counters (optional)
};
// The in-projection of the attention layer BEHIND the chain's last layer (rms_norm + quantization + rows of wq, wk,
// wv), run as the chain's last stage; its outputs go to ordinary memory for the attention kernels that follow.
struct ChainTail {
    it_gptr<const float> norm_w;
    it_gptr<const uint8_t> q_q, q_s, k_q, k_s, v_q, v_s;   // wq (8192 rows: query and gate of every head), wk, wv (512 rows each)
    it_gptr<float> out_q, out_k, out_v;
    float eps;
};
// A whole attention mixer inside the chain (has_mixer == 3): in-projection, norm + rotation of the query heads and of
// the new key, the cache rows of the new position, attention over the context split over the blocks, merge + sigmoid
// gate; the out-projection's matrix is the layer's ChainMixer o_q / o_s.  16 query heads of 256 on 2 KV heads.
struct ChainAttn {
    it_gptr<const float> norm_w;
    it_gptr<const uint8_t> q_q, q_s, k_q, k_s, v_q, v_s;   // wq (8192 rows: query and gate of every head), wk, wv (512 rows each)
    it_gptr<const float> q_norm, k_norm;
    it_gptr<const float2> rope;      // [pos][n_rot / 2] (cos, sin)
    it_gptr<uint16_t> k_slab, v_slab;   // f16 [pos][512]
    it_gptr<const int> n_pos;        // device word: positions in the context, this token's included
    float eps, eps_head, scale;
    int n_rot;
};
struct ChainLayer {
    // 0: the layer's mixer ran before the chain; 1: a Gated DeltaNet mixer; 2: an attention layer whose out-projection
    // (+ residual) opens the chain (first layer only: its input is in ordinary memory when the kernel starts);
    // 3: an attention mixer, all of it
    int has_mixer;
    ChainMixer m;
    ChainFfn f;
    ChainAttn a;
};
// layers of one chain: a model's whole token when every block of it fits the stages.  They travel in the kernel's
// argument block (30 KB at this limit, which the runtime takes, also for a captured launch), where the compiler knows
// them to be readable and unchanging and loads them ahead of their uses; a table in device memory, which it must load
// where each value is used, measured 2.7 % slower per token.
constexpr int CHAIN_MAX_LAYERS = 56;
constexpr int CHAIN_BLOCKS = 256;
constexpr int CHAIN_ATTN_SPLITS = 128;     // key ranges of an in-chain attention (two KV heads x 128 ranges = the grid)
constexpr size_t CHAIN_LL_STAGE_WORDS = 24576;   // 8-byte words of hand-off space of the stages
// ... and behind them the attention partials: per (query head, key range) 256 sums, the range's maximum and its weight
constexpr size_t CHAIN_LL_WORDS = CHAIN_LL_STAGE_WORDS + (size_t)16 * CHAIN_ATTN_SPLITS * 258;
template <int NL> struct ChainPT {
    int n_layers;
    int has_tail;
    ChainTail tail;
    int sh_fmt;                  // the shared expert's format (W_Q8_0 or W_NVFP4)
    int rf;                      // 1: the router, the shared expert's gate-logit row and ssm alpha / beta are F32 matrices (as real
                                 // files keep them; their *_q pointers hold floats, their *_s are null), 0: Q8_0
    it_gptr<float> x;                    // residual stream [2048], read at the start and current after every layer
    it_gptr<unsigned long long> ll;      // CHAIN_LL_WORDS words of uncached device memory, zero before the first chain
    it_gptr<unsigned> epoch;             // device word: the last epoch any chain has used (starts at 0)
    it_gptr<unsigned> abort_flag;        // uncached device word: set when a bounded wait gave up (the results are then void)
    it_gptr<unsigned long long> tally;   // expert read tally (optional)
    int spin_limit;              // polls a wait may take before it gives up
    ChainLayer layer[NL];   // (last: host code copies and clears the n_layers entries in use, not all 30 KB)
};
typedef ChainPT<CHAIN_MAX_LAYERS> ChainP;
// A chain of up to this many layers is launched with a small argument block: a launch queued outside a graph pays the
// host's copy of its arguments (8-10 us for 30 KB against 2.5 us for 2 KB, measured; a replayed graph pays neither).
constexpr int CHAIN_SHORT_LAYERS = 4;
// whether this device can hold the chain's grid (one block per compute unit, all resident at once)
bool layer_chain_fits();
// false: not launched
bool layer_chain(const ChainP& p, hipStream_t s);

}  // namespace itk
