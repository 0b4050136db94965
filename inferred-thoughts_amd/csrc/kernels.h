// Launch wrappers for every HIP kernel in the library.  Plain pointers and sizes
// only; every pointer is a device pointer.  `dyn` pointers, when non-null, name a
// device int that overrides the by-value scalar beside them — that is what lets a
// captured decode graph stay valid while the position advances.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace itk {

// ---- weight formats on the device (repacked at upload) ----------------------
// Q8_0:  quants int8 [n_rows][n_in], scales f16 [n_rows][n_in/32]
// NVFP4: nibbles u8 [n_rows][n_in/2] (byte j of sub-block s = elements j, j+8 of
//        that sub-block, as in the file), scales u8 [n_rows][n_in/16]
// F32/F16/BF16: file layout (row-major), read as is.
enum WFmt : int { W_F32 = 0, W_F16 = 1, W_Q8_0 = 8, W_BF16 = 30, W_NVFP4 = 40 };

struct WView {
    const void* q;       // quants / nibbles / raw rows
    const void* scales;  // per-block scales (null for F32/F16/BF16)
    int fmt;
    int n_in, n_out;
};

// repack kernels: file layout -> device layout
// batch runs of elementwise ops as one kernel each (fast mode); false: not a case for the fused form
bool conv_split_l2(float* state, const float* x, const float* w, int kernel, int nc, int n_tok, float* q_out, float* k_out,
                   float* v_out, int kdim, float eps, hipStream_t s);
bool gated_norm_silu_q8(const float* core, const float* w, float* z, float* scales, int8_t* quants, int64_t n_heads, float eps,
                        hipStream_t s);
// two unquantized matrices of one element type over the same batch of activations, one launch (fast mode, > 16 tokens)
bool float_matmul_pair(const WView& a, const WView& b, const float* x, int n_tok, float* out_a, float* out_b, hipStream_t s);
void repack_q8_0(const uint8_t* raw, int8_t* q, uint16_t* scales, int64_t n_rows, int n_in, hipStream_t s);
void repack_nvfp4(const uint8_t* raw, uint8_t* nib, uint8_t* scales, int64_t n_rows, int n_in, hipStream_t s);

// ---- activation quantization --------------------------------------------------
void quantize_q8_0(const float* x, float* scales, int8_t* quants, int64_t n, hipStream_t s);

// ---- matmul family -------------------------------------------------------------
// out[t][j] = dot(w.row(j), x[t]); act is the Q8_0 form of x for quantized formats.
void matmul(const WView& w, const float* x, const float* act_scales, const int8_t* act_quants, int n_tok,
            float* out, float out_scale, int exact, hipStream_t s);

// The same product for 16 or more tokens on the int8 matrix cores (Q8_0 weights only): bit-identical
// to `matmul`.  Returns false without launching when the shape or format is not handled.
// fma: the scaled block sum is added with one rounding instead of two (fast mode only: not the CPU path's bits)
bool q8_gemm(const WView& w, const float* act_scales, const int8_t* act_quants, int n_tok, float* out, float out_scale,
             hipStream_t s, bool fma = false);

struct ExpertsView {
    const void* q;       // expert e at q + e*q_stride
    const void* scales;  // expert e at scales + e*s_stride
    int64_t q_stride, s_stride;
    int fmt, n_in, n_out, n_expert;
    const float* scale2;  // per-expert second scale or null
    uint32_t* counts;     // this tensor's per-expert read counters (device), or null
    // Two-tier placement (device arrays of n_expert entries, or null when every expert sits in device memory at its
    // stride): where expert e's quants and scales are, in a device slot or in pinned host memory that the device
    // reads across the bus, and which of the two (0 device, 1 host) for the read tallies.
    const uint8_t* const* q_tab;
    const uint8_t* const* s_tab;
    const uint8_t* tier;
};
// One matmul per pick.  x rows: mode 0 = one row per pick, 1 = one row per token
// (pick i reads row i / n_used), 2 = a single shared row.
void matmul_experts(const ExpertsView& w, const int32_t* ids, int n_picks, int n_used, int x_mode,
                    const float* act_scales, const int8_t* act_quants, float* out, hipStream_t s);
// The same products (up == null) or the gate/up pair with silu-mul (up != null) for a batch of 32 or more
// pairs: pairs are grouped by expert and multiplied on the int8 matrix cores, a matrix read once per 16
// pairs; bit-identical to the per-pair kernels.  `work` is device scratch of experts_group_work_ints ints.
// Returns false without launching when the shape, format or scratch does not fit.
size_t experts_group_work_ints(int n_picks, int n_expert);
// NVFP4 only, fast mode: the same products on the f16 matrix cores, weights expanded exactly to f16 and the
// Q8_0 activations as an f16 hi/lo pair; results agree with the int8 kernels to ~1e-6 relative.
// work: experts_f16_work_ints ints; fwork: experts_f16_work_bytes bytes, 16-byte aligned.
size_t experts_f16_work_ints(int n_picks, int n_expert);
// pairs sorted into per-expert lists cut into tiles of at most tile_pairs: n_tiles[0] = tile count, tiles = {expert,
// first slot, pairs, 0}, order[slot] = pair
void moe_group(const int32_t* ids, int n_picks, int n_expert, int tile_pairs, int32_t* n_tiles, int4* tiles,
               int32_t* order, hipStream_t s);
size_t experts_f16_work_bytes(int x_rows, int n_in);
// whether experts_gemm_f16 takes these operands (shape, format, alignment), given scratch of the sizes above
bool experts_f16_takes(const ExpertsView& w, const ExpertsView* up, int n_picks, const int8_t* act_quants, const float* out);
bool experts_gemm_f16(const ExpertsView& w, const ExpertsView* up, const int32_t* ids, int n_picks, int n_used,
                      int x_mode, const float* act_scales, const int8_t* act_quants, float* out, int32_t* work,
                      size_t work_ints, void* fwork, size_t fwork_bytes, bool grouped, hipStream_t s);
// NVFP4 experts with few pairs per expert in fast mode (k_gemm_f16s.hip): tiles of 16 pairs on MFMA 16x16x32 f16, no LDS;
// the grouping has the layout of experts_gemm's (tiles of 16 pairs).  Scratch as for experts_gemm_f16.
bool experts_f16s_takes(const ExpertsView& w, const ExpertsView* up, int n_picks, const int8_t* act_quants, const float* out);
bool experts_gemm_f16s(const ExpertsView& w, const ExpertsView* up, const int32_t* ids, int n_picks, int n_used,
                       int x_mode, const float* act_scales, const int8_t* act_quants, float* out, int32_t* work,
                       size_t work_ints, void* fwork, size_t fwork_bytes, bool grouped, hipStream_t s);
// Small batches in fast mode (k_moe_rows.hip): pairs sorted by expert in tiles of 8 or 16, every weight row of a tile's
// expert streamed once and multiplied with all its pairs by integer dots.  ids null: one dense matrix (strides
// ignored), tile t = tokens 8 t .. 8 t + 7.  False: nothing launched (shape, alignment or scratch do not fit).
bool expert_rows_takes(const ExpertsView& w, const ExpertsView* up, const int8_t* act_quants);
int expert_rows_tile(int n_picks, int n_expert, int n_in);   // pairs per tile the launch groups for
bool expert_rows(const ExpertsView& w, const ExpertsView* up, const int32_t* ids, int n_picks, int n_used, int x_mode,
                 const float* act_scales, const int8_t* act_quants, float* out, float out_scale, int32_t* work,
                 size_t work_ints, bool grouped, hipStream_t s);
bool experts_gemm(const ExpertsView& w, const ExpertsView* up, const int32_t* ids, int n_picks, int n_used, int x_mode,
                  const float* act_scales, const int8_t* act_quants, float* out, int32_t* work, size_t work_ints,
                  bool grouped, hipStream_t s);
// out[i] = silu(gate_e . x * sg_e) * (up_e . x * su_e)
void moe_glu(const ExpertsView& gate, const ExpertsView& up, const int32_t* ids, int n_picks, int n_used,
             int x_mode, const float* act_scales, const int8_t* act_quants, float* out, hipStream_t s);

// ---- expert read counters -------------------------------------------------------
// counts_a[ids[i]] += 1 (and counts_b, when given: a second tensor read with the same picks) for every pick, and
// tally[0] += the reads counted: the device-side read counters of the expert cache (reads served from device memory;
// tally[1], reads served from a host tier, stays 0 when every expert is resident)
void expert_count(const int32_t* ids, int n_picks, int n_expert, uint32_t* counts_a, uint32_t* counts_b,
                  unsigned long long* tally, hipStream_t s, const uint8_t* tier_a = nullptr, const uint8_t* tier_b = nullptr);

// one entry of a tensor's placement table changes: the expert's quants, scales and tier byte (written by one thread)
struct ExpertPatch {
    const uint8_t** q_at;
    const uint8_t** s_at;
    uint8_t* tier_at;
    const uint8_t* q;
    const uint8_t* s;
    uint32_t tier, pad;
};
void expert_patch(const ExpertPatch* patches, int n, hipStream_t s);

// ---- router ----------------------------------------------------------------------
void softmax_rows(float* x, int64_t n_rows, int row, int exact, hipStream_t s);
void route_topk(const float* probs, int n_tok, int n_expert, int n_used, int32_t* ids, float* weights,
                hipStream_t s);
void moe_finish(float* out, int64_t at, int n, const float* rows, const float* weights, int n_tok, int n_used,
                const float* shared, const float* logit, int64_t logit_at, int exact, hipStream_t s);

// ---- norms and elementwise ------------------------------------------------------
// q_scales / q_quants (optional, nd a multiple of 32): the Q8_0 form of `out` is written as well, bit for bit what
// quantize_q8_0 gives on it
void rms_norm(const float* x, const float* w, float eps, float* out, int64_t n_rows, int nd, int exact,
              hipStream_t s, float* q_scales = nullptr, int8_t* q_quants = nullptr);
// whether rms_norm writes the Q8_0 form when given the buffers for it (row length and alignments): the caller marks the
// quantized form valid only then
bool rms_norm_writes_q8(const float* x, const float* w, const float* out, int nd);
void rms_norm_heads(float* x, const float* w, int head_dim, float eps, int64_t n_heads, int exact,
                    hipStream_t s);
void l2_norm_heads(float* x, int head_dim, float eps, int64_t n_heads, int exact, hipStream_t s);
void rope_neox(float* x, const float2* table, int table_half, int64_t n_tok, int pos, const int* pos_dyn,
               int head_dim, int n_rot, int n_heads, hipStream_t s);
// exact = 0: long batches take the exponential on the transcendental unit (fast mode)
void silu_mul(float* gate, const float* up, int64_t n, int exact, hipStream_t s);
void sigmoid_mul(float* x, const float* g, int64_t n, int exact, hipStream_t s);
void add_assign(float* a, const float* b, int64_t n, hipStream_t s);
void scale(float* a, float v, int64_t n, hipStream_t s);
void add_scaled(float* a, const float* b, float v, int64_t n, hipStream_t s);
void add_scaled_rows(float* acc, int64_t n, const float* rows, const float* scales, int n_scales,
                     hipStream_t s);
void add_scaled_sigmoid(float* acc, const float* b, int64_t n, const float* logit, hipStream_t s);
void gather_chunks(const float* src, int64_t chunk, int64_t stride, int64_t offset, float* out,
                   int64_t out_len, hipStream_t s);
void scatter_chunks(const float* src, int64_t src_len, int64_t chunk, int64_t stride, int64_t offset,
                    float* dst, hipStream_t s);
void kv_write(uint16_t* slab, int64_t offset, const int* offset_dyn, int64_t offset_mul, const float* src,
              int64_t n, hipStream_t s);
void fill_zero(void* p, int64_t bytes, hipStream_t s);
// n <= POKE_MAX host ints to device memory as one small kernel whose argument block carries them (the host array may be
// reused as soon as the call returns); false: too many, nothing was launched
constexpr int POKE_MAX = 256;
bool poke_ints(int* dst, const int* host_values, int n, hipStream_t s);
void argmax(const float* x, int64_t n, int32_t* out, int32_t* scratch_idx, float* scratch_val, hipStream_t s);
// x = dequantized row `*token` of an embedding table (Q8_0 repacked, F16, BF16 or F32); the id goes to
// ring[ring_dyn ? *ring_dyn : ring_idx] when ring is non-null
// arg-max of the logits and the embedding row of the winner (the two above) in two launches instead of three
void argmax_embed(const float* logits, int64_t n, int32_t* out, int32_t* scratch_idx, float* scratch_val, const WView& w,
                  float* x, int32_t* ring, int ring_idx, const int* ring_dyn, hipStream_t s);
void embed_row(const WView& w, const int32_t* token, float* x, int32_t* ring, int ring_idx, const int* ring_dyn,
               hipStream_t s);

// ---- gated delta net ---------------------------------------------------------------
void ssm_conv(float* state, const float* x, const float* w, int kernel, int nc, int n_tok, float* out, int exact,
              hipStream_t s);
struct DeltaArgs {
    const float *q, *k, *v, *alpha, *beta, *ssm_a, *dt_bias;
    int n_tokens, head_k_dim, head_v_dim, n_k_heads, n_v_heads;
};
// work: scratch of gdn_chunk_work_floats() floats for the chunked MFMA form (fast mode, 64 tokens and more); may be null
void delta_rule(const DeltaArgs& d, float* state, float* out, int exact, float* work, size_t work_floats, hipStream_t s);
size_t gdn_chunk_work_floats(int n_tokens, int n_v_heads);
bool delta_rule_chunked(const DeltaArgs& d, float* state, float* out, float* work, size_t work_floats, hipStream_t s);

// ---- attention -------------------------------------------------------------------------
struct AttnArgs {
    const float* q;
    const uint16_t *k, *v;
    int n_q, kv_dim, n_pos, head_dim, n_head, n_head_kv;
    float scale;
    const int* n_pos_dyn;  // overrides n_pos when non-null (decode graphs)
};
// exact: the oracle's order (scores, serial softmax sum, positions outermost).
// scratch: n_q * n_head * n_pos floats.
void attend_exact(const AttnArgs& a, float* scratch, float* out, hipStream_t s);
// split-K flash decoding; scratch: n_q*n_head*n_split*(head_dim+2) floats.
int attend_split_count(int n_pos_max, int n_q, int head_dim, int group);
bool attend_split(const AttnArgs& a, int n_split_max, float* scratch, float* out, hipStream_t s);  // false: not launched
// more than 16 queries, fast mode: one pass over the keys on the f16 matrix cores; false when the shape is not taken
bool attend_prefill(const AttnArgs& a, float* out, hipStream_t s);
bool attend_prefill_takes(const AttnArgs& a, const float* out);
// What one decode token's attention needs before it can attend, folded into the tile kernel: the
// query heads' norm + rotation (every block, for its own heads) and the new position's key
// (norm + rotation) and value rows, written to the slabs by the block whose tile holds them.
struct TilePrepP {
    const float *qg, *kproj, *vproj;  // wq output [n_head][2 * head_dim] (q then gate), k and v projections
    const float *q_norm, *k_norm;
    const float2* rope;               // [pos][n_rot / 2] (cos, sin)
    int n_rot;
    float eps;
    uint16_t *k_slab, *v_slab;
};
bool attend_tile_prep_ok(const AttnArgs& a, const TilePrepP& pr);
bool attend_split_gated_prep(const AttnArgs& a, const TilePrepP& pr, int n_split, float* scratch, float* out,
                             const float* gate, int gate_stride, hipStream_t s);
// the same with the merge multiplying by sigmoid(gate[head * gate_stride + i]) (n_q == 1)
bool attend_split_gated(const AttnArgs& a, int n_split_max, float* scratch, float* out, const float* gate,
                        int gate_stride, hipStream_t s);

}  // namespace itk
