/* inferred_hip.h — C ABI of the MI355X (gfx950) backend for the per-token model loop.
 *
 * Every `it_hip_*` op below replaces one method of the reference's backend seam,
 * `trait Ops` (/root/reference src/ops/mod.rs:489-1426), with the same argument
 * order and meaning: Rust slices become (pointer, length) pairs, the argument
 * structs become the plain-old-data structs declared here, and `&self` becomes the
 * opaque `it_hip*`.  All pointers are HOST pointers, exactly as at the seam: the
 * backend keeps device copies keyed on the host address (activation mirrors,
 * resident weights, device-owned KV and recurrent-state slabs) and moves data only
 * at `host_wrote` / `host_needs` / first touch.
 *
 * Conventions carried over from the reference:
 *  - batch size is derived from buffer lengths, never passed (mod.rs:462-488);
 *  - ops return nothing; the first error is kept and later calls keep going; poll
 *    it_hip_take_error() after the run (src/ops/cuda/ops/mod.rs:91-110);
 *  - one host thread drives one backend; all device work is issued in call order;
 *  - never pass a sub-slice of an activation (a prefix is fine).
 */
#ifndef INFERRED_HIP_H
#define INFERRED_HIP_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ggml type codes (src/gguf/types.rs:62-100) */
enum { IT_F32 = 0, IT_F16 = 1, IT_Q8_0 = 8, IT_BF16 = 30, IT_NVFP4 = 40 };

/* struct Weights, src/ops/mod.rs:62-92 */
typedef struct {
    const uint8_t* data;
    uint64_t len; /* bytes */
    uint32_t ty;
    uint32_t pooled;
    uint64_t n_in, n_out;
} it_weights;

/* struct Experts, src/ops/mod.rs:107-152 */
typedef struct {
    const uint8_t* data;
    uint64_t len;
    uint32_t ty;
    uint32_t _pad;
    uint64_t n_in, n_out, n_expert;
    const uint8_t* scale; /* n_expert little-endian f32, NULL when the file has none */
    uint64_t scale_len;   /* bytes */
} it_experts;

/* struct Attn, src/ops/mod.rs:228-276; n_q is derived from q_len */
typedef struct {
    const float* q;
    uint64_t q_len;
    const uint16_t* k;
    const uint16_t* v;
    uint64_t kv_len; /* elements in each slab */
    uint64_t kv_dim, n_pos, head_dim, n_head, n_head_kv;
    float scale;
} it_attn;

/* struct Delta, src/ops/mod.rs:337-358; n_tokens = v_len / (n_v_heads * head_v_dim) */
typedef struct {
    const float *q, *k, *v, *alpha, *beta, *ssm_a, *dt_bias;
    uint64_t n_tokens;
    uint64_t head_k_dim, head_v_dim, n_k_heads, n_v_heads;
} it_delta;

/* enum Route, src/ops/mod.rs:176-218 */
enum { IT_ROUTE_HOST = 0, IT_ROUTE_DEVICE = 1 };
typedef struct {
    uint32_t kind;
    uint32_t _pad;
    const uint64_t* ids;  /* Host: n_tok * n_used expert ids, token-major */
    const float* weights; /* Host: normalized weights, same order */
    uint64_t n_used, n_tok;
} it_route;

/* struct TierCounters, src/ops/mod.rs:364-401 */
typedef struct {
    uint64_t fetched, fetch_bytes, read_us, upload_us, writes_us, picks_wait_us, picks_copy_us;
    uint64_t prefetch_reads, prefetch_used, lookups, host_reads, slot_bytes;
    uint64_t vram_free, vram_total, mirrors, mirror_bytes;
    uint32_t oversubscribed, _pad;
    uint64_t slots, resident_bytes, weight_bytes, kv_bytes, quant_bytes, pool_bytes;
} it_tier_counters;

/* struct ExpertStats, src/ops/cuda/experts.rs:210-315: hits = reads served from device memory, lookups - hits = reads
 * that crossed the bus to the pinned host tier, host_slots = experts in that tier, fetched = cold experts brought into
 * device memory from the model file, evictions = experts that left device memory (exchanged by counts, or displaced
 * by a fetched one), oversubscribed = some expert is cold (both tiers filled before the pool did) */
typedef struct {
    uint64_t slots, slot_bytes, resident, pool, host_slots, evictions, fetched, lookups, hits;
    uint32_t oversubscribed, _pad;
} it_expert_stats;

typedef struct it_hip it_hip;

/* flags for it_hip_create */
enum {
    IT_HIP_EXACT = 1,    /* every reduction in the CPU path's order (bit-identical results) */
    IT_HIP_NO_GRAPH = 2, /* never capture decode passes into a HIP graph */
    IT_HIP_NO_FUSE = 4,  /* capture decode passes op by op, without the fused kernels */
    IT_HIP_NO_CHAIN = 8, /* keep every fused decode stage a launch of its own (no persistent kernel over runs of layers) */
};

/* Cuda::new, src/ops/cuda/mod.rs:757-935.  NULL on failure with a message in err. */
it_hip* it_hip_create(uint32_t flags, int device, char* err, size_t err_len);
void it_hip_destroy(it_hip* be);
/* Cuda::take_error: 1 and the message when an error is pending (and clears it), else 0 */
int it_hip_take_error(it_hip* be, char* msg, size_t msg_len);
/* 1 when an error is already recorded; never waits for the device (extension) */
int it_hip_has_error(it_hip* be);
/* check_expert_types, src/ops/mod.rs:29-55, for this backend: 0 = supported */
int it_hip_check_expert_types(uint32_t gate, uint32_t up, uint32_t down, char* msg, size_t msg_len);

/* ---- required trait methods ---- */
void it_hip_rms_norm(it_hip*, const float* x, uint64_t x_len, const float* weight, uint64_t w_len, float eps,
                     float* out, uint64_t out_len); /* mod.rs:497 */
void it_hip_rms_norm_heads(it_hip*, float* x, uint64_t x_len, const float* weight, uint64_t w_len,
                           uint64_t head_dim, float eps); /* mod.rs:502 */
void it_hip_matmul(it_hip*, const it_weights* w, const float* x, uint64_t x_len, float* out,
                   uint64_t out_len); /* mod.rs:520 */
void it_hip_rope_neox(it_hip*, float* x, uint64_t x_len, uint64_t pos, uint64_t head_dim, uint64_t n_rot,
                      uint64_t n_heads, float theta_base); /* mod.rs:545 */
void it_hip_softmax(it_hip*, float* x, uint64_t x_len, uint64_t row);   /* mod.rs:567 */
void it_hip_attend(it_hip*, const it_attn* a, float* out, uint64_t out_len); /* mod.rs:589 */
void it_hip_silu_mul(it_hip*, float* gate, uint64_t gate_len, const float* up, uint64_t up_len); /* :592 */
void it_hip_l2_norm_heads(it_hip*, float* x, uint64_t x_len, uint64_t head_dim, float eps); /* :613 */
void it_hip_ssm_conv(it_hip*, float* state, uint64_t state_len, const float* x, uint64_t x_len,
                     const float* weight, uint64_t w_len, uint64_t kernel, float* out,
                     uint64_t out_len); /* mod.rs:647 */
void it_hip_gather_chunks(it_hip*, const float* src, uint64_t src_len, uint64_t chunk, uint64_t stride,
                          uint64_t offset, float* out, uint64_t out_len); /* mod.rs:664 */
void it_hip_sigmoid_mul(it_hip*, float* x, uint64_t x_len, const float* g, uint64_t g_len); /* :746 */
void it_hip_delta_rule(it_hip*, const it_delta* d, float* state, uint64_t state_len, float* out,
                       uint64_t out_len); /* mod.rs:785 */
void it_hip_add_assign(it_hip*, float* a, uint64_t a_len, const float* b, uint64_t b_len); /* :788 */

/* ---- methods whose defaults touch host memory, overridden for the device ---- */
void it_hip_scale(it_hip*, float* buf, uint64_t len, float s); /* mod.rs:600 */
void it_hip_scatter_chunks(it_hip*, const float* src, uint64_t src_len, uint64_t chunk, uint64_t stride,
                           uint64_t offset, float* dst, uint64_t dst_len); /* mod.rs:730 */
void it_hip_matmul_pair(it_hip*, const it_weights* a, const it_weights* b, const float* x, uint64_t x_len,
                        float* out_a, uint64_t out_a_len, float* out_b, uint64_t out_b_len); /* :1012 */
void it_hip_matmul_experts(it_hip*, const it_experts* w, const it_route* route, const float* x,
                           uint64_t x_len, float* out, uint64_t out_len); /* mod.rs:1049 */
void it_hip_moe_glu(it_hip*, const it_experts* gate, const it_experts* up, const it_route* route,
                    const float* x, uint64_t x_len, float* out, uint64_t out_len, float* scratch,
                    uint64_t scratch_len); /* mod.rs:1105 */
void it_hip_moe_finish(it_hip*, float* out, uint64_t out_len, uint64_t at, uint64_t n, const float* rows,
                       uint64_t rows_len, const it_route* route, const float* shared, uint64_t shared_len,
                       const float* logit, uint64_t logit_len, uint64_t logit_at); /* mod.rs:1134 */
/* Ops::route (mod.rs:1191): the choice stays on the device; *out is a Device route */
void it_hip_route(it_hip*, float* probs, uint64_t probs_len, uint64_t n_expert, uint64_t n_used,
                  it_route* out);
void it_hip_add_scaled_rows(it_hip*, float* acc, uint64_t acc_len, const float* rows, uint64_t rows_len,
                            const float* scales, uint64_t scales_len); /* mod.rs:1228 */
void it_hip_add_scaled_sigmoid(it_hip*, float* acc, uint64_t acc_len, const float* b, uint64_t b_len,
                               const float* logit, uint64_t logit_len); /* mod.rs:1250 */
void it_hip_add_scaled(it_hip*, float* a, uint64_t a_len, const float* b, uint64_t b_len,
                       float scale); /* mod.rs:1265 */
void it_hip_kv_write(it_hip*, uint16_t* slab, uint64_t slab_len, uint64_t offset, const float* src,
                     uint64_t src_len); /* mod.rs:1421 */

/* ---- methods only the qwen4exp architecture calls (mod.rs:705-966): hyper-connection streams, PLE, QSA sparse
 * attention.  That architecture is outside this backend's path; each entry point exists so that a binding covers the
 * whole trait, launches nothing, and records the sticky error "<op>: qwen4exp-only op, not implemented by the hip
 * backend" (the reference refuses unsupported work the same way: first error kept, polled after the run). ---- */
typedef struct {
    uint64_t from, to, ratio, dim;
    const float* norm;
    uint64_t norm_len;
    float eps;
    uint32_t _pad;
    uint64_t n_rot;
    float theta;
    uint32_t _pad2;
} it_qsa_pool; /* struct QsaPool, mod.rs:279-289 */
typedef struct {
    uint64_t n_head, dim, n_blocks, start_pos, ratio, budget;
} it_qsa_select; /* struct QsaSelect, mod.rs:294-305 */
void it_hip_mean_streams(it_hip*, const float* src, uint64_t src_len, uint64_t n_stream, uint64_t nd, float inv,
                         float* out, uint64_t out_len); /* mod.rs:705 */
void it_hip_mul_rows(it_hip*, float* x, uint64_t x_len, const float* w, uint64_t w_len); /* mod.rs:801 */
void it_hip_silu(it_hip*, float* x, uint64_t x_len);                                       /* mod.rs:811 */
void it_hip_sigmoid(it_hip*, float* x, uint64_t x_len);                                    /* mod.rs:818 */
void it_hip_mul_streams(it_hip*, float* out, uint64_t out_len, const float* h, uint64_t h_len, const float* w,
                        uint64_t w_len, uint64_t n_stream); /* mod.rs:828 */
void it_hip_row_dot(it_hip*, const float* a, uint64_t a_len, const float* b, uint64_t b_len, uint64_t width,
                    float* out, uint64_t out_len); /* mod.rs:846 */
void it_hip_signed_sqrt_sigmoid(it_hip*, float* s, uint64_t s_len); /* mod.rs:861 */
void it_hip_dilated_conv(it_hip*, float* state, uint64_t state_len, const float* x, uint64_t x_len, const float* weight,
                         uint64_t w_len, uint64_t kernel, uint64_t dilation, float* out, uint64_t out_len); /* :884 */
void it_hip_qsa_pool(it_hip*, const uint16_t* raw, uint64_t raw_len, float* pooled, uint64_t pooled_len,
                     const it_qsa_pool* p); /* mod.rs:941 */
void it_hip_qsa_select(it_hip*, const float* q, uint64_t q_len, const float* pooled, uint64_t pooled_len,
                       const it_qsa_select* s, float* scores, uint64_t scores_len, uint32_t* cells,
                       uint64_t cells_len); /* mod.rs:954 */
void it_hip_attend_sparse(it_hip*, const it_attn* a, const uint32_t* cells, uint64_t cells_len,
                          const it_qsa_select* sel, float* out, uint64_t out_len); /* mod.rs:966 */

/* ---- residency protocol (mod.rs:1360-1419) ---- */
void it_hip_host_wrote(it_hip*, const float* buf, uint64_t len);
void it_hip_host_needs(it_hip*, float* buf, uint64_t len);
void it_hip_begin_pass(it_hip*, uint64_t n_tokens);
void it_hip_end_pass(it_hip*);
void it_hip_forget_state(it_hip*);
void it_hip_read_state(it_hip*, float* host, uint64_t len);
/* the KV analogue of read_state, for checkpoints: bring a slab's device copy home */
void it_hip_read_kv(it_hip*, uint16_t* slab, uint64_t len);

/* ---- reporting hooks (mod.rs:1300-1358) ---- */
void it_hip_device_report(it_hip*);
void it_hip_reserve_activations(it_hip*, uint64_t bytes);
int it_hip_tier_counters(it_hip*, it_tier_counters* out);
/* "label=value\n" lines into buf; returns bytes written */
size_t it_hip_config_report(it_hip*, char* buf, size_t buf_len);
/* one-time cost charged to the first passes (weight upload + repack), microseconds */
uint64_t it_hip_setup_cost(it_hip*, char* label, size_t label_len);
void it_hip_prefetch_hint(it_hip*, const it_weights* next_router, const float* x, uint64_t x_len, uint64_t k);

/* ---- expert cache API (src/ops/cuda/ops/placement.rs:15-363, src/ops/cuda/experts.rs:34-62) ----
 * 288 GB of device memory hold every expert of the models this backend is measured on, so the cache normally is one
 * tier: each expert matrix of a pooled tensor takes a device slot at first sight of its tensor.  The slab keeps the
 * reference's shape: one uniform slot size (the bytes of one expert matrix; a tensor of another size is refused,
 * experts.rs:890-901), a capacity in slots fixed when the first pooled tensor arrives (set_expert_slots, else
 * set_expert_budget, else free device memory minus the reserves), and per-expert read counters on the device that
 * the expert kernels write.
 * A pool larger than the capacity spills into a second tier, as in the reference: the experts that do not fit live in
 * page-locked host memory mapped into the device's address space (up to set_expert_host_budget bytes), every pooled
 * tensor is then read through a device table of per-expert addresses, and a kernel dereferences an expert wherever it
 * lies, so a miss is slow (it crosses the bus) but never blocks and never changes a value.  Placement is first touch
 * wins device memory; every 64 tokens, at a pass boundary, a bounded number of busy host-tier experts change places
 * with idle device-tier ones (placement.rs:33-80), and replace_experts_by_counts runs that exchange to completion.
 * A pool that outgrows both tiers has cold experts (experts.rs:67-93): no copy of them is held; before an expert kernel
 * runs the picks are read back (such passes never run from a graph; the exchange by counts is paused), and
 * each cold pick is fetched from the model file (set_model_path + set_map_base; else from the tensor's mapping) into a
 * device slot taken by GCLOCK from an expert the routing decision did not pick.  The device tier must hold one
 * decision's picks of a layer's three tensors, else the call is refused with a sticky error.  prefetch_hint (the next
 * layer's router on this layer's input) starts reading the next layer's likely cold experts while this one computes. */
void it_hip_set_expert_budget(it_hip*, uint64_t bytes);      /* placement.rs:178 */
void it_hip_set_expert_host_budget(it_hip*, uint64_t bytes); /* placement.rs:322; 0 = 64 GiB */
void it_hip_set_expert_slots(it_hip*, uint64_t n);           /* placement.rs:157; 0 = by budget */
void it_hip_set_expert_pool(it_hip*, uint64_t n);            /* sizes the read counters, experts.rs:424-438 */
void it_hip_reserve_for_weights(it_hip*, uint64_t dense_bytes); /* placement.rs:203 */
void it_hip_reserve_for_kv(it_hip*, uint64_t bytes);         /* placement.rs:341 */
void it_hip_set_prefetch(it_hip*, int on);                   /* placement.rs:164; nothing to fetch when all resident */
void it_hip_set_model_path(it_hip*, const char* path);       /* placement.rs:357 */
/* reads of cold experts from the model file so far: out[0] through the unbuffered (O_DIRECT) descriptor, out[1] in all
 * (src/ops/cuda/experts.rs:310-312, 510-511: on by default on Linux, INFERRED_FETCH_DIRECT=0 / =1 overrides, a file
 * system that refuses the flag is read buffered) */
void it_hip_fetch_read_counts(it_hip*, uint64_t out[2]);
void it_hip_set_map_base(it_hip*, uint64_t base);            /* placement.rs:363 */
/* lookups / hits come from the device counters (waits for the device), placement.rs:15 */
void it_hip_expert_stats(it_hip*, it_expert_stats* out);
/* share of all expert reads taken by the busiest slab-many matrices, and the reads counted (placement.rs:347,
 * experts.rs:861-873); 0 = ok, 1 = no pooled tensor yet */
int it_hip_expert_coverage(it_hip*, double* fraction, uint64_t* total_reads);
/* re-place the pool by the reads counted so far: busy host-tier experts change places with idle device-tier ones;
 * returns the experts moved into device memory (0 with the whole pool there), -1 on a device error (placement.rs:113) */
int64_t it_hip_replace_experts_by_counts(it_hip*);
/* extension: the per-expert read counts of one tensor (keyed on its data pointer), expert order; returns entries */
uint64_t it_hip_expert_counts(it_hip*, const uint8_t* tensor_data, uint32_t* out, uint64_t cap);
/* GCLOCK victim choice (src/ops/cuda/experts.rs:2215-2233) as a pure function over a
 * ring of heat counters and lease flags; returns the victim index or -1 when every
 * slot is leased.  Never selects a victim in the all-resident tier; kept for tests. */
int64_t it_hip_clock_pick(uint8_t* heat, const uint8_t* leased, uint64_t n, uint64_t* hand);

/* ---- extensions (no counterpart in the reference's trait) ---- */
/* first strict maximum of a device-current activation, computed on the device
 * (the rule of Profile::record_token, src/profile.rs:192-213) */
uint32_t it_hip_argmax(it_hip*, const float* buf, uint64_t len);
/* Greedy feedback without a host round trip: picks the first strict maximum of `logits`
 * (as it_hip_argmax), writes the dequantized row of `table` for that id into `x`
 * (Model::embed, src/model/qwen35.rs:855-873: Q8_0, F16, BF16 or F32 tables) and files the
 * id at ring_index in a device ring of 65536 ids.  Called inside a pass in place of the host
 * embedding; `logits` names the device copy the previous pass left (the host copy is not
 * consulted).  Returns 0 without doing anything when the table type is not handled or the
 * logits have no device copy. */
int it_hip_embed_argmax(it_hip*, const it_weights* table, const float* logits, uint64_t logits_len, float* x,
                        uint64_t x_len, uint64_t ring_index);
/* ids filed by it_hip_embed_argmax at ring indices first_index .. first_index + n (waits for the device) */
void it_hip_read_tokens(it_hip*, uint64_t first_index, uint64_t n, uint32_t* out);
void it_hip_sync(it_hip*);
/* per-kernel-family device time, measured with HIP events recorded on the launch
 * stream around every launch between begin and end (at most 16384 launches) */
typedef struct {
    char name[48];
    uint64_t launches;
    double ms_total;
    uint64_t bytes_total; /* algorithmic bytes: weights read once + activations in and out */
} it_profile_row;
void it_hip_profile_begin(it_hip*);
int it_hip_profile_end(it_hip*, it_profile_row* rows, int max_rows);
/* forget the device copy keyed on one host address: call before freeing a buffer
 * the backend has seen, or a later allocation at the same address reads stale data */
void it_hip_release(it_hip*, const void* host);
/* forget every mirror and resident weight (call when the model file is unmapped) */
void it_hip_drop_mirrors(it_hip*);
uint64_t it_hip_launch_count(it_hip*);
/* decode graphs: captures, replays, fallbacks to eager, kernel launches in the captured graph */
void it_hip_graph_stats(it_hip*, uint64_t out[4]);
/* layer chains (runs of decode layers as one persistent kernel, fast mode; no counterpart in the reference, whose
 * graph keeps one node per kernel: src/ops/cuda/mod.rs:600-647): chain launches in the last fused pass, layers they
 * cover, 1 while chains are enabled for this backend, the bound on a hand-off wait in polls */
void it_hip_chain_stats(it_hip*, uint64_t out[4]);
/* The caller has zeroed the host copy of every recurrent-state slab (a sequence reset): the device copies are
 * zeroed in place, where forget_state (mod.rs:1360-1419) would upload the zeros again at their next use. */
void it_hip_zero_state(it_hip*);
/* This card's matrix-core ceiling, measured: back-to-back MFMA instructions on eight independent
 * accumulators per wave, two waves on every SIMD, no memory in the loop (the method of the reference's
 * own ceilings, tests/cuda_ops.rs:56-72).  kind: 0 int8 16x16x64, 1 int8 16x16x32, 2 f16 32x32x16,
 * 3 f16 16x16x32, 4 f32 16x16x4; iters = instructions per accumulator.  Writes operations per second
 * (2 per multiply-accumulate).  0 = ok, 1 = bad argument, 2 = device error */
int it_hip_mfma_ceiling(it_hip*, int kind, int iters, double* ops_per_s);

/* ---- one entry point that allocates nothing ----
 * No counterpart in the reference (its device backend sizes its pools with the driver's allocator as it goes,
 * src/ops/cuda/mod.rs:1011-1158).  For callers that cannot allocate: code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc.  The computation is it_hip_attend's split-K form (fast mode) for at most 16
 * query rows: same kernels, same split count, bit-identical output.  Differences from it_hip_attend:
 *  - every pointer in `a`, and `out`, is a DEVICE pointer the caller owns (nothing is mirrored or copied);
 *  - `stream` is a hipStream_t (NULL = the null stream); the call only enqueues work on it;
 *  - the split-K partial results live in a fixed array of IT_HIP_NOALLOC_SCRATCH_BYTES inside the library's code
 *    object, one copy per GPU, held until the process ends and shared by every call on that GPU: calls that overlap
 *    on one GPU race.  A problem whose partials (n_q * n_head * n_split * (head_dim + 2) floats; n_split =
 *    ceil(n_pos / 64) capped at 256 for head_dim 64, 128 and 256, ceil(n_pos / 128) otherwise) do not fit is refused;
 *  - it calls no hipMalloc, hipFree or allocating library routine, and needs no it_hip handle;
 *  - the scratch's device address is looked up once per GPU (hipGetSymbolAddress, and an attribute of the tile
 *    kernel set): at it_hip_create, else inside the first call on that GPU.  That first call is therefore not one to
 *    make while a stream is capturing: create a backend, or make one warm-up call, before using it under capture.
 * Returns 0 = enqueued, 1 = bad argument, 2 = too large for the fixed scratch, 3 = device error; the message goes to
 * err. */
#define IT_HIP_NOALLOC_SCRATCH_BYTES (8ull << 20)
int it_hip_attend_noalloc(const it_attn* a, float* out, uint64_t out_len, void* stream, char* err, size_t err_len);

/* ---- model + engine: the host side of the loop over this backend ----------
 * Qwen35::load / forward (src/model/qwen35.rs:755-858, 956-1127) and
 * Engine::{new, prefill, decode, generate, reset} (src/engine/mod.rs:147-437). */
typedef struct it_model it_model;
typedef struct it_engine it_engine;
typedef void (*it_trace_fn)(void* user, const char* name, uint32_t layer, const float* data, uint64_t n);

it_model* it_model_open(const char* gguf_path, char* err, size_t err_len);
void it_model_close(it_model*);
/* n_layer n_embd n_vocab n_head n_head_kv head_dim n_expert n_expert_used expert_ff n_rot */
void it_model_dims(const it_model*, uint64_t out[10]);
/* weight bytes one decode token reads (src/model/qwen35.rs:875-939) */
uint64_t it_model_decode_weight_bytes(const it_model*);
/* multiply-accumulates of one token's pass without the output head: dense matrices, routed expert gate+up,
 * routed expert down (the matrices of src/model/qwen35.rs:875-939) */
void it_model_token_macs(const it_model*, uint64_t out[3]);
it_engine* it_engine_new(it_model*, it_hip*, uint64_t n_ctx, uint64_t max_batch);
void it_engine_free(it_engine*);
void it_engine_reset(it_engine*);
void it_engine_set_trace(it_engine*, it_trace_fn fn, void* user);
uint64_t it_engine_pos(const it_engine*);
/* Engine::checkpoint / restore / rewind (src/engine/mod.rs:223-294).  state_sizes: floats of the conv and ssm slabs
 * (all layers).  checkpoint: brings the device's recurrent state home (read_state per layer), copies both slabs out
 * and returns the position.  restore: 0 = ok; truncates the sequence to pos, reloads the slabs and has the backend
 * forget its copies; the next token must be fed from the host (it_engine_forward).  rewind: 1 = done, 0 = refused
 * (always refused when the model has recurrent layers). */
void it_engine_state_sizes(const it_engine*, uint64_t out[2]);
uint64_t it_engine_checkpoint(it_engine*, float* conv_out, float* ssm_out);
int it_engine_restore(it_engine*, uint64_t pos, const float* conv_in, const float* ssm_in);
int it_engine_rewind(it_engine*, uint64_t len);
/* one forward pass at the current position; logits (n_vocab) may be NULL. 0 = ok */
int it_engine_forward(it_engine*, const uint32_t* tokens, uint64_t n, float* logits);
/* chunked prefill; logits of the last token (may be NULL) */
int it_engine_prefill(it_engine*, const uint32_t* tokens, uint64_t n, float* logits);
/* greedy generation; returns tokens produced or a negative error */
int64_t it_engine_generate(it_engine*, const uint32_t* prompt, uint64_t n_prompt, uint64_t max_new,
                           uint32_t* out_ids, float* last_logits);
/* greedy decode of `n` more tokens from the last logits, argmax on the device; for
 * throughput runs.  Returns tokens produced. */
int64_t it_engine_decode_greedy(it_engine*, uint64_t n, uint32_t* out_ids);
const char* it_engine_last_error(it_engine*);
/* bring device-owned state home and return host pointers (parity tests, checkpoints) */
const float* it_engine_ssm_state(it_engine*, uint64_t layer, uint64_t* len);
const float* it_engine_conv_state(it_engine*, uint64_t layer, uint64_t* len);
const uint16_t* it_engine_k_slab(it_engine*, uint64_t slot, uint64_t* len);
const uint16_t* it_engine_v_slab(it_engine*, uint64_t slot, uint64_t* len);

/* ---- synthetic GGUF writer (the reference ships none; its model tests need real
 * files, tests/common/mod.rs:10-44) ---- */
#define IT_SYNTH_ROUTER_F32 0xffffffffu
typedef struct {
    uint64_t n_layer, n_embd, n_vocab;
    uint64_t n_head, n_head_kv, head_dim, n_rot;
    uint64_t n_expert, n_expert_used, expert_ff, shared_ff;
    uint64_t ssm_d_conv, ssm_d_state, ssm_n_group, ssm_dt_rank; /* d_inner = d_state * dt_rank */
    uint64_t full_attention_interval;
    float rope_theta, rms_eps;
    uint32_t dense_type;  /* IT_Q8_0 */
    uint32_t expert_type; /* IT_Q8_0 or IT_NVFP4 */
    uint32_t router_type; /* router, shared-gate and ssm alpha/beta matrices: 0 = as dense_type, IT_Q8_0, or
                             IT_SYNTH_ROUTER_F32 for F32 (what real files keep them in; IT_F32 itself is 0) */
    uint32_t shared_type; /* the shared expert's matrices: 0 = as dense_type; IT_NVFP4 = NVFP4 with a second, per-tensor
                             scale each (ffn_*_shexp.scale), which is how an NVFP4 file of this model stores them */
    uint64_t seed;
    float weight_std; /* N(0, std) for Q8_0 matrices */
    uint32_t n_threads;
} it_synth_config;
/* 0 = ok */
int it_synth_write_gguf(const char* path, const it_synth_config* cfg, char* err, size_t err_len);

#ifdef __cplusplus
}
#endif
#endif
