/* TEST INFRASTRUCTURE — the CPU oracle's C interface.
 *
 * A scalar restatement of the reference's CPU path for the per-token model
 * loop.  Only tests, the smoke check and the benchmark's cpu_baseline leg may
 * load this library; the shipped HIP library never does.
 *
 * Every op takes the same plain-old-data arguments as the HIP C ABI in
 * include/inferred_hip.h, so a parity test calls both with the same buffers.
 */
#ifndef ORC_ORACLE_H
#define ORC_ORACLE_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ggml type codes, src/gguf/types.rs:62-100 */
enum { ORC_F32 = 0, ORC_F16 = 1, ORC_Q8_0 = 8, ORC_BF16 = 30, ORC_NVFP4 = 40 };

typedef struct {
    const uint8_t* data;
    uint64_t len;
    uint32_t ty;
    uint32_t pooled;
    uint64_t n_in, n_out;
} orc_weights;

typedef struct {
    const uint8_t* data;
    uint64_t len;
    uint32_t ty;
    uint32_t _pad;
    uint64_t n_in, n_out, n_expert;
    const uint8_t* scale; /* n_expert little-endian f32, or NULL */
    uint64_t scale_len;   /* bytes */
} orc_experts;

typedef struct {
    const float* q;
    uint64_t q_len;
    const uint16_t* k;
    const uint16_t* v;
    uint64_t kv_len;
    uint64_t kv_dim, n_pos, head_dim, n_head, n_head_kv;
    float scale;
} orc_attn;

typedef struct {
    const float *q, *k, *v, *alpha, *beta, *ssm_a, *dt_bias;
    uint64_t n_tokens;
    uint64_t head_k_dim, head_v_dim, n_k_heads, n_v_heads;
} orc_delta;

/* ---- scalar formats ---- */
float orc_c_f16_to_f32(uint16_t h);
uint16_t orc_c_f32_to_f16(float f);
float orc_c_bf16_to_f32(uint16_t h);
float orc_c_ue4m3_to_f32(uint8_t x);
float orc_c_expf(float x);
float orc_c_logf(float x);
uint64_t orc_type_bytes(uint32_t ty, uint64_t n_elems);
int orc_dequantize(uint32_t ty, const uint8_t* data, uint64_t n, float* out);

/* ---- Q8_0 activations and the integer dots ---- */
void orc_quantize_q8_0(const float* x, uint64_t n, float* scales, int8_t* quants);
void orc_q8_0_blocks(const float* x, uint64_t n, uint8_t* out);
float orc_dot_q8_0_q8_0(const uint8_t* row, uint64_t n, const float* scales, const int8_t* quants);
float orc_dot_nvfp4_q8_0(const uint8_t* row, uint64_t n, const float* scales, const int8_t* quants);

/* ---- the seam's ops (src/ops/mod.rs trait Ops, src/ops/naive.rs) ---- */
void orc_set_threads(int n); /* 1 = naive; >1 = rows / (row,kv head) units split like src/ops/spin.rs */
int orc_get_threads(void);
void orc_rms_norm(const float* x, uint64_t x_len, const float* w, uint64_t nd, float eps, float* out);
void orc_rms_norm_heads(float* x, uint64_t x_len, const float* w, uint64_t head_dim, float eps);
void orc_matmul(const orc_weights* w, const float* x, uint64_t x_len, float* out);
void orc_matmul_pair(const orc_weights* a, const orc_weights* b, const float* x, uint64_t x_len, float* out_a,
                     float* out_b);
void orc_rope_neox(float* x, uint64_t x_len, uint64_t pos, uint64_t head_dim, uint64_t n_rot, uint64_t n_heads,
                   float theta);
void orc_softmax(float* x, uint64_t x_len, uint64_t row);
void orc_attend(const orc_attn* a, float* out);
void orc_silu_mul(float* gate, const float* up, uint64_t n);
void orc_scale(float* buf, uint64_t n, float s);
void orc_l2_norm_heads(float* x, uint64_t x_len, uint64_t head_dim, float eps);
void orc_ssm_conv(float* state, const float* x, uint64_t x_len, const float* weight, uint64_t w_len,
                  uint64_t kernel, float* out);
void orc_gather_chunks(const float* src, uint64_t chunk, uint64_t stride, uint64_t offset, float* out,
                       uint64_t out_len);
void orc_scatter_chunks(const float* src, uint64_t src_len, uint64_t chunk, uint64_t stride, uint64_t offset,
                        float* dst);
void orc_sigmoid_mul(float* x, const float* g, uint64_t n);
void orc_delta_rule(const orc_delta* d, float* state, float* out);
void orc_add_assign(float* a, const float* b, uint64_t n);
void orc_add_scaled(float* a, const float* b, uint64_t n, float scale);
void orc_add_scaled_rows(float* acc, uint64_t n, const float* rows, const float* scales, uint64_t n_scales);
void orc_add_scaled_sigmoid(float* acc, const float* b, uint64_t n, const float* logit);
void orc_kv_write(uint16_t* slab, uint64_t offset, const float* src, uint64_t n);
/* route: probs [n_tok, n_expert] -> ids (u32) and weights, token-major, n_used each */
void orc_route(const float* probs, uint64_t n_tok, uint64_t n_expert, uint64_t n_used, uint32_t* ids,
               float* weights);
void orc_matmul_experts(const orc_experts* w, const uint32_t* ids, uint64_t n_picks, uint64_t n_used,
                        const float* x, uint64_t x_len, float* out);
void orc_moe_glu(const orc_experts* gate, const orc_experts* up, const uint32_t* ids, uint64_t n_picks,
                 uint64_t n_used, const float* x, uint64_t x_len, float* out, float* scratch);
void orc_moe_finish(float* out, uint64_t at, uint64_t n, const float* rows, const float* weights,
                    uint64_t n_tok, uint64_t n_used, const float* shared, const float* logit,
                    uint64_t logit_at);
uint32_t orc_argmax(const float* logits, uint64_t n);

/* ---- model + engine (src/model/qwen35.rs, src/engine/mod.rs) ---- */
typedef struct orc_model orc_model;
typedef struct orc_engine orc_engine;
/* trace hook: called after each named intermediate, like src/model/qwen35.rs ctx.trace */
typedef void (*orc_trace_fn)(void* user, const char* name, uint32_t layer, const float* data, uint64_t n);

orc_model* orc_model_open(const char* gguf_path, char* err, size_t err_len);
void orc_model_close(orc_model* m);
/* writes: n_layer n_embd n_vocab n_head n_head_kv head_dim n_expert n_expert_used expert_ff n_rot */
void orc_model_dims(const orc_model* m, uint64_t out[10]);
uint64_t orc_model_decode_weight_bytes(const orc_model* m);
orc_engine* orc_engine_new(orc_model* m, uint64_t n_ctx, uint64_t max_batch);
void orc_engine_free(orc_engine* e);
void orc_engine_reset(orc_engine* e);
void orc_engine_set_trace(orc_engine* e, orc_trace_fn fn, void* user);
uint64_t orc_engine_pos(const orc_engine* e);
/* one forward pass over n tokens at the current position; logits [n_vocab] out. 0 = ok */
int orc_engine_forward(orc_engine* e, const uint32_t* tokens, uint64_t n, float* logits);
/* chunked prefill (max_batch) then greedy decode; returns number produced, <0 on error */
int64_t orc_engine_generate(orc_engine* e, const uint32_t* prompt, uint64_t n_prompt, uint64_t max_new,
                            uint32_t* out_ids, float* last_logits);
/* state access for parity tests */
const float* orc_engine_ssm_state(orc_engine* e, uint64_t layer, uint64_t* len);
const float* orc_engine_conv_state(orc_engine* e, uint64_t layer, uint64_t* len);
const uint16_t* orc_engine_k_slab(orc_engine* e, uint64_t slot, uint64_t* len);
const uint16_t* orc_engine_v_slab(orc_engine* e, uint64_t slot, uint64_t* len);

#ifdef __cplusplus
}
#endif
#endif
