// TEST INFRASTRUCTURE — the CPU oracle's ops.  Not part of the shipped library.
//
// A scalar restatement of /root/reference src/ops/naive.rs (the reference's own
// oracle), the default methods of `trait Ops` in src/ops/mod.rs, and the thread
// split of src/ops/spin.rs.  Arithmetic order is the reference's, line for line;
// build with -ffp-contract=off and without fast-math.
//
// Parity status of each function (what pins it) is listed in oracle/README.md.
#include "oracle.h"
#include "orc_math.h"

#include <atomic>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <thread>
#include <vector>

// ------------------------------------------------------------------ thread pool
// src/ops/pool.rs: persistent workers released by a generation counter; unit
// ranges are contiguous spans of ceil(len/n) (Rows::range, pool.rs:240-245).
namespace {

struct Pool {
    int n = 1;
    std::vector<std::thread> workers;
    std::atomic<uint64_t> gen{0};
    std::atomic<int> done{0};
    std::atomic<bool> stop{false};
    const std::function<void(int, int)>* job = nullptr;

    void start(int threads) {
        shutdown();
        n = threads < 1 ? 1 : threads;
        stop = false;
        gen = 0;
        for (int i = 1; i < n; i++) {
            workers.emplace_back([this, i] {
                uint64_t seen = 0;
                for (;;) {
                    int spins = 0;
                    while (gen.load(std::memory_order_acquire) == seen) {
                        if (stop.load(std::memory_order_relaxed)) return;
                        if (++spins > 2000) {
                            std::this_thread::yield();
                        }
                    }
                    seen = gen.load(std::memory_order_acquire);
                    (*job)(i, n);
                    done.fetch_add(1, std::memory_order_release);
                }
            });
        }
    }
    void shutdown() {
        if (workers.empty()) return;
        stop = true;
        for (auto& w : workers) w.join();
        workers.clear();
        n = 1;
    }
    void run(const std::function<void(int, int)>& f) {
        if (n == 1) {
            f(0, 1);
            return;
        }
        job = &f;
        done.store(0, std::memory_order_relaxed);
        gen.fetch_add(1, std::memory_order_release);
        f(0, n);
        while (done.load(std::memory_order_acquire) != n - 1) {
        }
    }
    ~Pool() { shutdown(); }
};

Pool g_pool;

inline void span_of(uint64_t len, int index, int n, uint64_t* start, uint64_t* end) {
    uint64_t per = (len + (uint64_t)n - 1) / (uint64_t)n;
    uint64_t s = per * (uint64_t)index;
    if (s > len) s = len;
    uint64_t e = s + per;
    if (e > len) e = len;
    *start = s;
    *end = e;
}

constexpr uint64_t QK8_0 = 32;
constexpr uint64_t MIN_ROWS = 64;  // src/ops/spin.rs: below this a matmul stays on the caller
constexpr uint64_t MIN_POS = 64;   // src/ops/spin.rs: attention threads only past this

}  // namespace

extern "C" {

void orc_set_threads(int n) { g_pool.start(n); }
int orc_get_threads(void) { return g_pool.n; }

float orc_c_f16_to_f32(uint16_t h) { return orc_f16_to_f32(h); }
uint16_t orc_c_f32_to_f16(float f) { return orc_f32_to_f16(f); }
float orc_c_bf16_to_f32(uint16_t h) { return orc_bf16_to_f32(h); }
float orc_c_ue4m3_to_f32(uint8_t x) { return orc_ue4m3_to_f32(x); }
float orc_c_expf(float x) { return orc_expf(x); }
float orc_c_logf(float x) { return orc_logf(x); }

// src/gguf/types.rs:143-210 — block size and bytes per block.
uint64_t orc_type_bytes(uint32_t ty, uint64_t n) {
    switch (ty) {
        case ORC_F32: return n * 4;
        case ORC_F16: return n * 2;
        case ORC_BF16: return n * 2;
        case ORC_Q8_0: return n / 32 * 34;
        case ORC_NVFP4: return n / 64 * 36;
        default: return 0;
    }
}

// src/quant/mod.rs:40-88 (dispatch), :96-106 (Q8_0), :344-357 (NVFP4).
int orc_dequantize(uint32_t ty, const uint8_t* data, uint64_t n, float* out) {
    switch (ty) {
        case ORC_F32:
            memcpy(out, data, n * 4);
            return 0;
        case ORC_F16:
            for (uint64_t i = 0; i < n; i++) {
                uint16_t h;
                memcpy(&h, data + 2 * i, 2);
                out[i] = orc_f16_to_f32(h);
            }
            return 0;
        case ORC_BF16:
            for (uint64_t i = 0; i < n; i++) {
                uint16_t h;
                memcpy(&h, data + 2 * i, 2);
                out[i] = orc_bf16_to_f32(h);
            }
            return 0;
        case ORC_Q8_0:
            for (uint64_t b = 0; b < n / 32; b++) {
                const uint8_t* blk = data + b * 34;
                uint16_t h;
                memcpy(&h, blk, 2);
                float d = orc_f16_to_f32(h);
                for (int i = 0; i < 32; i++) out[b * 32 + i] = (float)(int8_t)blk[2 + i] * d;
            }
            return 0;
        case ORC_NVFP4:
            for (uint64_t b = 0; b < n / 64; b++) {
                const uint8_t* blk = data + b * 36;
                float* y = out + b * 64;
                for (int s = 0; s < 4; s++) {
                    float d = orc_ue4m3_to_f32(blk[s]);
                    const uint8_t* qs = blk + 4 + s * 8;
                    for (int j = 0; j < 8; j++) {
                        y[s * 16 + j] = (float)ORC_KVALUES_MXFP4[qs[j] & 0xf] * d;
                        y[s * 16 + j + 8] = (float)ORC_KVALUES_MXFP4[qs[j] >> 4] * d;
                    }
                }
            }
            return 0;
        default: return -1;
    }
}

// src/ops/naive.rs:652-675 QuantizedRow::from_f32 (ggml quantize_row_q8_0_ref).
void orc_quantize_q8_0(const float* x, uint64_t n, float* scales, int8_t* quants) {
    for (uint64_t b = 0; b < n / QK8_0; b++) {
        const float* blk = x + b * QK8_0;
        float amax = 0.0f;
        for (uint64_t i = 0; i < QK8_0; i++) {
            float a = fabsf(blk[i]);
            // f32::max: a NaN operand is skipped
            if (a > amax || amax != amax) amax = a;
        }
        float d = amax / 127.0f;
        float id = d != 0.0f ? 1.0f / d : 0.0f;
        scales[b] = orc_f16_to_f32(orc_f32_to_f16(d));
        for (uint64_t i = 0; i < QK8_0; i++) {
            float r = roundf(blk[i] * id);  // half away from zero
            // Rust `as i8` saturates; NaN -> 0
            int8_t q;
            if (r != r) q = 0;
            else if (r >= 127.0f) q = 127;
            else if (r <= -128.0f) q = -128;
            else q = (int8_t)r;
            quants[b * QK8_0 + i] = q;
        }
    }
}

// src/ops/naive.rs:679-686 to_blocks.
void orc_q8_0_blocks(const float* x, uint64_t n, uint8_t* out) {
    std::vector<float> sc(n / QK8_0);
    std::vector<int8_t> q(n);
    orc_quantize_q8_0(x, n, sc.data(), q.data());
    for (uint64_t b = 0; b < n / QK8_0; b++) {
        uint16_t h = orc_f32_to_f16(sc[b]);
        memcpy(out + b * 34, &h, 2);
        memcpy(out + b * 34 + 2, q.data() + b * QK8_0, QK8_0);
    }
}

// src/ops/naive.rs:691-704.
float orc_dot_q8_0_q8_0(const uint8_t* row, uint64_t n, const float* scales, const int8_t* quants) {
    float sumf = 0.0f;
    for (uint64_t i = 0; i < n / QK8_0; i++) {
        const uint8_t* blk = row + i * 34;
        uint16_t h;
        memcpy(&h, blk, 2);
        float dw = orc_f16_to_f32(h);
        const int8_t* qs = quants + i * QK8_0;
        int32_t sumi = 0;
        for (uint64_t j = 0; j < QK8_0; j++) sumi += (int32_t)(int8_t)blk[2 + j] * (int32_t)qs[j];
        sumf += (float)sumi * (dw * scales[i]);
    }
    return sumf;
}

// src/ops/naive.rs:714-734.
float orc_dot_nvfp4_q8_0(const uint8_t* row, uint64_t n, const float* scales, const int8_t* quants) {
    float sumf = 0.0f;
    for (uint64_t ib = 0; ib < n / 64; ib++) {
        const uint8_t* blk = row + ib * 36;
        for (int s = 0; s < 4; s++) {
            float d = orc_ue4m3_to_f32(blk[s]);
            uint64_t q8 = 2 * ib + (uint64_t)(s / 2);
            int off = (s % 2) * 16;
            float dy = scales[q8];
            const int8_t* qa = quants + q8 * QK8_0;
            int32_t lo = 0, hi = 0;
            for (int j = 0; j < 8; j++) {
                uint8_t qv = blk[4 + s * 8 + j];
                lo += (int32_t)qa[off + j] * (int32_t)ORC_KVALUES_MXFP4[qv & 0xf];
                hi += (int32_t)qa[off + j + 8] * (int32_t)ORC_KVALUES_MXFP4[qv >> 4];
            }
            sumf += dy * d * (float)(lo + hi);
        }
    }
    return sumf;
}

}  // extern "C"

namespace {

// src/ops/naive.rs:843-861 dot_row: serial f32 fold from zero.
float dot_row(uint32_t ty, const uint8_t* row, const float* x, uint64_t n) {
    float sum = 0.0f;
    if (ty == ORC_F32) {
        for (uint64_t i = 0; i < n; i++) {
            float w;
            memcpy(&w, row + 4 * i, 4);
            sum += w * x[i];
        }
    } else if (ty == ORC_F16) {
        for (uint64_t i = 0; i < n; i++) {
            uint16_t h;
            memcpy(&h, row + 2 * i, 2);
            sum += orc_f16_to_f32(h) * x[i];
        }
    } else if (ty == ORC_BF16) {
        for (uint64_t i = 0; i < n; i++) {
            uint16_t h;
            memcpy(&h, row + 2 * i, 2);
            sum += orc_bf16_to_f32(h) * x[i];
        }
    }
    return sum;
}

struct Act {
    std::vector<float> scales;
    std::vector<int8_t> quants;
    bool quantized = false;
    void of(uint32_t ty, const float* x, uint64_t n) {
        quantized = (ty == ORC_Q8_0 || ty == ORC_NVFP4);
        if (quantized) {
            scales.resize(n / QK8_0);
            quants.resize(n);
            orc_quantize_q8_0(x, n, scales.data(), quants.data());
        }
    }
    float dot(uint32_t ty, const uint8_t* row, const float* x, uint64_t n) const {
        if (ty == ORC_Q8_0) return orc_dot_q8_0_q8_0(row, n, scales.data(), quants.data());
        if (ty == ORC_NVFP4) return orc_dot_nvfp4_q8_0(row, n, scales.data(), quants.data());
        return dot_row(ty, row, x, n);
    }
};

// src/ops/naive.rs:38-83 matmul_row.
void matmul_row(const orc_weights* w, const float* x, float* out) {
    Act qx;
    qx.of(w->ty, x, w->n_in);
    uint64_t stride = orc_type_bytes(w->ty, w->n_in);
    for (uint64_t j = 0; j < w->n_out; j++) out[j] = qx.dot(w->ty, w->data + j * stride, x, w->n_in);
}

// src/ops/naive.rs:633-640.
float rms_scale(const float* x, uint64_t n, float eps) {
    double sum = 0.0;
    for (uint64_t i = 0; i < n; i++) sum += (double)(x[i] * x[i]);
    float mean = (float)(sum / (double)n);
    return 1.0f / sqrtf(mean + eps);
}

// src/ops/naive.rs:362-376.
void softmax_in_place(float* x, uint64_t n) {
    if (n == 0) return;
    float max = -INFINITY;
    for (uint64_t i = 0; i < n; i++) {
        // f32::max skips NaN
        if (x[i] > max || max != max) max = x[i];
    }
    float sum = 0.0f;
    for (uint64_t i = 0; i < n; i++) {
        x[i] = orc_expf(x[i] - max);
        sum += x[i];
    }
    for (uint64_t i = 0; i < n; i++) x[i] /= sum;
}

struct AttnScratch {
    std::vector<float> scores, conv;
};

// src/ops/naive.rs:420-466 attend_kv_head.
void attend_kv_head(const orc_attn* a, uint64_t t, uint64_t h_kv, float* out, AttnScratch& sc) {
    uint64_t hd = a->head_dim, group = a->n_head / a->n_head_kv;
    uint64_t n_q = a->q_len / (a->n_head * hd);
    uint64_t n_pos = a->n_pos - n_q + 1 + t;  // Attn::n_pos_of, src/ops/mod.rs:273-275
    uint64_t off = h_kv * hd;
    uint64_t q_row = t * a->n_head * hd;
    sc.scores.resize(group * a->n_pos);
    sc.conv.resize(hd);
    for (uint64_t s = 0; s < n_pos; s++) {
        const uint16_t* key = a->k + s * a->kv_dim + off;
        for (uint64_t i = 0; i < hd; i++) sc.conv[i] = orc_f16_to_f32(key[i]);
        for (uint64_t g = 0; g < group; g++) {
            const float* q = a->q + q_row + (h_kv * group + g) * hd;
            float dot = 0.0f;
            for (uint64_t i = 0; i < hd; i++) dot += q[i] * sc.conv[i];
            sc.scores[g * n_pos + s] = dot * a->scale;
        }
    }
    for (uint64_t g = 0; g < group; g++) softmax_in_place(sc.scores.data() + g * n_pos, n_pos);
    for (uint64_t i = 0; i < group * hd; i++) out[i] = 0.0f;
    for (uint64_t s = 0; s < n_pos; s++) {
        const uint16_t* val = a->v + s * a->kv_dim + off;
        for (uint64_t i = 0; i < hd; i++) sc.conv[i] = orc_f16_to_f32(val[i]);
        for (uint64_t g = 0; g < group; g++) {
            float w = sc.scores[g * n_pos + s];
            float* o = out + g * hd;
            for (uint64_t i = 0; i < hd; i++) o[i] += w * sc.conv[i];
        }
    }
}

}  // namespace

extern "C" {

// src/ops/naive.rs:139-152.
void orc_rms_norm(const float* x, uint64_t x_len, const float* w, uint64_t nd, float eps, float* out) {
    for (uint64_t r = 0; r < x_len / nd; r++) {
        const float* row = x + r * nd;
        float* o = out + r * nd;
        float scale = rms_scale(row, nd, eps);
        for (uint64_t i = 0; i < nd; i++) o[i] = row[i] * scale * w[i];
    }
}

// src/ops/naive.rs:154-164.
void orc_rms_norm_heads(float* x, uint64_t x_len, const float* w, uint64_t head_dim, float eps) {
    for (uint64_t r = 0; r < x_len / head_dim; r++) {
        float* head = x + r * head_dim;
        float scale = rms_scale(head, head_dim, eps);
        for (uint64_t i = 0; i < head_dim; i++) head[i] = head[i] * scale * w[i];
    }
}

// src/ops/naive.rs:166-178 (serial) and src/ops/spin.rs:157-205 (threaded; same dots,
// rows split in contiguous spans, bit-identical by construction).
void orc_matmul(const orc_weights* w, const float* x, uint64_t x_len, float* out) {
    uint64_t n = x_len / w->n_in;
    if (w->n_out < MIN_ROWS || g_pool.n == 1) {
        for (uint64_t t = 0; t < n; t++) matmul_row(w, x + t * w->n_in, out + t * w->n_out);
        return;
    }
    std::vector<Act> qx(n);
    for (uint64_t t = 0; t < n; t++) qx[t].of(w->ty, x + t * w->n_in, w->n_in);
    uint64_t stride = orc_type_bytes(w->ty, w->n_in);
    const uint64_t TOKEN_TILE = 8;
    g_pool.run([&](int index, int nw) {
        uint64_t start, end;
        span_of(w->n_out, index, nw, &start, &end);
        for (uint64_t lo = 0; lo < n; lo += TOKEN_TILE) {
            uint64_t hi = lo + TOKEN_TILE < n ? lo + TOKEN_TILE : n;
            for (uint64_t j = start; j < end; j++) {
                const uint8_t* row = w->data + j * stride;
                for (uint64_t t = lo; t < hi; t++)
                    out[t * w->n_out + j] = qx[t].dot(w->ty, row, x + t * w->n_in, w->n_in);
            }
        }
    });
}

// src/ops/mod.rs:1012-1022.
void orc_matmul_pair(const orc_weights* a, const orc_weights* b, const float* x, uint64_t x_len, float* out_a,
                     float* out_b) {
    orc_matmul(a, x, x_len, out_a);
    orc_matmul(b, x, x_len, out_b);
}

// src/ops/naive.rs:180-218.
void orc_rope_neox(float* x, uint64_t x_len, uint64_t pos, uint64_t head_dim, uint64_t n_rot, uint64_t n_heads,
                   float theta) {
    uint64_t per_row = head_dim * n_heads;
    uint64_t half = n_rot / 2;
    for (uint64_t t = 0; t < x_len / per_row; t++) {
        uint64_t p = pos + t;
        for (uint64_t h = 0; h < n_heads; h++) {
            float* head = x + t * per_row + h * head_dim;
            for (uint64_t i = 0; i < half; i++) {
                double freq = pow((double)theta, -2.0 * (double)i / (double)n_rot);
                double th = (double)p * freq;
                float sn = (float)sin(th), cs = (float)cos(th);
                float x0 = head[i], x1 = head[i + half];
                head[i] = x0 * cs - x1 * sn;
                head[i + half] = x0 * sn + x1 * cs;
            }
        }
    }
}

// src/ops/naive.rs:220-227.
void orc_softmax(float* x, uint64_t x_len, uint64_t row) {
    if (row == 0) return;
    for (uint64_t at = 0; at < x_len; at += row) {
        uint64_t n = at + row <= x_len ? row : x_len - at;
        softmax_in_place(x + at, n);
    }
}

// src/ops/naive.rs:229-244 (serial) and src/ops/spin.rs:213-249 (threaded over (t, h_kv)).
void orc_attend(const orc_attn* a, float* out) {
    uint64_t hd = a->head_dim;
    uint64_t n_q = a->q_len / (a->n_head * hd);
    uint64_t group = a->n_head / a->n_head_kv;
    uint64_t per_kv = group * hd, per_row = a->n_head * hd;
    uint64_t units = n_q * a->n_head_kv;
    if (a->n_pos < MIN_POS || (a->n_head_kv < 2 && n_q < 2) || g_pool.n == 1) {
        AttnScratch sc;
        for (uint64_t u = 0; u < units; u++) {
            uint64_t t = u / a->n_head_kv, h = u % a->n_head_kv;
            attend_kv_head(a, t, h, out + t * per_row + h * per_kv, sc);
        }
        return;
    }
    g_pool.run([&](int index, int nw) {
        uint64_t first, last;
        span_of(units, index, nw, &first, &last);
        AttnScratch sc;
        for (uint64_t u = first; u < last; u++) {
            uint64_t t = u / a->n_head_kv, h = u % a->n_head_kv;
            attend_kv_head(a, t, h, out + t * per_row + h * per_kv, sc);
        }
    });
}

// src/ops/naive.rs:246-252.
void orc_silu_mul(float* gate, const float* up, uint64_t n) {
    for (uint64_t i = 0; i < n; i++) {
        float g = gate[i];
        gate[i] = g / (1.0f + orc_expf(-g)) * up[i];
    }
}

// src/ops/mod.rs:600-604.
void orc_scale(float* buf, uint64_t n, float s) {
    for (uint64_t i = 0; i < n; i++) buf[i] *= s;
}

// src/ops/naive.rs:254-273.
void orc_l2_norm_heads(float* x, uint64_t x_len, uint64_t head_dim, float eps) {
    for (uint64_t r = 0; r < x_len / head_dim; r++) {
        float* head = x + r * head_dim;
        double sum = 0.0;
        for (uint64_t i = 0; i < head_dim; i++) sum += (double)(head[i] * head[i]);
        float nrm = sqrtf((float)sum);
        // f32::max(eps): NaN operand skipped
        float m = (nrm > eps || eps != eps) ? nrm : eps;
        if (nrm != nrm) m = eps;
        float scale = 1.0f / m;
        for (uint64_t i = 0; i < head_dim; i++) head[i] *= scale;
    }
}

// src/ops/naive.rs:275-315.
void orc_ssm_conv(float* state, const float* x, uint64_t x_len, const float* weight, uint64_t w_len,
                  uint64_t kernel, float* out) {
    uint64_t keep = kernel - 1;
    uint64_t nc = w_len / kernel;
    for (uint64_t t = 0; t < x_len / nc; t++) {
        const float* xt = x + t * nc;
        float* ot = out + t * nc;
        for (uint64_t c = 0; c < nc; c++) {
            float* past = state + c * keep;
            float sum = 0.0f;
            for (uint64_t k = 0; k < keep; k++) sum += past[k] * weight[c * kernel + k];
            sum += xt[c] * weight[c * kernel + keep];
            ot[c] = sum / (1.0f + orc_expf(-sum));
            for (uint64_t k = 0; k + 1 < keep; k++) past[k] = past[k + 1];
            past[keep - 1] = xt[c];
        }
    }
}

// src/ops/naive.rs:317-330.
void orc_gather_chunks(const float* src, uint64_t chunk, uint64_t stride, uint64_t offset, float* out,
                       uint64_t out_len) {
    for (uint64_t c = 0; c < out_len / chunk; c++) memcpy(out + c * chunk, src + c * stride + offset, chunk * 4);
}

// src/ops/mod.rs:730-742.
void orc_scatter_chunks(const float* src, uint64_t src_len, uint64_t chunk, uint64_t stride, uint64_t offset,
                        float* dst) {
    for (uint64_t i = 0; i < src_len / chunk; i++) memcpy(dst + offset + i * stride, src + i * chunk, chunk * 4);
}

// src/ops/naive.rs:332-337.
void orc_sigmoid_mul(float* x, const float* g, uint64_t n) {
    for (uint64_t i = 0; i < n; i++) x[i] *= 1.0f / (1.0f + orc_expf(-g[i]));
}

// src/ops/naive.rs:86-135 (one token), :339-350 (batch), Delta helpers src/ops/mod.rs:403-455.
void orc_delta_rule(const orc_delta* d, float* state, float* out) {
    uint64_t sk = d->head_k_dim, sv = d->head_v_dim;
    uint64_t kper = d->n_k_heads * sk, vper = d->n_v_heads * sv;
    float q_scale = 1.0f / sqrtf((float)sk);
    for (uint64_t t = 0; t < d->n_tokens; t++) {
        const float* qt = d->q + t * kper;
        const float* kt = d->k + t * kper;
        const float* vt = d->v + t * vper;
        const float* alpha = d->alpha + t * d->n_v_heads;
        const float* beta_raw = d->beta + t * d->n_v_heads;
        float* ot = out + t * vper;
        for (uint64_t h = 0; h < d->n_v_heads; h++) {
            uint64_t kh = h % d->n_k_heads;
            const float* q = qt + kh * sk;
            const float* k = kt + kh * sk;
            const float* v = vt + h * sv;
            float* s = state + h * sk * sv;
            float a = alpha[h] + d->dt_bias[h];
            float softplus = a > 20.0f ? a : orc_logf(1.0f + orc_expf(a));
            float g = orc_expf(softplus * d->ssm_a[h]);
            float beta = 1.0f / (1.0f + orc_expf(-beta_raw[h]));
            for (uint64_t i = 0; i < sk * sv; i++) s[i] *= g;
            for (uint64_t j = 0; j < sv; j++) {
                float* row = s + j * sk;
                float pred = 0.0f;
                for (uint64_t i = 0; i < sk; i++) pred += row[i] * k[i];
                float delta = beta * (v[j] - pred);
                for (uint64_t i = 0; i < sk; i++) row[i] += k[i] * delta;
                float o = 0.0f;
                for (uint64_t i = 0; i < sk; i++) o += row[i] * (q[i] * q_scale);
                ot[h * sv + j] = o;
            }
        }
    }
}

// src/ops/naive.rs:352-357.
void orc_add_assign(float* a, const float* b, uint64_t n) {
    for (uint64_t i = 0; i < n; i++) a[i] += b[i];
}

// src/ops/mod.rs:1265-1270.
void orc_add_scaled(float* a, const float* b, uint64_t n, float scale) {
    for (uint64_t i = 0; i < n; i++) a[i] += b[i] * scale;
}

// src/ops/mod.rs:1228-1238.
void orc_add_scaled_rows(float* acc, uint64_t n, const float* rows, const float* scales, uint64_t n_scales) {
    for (uint64_t j = 0; j < n; j++) {
        float v = 0.0f;
        for (uint64_t e = 0; e < n_scales; e++) v += scales[e] * rows[e * n + j];
        acc[j] = v;
    }
}

// src/ops/mod.rs:1250-1253.
void orc_add_scaled_sigmoid(float* acc, const float* b, uint64_t n, const float* logit) {
    float s = 1.0f / (1.0f + orc_expf(-logit[0]));
    orc_add_scaled(acc, b, n, s);
}

// src/ops/mod.rs:1421-1425.
void orc_kv_write(uint16_t* slab, uint64_t offset, const float* src, uint64_t n) {
    for (uint64_t i = 0; i < n; i++) slab[offset + i] = orc_f32_to_f16(src[i]);
}

// src/ops/mod.rs:1191-1216.
void orc_route(const float* probs, uint64_t n_tok, uint64_t n_expert, uint64_t n_used, uint32_t* ids,
               float* weights) {
    for (uint64_t t = 0; t < n_tok; t++) {
        const float* p = probs + t * n_expert;
        uint32_t* mine = ids + t * n_used;
        for (uint64_t r = 0; r < n_used; r++) {
            uint64_t best = UINT64_MAX;
            for (uint64_t e = 0; e < n_expert; e++) {
                bool taken = false;
                for (uint64_t k = 0; k < r; k++) taken |= (mine[k] == e);
                if (taken) continue;
                if (best == UINT64_MAX || p[e] > p[best]) best = e;
            }
            mine[r] = (uint32_t)best;
        }
        float sum = 0.0f;
        for (uint64_t r = 0; r < n_used; r++) sum += p[mine[r]];
        float denom = sum > 6.103515625e-5f ? sum : 6.103515625e-5f;
        for (uint64_t r = 0; r < n_used; r++) weights[t * n_used + r] = p[mine[r]] / denom;
    }
}

// src/ops/mod.rs:1049-1088.
void orc_matmul_experts(const orc_experts* w, const uint32_t* ids, uint64_t n_picks, uint64_t n_used,
                        const float* x, uint64_t x_len, float* out) {
    if (n_used == 0) n_used = 1;
    uint64_t rows = x_len / w->n_in;
    uint64_t stride = orc_type_bytes(w->ty, w->n_in) * w->n_out;
    for (uint64_t i = 0; i < n_picks; i++) {
        uint64_t e = ids[i];
        uint64_t r = rows == n_picks ? i : (rows > 1 ? i / n_used : 0);
        orc_weights one = {w->data + e * stride, stride, w->ty, 1, w->n_in, w->n_out};
        float* row = out + i * w->n_out;
        orc_matmul(&one, x + r * w->n_in, w->n_in, row);
        if (w->scale_len != 0) {
            float s;
            memcpy(&s, w->scale + e * 4, 4);
            orc_scale(row, w->n_out, s);
        }
    }
}

// src/ops/mod.rs:1105-1117.
void orc_moe_glu(const orc_experts* gate, const orc_experts* up, const uint32_t* ids, uint64_t n_picks,
                 uint64_t n_used, const float* x, uint64_t x_len, float* out, float* scratch) {
    orc_matmul_experts(gate, ids, n_picks, n_used, x, x_len, out);
    orc_matmul_experts(up, ids, n_picks, n_used, x, x_len, scratch);
    orc_silu_mul(out, scratch, n_picks * gate->n_out);
}

// src/ops/mod.rs:1134-1171.
void orc_moe_finish(float* out, uint64_t at, uint64_t n, const float* rows, const float* weights,
                    uint64_t n_tok, uint64_t n_used, const float* shared, const float* logit,
                    uint64_t logit_at) {
    for (uint64_t t = 0; t < n_tok; t++) {
        float g = 1.0f / (1.0f + orc_expf(-logit[logit_at + t]));
        const float* w = weights + t * n_used;
        for (uint64_t j = 0; j < n; j++) {
            float v = 0.0f;
            for (uint64_t e = 0; e < n_used; e++) v += w[e] * rows[(t * n_used + e) * n + j];
            v += shared[t * n + j] * g;
            out[at + t * n + j] = v;
        }
    }
}

// src/profile.rs:192-213 record_token: first strict maximum.
uint32_t orc_argmax(const float* logits, uint64_t n) {
    uint64_t i1 = 0;
    for (uint64_t i = 1; i < n; i++)
        if (logits[i] > logits[i1]) i1 = i;
    return (uint32_t)i1;
}

}  // extern "C"
