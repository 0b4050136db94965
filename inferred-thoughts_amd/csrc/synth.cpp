// Seeded synthetic qwen35moe GGUF writer.
//
// The reference ships no synthetic model: every model-level test of it needs a
// real GGUF (/root/reference tests/common/mod.rs:10-44).  This writes one with the
// tensor names, shapes and metadata keys its loader reads
// (src/model/qwen35.rs:333-431, 776-831), so the CPU oracle and the HIP path can
// be run on the same file.
//
// Choices the shapes leave open, fixed here for both sides:
//   PRNG        splitmix64 keyed by (seed, tensor index, element index); normals by Box-Muller
//   matrices    N(0, weight_std) quantized to Q8_0 with ggml's rule; NVFP4 experts draw the
//               nibbles uniformly over the 16 codes and the UE4M3 scales from |N(0,1)|, with a
//               per-expert f32 second scale that brings the weights to about weight_std
//   norms       1.0 (F32); ssm_a = -exp(N(0,1)) (must be negative); ssm_dt.bias, conv taps N(0, .5)
#include <fcntl.h>
#include <sys/mman.h>
#include <unistd.h>

#include <cmath>
#include <cstdio>
#include <cstring>
#include <functional>
#include <string>
#include <thread>
#include <vector>

#include "../../include/inferred_hip.h"
#include "gguf.h"
#include "host_formats.h"

namespace {

inline uint64_t splitmix(uint64_t x) {
    x += 0x9e3779b97f4a7c15ull;
    x = (x ^ (x >> 30)) * 0xbf58476d1ce4e5b9ull;
    x = (x ^ (x >> 27)) * 0x94d049bb133111ebull;
    return x ^ (x >> 31);
}
inline uint64_t key_of(uint64_t seed, uint64_t tensor, uint64_t i) {
    return splitmix(splitmix(seed * 0x2545f4914f6cdd1dull + tensor) + i);
}
inline double unit(uint64_t h) { return ((double)(h >> 11) + 0.5) * (1.0 / 9007199254740992.0); }
inline float normal(uint64_t seed, uint64_t tensor, uint64_t i) {
    uint64_t h = key_of(seed, tensor, i);
    double u1 = unit(h), u2 = unit(splitmix(h));
    return (float)(std::sqrt(-2.0 * std::log(u1)) * std::cos(6.283185307179586 * u2));
}

struct Spec {
    std::string name;
    std::vector<uint64_t> dims;
    uint32_t ty;
    int kind;  // 0 normal matrix, 1 ones, 2 ssm_a, 3 N(0,0.5) f32, 4 nvfp4 experts, 5 expert scale
    uint64_t offset = 0, bytes = 0;
};

struct Out {
    std::vector<uint8_t> b;
    template <class T> void put(T v) { const uint8_t* p = (const uint8_t*)&v; b.insert(b.end(), p, p + sizeof(T)); }
    void str(const std::string& s) { put<uint64_t>(s.size()); b.insert(b.end(), s.begin(), s.end()); }
    void kv_u32(const std::string& k, uint32_t v) { str(k); put<uint32_t>(4); put<uint32_t>(v); }
    void kv_f32(const std::string& k, float v) { str(k); put<uint32_t>(6); put<float>(v); }
    void kv_str(const std::string& k, const std::string& v) { str(k); put<uint32_t>(8); str(v); }
    void kv_i32s(const std::string& k, const std::vector<int32_t>& v) {
        str(k); put<uint32_t>(9); put<uint32_t>(5); put<uint64_t>(v.size());
        for (auto x : v) put<int32_t>(x);
    }
};

void parallel_rows(uint64_t n, unsigned threads, const std::function<void(uint64_t, uint64_t)>& f) {
    if (threads <= 1 || n < 64) {
        f(0, n);
        return;
    }
    std::vector<std::thread> th;
    uint64_t per = (n + threads - 1) / threads;
    for (unsigned t = 0; t < threads; t++) {
        uint64_t lo = per * t, hi = lo + per < n ? lo + per : n;
        if (lo >= hi) break;
        th.emplace_back([=, &f] { f(lo, hi); });
    }
    for (auto& t : th) t.join();
}

}  // namespace

extern "C" int it_synth_write_gguf(const char* path, const it_synth_config* c, char* err, size_t err_len) {
    auto bad = [&](const std::string& m) {
        if (err && err_len) snprintf(err, err_len, "%s", m.c_str());
        return 1;
    };
    if (!c || !path) return bad("null argument");
    if (c->n_embd % 64 || c->expert_ff % 64 || c->shared_ff % 64 || c->head_dim % 32)
        return bad("n_embd, expert_ff, shared_ff must be multiples of 64 and head_dim of 32");
    if (c->expert_type != IT_Q8_0 && c->expert_type != IT_NVFP4) return bad("expert_type must be Q8_0 or NVFP4");
    if (c->shared_type != 0 && c->shared_type != IT_NVFP4) return bad("shared_type must be 0 (as the dense matrices) or NVFP4");
    const uint64_t nd = c->n_embd, dk = c->ssm_d_state, nv = c->ssm_dt_rank, nk = c->ssm_n_group;
    const uint64_t d_inner = dk * nv, key_dim = dk * nk, conv_dim = 2 * key_dim + d_inner;
    const uint64_t qd = c->head_dim * c->n_head, kvd = c->head_dim * c->n_head_kv;
    const uint32_t D = c->dense_type ? c->dense_type : IT_Q8_0;
    const uint32_t R = c->router_type == IT_SYNTH_ROUTER_F32 ? (uint32_t)IT_F32 : (c->router_type ? c->router_type : D);
    std::vector<Spec> specs;
    auto add = [&](const std::string& n, std::vector<uint64_t> dims, uint32_t ty, int kind) {
        specs.push_back(Spec{n, dims, ty, kind});
    };
    add("token_embd.weight", {nd, c->n_vocab}, D, 0);
    add("output_norm.weight", {nd}, IT_F32, 1);
    add("output.weight", {nd, c->n_vocab}, D, 0);
    for (uint64_t i = 0; i < c->n_layer; i++) {
        auto nm = [&](const char* s) { return "blk." + std::to_string(i) + "." + s; };
        bool rec = (i + 1) % c->full_attention_interval != 0;
        add(nm("attn_norm.weight"), {nd}, IT_F32, 1);
        add(nm("post_attention_norm.weight"), {nd}, IT_F32, 1);
        if (rec) {
            add(nm("attn_qkv.weight"), {nd, conv_dim}, D, 0);
            add(nm("attn_gate.weight"), {nd, d_inner}, D, 0);
            add(nm("ssm_conv1d.weight"), {c->ssm_d_conv, conv_dim}, IT_F32, 3);
            add(nm("ssm_beta.weight"), {nd, nv}, R, 0);
            add(nm("ssm_alpha.weight"), {nd, nv}, R, 0);
            add(nm("ssm_a"), {nv}, IT_F32, 2);
            add(nm("ssm_dt.bias"), {nv}, IT_F32, 3);
            add(nm("ssm_norm.weight"), {dk}, IT_F32, 1);
            add(nm("ssm_out.weight"), {d_inner, nd}, D, 0);
        } else {
            add(nm("attn_q.weight"), {nd, 2 * qd}, D, 0);
            add(nm("attn_k.weight"), {nd, kvd}, D, 0);
            add(nm("attn_v.weight"), {nd, kvd}, D, 0);
            add(nm("attn_output.weight"), {qd, nd}, D, 0);
            add(nm("attn_q_norm.weight"), {c->head_dim}, IT_F32, 1);
            add(nm("attn_k_norm.weight"), {c->head_dim}, IT_F32, 1);
        }
        add(nm("ffn_gate_inp.weight"), {nd, c->n_expert}, R, 0);
        int ek = c->expert_type == IT_NVFP4 ? 4 : 0;
        add(nm("ffn_gate_exps.weight"), {nd, c->expert_ff, c->n_expert}, c->expert_type, ek);
        add(nm("ffn_up_exps.weight"), {nd, c->expert_ff, c->n_expert}, c->expert_type, ek);
        add(nm("ffn_down_exps.weight"), {c->expert_ff, nd, c->n_expert}, c->expert_type, ek);
        if (c->expert_type == IT_NVFP4) {
            add(nm("ffn_gate_exps.scale"), {c->n_expert}, IT_F32, 5);
            add(nm("ffn_up_exps.scale"), {c->n_expert}, IT_F32, 5);
            add(nm("ffn_down_exps.scale"), {c->n_expert}, IT_F32, 5);
        }
        if (c->shared_type == IT_NVFP4) {
            add(nm("ffn_gate_shexp.weight"), {nd, c->shared_ff}, IT_NVFP4, 4);
            add(nm("ffn_up_shexp.weight"), {nd, c->shared_ff}, IT_NVFP4, 4);
            add(nm("ffn_down_shexp.weight"), {c->shared_ff, nd}, IT_NVFP4, 4);
            add(nm("ffn_gate_shexp.scale"), {1}, IT_F32, 5);
            add(nm("ffn_up_shexp.scale"), {1}, IT_F32, 5);
            add(nm("ffn_down_shexp.scale"), {1}, IT_F32, 5);
        } else {
            add(nm("ffn_gate_shexp.weight"), {nd, c->shared_ff}, D, 0);
            add(nm("ffn_up_shexp.weight"), {nd, c->shared_ff}, D, 0);
            add(nm("ffn_down_shexp.weight"), {c->shared_ff, nd}, D, 0);
        }
        add(nm("ffn_gate_inp_shexp.weight"), {nd}, R, 0);
    }
    const uint64_t align = 32;
    uint64_t off = 0;
    for (Spec& s : specs) {
        uint64_t n = 1;
        for (auto d : s.dims) n *= d;
        s.bytes = itg::type_bytes(s.ty, n);
        if (s.bytes == 0) return bad("tensor " + s.name + ": shape is not a whole number of blocks");
        s.offset = off;
        off = (off + s.bytes + align - 1) / align * align;
    }
    Out h;
    h.b.insert(h.b.end(), {'G', 'G', 'U', 'F'});
    h.put<uint32_t>(3);
    h.put<int64_t>((int64_t)specs.size());
    const std::string a = "qwen35moe";
    std::vector<std::pair<std::string, uint32_t>> u32s = {
        {"block_count", (uint32_t)c->n_layer}, {"embedding_length", (uint32_t)nd},
        {"expert_count", (uint32_t)c->n_expert}, {"expert_used_count", (uint32_t)c->n_expert_used},
        {"expert_feed_forward_length", (uint32_t)c->expert_ff},
        {"expert_shared_feed_forward_length", (uint32_t)c->shared_ff},
        {"attention.head_count", (uint32_t)c->n_head}, {"attention.head_count_kv", (uint32_t)c->n_head_kv},
        {"attention.key_length", (uint32_t)c->head_dim}, {"attention.value_length", (uint32_t)c->head_dim},
        {"rope.dimension_count", (uint32_t)c->n_rot}, {"ssm.conv_kernel", (uint32_t)c->ssm_d_conv},
        {"ssm.inner_size", (uint32_t)d_inner}, {"ssm.state_size", (uint32_t)dk},
        {"ssm.time_step_rank", (uint32_t)nv}, {"ssm.group_count", (uint32_t)nk},
        {"full_attention_interval", (uint32_t)c->full_attention_interval}};
    h.put<int64_t>((int64_t)(u32s.size() + 5));
    h.kv_str("general.architecture", a);
    h.kv_u32("general.alignment", (uint32_t)align);
    for (auto& kv : u32s) h.kv_u32(a + "." + kv.first, kv.second);
    h.kv_f32(a + ".rope.freq_base", c->rope_theta);
    h.kv_f32(a + ".attention.layer_norm_rms_epsilon", c->rms_eps);
    int32_t r4 = (int32_t)(c->n_rot / 4);
    h.kv_i32s(a + ".rope.dimension_sections", {r4 + (int32_t)(c->n_rot / 2 - 3 * r4 > 0 ? 0 : 0), r4, (int32_t)(c->n_rot / 2) - 2 * r4, 0});
    for (const Spec& s : specs) {
        h.str(s.name);
        h.put<uint32_t>((uint32_t)s.dims.size());
        for (auto d : s.dims) h.put<int64_t>((int64_t)d);
        h.put<uint32_t>(s.ty);
        h.put<uint64_t>(s.offset);
    }
    uint64_t data_start = (h.b.size() + align - 1) / align * align;
    uint64_t total = data_start + off;
    int fd = ::open(path, O_RDWR | O_CREAT | O_TRUNC, 0644);
    if (fd < 0) return bad(std::string("cannot create ") + path);
    if (ftruncate(fd, (off_t)total) != 0) {
        close(fd);
        return bad("cannot size the output file (disk full?)");
    }
    uint8_t* base = (uint8_t*)mmap(nullptr, total, PROT_READ | PROT_WRITE, MAP_SHARED, fd, 0);
    if (base == MAP_FAILED) {
        close(fd);
        return bad("cannot map the output file");
    }
    memcpy(base, h.b.data(), h.b.size());
    unsigned threads = c->n_threads ? c->n_threads : 1;
    const float std_w = c->weight_std > 0 ? c->weight_std : 0.02f;
    // |N(0,1)| -> UE4M3 code lookup over 4096 quantiles
    std::vector<uint8_t> scale_lut(4096);
    {
        // quantiles by bisection on erf
        for (int k = 0; k < 4096; k++) {
            double q = (k + 0.5) / 4096.0, lo = 0, hi = 8;
            for (int it = 0; it < 60; it++) {
                double mid = 0.5 * (lo + hi);
                if (std::erf(mid / std::sqrt(2.0)) < q) lo = mid; else hi = mid;
            }
            uint8_t code = ith::ue4m3_encode((float)(0.5 * (lo + hi)));
            scale_lut[k] = code == 0 ? 1 : code;
        }
    }
    for (size_t ti = 0; ti < specs.size(); ti++) {
        const Spec& s = specs[ti];
        uint8_t* dst = base + data_start + s.offset;
        uint64_t n = 1;
        for (auto d : s.dims) n *= d;
        const uint64_t seed = c->seed;
        switch (s.kind) {
            case 0: {
                if (s.ty == IT_Q8_0) {
                    parallel_rows(n / 32, threads, [&](uint64_t lo, uint64_t hi) {
                        float blk[32];
                        for (uint64_t b = lo; b < hi; b++) {
                            for (int i = 0; i < 32; i++) blk[i] = std_w * normal(seed, ti, b * 32 + i);
                            ith::quantize_block_q8_0(blk, dst + b * 34);
                        }
                    });
                } else if (s.ty == IT_F32) {
                    parallel_rows(n, threads, [&](uint64_t lo, uint64_t hi) {
                        for (uint64_t i = lo; i < hi; i++) {
                            float v = std_w * normal(seed, ti, i);
                            memcpy(dst + i * 4, &v, 4);
                        }
                    });
                } else {
                    munmap(base, total);
                    close(fd);
                    return bad("dense/router type must be Q8_0 or F32");
                }
                break;
            }
            case 1:
                for (uint64_t i = 0; i < n; i++) { float v = 1.0f; memcpy(dst + i * 4, &v, 4); }
                break;
            case 2:
                for (uint64_t i = 0; i < n; i++) { float v = -std::exp(normal(seed, ti, i)); memcpy(dst + i * 4, &v, 4); }
                break;
            case 3:
                for (uint64_t i = 0; i < n; i++) { float v = 0.5f * normal(seed, ti, i); memcpy(dst + i * 4, &v, 4); }
                break;
            case 4:
                parallel_rows(n / 64, threads, [&](uint64_t lo, uint64_t hi) {
                    for (uint64_t b = lo; b < hi; b++) {
                        uint8_t* blk = dst + b * 36;
                        uint64_t hsc = key_of(seed, ti, b * 5);
                        for (int k = 0; k < 4; k++) blk[k] = scale_lut[(hsc >> (12 * k)) & 4095];
                        for (int w = 0; w < 4; w++) {
                            uint64_t hv = key_of(seed, ti, b * 5 + 1 + w);
                            memcpy(blk + 4 + 8 * w, &hv, 8);
                        }
                    }
                });
                break;
            case 5:
                // E[(e2m1 * ue4m3)^2] ~ 8.56 * 1.0 for these draws -> std ~ 2.93
                for (uint64_t i = 0; i < n; i++) {
                    float v = (std_w / 2.93f) * (float)(0.75 + 0.5 * unit(key_of(seed, ti, i)));
                    memcpy(dst + i * 4, &v, 4);
                }
                break;
        }
    }
    msync(base, total, MS_ASYNC);
    munmap(base, total);
    close(fd);
    return 0;
}
