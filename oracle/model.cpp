// TEST INFRASTRUCTURE — the CPU oracle's model loop.  Not part of the shipped library.
//
// Restates, on top of oracle/ops.cpp:
//   src/gguf/mod.rs:143-296, src/gguf/metadata.rs:131-205   GGUF v3 container
//   src/model/mod.rs:261-418                                tensor views + shape checks
//   src/model/qwen35.rs:193-489                             Config::from_gguf
//   src/model/qwen35.rs:584-729                             Scratch sizes
//   src/model/qwen35.rs:755-873                             load, kv_slot, embed
//   src/model/qwen35.rs:956-1328                            forward / attention / gated_delta
//   src/model/qwen35.rs:1587-1700                           moe_batch
//   src/cache/mod.rs:33-65,215-252, src/cache/recurrent.rs  KV slabs, recurrent state
//   src/engine/mod.rs:310-437, src/profile.rs:192-213       chunked prefill, greedy generate
#include "oracle.h"
#include "orc_math.h"

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cmath>
#include <cstdio>
#include <cstring>
#include <map>
#include <string>
#include <vector>

namespace {

struct TensorInfo {
    std::vector<uint64_t> dims;
    uint32_t ty = 0;
    uint64_t offset = 0;
};

struct Gguf {
    int fd = -1;
    const uint8_t* base = nullptr;
    size_t size = 0;
    size_t data_start = 0;
    std::map<std::string, uint64_t> u;      // any integer-valued key
    std::map<std::string, double> f;        // f32/f64 keys
    std::map<std::string, std::string> s;   // string keys
    std::map<std::string, std::vector<int32_t>> i32_arrays;
    std::map<std::string, TensorInfo> tensors;
    std::string err;

    ~Gguf() {
        if (base) munmap((void*)base, size);
        if (fd >= 0) close(fd);
    }

    struct Cur {
        const uint8_t* p;
        const uint8_t* end;
        bool ok = true;
        template <class T>
        T get() {
            T v{};
            if (p + sizeof(T) > end) {
                ok = false;
                return v;
            }
            memcpy(&v, p, sizeof(T));
            p += sizeof(T);
            return v;
        }
        std::string str() {
            uint64_t n = get<uint64_t>();
            if (!ok || p + n > end) {
                ok = false;
                return {};
            }
            std::string r((const char*)p, n);
            p += n;
            return r;
        }
    };

    static size_t scalar_size(uint32_t t) {
        switch (t) {
            case 0: case 1: case 7: return 1;
            case 2: case 3: return 2;
            case 4: case 5: case 6: return 4;
            case 10: case 11: case 12: return 8;
            default: return 0;
        }
    }

    bool read_value(Cur& c, const std::string& key, uint32_t vt) {
        switch (vt) {
            case 0: u[key] = c.get<uint8_t>(); break;
            case 1: u[key] = (uint64_t)(int64_t)c.get<int8_t>(); break;
            case 2: u[key] = c.get<uint16_t>(); break;
            case 3: u[key] = (uint64_t)(int64_t)c.get<int16_t>(); break;
            case 4: u[key] = c.get<uint32_t>(); break;
            case 5: u[key] = (uint64_t)(int64_t)c.get<int32_t>(); break;
            case 6: f[key] = c.get<float>(); break;
            case 7: u[key] = c.get<uint8_t>(); break;
            case 8: s[key] = c.str(); break;
            case 10: u[key] = c.get<uint64_t>(); break;
            case 11: u[key] = (uint64_t)c.get<int64_t>(); break;
            case 12: f[key] = c.get<double>(); break;
            case 9: {
                uint32_t et = c.get<uint32_t>();
                uint64_t n = c.get<uint64_t>();
                if (et == 8) {
                    for (uint64_t i = 0; i < n && c.ok; i++) c.str();
                } else if (et == 5) {
                    std::vector<int32_t> v(n);
                    for (uint64_t i = 0; i < n; i++) v[i] = c.get<int32_t>();
                    i32_arrays[key] = v;
                } else {
                    size_t sz = scalar_size(et);
                    if (sz == 0) return false;
                    if (c.p + sz * n > c.end) return false;
                    c.p += sz * n;
                }
                break;
            }
            default: return false;
        }
        return c.ok;
    }

    bool open(const char* path) {
        fd = ::open(path, O_RDONLY);
        if (fd < 0) {
            err = std::string("cannot open ") + path;
            return false;
        }
        struct stat st;
        fstat(fd, &st);
        size = (size_t)st.st_size;
        void* m = mmap(nullptr, size, PROT_READ, MAP_PRIVATE, fd, 0);
        if (m == MAP_FAILED) {
            err = "mmap failed";
            return false;
        }
        base = (const uint8_t*)m;
        Cur c{base, base + size};
        if (size < 24 || memcmp(base, "GGUF", 4) != 0) {
            err = "bad magic";
            return false;
        }
        c.p += 4;
        uint32_t version = c.get<uint32_t>();
        if (version != 3 && version != 2) {
            err = "unsupported GGUF version";
            return false;
        }
        int64_t n_tensors = c.get<int64_t>();
        int64_t n_kv = c.get<int64_t>();
        for (int64_t i = 0; i < n_kv; i++) {
            std::string key = c.str();
            uint32_t vt = c.get<uint32_t>();
            if (!c.ok || !read_value(c, key, vt)) {
                err = "bad metadata at key " + key;
                return false;
            }
        }
        for (int64_t i = 0; i < n_tensors; i++) {
            std::string name = c.str();
            uint32_t nd = c.get<uint32_t>();
            if (!c.ok || nd > 4) {
                err = "bad tensor info";
                return false;
            }
            TensorInfo ti;
            for (uint32_t d = 0; d < nd; d++) ti.dims.push_back((uint64_t)c.get<int64_t>());
            ti.ty = c.get<uint32_t>();
            ti.offset = c.get<uint64_t>();
            if (tensors.count(name)) {
                err = "duplicate tensor " + name;
                return false;
            }
            tensors[name] = ti;
        }
        if (!c.ok) {
            err = "truncated header";
            return false;
        }
        uint64_t align = u.count("general.alignment") ? u["general.alignment"] : 32;
        size_t pos = (size_t)(c.p - base);
        data_start = (pos + align - 1) / align * align;
        if (data_start > size) {
            err = "data blob starts past the end of the file";
            return false;
        }
        for (auto& kv : tensors) {
            uint64_t n = 1;
            for (auto d : kv.second.dims)
                if (__builtin_mul_overflow(n, d, &n) || n > (1ull << 56)) {
                    err = "tensor element count overflows: " + kv.first;
                    return false;
                }
            uint64_t bytes = orc_type_bytes(kv.second.ty, n);
            if (bytes == 0 && n != 0) {
                err = "unsupported tensor type in " + kv.first;
                return false;
            }
            if (kv.second.offset > size - data_start || bytes > size - data_start - kv.second.offset) {
                err = "tensor past end of file: " + kv.first;
                return false;
            }
        }
        return true;
    }

    const uint8_t* bytes(const TensorInfo& t) const { return base + data_start + t.offset; }
    static uint64_t n_elems(const TensorInfo& t) {
        uint64_t n = 1;
        for (auto d : t.dims) n *= d;
        return n;
    }
};

// src/model/mod.rs:261-271.
bool shape_is(const std::vector<uint64_t>& got, std::initializer_list<uint64_t> want_l) {
    std::vector<uint64_t> want(want_l);
    auto trim = [](const std::vector<uint64_t>& d) {
        size_t n = d.size();
        while (n > 0 && d[n - 1] == 1) n--;
        return n;
    };
    size_t g = trim(got), w = trim(want);
    if (g != w) return false;
    for (size_t i = 0; i < g; i++)
        if (got[i] != want[i]) return false;
    return true;
}

struct Cfg {
    uint64_t n_layer, n_embd, n_ff, n_head, n_head_kv, head_dim, n_vocab;
    float rope_theta, rms_eps;
    uint64_t n_rot;
    uint64_t d_conv, d_inner, d_state, dt_rank, n_group, interval, nextn;
    uint64_t n_expert, n_used, expert_ff, shared_ff;
    uint64_t q_gate_dim() const { return head_dim * 2 * n_head; }
    uint64_t kv_dim() const { return n_head_kv * head_dim; }
    uint64_t head_k_dim() const { return d_state; }
    uint64_t head_v_dim() const { return d_inner / dt_rank; }
    uint64_t n_k_heads() const { return n_group; }
    uint64_t n_v_heads() const { return dt_rank; }
    uint64_t key_dim() const { return head_k_dim() * n_k_heads(); }
    uint64_t value_dim() const { return head_v_dim() * n_v_heads(); }
    uint64_t conv_dim() const { return key_dim() * 2 + value_dim(); }
    uint64_t ssm_state_len() const { return head_k_dim() * head_v_dim() * n_v_heads(); }
    uint64_t conv_state_len() const { return (d_conv - 1) * conv_dim(); }
    uint64_t n_main() const { return n_layer - nextn; }
    bool is_recurrent(uint64_t il) const { return il < n_main() && (il + 1) % interval != 0; }
};

struct Layer {
    std::vector<float> attn_norm, ffn_norm;
    bool recurrent = false;
    // attention
    orc_weights wq{}, wk{}, wv{}, wo{};
    std::vector<float> q_norm, k_norm;
    // delta
    orc_weights wqkv{}, wgate{}, ssm_beta{}, ssm_alpha{}, ssm_out{};
    std::vector<float> conv1d, ssm_a, dt_bias, ssm_norm;
    // moe
    orc_weights gate_inp{}, shared_gate{}, shared_up{}, shared_down{}, shared_gate_inp{};
    orc_experts gate{}, up{}, down{};
    bool has_gate_s = false, has_up_s = false, has_down_s = false;
    float gate_s = 1, up_s = 1, down_s = 1;
};

}  // namespace

struct orc_model {
    Gguf g;
    Cfg c{};
    orc_weights tok_embd{}, output{};
    bool has_output_s = false;
    float output_s = 1;
    std::vector<float> output_norm;
    std::vector<Layer> layers;
    std::vector<uint64_t> kv_slot;
    uint64_t n_kv_layer = 0;
    std::string err;

    bool need_u(const std::string& k, uint64_t* out) {
        std::string full = g.s["general.architecture"] + "." + k;
        auto it = g.u.find(full);
        if (it == g.u.end()) {
            err = "missing key " + full;
            return false;
        }
        *out = it->second;
        return true;
    }
    bool need_f(const std::string& k, float* out) {
        std::string full = g.s["general.architecture"] + "." + k;
        auto it = g.f.find(full);
        if (it == g.f.end()) {
            err = "missing key " + full;
            return false;
        }
        *out = (float)it->second;
        return true;
    }
    const TensorInfo* tensor(const std::string& name) {
        auto it = g.tensors.find(name);
        if (it == g.tensors.end()) {
            err = "missing tensor " + name;
            return nullptr;
        }
        return &it->second;
    }
    bool matrix(const std::string& name, uint64_t n_in, uint64_t n_out, orc_weights* w) {
        const TensorInfo* t = tensor(name);
        if (!t) return false;
        if (!shape_is(t->dims, {n_in, n_out})) {
            err = "shape mismatch " + name;
            return false;
        }
        *w = {g.bytes(*t), orc_type_bytes(t->ty, Gguf::n_elems(*t)), t->ty, 0, n_in, n_out};
        return true;
    }
    bool row_matrix(const std::string& name, uint64_t n_in, orc_weights* w) {
        const TensorInfo* t = tensor(name);
        if (!t) return false;
        if (!shape_is(t->dims, {n_in})) {
            err = "shape mismatch " + name;
            return false;
        }
        *w = {g.bytes(*t), orc_type_bytes(t->ty, n_in), t->ty, 0, n_in, 1};
        return true;
    }
    bool vector(const std::string& name, uint64_t len, std::vector<float>* out) {
        const TensorInfo* t = tensor(name);
        if (!t) return false;
        if (!shape_is(t->dims, {len})) {
            err = "shape mismatch " + name;
            return false;
        }
        out->resize(len);
        if (orc_dequantize(t->ty, g.bytes(*t), len, out->data()) != 0) {
            err = "unsupported type for " + name;
            return false;
        }
        return true;
    }
    bool conv_weights(const std::string& name, uint64_t kernel, uint64_t nc, std::vector<float>* out) {
        const TensorInfo* t = tensor(name);
        if (!t) return false;
        if (!shape_is(t->dims, {kernel, nc})) {
            err = "shape mismatch " + name;
            return false;
        }
        out->resize(kernel * nc);
        if (orc_dequantize(t->ty, g.bytes(*t), kernel * nc, out->data()) != 0) {
            err = "unsupported type for " + name;
            return false;
        }
        return true;
    }
    bool experts(const std::string& name, uint64_t n_in, uint64_t n_out, uint64_t n_expert, orc_experts* e) {
        const TensorInfo* t = tensor(name);
        if (!t) return false;
        if (!shape_is(t->dims, {n_in, n_out, n_expert})) {
            err = "shape mismatch " + name;
            return false;
        }
        *e = {g.bytes(*t), orc_type_bytes(t->ty, Gguf::n_elems(*t)), t->ty, 0, n_in, n_out, n_expert, nullptr, 0};
        std::string sn = name;
        size_t at = sn.find(".weight");
        if (at != std::string::npos) sn.replace(at, 7, ".scale");
        auto it = g.tensors.find(sn);
        if (it != g.tensors.end()) {
            if (!shape_is(it->second.dims, {n_expert}) || it->second.ty != ORC_F32) {
                err = "bad expert scale " + sn;
                return false;
            }
            e->scale = g.bytes(it->second);
            e->scale_len = n_expert * 4;
        }
        return true;
    }
    bool optional_scalar(const std::string& name, bool* has, float* v) {
        auto it = g.tensors.find(name);
        *has = false;
        if (it == g.tensors.end()) return true;
        std::vector<float> one;
        if (!vector(name, 1, &one)) return false;
        *has = true;
        *v = one[0];
        return true;
    }

    bool load(const char* path) {
        if (!g.open(path)) {
            err = g.err;
            return false;
        }
        std::string arch = g.s["general.architecture"];
        if (arch != "qwen35moe") {
            err = "unsupported architecture '" + arch + "' (oracle covers qwen35moe)";
            return false;
        }
        uint64_t v_len = 0;
        if (!need_u("block_count", &c.n_layer) || !need_u("embedding_length", &c.n_embd) ||
            !need_u("expert_count", &c.n_expert) || !need_u("expert_used_count", &c.n_used) ||
            !need_u("expert_feed_forward_length", &c.expert_ff) ||
            !need_u("expert_shared_feed_forward_length", &c.shared_ff) ||
            !need_u("attention.head_count", &c.n_head) || !need_u("attention.head_count_kv", &c.n_head_kv) ||
            !need_u("attention.key_length", &c.head_dim) || !need_u("attention.value_length", &v_len) ||
            !need_f("rope.freq_base", &c.rope_theta) || !need_f("attention.layer_norm_rms_epsilon", &c.rms_eps) ||
            !need_u("rope.dimension_count", &c.n_rot) || !need_u("ssm.conv_kernel", &c.d_conv) ||
            !need_u("ssm.inner_size", &c.d_inner) || !need_u("ssm.state_size", &c.d_state) ||
            !need_u("ssm.time_step_rank", &c.dt_rank) || !need_u("ssm.group_count", &c.n_group))
            return false;
        c.n_ff = c.expert_ff;
        if (!need_u("full_attention_interval", &c.interval)) {
            c.interval = 4;
            err.clear();
        }
        if (!need_u("nextn_predict_layers", &c.nextn)) {
            c.nextn = 0;
            err.clear();
        }
        auto sec = g.i32_arrays.find(arch + ".rope.dimension_sections");
        if (sec == g.i32_arrays.end() || sec->second.size() != 4) {
            err = "rope.dimension_sections must be an i32 array of 4";
            return false;
        }
        if (c.n_head_kv == 0 || c.n_head % c.n_head_kv != 0) { err = "GQA grouping"; return false; }
        if (v_len != c.head_dim) { err = "key_length != value_length"; return false; }
        if (c.n_used == 0 || c.n_used > c.n_expert) { err = "expert_used_count"; return false; }
        if (c.dt_rank == 0 || c.d_inner % c.dt_rank != 0) { err = "ssm.inner_size / ssm.time_step_rank"; return false; }
        if (c.n_group == 0 || c.dt_rank % c.n_group != 0) { err = "delta rule grouping"; return false; }
        if (c.head_v_dim() != c.head_k_dim()) { err = "delta rule head dimensions"; return false; }
        if (c.interval == 0) { err = "full_attention_interval"; return false; }
        if (c.n_rot > c.head_dim) { err = "rope.dimension_count"; return false; }

        const TensorInfo* te = tensor("token_embd.weight");
        if (!te || te->dims.size() < 2) { err = "token_embd.weight: expected 2 dimensions"; return false; }
        c.n_vocab = te->dims[1];
        if (!matrix("token_embd.weight", c.n_embd, c.n_vocab, &tok_embd)) return false;
        if (g.tensors.count("output.weight")) {
            if (!matrix("output.weight", c.n_embd, c.n_vocab, &output)) return false;
            if (!optional_scalar("output.scale", &has_output_s, &output_s)) return false;
        } else {
            output = tok_embd;
        }
        layers.resize(c.n_main());
        for (uint64_t i = 0; i < c.n_main(); i++) {
            Layer& L = layers[i];
            auto p = [&](const char* n) { return "blk." + std::to_string(i) + "." + n; };
            L.recurrent = c.is_recurrent(i);
            if (L.recurrent) {
                if (!matrix(p("attn_qkv.weight"), c.n_embd, c.conv_dim(), &L.wqkv) ||
                    !matrix(p("attn_gate.weight"), c.n_embd, c.value_dim(), &L.wgate) ||
                    !conv_weights(p("ssm_conv1d.weight"), c.d_conv, c.conv_dim(), &L.conv1d) ||
                    !matrix(p("ssm_beta.weight"), c.n_embd, c.n_v_heads(), &L.ssm_beta) ||
                    !matrix(p("ssm_alpha.weight"), c.n_embd, c.n_v_heads(), &L.ssm_alpha) ||
                    !vector(p("ssm_a"), c.n_v_heads(), &L.ssm_a) ||
                    !vector(p("ssm_dt.bias"), c.n_v_heads(), &L.dt_bias) ||
                    !vector(p("ssm_norm.weight"), c.head_v_dim(), &L.ssm_norm) ||
                    !matrix(p("ssm_out.weight"), c.value_dim(), c.n_embd, &L.ssm_out))
                    return false;
            } else {
                if (!matrix(p("attn_q.weight"), c.n_embd, c.q_gate_dim(), &L.wq) ||
                    !matrix(p("attn_k.weight"), c.n_embd, c.kv_dim(), &L.wk) ||
                    !matrix(p("attn_v.weight"), c.n_embd, c.kv_dim(), &L.wv) ||
                    !matrix(p("attn_output.weight"), c.head_dim * c.n_head, c.n_embd, &L.wo) ||
                    !vector(p("attn_q_norm.weight"), c.head_dim, &L.q_norm) ||
                    !vector(p("attn_k_norm.weight"), c.head_dim, &L.k_norm))
                    return false;
            }
            if (!matrix(p("ffn_gate_inp.weight"), c.n_embd, c.n_expert, &L.gate_inp) ||
                !experts(p("ffn_gate_exps.weight"), c.n_embd, c.expert_ff, c.n_expert, &L.gate) ||
                !experts(p("ffn_up_exps.weight"), c.n_embd, c.expert_ff, c.n_expert, &L.up) ||
                !experts(p("ffn_down_exps.weight"), c.expert_ff, c.n_embd, c.n_expert, &L.down) ||
                !matrix(p("ffn_gate_shexp.weight"), c.n_embd, c.shared_ff, &L.shared_gate) ||
                !matrix(p("ffn_up_shexp.weight"), c.n_embd, c.shared_ff, &L.shared_up) ||
                !matrix(p("ffn_down_shexp.weight"), c.shared_ff, c.n_embd, &L.shared_down) ||
                !row_matrix(p("ffn_gate_inp_shexp.weight"), c.n_embd, &L.shared_gate_inp) ||
                !optional_scalar(p("ffn_gate_shexp.scale"), &L.has_gate_s, &L.gate_s) ||
                !optional_scalar(p("ffn_up_shexp.scale"), &L.has_up_s, &L.up_s) ||
                !optional_scalar(p("ffn_down_shexp.scale"), &L.has_down_s, &L.down_s) ||
                !vector(p("attn_norm.weight"), c.n_embd, &L.attn_norm) ||
                !vector(p("post_attention_norm.weight"), c.n_embd, &L.ffn_norm))
                return false;
        }
        uint64_t next = 0;
        for (uint64_t il = 0; il < c.n_main(); il++) {
            kv_slot.push_back(next);
            if (!c.is_recurrent(il)) next++;
        }
        n_kv_layer = next;
        return vector("output_norm.weight", c.n_embd, &output_norm);
    }
};

struct orc_engine {
    orc_model* m;
    uint64_t n_ctx, max_batch;
    uint64_t len = 0;  // committed positions
    std::vector<uint16_t> k_slabs, v_slabs;  // [n_kv_layer][n_ctx*kv_dim]
    std::vector<float> conv, ssm;            // [n_main][conv_state_len], [n_main][ssm_state_len]
    orc_trace_fn trace = nullptr;
    void* trace_user = nullptr;
    // scratch (src/model/qwen35.rs:584-635)
    std::vector<float> x, normed, mixed, ffn_out, qg, q, g, k, v, attn, qkv, z, alpha, beta, convo, q_part,
        k_part, v_part, core, router, e_gate, e_up, e_out, e_in, g_all, u_all, o_all, shexp_logit, last,
        final_norm, logits, route_w;
    std::vector<uint32_t> route_ids;

    void tr(const char* name, uint64_t il, const std::vector<float>& t, uint64_t n) {
        if (trace) trace(trace_user, name, (uint32_t)il, t.data(), n);
    }
};

namespace {
const uint64_t MOE_CHUNK = 512;  // src/model/qwen35.rs:650

void fit(orc_engine* e, uint64_t n) {
    const Cfg& c = e->m->c;
    auto z = [&](std::vector<float>& b, uint64_t k) { if (b.size() < n * k) b.resize(n * k, 0.0f); };
    z(e->x, c.n_embd); z(e->normed, c.n_embd); z(e->mixed, c.n_embd); z(e->ffn_out, c.n_embd);
    z(e->qg, c.q_gate_dim()); z(e->q, c.head_dim * c.n_head); z(e->g, c.head_dim * c.n_head);
    z(e->k, c.kv_dim()); z(e->v, c.kv_dim()); z(e->attn, c.head_dim * c.n_head);
    z(e->qkv, c.conv_dim()); z(e->z, c.value_dim()); z(e->alpha, c.n_v_heads()); z(e->beta, c.n_v_heads());
    z(e->convo, c.conv_dim()); z(e->q_part, c.key_dim()); z(e->k_part, c.key_dim());
    z(e->v_part, c.value_dim()); z(e->core, c.value_dim());
    uint64_t nt = n < MOE_CHUNK ? n : MOE_CHUNK;
    auto zz = [&](std::vector<float>& b, uint64_t k) { if (b.size() < k) b.resize(k, 0.0f); };
    uint64_t ff = c.expert_ff > c.shared_ff ? c.expert_ff : c.shared_ff;
    zz(e->router, nt * c.n_expert); zz(e->e_gate, nt * ff); zz(e->e_up, nt * ff);
    zz(e->e_out, nt * c.n_embd); zz(e->e_in, nt * c.n_embd);
    zz(e->g_all, nt * c.n_used * c.expert_ff); zz(e->u_all, nt * c.n_used * c.expert_ff);
    zz(e->o_all, nt * c.n_used * c.n_embd); zz(e->shexp_logit, nt);
    zz(e->route_w, nt * c.n_used);
    if (e->route_ids.size() < nt * c.n_used) e->route_ids.resize(nt * c.n_used);
    zz(e->last, c.n_embd); zz(e->final_norm, c.n_embd); zz(e->logits, c.n_vocab);
}

// src/model/qwen35.rs:1587-1700.
void moe_batch(orc_engine* e, const Layer& L, uint64_t at, uint64_t n) {
    const Cfg& c = e->m->c;
    uint64_t nd = c.n_embd;
    orc_gather_chunks(e->normed.data(), n * nd, n * nd, at, e->e_in.data(), n * nd);
    const float* x = e->e_in.data();
    orc_matmul_pair(&L.gate_inp, &L.shared_gate_inp, x, n * nd, e->router.data(), e->shexp_logit.data());
    orc_softmax(e->router.data(), n * c.n_expert, c.n_expert);
    orc_route(e->router.data(), n, c.n_expert, c.n_used, e->route_ids.data(), e->route_w.data());
    uint64_t pairs = n * c.n_used;
    uint64_t ff = pairs * c.expert_ff;
    orc_moe_glu(&L.gate, &L.up, e->route_ids.data(), pairs, c.n_used, x, n * nd, e->g_all.data(), e->u_all.data());
    orc_matmul_experts(&L.down, e->route_ids.data(), pairs, c.n_used, e->g_all.data(), ff, e->o_all.data());
    uint64_t sff = n * c.shared_ff;
    orc_matmul(&L.shared_gate, x, n * nd, e->e_gate.data());
    orc_matmul(&L.shared_up, x, n * nd, e->e_up.data());
    if (L.has_up_s) orc_scale(e->e_up.data(), sff, L.up_s);
    if (L.has_gate_s) orc_scale(e->e_gate.data(), sff, L.gate_s);
    orc_silu_mul(e->e_gate.data(), e->e_up.data(), sff);
    orc_matmul(&L.shared_down, e->e_gate.data(), sff, e->e_out.data());
    if (L.has_down_s) orc_scale(e->e_out.data(), n * nd, L.down_s);
    orc_moe_finish(e->ffn_out.data(), at, nd, e->o_all.data(), e->route_w.data(), n, c.n_used, e->e_out.data(),
                   e->shexp_logit.data(), 0);
}

// src/model/qwen35.rs:1138-1223.
void attention(orc_engine* e, const Layer& L, uint64_t il, uint64_t start_pos, uint64_t n) {
    const Cfg& c = e->m->c;
    uint64_t hd = c.head_dim, kd = c.kv_dim(), nd = c.n_embd;
    orc_matmul(&L.wq, e->normed.data(), n * nd, e->qg.data());
    e->tr("Qcur_full", il, e->qg, n * c.q_gate_dim());
    orc_gather_chunks(e->qg.data(), hd, 2 * hd, 0, e->q.data(), n * hd * c.n_head);
    orc_gather_chunks(e->qg.data(), hd, 2 * hd, hd, e->g.data(), n * hd * c.n_head);
    orc_matmul(&L.wk, e->normed.data(), n * nd, e->k.data());
    orc_matmul(&L.wv, e->normed.data(), n * nd, e->v.data());
    orc_rms_norm_heads(e->q.data(), n * hd * c.n_head, L.q_norm.data(), hd, c.rms_eps);
    e->tr("Qcur_normed", il, e->q, n * hd * c.n_head);
    orc_rms_norm_heads(e->k.data(), n * kd, L.k_norm.data(), hd, c.rms_eps);
    e->tr("Kcur_normed", il, e->k, n * kd);
    orc_rope_neox(e->q.data(), n * hd * c.n_head, start_pos, hd, c.n_rot, c.n_head, c.rope_theta);
    e->tr("Qcur", il, e->q, n * hd * c.n_head);
    orc_rope_neox(e->k.data(), n * kd, start_pos, hd, c.n_rot, c.n_head_kv, c.rope_theta);
    e->tr("Kcur", il, e->k, n * kd);
    uint64_t slot = e->m->kv_slot[il];
    uint16_t* ks = e->k_slabs.data() + slot * e->n_ctx * kd;
    uint16_t* vs = e->v_slabs.data() + slot * e->n_ctx * kd;
    orc_kv_write(ks, start_pos * kd, e->k.data(), n * kd);
    orc_kv_write(vs, start_pos * kd, e->v.data(), n * kd);
    orc_attn a = {e->q.data(), n * hd * c.n_head, ks, vs, e->n_ctx * kd, kd, start_pos + n, hd, c.n_head,
                  c.n_head_kv, 1.0f / sqrtf((float)hd)};
    orc_attend(&a, e->attn.data());
    e->tr("attn_pregate", il, e->attn, n * hd * c.n_head);
    orc_sigmoid_mul(e->attn.data(), e->g.data(), n * hd * c.n_head);
    e->tr("attn_gated", il, e->attn, n * hd * c.n_head);
    orc_matmul(&L.wo, e->attn.data(), n * hd * c.n_head, e->mixed.data());
    e->tr("attn_output", il, e->mixed, n * nd);
}

// src/model/qwen35.rs:1232-1328.
void gated_delta(orc_engine* e, const Layer& L, uint64_t il, uint64_t n) {
    const Cfg& c = e->m->c;
    uint64_t kdim = c.key_dim(), vdim = c.value_dim(), cdim = c.conv_dim(), nd = c.n_embd;
    orc_matmul(&L.wqkv, e->normed.data(), n * nd, e->qkv.data());
    e->tr("linear_attn_qkv_mixed", il, e->qkv, n * cdim);
    orc_matmul(&L.wgate, e->normed.data(), n * nd, e->z.data());
    e->tr("z", il, e->z, n * vdim);
    orc_matmul_pair(&L.ssm_alpha, &L.ssm_beta, e->normed.data(), n * nd, e->alpha.data(), e->beta.data());
    orc_ssm_conv(e->conv.data() + il * c.conv_state_len(), e->qkv.data(), n * cdim, L.conv1d.data(),
                 L.conv1d.size(), c.d_conv, e->convo.data());
    e->tr("conv_output_silu", il, e->convo, n * cdim);
    orc_gather_chunks(e->convo.data(), kdim, cdim, 0, e->q_part.data(), n * kdim);
    orc_gather_chunks(e->convo.data(), kdim, cdim, kdim, e->k_part.data(), n * kdim);
    orc_gather_chunks(e->convo.data(), vdim, cdim, 2 * kdim, e->v_part.data(), n * vdim);
    orc_l2_norm_heads(e->q_part.data(), n * kdim, c.head_k_dim(), c.rms_eps);
    orc_l2_norm_heads(e->k_part.data(), n * kdim, c.head_k_dim(), c.rms_eps);
    e->tr("q_conv_predelta", il, e->q_part, n * kdim);
    e->tr("k_conv_predelta", il, e->k_part, n * kdim);
    orc_delta d = {e->q_part.data(), e->k_part.data(), e->v_part.data(), e->alpha.data(), e->beta.data(),
                   L.ssm_a.data(), L.dt_bias.data(), n, c.head_k_dim(), c.head_v_dim(), c.n_k_heads(),
                   c.n_v_heads()};
    orc_delta_rule(&d, e->ssm.data() + il * c.ssm_state_len(), e->core.data());
    e->tr("dnet_out", il, e->core, n * vdim);
    orc_rms_norm_heads(e->core.data(), n * vdim, L.ssm_norm.data(), c.head_v_dim(), c.rms_eps);
    orc_silu_mul(e->z.data(), e->core.data(), n * vdim);
    e->tr("final_output", il, e->z, n * vdim);
    orc_matmul(&L.ssm_out, e->z.data(), n * vdim, e->mixed.data());
    e->tr("linear_attn_out", il, e->mixed, n * nd);
}

// src/model/qwen35.rs:956-1127.
int forward(orc_engine* e, const uint32_t* tokens, uint64_t n, uint64_t start_pos, float* logits_out) {
    orc_model* m = e->m;
    const Cfg& c = m->c;
    if (n == 0) return -1;
    if (start_pos + n > e->n_ctx) return -2;  // ContextOverflow, before any write
    for (uint64_t t = 0; t < n; t++)
        if (tokens[t] >= c.n_vocab) return -3;  // TokenOutOfRange
    uint64_t nd = c.n_embd;
    fit(e, n);
    uint64_t emb_stride = orc_type_bytes(m->tok_embd.ty, nd);
    for (uint64_t t = 0; t < n; t++)
        orc_dequantize(m->tok_embd.ty, m->tok_embd.data + tokens[t] * emb_stride, nd, e->x.data() + t * nd);
    e->tr("inp_embd", 0, e->x, n * nd);
    for (uint64_t il = 0; il < c.n_main(); il++) {
        const Layer& L = m->layers[il];
        orc_rms_norm(e->x.data(), n * nd, L.attn_norm.data(), nd, c.rms_eps, e->normed.data());
        e->tr("attn_norm", il, e->normed, n * nd);
        if (L.recurrent) gated_delta(e, L, il, n);
        else attention(e, L, il, start_pos, n);
        orc_add_assign(e->x.data(), e->mixed.data(), n * nd);
        e->tr("attn_residual", il, e->x, n * nd);
        orc_rms_norm(e->x.data(), n * nd, L.ffn_norm.data(), nd, c.rms_eps, e->normed.data());
        for (uint64_t t = 0; t < n;) {
            uint64_t take = MOE_CHUNK < n - t ? MOE_CHUNK : n - t;
            moe_batch(e, L, t * nd, take);
            t += take;
        }
        e->tr("ffn_moe_out", il, e->ffn_out, n * nd);
        orc_add_assign(e->x.data(), e->ffn_out.data(), n * nd);
        e->tr("post_ffn", il, e->x, n * nd);
    }
    e->len = start_pos + n;
    orc_gather_chunks(e->x.data(), nd, nd, (n - 1) * nd, e->last.data(), nd);
    orc_rms_norm(e->last.data(), nd, m->output_norm.data(), nd, c.rms_eps, e->final_norm.data());
    e->tr("result_norm", 0, e->final_norm, nd);
    orc_matmul(&m->output, e->final_norm.data(), nd, e->logits.data());
    if (m->has_output_s) orc_scale(e->logits.data(), c.n_vocab, m->output_s);
    e->tr("result_output", 0, e->logits, c.n_vocab);
    if (logits_out) memcpy(logits_out, e->logits.data(), c.n_vocab * 4);
    return 0;
}
}  // namespace

extern "C" {

orc_model* orc_model_open(const char* path, char* err, size_t err_len) {
    orc_model* m = new orc_model();
    if (!m->load(path)) {
        if (err && err_len) snprintf(err, err_len, "%s", m->err.c_str());
        delete m;
        return nullptr;
    }
    return m;
}
void orc_model_close(orc_model* m) { delete m; }

void orc_model_dims(const orc_model* m, uint64_t out[10]) {
    const Cfg& c = m->c;
    uint64_t v[10] = {c.n_main(), c.n_embd, c.n_vocab, c.n_head, c.n_head_kv,
                      c.head_dim, c.n_expert, c.n_used, c.expert_ff, c.n_rot};
    memcpy(out, v, sizeof v);
}

// Bytes of weights one decode token reads: every dense matrix once, n_used routed
// experts per layer, router, shared expert, LM head (cf. src/model/qwen35.rs:875-939).
uint64_t orc_model_decode_weight_bytes(const orc_model* m) {
    uint64_t b = m->output.len;
    for (const Layer& L : m->layers) {
        if (L.recurrent) b += L.wqkv.len + L.wgate.len + L.ssm_beta.len + L.ssm_alpha.len + L.ssm_out.len;
        else b += L.wq.len + L.wk.len + L.wv.len + L.wo.len;
        b += L.gate_inp.len + L.shared_gate.len + L.shared_up.len + L.shared_down.len + L.shared_gate_inp.len;
        b += (L.gate.len + L.up.len + L.down.len) / m->c.n_expert * m->c.n_used;
    }
    return b;
}

orc_engine* orc_engine_new(orc_model* m, uint64_t n_ctx, uint64_t max_batch) {
    orc_engine* e = new orc_engine();
    e->m = m;
    e->n_ctx = n_ctx;
    e->max_batch = max_batch ? max_batch : 512;  // DEFAULT_MAX_BATCH, src/engine/mod.rs:87
    const Cfg& c = m->c;
    e->k_slabs.assign(m->n_kv_layer * n_ctx * c.kv_dim(), 0);
    e->v_slabs.assign(m->n_kv_layer * n_ctx * c.kv_dim(), 0);
    e->conv.assign(c.n_main() * c.conv_state_len(), 0.0f);
    e->ssm.assign(c.n_main() * c.ssm_state_len(), 0.0f);
    return e;
}
void orc_engine_free(orc_engine* e) { delete e; }
void orc_engine_reset(orc_engine* e) {
    e->len = 0;
    std::fill(e->conv.begin(), e->conv.end(), 0.0f);
    std::fill(e->ssm.begin(), e->ssm.end(), 0.0f);
}
void orc_engine_set_trace(orc_engine* e, orc_trace_fn fn, void* user) {
    e->trace = fn;
    e->trace_user = user;
}
uint64_t orc_engine_pos(const orc_engine* e) { return e->len; }

int orc_engine_forward(orc_engine* e, const uint32_t* tokens, uint64_t n, float* logits) {
    return forward(e, tokens, n, e->len, logits);
}

// src/engine/mod.rs:366-437.
int64_t orc_engine_generate(orc_engine* e, const uint32_t* prompt, uint64_t n_prompt, uint64_t max_new,
                            uint32_t* out_ids, float* last_logits) {
    for (uint64_t at = 0; at < n_prompt; at += e->max_batch) {
        uint64_t take = e->max_batch < n_prompt - at ? e->max_batch : n_prompt - at;
        int rc = forward(e, prompt + at, take, e->len, nullptr);
        if (rc != 0) return rc;
    }
    uint64_t produced = 0;
    for (uint64_t i = 0; i < max_new; i++) {
        uint64_t pos = e->len;
        uint32_t next = orc_argmax(e->logits.data(), e->m->c.n_vocab);
        out_ids[produced++] = next;
        if (produced == max_new) break;
        if (pos + 1 >= e->n_ctx) break;
        int rc = forward(e, &next, 1, e->len, nullptr);
        if (rc != 0) return rc;
    }
    if (last_logits) memcpy(last_logits, e->logits.data(), e->m->c.n_vocab * 4);
    return (int64_t)produced;
}

const float* orc_engine_ssm_state(orc_engine* e, uint64_t layer, uint64_t* len) {
    *len = e->m->c.ssm_state_len();
    return e->ssm.data() + layer * *len;
}
const float* orc_engine_conv_state(orc_engine* e, uint64_t layer, uint64_t* len) {
    *len = e->m->c.conv_state_len();
    return e->conv.data() + layer * *len;
}
const uint16_t* orc_engine_k_slab(orc_engine* e, uint64_t slot, uint64_t* len) {
    *len = e->n_ctx * e->m->c.kv_dim();
    return e->k_slabs.data() + slot * *len;
}
const uint16_t* orc_engine_v_slab(orc_engine* e, uint64_t slot, uint64_t* len) {
    *len = e->n_ctx * e->m->c.kv_dim();
    return e->v_slabs.data() + slot * *len;
}

}  // extern "C"
