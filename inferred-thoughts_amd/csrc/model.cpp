// Host side of the per-token model loop, driving the HIP backend through the same
// C ABI a binding of the reference's `trait Ops` would use.
//
// Mirrors (file:line under /root/reference):
//   Config::from_gguf            src/model/qwen35.rs:333-489
//   tensor views + shape checks  src/model/mod.rs:261-418
//   Qwen35::load, kv_slot, embed src/model/qwen35.rs:755-873
//   Scratch::fit                 src/model/qwen35.rs:673-729 (stable host addresses)
//   forward/attention/gated_delta src/model/qwen35.rs:956-1328
//   moe_batch                    src/model/qwen35.rs:1587-1700
//   KvCache / RecurrentState     src/cache/mod.rs:33-65,215-252, src/cache/recurrent.rs:31-142
//   Engine run/prefill/generate  src/engine/mod.rs:310-437
#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <memory>
#include <string>
#include <vector>

#include "../../include/inferred_hip.h"
#include "gguf.h"
#include "host_formats.h"

namespace {

struct Dims {
    uint64_t n_layer = 0, n_embd = 0, n_vocab = 0, n_head = 0, n_head_kv = 0, head_dim = 0, n_rot = 0;
    uint64_t n_expert = 0, n_used = 0, expert_ff = 0, shared_ff = 0;
    uint64_t d_conv = 0, d_inner = 0, d_state = 0, dt_rank = 0, n_group = 0, interval = 4, nextn = 0;
    float theta = 0, eps = 0;
    uint64_t layers() const { return n_layer - nextn; }
    bool recurrent(uint64_t il) const { return il < layers() && (il + 1) % interval != 0; }
    uint64_t q_gate() const { return head_dim * 2 * n_head; }
    uint64_t q_dim() const { return head_dim * n_head; }
    uint64_t kv_dim() const { return head_dim * n_head_kv; }
    uint64_t dk() const { return d_state; }
    uint64_t dv() const { return d_inner / dt_rank; }
    uint64_t key_dim() const { return dk() * n_group; }
    uint64_t value_dim() const { return dv() * dt_rank; }
    uint64_t conv_dim() const { return 2 * key_dim() + value_dim(); }
    uint64_t ssm_len() const { return dk() * dv() * dt_rank; }
    uint64_t conv_len() const { return (d_conv - 1) * conv_dim(); }
};

struct Block {
    bool recurrent = false;
    std::vector<float> attn_norm, ffn_norm;
    it_weights wq{}, wk{}, wv{}, wo{};
    std::vector<float> q_norm, k_norm;
    it_weights wqkv{}, wgate{}, w_alpha{}, w_beta{}, w_out{};
    std::vector<float> conv1d, ssm_a, dt_bias, ssm_norm;
    it_weights router{}, sh_gate{}, sh_up{}, sh_down{}, sh_gate_inp{};
    it_experts gate{}, up{}, down{};
    float sh_scale[3] = {1, 1, 1};
    bool sh_has[3] = {false, false, false};
};

}  // namespace

struct it_model {
    itg::File file;
    std::string path;
    Dims d;
    it_weights tok_embd{}, output{};
    bool has_output_scale = false;
    float output_scale = 1.0f;
    std::vector<float> output_norm;
    std::vector<Block> blocks;
    std::vector<uint64_t> kv_slot;
    uint64_t n_kv_layer = 0;
    std::string err;

    bool fail(const std::string& m) {
        if (err.empty()) err = m;
        return false;
    }
    const itg::Tensor* need(const std::string& name) {
        const itg::Tensor* t = file.tensor(name);
        if (!t) fail("missing tensor " + name);
        return t;
    }
    static bool shape_is(const std::vector<uint64_t>& got, std::vector<uint64_t> want) {
        auto g = got;
        while (!g.empty() && g.back() == 1) g.pop_back();
        while (!want.empty() && want.back() == 1) want.pop_back();
        return g == want;
    }
    bool shape_err(const std::string& name, const std::vector<uint64_t>& want, const std::vector<uint64_t>& got) {
        std::string m = "tensor " + name + ": expected {";
        for (auto v : want) m += std::to_string(v) + ",";
        m += "} got {";
        for (auto v : got) m += std::to_string(v) + ",";
        return fail(m + "}");
    }
    bool matrix(const std::string& name, uint64_t n_in, uint64_t n_out, it_weights* w) {
        const itg::Tensor* t = need(name);
        if (!t) return false;
        if (!shape_is(t->dims, {n_in, n_out})) return shape_err(name, {n_in, n_out}, t->dims);
        *w = it_weights{file.bytes(*t), itg::type_bytes(t->ty, t->n_elems()), t->ty, 0, n_in, n_out};
        return true;
    }
    bool row_matrix(const std::string& name, uint64_t n_in, it_weights* w) {
        const itg::Tensor* t = need(name);
        if (!t) return false;
        if (!shape_is(t->dims, {n_in})) return shape_err(name, {n_in}, t->dims);
        *w = it_weights{file.bytes(*t), itg::type_bytes(t->ty, n_in), t->ty, 0, n_in, 1};
        return true;
    }
    bool vec(const std::string& name, std::vector<uint64_t> shape, std::vector<float>* out) {
        const itg::Tensor* t = need(name);
        if (!t) return false;
        if (!shape_is(t->dims, shape)) return shape_err(name, shape, t->dims);
        out->resize(t->n_elems());
        if (!ith::dequantize(t->ty, file.bytes(*t), t->n_elems(), out->data()))
            return fail("tensor " + name + ": unsupported type for a vector");
        return true;
    }
    bool experts(const std::string& name, uint64_t n_in, uint64_t n_out, uint64_t n_expert, it_experts* e) {
        const itg::Tensor* t = need(name);
        if (!t) return false;
        if (!shape_is(t->dims, {n_in, n_out, n_expert})) return shape_err(name, {n_in, n_out, n_expert}, t->dims);
        *e = it_experts{file.bytes(*t), itg::type_bytes(t->ty, t->n_elems()), t->ty, 0, n_in, n_out, n_expert, nullptr, 0};
        std::string sn = name;
        size_t at = sn.rfind(".weight");
        if (at != std::string::npos) sn.replace(at, 7, ".scale");
        if (const itg::Tensor* s = file.tensor(sn)) {
            if (!shape_is(s->dims, {n_expert})) return shape_err(sn, {n_expert}, s->dims);
            if (s->ty != IT_F32) return fail("tensor " + sn + ": per-expert scales must be F32");
            e->scale = file.bytes(*s);
            e->scale_len = n_expert * 4;
        }
        return true;
    }
    bool scalar_opt(const std::string& name, bool* has, float* v) {
        *has = false;
        if (!file.tensor(name)) return true;
        std::vector<float> one;
        if (!vec(name, {1}, &one)) return false;
        *has = true;
        *v = one[0];
        return true;
    }

    bool load(const std::string& path_in) {
        path = path_in;
        if (!file.open(path, &err)) return false;
        std::string arch;
        if (!file.get_string("general.architecture", &arch)) return fail("missing general.architecture");
        if (arch != "qwen35moe") return fail("unsupported architecture '" + arch + "' (this backend's loop covers qwen35moe)");
        auto u = [&](const char* k, uint64_t* out) {
            if (file.get_uint(arch + "." + k, out)) return true;
            return fail(std::string("missing key ") + arch + "." + k);
        };
        auto f = [&](const char* k, float* out) {
            if (file.get_float(arch + "." + k, out)) return true;
            return fail(std::string("missing key ") + arch + "." + k);
        };
        uint64_t v_len = 0;
        if (!u("block_count", &d.n_layer) || !u("embedding_length", &d.n_embd) || !u("expert_count", &d.n_expert) ||
            !u("expert_used_count", &d.n_used) || !u("expert_feed_forward_length", &d.expert_ff) ||
            !u("expert_shared_feed_forward_length", &d.shared_ff) || !u("attention.head_count", &d.n_head) ||
            !u("attention.head_count_kv", &d.n_head_kv) || !u("attention.key_length", &d.head_dim) ||
            !u("attention.value_length", &v_len) || !f("rope.freq_base", &d.theta) ||
            !f("attention.layer_norm_rms_epsilon", &d.eps) || !u("rope.dimension_count", &d.n_rot) ||
            !u("ssm.conv_kernel", &d.d_conv) || !u("ssm.inner_size", &d.d_inner) || !u("ssm.state_size", &d.d_state) ||
            !u("ssm.time_step_rank", &d.dt_rank) || !u("ssm.group_count", &d.n_group))
            return false;
        file.get_uint(arch + ".full_attention_interval", &d.interval);
        file.get_uint(arch + ".nextn_predict_layers", &d.nextn);
        const std::vector<int32_t>* sec = file.get_i32_array(arch + ".rope.dimension_sections");
        if (!sec || sec->size() != 4) return fail("rope.dimension_sections: expected an i32 array of 4 entries");
        if (d.n_head_kv == 0 || d.n_head % d.n_head_kv) return fail("GQA grouping: query heads do not divide into kv heads");
        if (v_len != d.head_dim) return fail("head dimension: key_length != value_length");
        if (d.n_used == 0 || d.n_used > d.n_expert) return fail("expert_used_count out of range");
        if (d.dt_rank == 0 || d.d_inner % d.dt_rank) return fail("ssm.inner_size does not divide into value heads");
        if (d.n_group == 0 || d.dt_rank % d.n_group) return fail("delta rule grouping: value heads do not divide into key heads");
        if (d.dv() != d.dk()) return fail("delta rule head dimensions: the recurrence assumes a square state");
        if (d.interval == 0) return fail("full_attention_interval must be non-zero");
        if (d.n_rot > d.head_dim) return fail("rope.dimension_count exceeds head_dim");
        if (d.nextn >= d.n_layer) return fail("nextn_predict_layers exceeds block_count");

        const itg::Tensor* te = need("token_embd.weight");
        if (!te) return false;
        if (te->dims.size() < 2) return fail("token_embd.weight: expected 2 dimensions");
        d.n_vocab = te->dims[1];
        if (!matrix("token_embd.weight", d.n_embd, d.n_vocab, &tok_embd)) return false;
        if (file.tensor("output.weight")) {
            if (!matrix("output.weight", d.n_embd, d.n_vocab, &output)) return false;
            if (!scalar_opt("output.scale", &has_output_scale, &output_scale)) return false;
        } else {
            output = tok_embd;
        }
        blocks.resize(d.layers());
        uint64_t slot = 0;
        for (uint64_t i = 0; i < d.layers(); i++) {
            Block& b = blocks[i];
            auto nm = [&](const char* s) { return "blk." + std::to_string(i) + "." + s; };
            b.recurrent = d.recurrent(i);
            kv_slot.push_back(slot);
            bool ok;
            if (b.recurrent) {
                ok = matrix(nm("attn_qkv.weight"), d.n_embd, d.conv_dim(), &b.wqkv) &&
                     matrix(nm("attn_gate.weight"), d.n_embd, d.value_dim(), &b.wgate) &&
                     vec(nm("ssm_conv1d.weight"), {d.d_conv, d.conv_dim()}, &b.conv1d) &&
                     matrix(nm("ssm_beta.weight"), d.n_embd, d.dt_rank, &b.w_beta) &&
                     matrix(nm("ssm_alpha.weight"), d.n_embd, d.dt_rank, &b.w_alpha) &&
                     vec(nm("ssm_a"), {d.dt_rank}, &b.ssm_a) && vec(nm("ssm_dt.bias"), {d.dt_rank}, &b.dt_bias) &&
                     vec(nm("ssm_norm.weight"), {d.dv()}, &b.ssm_norm) &&
                     matrix(nm("ssm_out.weight"), d.value_dim(), d.n_embd, &b.w_out);
            } else {
                slot++;
                ok = matrix(nm("attn_q.weight"), d.n_embd, d.q_gate(), &b.wq) &&
                     matrix(nm("attn_k.weight"), d.n_embd, d.kv_dim(), &b.wk) &&
                     matrix(nm("attn_v.weight"), d.n_embd, d.kv_dim(), &b.wv) &&
                     matrix(nm("attn_output.weight"), d.q_dim(), d.n_embd, &b.wo) &&
                     vec(nm("attn_q_norm.weight"), {d.head_dim}, &b.q_norm) &&
                     vec(nm("attn_k_norm.weight"), {d.head_dim}, &b.k_norm);
            }
            ok = ok && matrix(nm("ffn_gate_inp.weight"), d.n_embd, d.n_expert, &b.router) &&
                 experts(nm("ffn_gate_exps.weight"), d.n_embd, d.expert_ff, d.n_expert, &b.gate) &&
                 experts(nm("ffn_up_exps.weight"), d.n_embd, d.expert_ff, d.n_expert, &b.up) &&
                 experts(nm("ffn_down_exps.weight"), d.expert_ff, d.n_embd, d.n_expert, &b.down) &&
                 matrix(nm("ffn_gate_shexp.weight"), d.n_embd, d.shared_ff, &b.sh_gate) &&
                 matrix(nm("ffn_up_shexp.weight"), d.n_embd, d.shared_ff, &b.sh_up) &&
                 matrix(nm("ffn_down_shexp.weight"), d.shared_ff, d.n_embd, &b.sh_down) &&
                 row_matrix(nm("ffn_gate_inp_shexp.weight"), d.n_embd, &b.sh_gate_inp) &&
                 scalar_opt(nm("ffn_gate_shexp.scale"), &b.sh_has[0], &b.sh_scale[0]) &&
                 scalar_opt(nm("ffn_up_shexp.scale"), &b.sh_has[1], &b.sh_scale[1]) &&
                 scalar_opt(nm("ffn_down_shexp.scale"), &b.sh_has[2], &b.sh_scale[2]) &&
                 vec(nm("attn_norm.weight"), {d.n_embd}, &b.attn_norm) &&
                 vec(nm("post_attention_norm.weight"), {d.n_embd}, &b.ffn_norm);
            if (!ok) return false;
            // refused at load, not per call (src/ops/mod.rs:29-55)
            char msg[256];
            if (it_hip_check_expert_types(b.gate.ty, b.up.ty, b.down.ty, msg, sizeof msg)) return fail(msg);
        }
        n_kv_layer = slot;
        return vec("output_norm.weight", {d.n_embd}, &output_norm);
    }
};

// A host buffer whose address never changes once it has reached its largest size
// (src/model/qwen35.rs:572-583, 653-673).
struct HostBuf {
    std::vector<float> v;
    // Growing moves the buffer: the backend's mirror and quantized copy are keyed on the OLD address and would
    // otherwise leak, or be inherited by whatever the allocator places there next.
    void fit(uint64_t n, it_hip* be) {
        if (v.size() >= n) return;
        if (!v.empty() && n > v.capacity()) it_hip_release(be, v.data());
        v.resize(n, 0.0f);
    }
    float* p() { return v.data(); }
};

struct it_engine {
    it_model* m;
    it_hip* be;
    uint64_t n_ctx, max_batch;
    uint64_t moe_chunk = 512;  // tokens per routed-FFN sub-batch
    uint64_t len = 0;
    uint64_t ring_next = 0;  // next slot of the backend's device token ring this engine files into
    std::vector<uint16_t> k_slabs, v_slabs;
    std::vector<float> conv, ssm;
    it_trace_fn trace = nullptr;
    void* trace_user = nullptr;
    std::string err;
    HostBuf x, normed, mixed, ffn_out, qg, q, g, k, v, attn, qkv, z, alpha, beta, convo, q_part, k_part, v_part,
        core, router, e_gate, e_up, e_out, e_in, g_all, u_all, o_all, shexp_logit, last, final_norm, logits;

    uint64_t kv_reserved = 0;  // bytes this engine asked the backend to keep free of the expert slab
    uint64_t slab_len() const { return n_ctx * m->d.kv_dim(); }
    uint16_t* k_slab(uint64_t slot) { return k_slabs.data() + slot * slab_len(); }
    uint16_t* v_slab(uint64_t slot) { return v_slabs.data() + slot * slab_len(); }
    float* conv_of(uint64_t il) { return conv.data() + il * m->d.conv_len(); }
    float* ssm_of(uint64_t il) { return ssm.data() + il * m->d.ssm_len(); }

    void tr(const char* name, uint64_t il, HostBuf& b, uint64_t n) {
        if (!trace) return;
        it_hip_host_needs(be, b.p(), n);
        trace(trace_user, name, (uint32_t)il, b.p(), n);
    }
};

namespace {
constexpr uint64_t PREFETCH_K = 10;  // src/model/qwen4exp.rs:45: how many of the next router's picks a hint guesses
constexpr uint64_t MOE_CHUNK = 512;  // src/model/qwen35.rs:650: the reference's routed-FFN sub-batch; a larger engine batch raises it (it_engine_new)

void fit(it_engine* e, uint64_t n) {
    const Dims& d = e->m->d;
    e->x.fit(n * d.n_embd, e->be); e->normed.fit(n * d.n_embd, e->be); e->mixed.fit(n * d.n_embd, e->be); e->ffn_out.fit(n * d.n_embd, e->be);
    e->qg.fit(n * d.q_gate(), e->be); e->q.fit(n * d.q_dim(), e->be); e->g.fit(n * d.q_dim(), e->be);
    e->k.fit(n * d.kv_dim(), e->be); e->v.fit(n * d.kv_dim(), e->be); e->attn.fit(n * d.q_dim(), e->be);
    e->qkv.fit(n * d.conv_dim(), e->be); e->z.fit(n * d.value_dim(), e->be); e->alpha.fit(n * d.dt_rank, e->be); e->beta.fit(n * d.dt_rank, e->be);
    e->convo.fit(n * d.conv_dim(), e->be); e->q_part.fit(n * d.key_dim(), e->be); e->k_part.fit(n * d.key_dim(), e->be);
    e->v_part.fit(n * d.value_dim(), e->be); e->core.fit(n * d.value_dim(), e->be);
    uint64_t nt = n < e->moe_chunk ? n : e->moe_chunk;
    uint64_t ff = d.expert_ff > d.shared_ff ? d.expert_ff : d.shared_ff;
    e->router.fit(nt * d.n_expert, e->be); e->e_gate.fit(nt * ff, e->be); e->e_up.fit(nt * ff, e->be); e->e_out.fit(nt * d.n_embd, e->be);
    e->e_in.fit(nt * d.n_embd, e->be); e->g_all.fit(nt * d.n_used * d.expert_ff, e->be); e->u_all.fit(nt * d.n_used * d.expert_ff, e->be);
    e->o_all.fit(nt * d.n_used * d.n_embd, e->be); e->shexp_logit.fit(nt, e->be);
    e->last.fit(d.n_embd, e->be); e->final_norm.fit(d.n_embd, e->be); e->logits.fit(d.n_vocab, e->be);
}

// next_router: the router of the next layer, for a single-token pass.  The reference's qwen35 loop does not hint; its
// qwen4exp loop does (src/model/qwen4exp.rs:1885-1896), between the routing decision and the expert products, and the
// hint changes no value.  The backend acts on it only while part of the expert pool is cold.
void moe_batch(it_engine* e, const Block& b, uint64_t at, uint64_t n, uint64_t total, const it_weights* next_router) {
    const Dims& d = e->m->d;
    it_hip* be = e->be;
    uint64_t nd = d.n_embd;
    it_hip_gather_chunks(be, e->normed.p(), total * nd, n * nd, n * nd, at, e->e_in.p(), n * nd);
    const float* x = e->e_in.p();
    it_hip_matmul_pair(be, &b.router, &b.sh_gate_inp, x, n * nd, e->router.p(), n * d.n_expert, e->shexp_logit.p(), n);
    it_hip_softmax(be, e->router.p(), n * d.n_expert, d.n_expert);
    it_route route;
    it_hip_route(be, e->router.p(), n * d.n_expert, d.n_expert, d.n_used, &route);
    if (total == 1 && next_router) it_hip_prefetch_hint(be, next_router, x, nd, PREFETCH_K);
    uint64_t pairs = n * d.n_used, ff = pairs * d.expert_ff;
    it_hip_moe_glu(be, &b.gate, &b.up, &route, x, n * nd, e->g_all.p(), ff, e->u_all.p(), ff);
    it_hip_matmul_experts(be, &b.down, &route, e->g_all.p(), ff, e->o_all.p(), pairs * nd);
    uint64_t sff = n * d.shared_ff;
    it_hip_matmul(be, &b.sh_gate, x, n * nd, e->e_gate.p(), sff);
    it_hip_matmul(be, &b.sh_up, x, n * nd, e->e_up.p(), sff);
    if (b.sh_has[1]) it_hip_scale(be, e->e_up.p(), sff, b.sh_scale[1]);
    if (b.sh_has[0]) it_hip_scale(be, e->e_gate.p(), sff, b.sh_scale[0]);
    it_hip_silu_mul(be, e->e_gate.p(), sff, e->e_up.p(), sff);
    it_hip_matmul(be, &b.sh_down, e->e_gate.p(), sff, e->e_out.p(), n * nd);
    if (b.sh_has[2]) it_hip_scale(be, e->e_out.p(), n * nd, b.sh_scale[2]);
    it_hip_moe_finish(be, e->ffn_out.p(), total * nd, at, nd, e->o_all.p(), pairs * nd, &route, e->e_out.p(),
                      n * nd, e->shexp_logit.p(), n, 0);
}

void attention(it_engine* e, const Block& b, uint64_t il, uint64_t start, uint64_t n) {
    const Dims& d = e->m->d;
    it_hip* be = e->be;
    uint64_t hd = d.head_dim, kd = d.kv_dim(), nd = d.n_embd, qd = d.q_dim();
    it_hip_matmul(be, &b.wq, e->normed.p(), n * nd, e->qg.p(), n * d.q_gate());
    e->tr("Qcur_full", il, e->qg, n * d.q_gate());
    it_hip_gather_chunks(be, e->qg.p(), n * d.q_gate(), hd, 2 * hd, 0, e->q.p(), n * qd);
    it_hip_gather_chunks(be, e->qg.p(), n * d.q_gate(), hd, 2 * hd, hd, e->g.p(), n * qd);
    it_hip_matmul(be, &b.wk, e->normed.p(), n * nd, e->k.p(), n * kd);
    it_hip_matmul(be, &b.wv, e->normed.p(), n * nd, e->v.p(), n * kd);
    it_hip_rms_norm_heads(be, e->q.p(), n * qd, b.q_norm.data(), hd, hd, d.eps);
    e->tr("Qcur_normed", il, e->q, n * qd);
    it_hip_rms_norm_heads(be, e->k.p(), n * kd, b.k_norm.data(), hd, hd, d.eps);
    e->tr("Kcur_normed", il, e->k, n * kd);
    it_hip_rope_neox(be, e->q.p(), n * qd, start, hd, d.n_rot, d.n_head, d.theta);
    e->tr("Qcur", il, e->q, n * qd);
    it_hip_rope_neox(be, e->k.p(), n * kd, start, hd, d.n_rot, d.n_head_kv, d.theta);
    e->tr("Kcur", il, e->k, n * kd);
    uint64_t slot = e->m->kv_slot[il];
    it_hip_kv_write(be, e->k_slab(slot), e->slab_len(), start * kd, e->k.p(), n * kd);
    it_hip_kv_write(be, e->v_slab(slot), e->slab_len(), start * kd, e->v.p(), n * kd);
    it_attn a{e->q.p(), n * qd, e->k_slab(slot), e->v_slab(slot), e->slab_len(), kd, start + n, hd, d.n_head,
              d.n_head_kv, 1.0f / std::sqrt((float)hd)};
    it_hip_attend(be, &a, e->attn.p(), n * qd);
    e->tr("attn_pregate", il, e->attn, n * qd);
    it_hip_sigmoid_mul(be, e->attn.p(), n * qd, e->g.p(), n * qd);
    e->tr("attn_gated", il, e->attn, n * qd);
    it_hip_matmul(be, &b.wo, e->attn.p(), n * qd, e->mixed.p(), n * nd);
    e->tr("attn_output", il, e->mixed, n * nd);
}

void gated_delta(it_engine* e, const Block& b, uint64_t il, uint64_t n) {
    const Dims& d = e->m->d;
    it_hip* be = e->be;
    uint64_t kdim = d.key_dim(), vdim = d.value_dim(), cdim = d.conv_dim(), nd = d.n_embd, nv = d.dt_rank;
    it_hip_matmul(be, &b.wqkv, e->normed.p(), n * nd, e->qkv.p(), n * cdim);
    e->tr("linear_attn_qkv_mixed", il, e->qkv, n * cdim);
    it_hip_matmul(be, &b.wgate, e->normed.p(), n * nd, e->z.p(), n * vdim);
    e->tr("z", il, e->z, n * vdim);
    it_hip_matmul_pair(be, &b.w_alpha, &b.w_beta, e->normed.p(), n * nd, e->alpha.p(), n * nv, e->beta.p(), n * nv);
    it_hip_ssm_conv(be, e->conv_of(il), d.conv_len(), e->qkv.p(), n * cdim, b.conv1d.data(), b.conv1d.size(), d.d_conv,
                    e->convo.p(), n * cdim);
    e->tr("conv_output_silu", il, e->convo, n * cdim);
    it_hip_gather_chunks(be, e->convo.p(), n * cdim, kdim, cdim, 0, e->q_part.p(), n * kdim);
    it_hip_gather_chunks(be, e->convo.p(), n * cdim, kdim, cdim, kdim, e->k_part.p(), n * kdim);
    it_hip_gather_chunks(be, e->convo.p(), n * cdim, vdim, cdim, 2 * kdim, e->v_part.p(), n * vdim);
    it_hip_l2_norm_heads(be, e->q_part.p(), n * kdim, d.dk(), d.eps);
    it_hip_l2_norm_heads(be, e->k_part.p(), n * kdim, d.dk(), d.eps);
    e->tr("q_conv_predelta", il, e->q_part, n * kdim);
    e->tr("k_conv_predelta", il, e->k_part, n * kdim);
    it_delta dl{e->q_part.p(), e->k_part.p(), e->v_part.p(), e->alpha.p(), e->beta.p(), b.ssm_a.data(),
                b.dt_bias.data(), n, d.dk(), d.dv(), d.n_group, nv};
    it_hip_delta_rule(be, &dl, e->ssm_of(il), d.ssm_len(), e->core.p(), n * vdim);
    e->tr("dnet_out", il, e->core, n * vdim);
    it_hip_rms_norm_heads(be, e->core.p(), n * vdim, b.ssm_norm.data(), d.dv(), d.dv(), d.eps);
    it_hip_silu_mul(be, e->z.p(), n * vdim, e->core.p(), n * vdim);
    e->tr("final_output", il, e->z, n * vdim);
    it_hip_matmul(be, &b.w_out, e->z.p(), n * vdim, e->mixed.p(), n * nd);
    e->tr("linear_attn_out", il, e->mixed, n * nd);
}

// Runs one pass; logits stay on the device unless `want_logits`.
// `tokens == nullptr` is the greedy feedback pass: one token, chosen on the device as the arg-max
// of the previous pass's logits and embedded there (its id lands at `ring_index` of the device ring).
int forward(it_engine* e, const uint32_t* tokens, uint64_t n, uint64_t start, bool want_logits,
            uint64_t ring_index = 0) {
    it_model* m = e->m;
    const Dims& d = m->d;
    it_hip* be = e->be;
    if (n == 0) { e->err = "forward: no tokens supplied"; return -1; }
    if (start + n > e->n_ctx) { e->err = "context overflow: position " + std::to_string(start + n - 1) + " with n_ctx " + std::to_string(e->n_ctx); return -2; }
    for (uint64_t t = 0; tokens && t < n; t++)
        if (tokens[t] >= d.n_vocab) { e->err = "token id " + std::to_string(tokens[t]) + " outside the vocabulary"; return -3; }
    uint64_t nd = d.n_embd;
    it_hip_begin_pass(be, n);
    fit(e, n);
    if (tokens) {
        uint64_t row_bytes = itg::type_bytes(m->tok_embd.ty, nd);
        for (uint64_t t = 0; t < n; t++)
            ith::dequantize(m->tok_embd.ty, m->tok_embd.data + tokens[t] * row_bytes, nd, e->x.p() + t * nd);
        it_hip_host_wrote(be, e->x.p(), n * nd);
    } else {
        if (!it_hip_embed_argmax(be, &m->tok_embd, e->logits.p(), d.n_vocab, e->x.p(), nd, ring_index)) {
            it_hip_end_pass(be);
            e->err = "the embedding table's type has no device form";
            return -4;
        }
    }
    e->tr("inp_embd", 0, e->x, n * nd);
    for (uint64_t il = 0; il < d.layers(); il++) {
        const Block& b = m->blocks[il];
        it_hip_rms_norm(be, e->x.p(), n * nd, b.attn_norm.data(), nd, d.eps, e->normed.p(), n * nd);
        e->tr("attn_norm", il, e->normed, n * nd);
        if (b.recurrent) gated_delta(e, b, il, n);
        else attention(e, b, il, start, n);
        it_hip_add_assign(be, e->x.p(), n * nd, e->mixed.p(), n * nd);
        e->tr("attn_residual", il, e->x, n * nd);
        it_hip_rms_norm(be, e->x.p(), n * nd, b.ffn_norm.data(), nd, d.eps, e->normed.p(), n * nd);
        for (uint64_t t = 0; t < n;) {
            uint64_t take = e->moe_chunk < n - t ? e->moe_chunk : n - t;
            moe_batch(e, b, t * nd, take, n, il + 1 < d.layers() ? &m->blocks[il + 1].router : nullptr);
            t += take;
        }
        e->tr("ffn_moe_out", il, e->ffn_out, n * nd);
        it_hip_add_assign(be, e->x.p(), n * nd, e->ffn_out.p(), n * nd);
        e->tr("post_ffn", il, e->x, n * nd);
    }
    e->len = start + n;
    it_hip_gather_chunks(be, e->x.p(), n * nd, nd, nd, (n - 1) * nd, e->last.p(), nd);
    it_hip_rms_norm(be, e->last.p(), nd, m->output_norm.data(), nd, d.eps, e->final_norm.p(), nd);
    e->tr("result_norm", 0, e->final_norm, nd);
    it_hip_matmul(be, &m->output, e->final_norm.p(), nd, e->logits.p(), d.n_vocab);
    if (m->has_output_scale) it_hip_scale(be, e->logits.p(), d.n_vocab, m->output_scale);
    it_hip_end_pass(be);
    if (want_logits) it_hip_host_needs(be, e->logits.p(), d.n_vocab);
    if (e->trace) e->tr("result_output", 0, e->logits, d.n_vocab);
    // a device-fed pass does not wait for the device: only an error already recorded is looked at,
    // and the caller polls once, with a wait, after its last pass
    if (!tokens && !it_hip_has_error(be)) return 0;
    char msg[512];
    if (it_hip_take_error(be, msg, sizeof msg)) {
        e->err = msg;
        return -10;
    }
    return 0;
}

uint32_t host_argmax(const float* l, uint64_t n) {  // src/profile.rs:192-213
    uint64_t best = 0;
    for (uint64_t i = 1; i < n; i++)
        if (l[i] > l[best]) best = i;
    return (uint32_t)best;
}
}  // namespace

extern "C" {

it_model* it_model_open(const char* path, char* err, size_t err_len) {
    auto m = std::make_unique<it_model>();
    if (!m->load(path)) {
        if (err && err_len) snprintf(err, err_len, "%s", m->err.c_str());
        return nullptr;
    }
    return m.release();
}
void it_model_close(it_model* m) { delete m; }

void it_model_dims(const it_model* m, uint64_t out[10]) {
    const Dims& d = m->d;
    uint64_t v[10] = {d.layers(), d.n_embd, d.n_vocab, d.n_head, d.n_head_kv, d.head_dim, d.n_expert, d.n_used,
                      d.expert_ff, d.n_rot};
    memcpy(out, v, sizeof v);
}

uint64_t it_model_decode_weight_bytes(const it_model* m) {
    uint64_t bytes = m->output.len;
    for (const Block& b : m->blocks) {
        if (b.recurrent) bytes += b.wqkv.len + b.wgate.len + b.w_alpha.len + b.w_beta.len + b.w_out.len;
        else bytes += b.wq.len + b.wk.len + b.wv.len + b.wo.len;
        bytes += b.router.len + b.sh_gate.len + b.sh_up.len + b.sh_down.len + b.sh_gate_inp.len;
        bytes += (b.gate.len + b.up.len + b.down.len) / m->d.n_expert * m->d.n_used;
    }
    return bytes;
}

void it_model_token_macs(const it_model* m, uint64_t out[3]) {
    uint64_t dense = 0, glu = 0, down = 0;
    auto macs = [](const it_weights& w) { return w.n_in * w.n_out; };
    for (const Block& b : m->blocks) {
        if (b.recurrent) dense += macs(b.wqkv) + macs(b.wgate) + macs(b.w_alpha) + macs(b.w_beta) + macs(b.w_out);
        else dense += macs(b.wq) + macs(b.wk) + macs(b.wv) + macs(b.wo);
        dense += macs(b.router) + macs(b.sh_gate) + macs(b.sh_up) + macs(b.sh_down) + macs(b.sh_gate_inp);
        glu += m->d.n_used * (b.gate.n_in * b.gate.n_out + b.up.n_in * b.up.n_out);
        down += m->d.n_used * b.down.n_in * b.down.n_out;
    }
    out[0] = dense;
    out[1] = glu;
    out[2] = down;
}

it_engine* it_engine_new(it_model* m, it_hip* be, uint64_t n_ctx, uint64_t max_batch) {
    if (!m || !be || n_ctx == 0) return nullptr;
    it_engine* e = new it_engine();
    e->m = m;
    e->be = be;
    e->n_ctx = n_ctx;
    e->max_batch = max_batch ? max_batch : 512;  // DEFAULT_MAX_BATCH, src/engine/mod.rs:87
    const Dims& d = m->d;
    // every expert's matrices are read once per routed-FFN sub-batch, so with memory to spare the sub-batch
    // follows the engine batch (the seam carries at most 65535 pairs per call)
    e->moe_chunk = std::max<uint64_t>(MOE_CHUNK, std::min<uint64_t>(e->max_batch, 65535 / std::max<uint64_t>(1, d.n_used)));
    e->k_slabs.assign(m->n_kv_layer * n_ctx * d.kv_dim(), 0);
    e->v_slabs.assign(m->n_kv_layer * n_ctx * d.kv_dim(), 0);
    e->conv.assign(d.layers() * d.conv_len(), 0.0f);
    e->ssm.assign(d.layers() * d.ssm_len(), 0.0f);
    // what the reference's CLI tells its device backend before the first pass (src/main.rs:545-560): the permanent
    // weights and the KV cache the expert slab must leave room for, and the size of the expert pool (one read
    // counter per expert matrix)
    uint64_t dense = m->output.len + m->tok_embd.len;
    for (const Block& b : m->blocks) {
        if (b.recurrent) dense += b.wqkv.len + b.wgate.len + b.w_alpha.len + b.w_beta.len + b.w_out.len;
        else dense += b.wq.len + b.wk.len + b.wv.len + b.wo.len;
        dense += b.router.len + b.sh_gate.len + b.sh_up.len + b.sh_down.len + b.sh_gate_inp.len;
    }
    // where the experts' bytes can be read from when they are not kept anywhere else (src/main.rs:559-560)
    it_hip_set_model_path(be, m->path.c_str());
    it_hip_set_map_base(be, (uint64_t)(uintptr_t)m->file.base());
    it_hip_reserve_for_weights(be, dense);
    it_hip_set_expert_pool(be, d.layers() * 3 * d.n_expert);
    e->kv_reserved = 2 * m->n_kv_layer * n_ctx * d.kv_dim() * sizeof(uint16_t) +
                     (d.layers() * (d.conv_len() + d.ssm_len())) * sizeof(float);
    it_hip_reserve_for_kv(be, e->kv_reserved);
    return e;
}
void it_engine_free(it_engine* e) {
    if (!e) return;
    // the host buffers are about to be freed: drop the device copies keyed on them
    HostBuf* bufs[] = {&e->x, &e->normed, &e->mixed, &e->ffn_out, &e->qg, &e->q, &e->g, &e->k, &e->v, &e->attn,
                       &e->qkv, &e->z, &e->alpha, &e->beta, &e->convo, &e->q_part, &e->k_part, &e->v_part, &e->core,
                       &e->router, &e->e_gate, &e->e_up, &e->e_out, &e->e_in, &e->g_all, &e->u_all, &e->o_all,
                       &e->shexp_logit, &e->last, &e->final_norm, &e->logits};
    for (HostBuf* b : bufs)
        if (!b->v.empty()) it_hip_release(e->be, b->p());
    for (uint64_t s = 0; s < e->m->n_kv_layer; s++) {
        it_hip_release(e->be, e->k_slab(s));
        it_hip_release(e->be, e->v_slab(s));
    }
    for (uint64_t il = 0; il < e->m->d.layers(); il++) {
        it_hip_release(e->be, e->conv_of(il));
        it_hip_release(e->be, e->ssm_of(il));
    }
    // the reserve is additive (placement.rs:341-343): give this engine's share back (unsigned wrap-around subtracts)
    it_hip_reserve_for_kv(e->be, (uint64_t)0 - e->kv_reserved);
    delete e;
}

// Engine::reset, src/engine/mod.rs:296-306
void it_engine_reset(it_engine* e) {
    e->len = 0;
    std::fill(e->conv.begin(), e->conv.end(), 0.0f);
    std::fill(e->ssm.begin(), e->ssm.end(), 0.0f);
    it_hip_zero_state(e->be);
}
// Engine::checkpoint / restore / rewind, src/engine/mod.rs:223-294.  The device owns the recurrent state once it has
// touched it: a checkpoint brings every layer's slabs home through read_state first, a restore writes the host slabs
// and tells the backend to forget its copies.  The KV needs no stored copy: positions past `pos` are no longer part of
// the sequence and the next pass overwrites them.
void it_engine_state_sizes(const it_engine* e, uint64_t out[2]) {
    out[0] = e->conv.size();
    out[1] = e->ssm.size();
}
uint64_t it_engine_checkpoint(it_engine* e, float* conv_out, float* ssm_out) {
    const Dims& d = e->m->d;
    for (uint64_t il = 0; il < d.layers(); il++) {
        if (!d.recurrent(il)) continue;
        it_hip_read_state(e->be, e->conv_of(il), d.conv_len());
        it_hip_read_state(e->be, e->ssm_of(il), d.ssm_len());
    }
    if (conv_out) memcpy(conv_out, e->conv.data(), e->conv.size() * sizeof(float));
    if (ssm_out) memcpy(ssm_out, e->ssm.data(), e->ssm.size() * sizeof(float));
    return e->len;
}
int it_engine_restore(it_engine* e, uint64_t pos, const float* conv_in, const float* ssm_in) {
    if (pos > e->n_ctx) {
        e->err = "checkpoint stands at " + std::to_string(pos) + " positions, context is " + std::to_string(e->n_ctx);
        return -1;
    }
    if (!conv_in || !ssm_in) {
        e->err = "restore: null state";
        return -2;
    }
    e->len = pos;
    memcpy(e->conv.data(), conv_in, e->conv.size() * sizeof(float));
    memcpy(e->ssm.data(), ssm_in, e->ssm.size() * sizeof(float));
    it_hip_forget_state(e->be);  // after both halves
    return 0;
}
int it_engine_rewind(it_engine* e, uint64_t len) {
    const Dims& d = e->m->d;
    for (uint64_t il = 0; il < d.layers(); il++)
        if (d.recurrent(il)) return 0;  // a recurrent state is not a log: it cannot drop tokens
    if (len > e->len) return 0;
    e->len = len;
    return 1;
}
void it_engine_set_trace(it_engine* e, it_trace_fn fn, void* user) {
    e->trace = fn;
    e->trace_user = user;
}
uint64_t it_engine_pos(const it_engine* e) { return e->len; }
const char* it_engine_last_error(it_engine* e) { return e->err.c_str(); }

int it_engine_forward(it_engine* e, const uint32_t* tokens, uint64_t n, float* logits) {
    int rc = forward(e, tokens, n, e->len, logits != nullptr);
    if (rc == 0 && logits) memcpy(logits, e->logits.p(), e->m->d.n_vocab * 4);
    return rc;
}

int it_engine_prefill(it_engine* e, const uint32_t* tokens, uint64_t n, float* logits) {
    for (uint64_t at = 0; at < n; at += e->max_batch) {
        uint64_t take = e->max_batch < n - at ? e->max_batch : n - at;
        bool last = at + take >= n;
        int rc = forward(e, tokens + at, take, e->len, last && logits != nullptr);
        if (rc) return rc;
    }
    if (logits) memcpy(logits, e->logits.p(), e->m->d.n_vocab * 4);
    return 0;
}

int64_t it_engine_generate(it_engine* e, const uint32_t* prompt, uint64_t n_prompt, uint64_t max_new,
                           uint32_t* out_ids, float* last_logits) {
    uint64_t nv = e->m->d.n_vocab;
    for (uint64_t at = 0; at < n_prompt; at += e->max_batch) {
        uint64_t take = e->max_batch < n_prompt - at ? e->max_batch : n_prompt - at;
        int rc = forward(e, prompt + at, take, e->len, at + take >= n_prompt);
        if (rc) return rc;
    }
    uint64_t produced = 0;
    for (uint64_t i = 0; i < max_new; i++) {
        uint64_t pos = e->len;
        uint32_t next = host_argmax(e->logits.p(), nv);
        out_ids[produced++] = next;
        if (produced == max_new) break;
        if (pos + 1 >= e->n_ctx) break;
        int rc = forward(e, &next, 1, e->len, true);
        if (rc) return rc;
    }
    if (last_logits) memcpy(last_logits, e->logits.p(), nv * 4);
    return (int64_t)produced;
}

// Greedy decoding with the token fed back on the device: passes are issued back to back and the
// host waits once, at the end, to read the ids.  Falls back to a host round trip per token when
// the embedding table has no device form.
int64_t it_engine_decode_greedy(it_engine* e, uint64_t n, uint32_t* out_ids) {
    uint64_t nv = e->m->d.n_vocab;
    uint64_t produced = 0;
    const uint32_t ty = e->m->tok_embd.ty;
    const bool on_device = ty == IT_Q8_0 || ty == IT_F16 || ty == IT_BF16 || ty == IT_F32;
    if (on_device) {
        const uint64_t first = e->ring_next;
        for (uint64_t i = 0; i < n && i < 65536; i++) {
            if (e->len + 1 > e->n_ctx) break;
            int rc = forward(e, nullptr, 1, e->len, false, e->ring_next);
            if (rc) return rc;
            e->ring_next++;
            produced++;
        }
        if (produced && out_ids) {
            it_hip_read_tokens(e->be, first, produced, out_ids);
            char msg[512];
            if (it_hip_take_error(e->be, msg, sizeof msg)) {
                e->err = msg;
                return -10;
            }
        }
        return (int64_t)produced;
    }
    for (uint64_t i = 0; i < n; i++) {
        if (e->len + 1 > e->n_ctx) break;
        uint32_t next = it_hip_argmax(e->be, e->logits.p(), nv);
        if (out_ids) out_ids[produced] = next;
        produced++;
        int rc = forward(e, &next, 1, e->len, false);
        if (rc) return rc;
    }
    return (int64_t)produced;
}

const float* it_engine_ssm_state(it_engine* e, uint64_t layer, uint64_t* len) {
    *len = e->m->d.ssm_len();
    it_hip_read_state(e->be, e->ssm_of(layer), *len);
    return e->ssm_of(layer);
}
const float* it_engine_conv_state(it_engine* e, uint64_t layer, uint64_t* len) {
    *len = e->m->d.conv_len();
    it_hip_read_state(e->be, e->conv_of(layer), *len);
    return e->conv_of(layer);
}
const uint16_t* it_engine_k_slab(it_engine* e, uint64_t slot, uint64_t* len) {
    *len = e->slab_len();
    it_hip_read_kv(e->be, e->k_slab(slot), *len);
    return e->k_slab(slot);
}
const uint16_t* it_engine_v_slab(it_engine* e, uint64_t slot, uint64_t* len) {
    *len = e->slab_len();
    it_hip_read_kv(e->be, e->v_slab(slot), *len);
    return e->v_slab(slot);
}

}  // extern "C"
