// Fast single-token kernels against the order-preserving ones, on the same random weights and
// activations, across formats (Q8_0, NVFP4), row lengths (256..4096), prologues (none, rms_norm,
// gated per-head norm) and epilogues (store, causal conv + silu, accumulate), and the routed
// FFN pair (router + gate/up GLU, down + finish + residual).  The order-preserving kernels are
// the ones the bit-exact model tests pin to the CPU oracle; this program holds the fast ones
// to 1e-4 of them (relative to the largest reference value) and to the same expert picks.
// Prints one line per comparison and exits non-zero on any mismatch.
#include <hip/hip_runtime.h>
#include <cstdio>
#include <vector>
#include <cstring>
#include <cstdlib>
#include <cmath>
#include <random>
#include "../../inferred-thoughts_amd/csrc/kernels.h"
#include "../../inferred-thoughts_amd/csrc/kernels_fused.h"
static int g_bad = 0;
using namespace itk;
#define CK(x) do{hipError_t e=(x); if(e!=hipSuccess){printf("err %s line %d\n",hipGetErrorString(e),__LINE__); exit(1);} }while(0)
static std::mt19937 rng(1);
template <class T> T* dev(const std::vector<T>& h) { T* d; CK(hipMalloc(&d, h.size() * sizeof(T) + 64)); CK(hipMemcpy(d, h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice)); return d; }
template <class T> std::vector<T> host(const T* d, size_t n) { std::vector<T> h(n); CK(hipDeviceSynchronize()); CK(hipMemcpy(h.data(), d, n * sizeof(T), hipMemcpyDeviceToHost)); return h; }
std::vector<float> randf(size_t n, float sd = 1.f) { std::normal_distribution<float> d(0, sd); std::vector<float> v(n); for (auto& x : v) x = d(rng); return v; }
uint16_t f2h(float f) { _Float16 h = (_Float16)f; uint16_t u; memcpy(&u, &h, 2); return u; }
struct Mat { uint8_t* q; uint8_t* s; int fmt, rows, n_in; };
Mat make_mat(int fmt, int rows, int n_in) {
    Mat m{nullptr, nullptr, fmt, rows, n_in};
    if (fmt == W_Q8_0) {
        std::vector<uint8_t> q((size_t)rows * n_in); for (auto& b : q) b = (uint8_t)(rng() & 0xff);
        std::vector<uint16_t> s((size_t)rows * n_in / 32); for (auto& x : s) x = f2h(0.001f + 0.002f * (rng() % 1000) / 1000.f);
        m.q = dev(q); m.s = (uint8_t*)dev(s);
    } else {
        std::vector<uint8_t> q((size_t)rows * n_in / 2); for (auto& b : q) b = (uint8_t)(rng() & 0xff);
        std::vector<uint8_t> s((size_t)rows * n_in / 16); for (auto& x : s) x = (uint8_t)(0x20 + rng() % 0x20);
        m.q = dev(q); m.s = dev(s);
    }
    return m;
}
double maxdiff(const std::vector<float>& a, const std::vector<float>& b, double* scale) {
    double d = 0, s = 0; for (size_t i = 0; i < a.size(); i++) { d = std::max(d, (double)std::fabs(a[i] - b[i])); s = std::max(s, (double)std::fabs(a[i])); if (a[i] != a[i] || b[i] != b[i]) d = 1e30; }
    *scale = s; return d;
}
void report(const char* what, const std::vector<float>& a, const std::vector<float>& b) {
    double s; double d = maxdiff(a, b, &s);
    printf("%-60s max|diff| %.3e  (max|ref| %.3e)  %s\n", what, d, s, d <= 1e-4 * std::max(1.0, s) ? "ok" : "MISMATCH");
    if (!(d <= 1e-4 * std::max(1.0, s))) g_bad++;
}
int main() {
    int fmts[2] = {W_Q8_0, W_NVFP4};
    // ---- fused_gemv
    for (int fmt : fmts) for (int n_in : {256, 512, 1024, 2048, 4096}) for (int mode : {0, 1, 2, 3}) for (int epi0 : {0, 1, 2, 3}) {
        int rows[3] = {1000, 512, 9};
        Mat m[3]; for (int i = 0; i < 3; i++) m[i] = make_mat(fmt, rows[i], n_in);
        auto x = randf(n_in), nw = randf(n_in, 0.5f), gate = randf(n_in);
        float *dx = dev(x), *dnw = dev(nw), *dgate = dev(gate);
        auto cs = randf(rows[0] * 3), cw = randf(rows[0] * 4);
        std::vector<float> res[2][3], xc[2], csr[2];
        auto init = randf(1000);
        for (int exact = 0; exact < 2; exact++) {
            float* dcs = dev(cs); float* dcw = dev(cw);
            float* out[3]; for (int i = 0; i < 3; i++) { auto o = init; o.resize(rows[i]); out[i] = dev(o); }
            float* dxc = dev(std::vector<float>(n_in, 0.f));
            FusedGemvP p{}; p.x = dx; p.norm_w = dnw; p.gate = dgate; p.x_copy = dxc; p.eps = 1e-6f; p.n_in = n_in; p.mode = mode; p.head_dim = 64; p.exact = exact; p.n_mats = 3;
            for (int i = 0; i < 3; i++) { p.m[i].q = m[i].q; p.m[i].s = m[i].s; p.m[i].out = out[i]; p.m[i].n_out = rows[i]; p.m[i].fmt = fmt; p.m[i].epi = i == 0 ? epi0 : 0; }
            p.conv_state = dcs; p.conv_w = dcw;
            fused_gemv(p, 0);
            for (int i = 0; i < 3; i++) res[exact][i] = host(out[i], rows[i]);
            xc[exact] = host(dxc, n_in); csr[exact] = host(dcs, rows[0] * 3);
        }
        char nm[128];
        for (int i = 0; i < 3; i++) { snprintf(nm, sizeof nm, "fused_gemv fmt=%d n_in=%d mode=%d epi0=%d mat%d", fmt, n_in, mode, epi0, i); report(nm, res[1][i], res[0][i]); }
        snprintf(nm, sizeof nm, "fused_gemv fmt=%d n_in=%d mode=%d epi0=%d x_copy", fmt, n_in, mode, epi0); report(nm, xc[1], xc[0]);
        if (epi0 == 1) { snprintf(nm, sizeof nm, "fused_gemv fmt=%d n_in=%d mode=%d conv state", fmt, n_in, mode); report(nm, csr[1], csr[0]); }
    }
    // ---- moe glu + down
    for (int efmt : fmts) for (int n_in : {512, 2048}) for (int ff : {256, 512}) {
        int ne = 64, nu = 10;
        size_t qs = (size_t)ff * (efmt == W_Q8_0 ? n_in : n_in / 2), ss = (size_t)ff * (efmt == W_Q8_0 ? n_in / 32 * 2 : n_in / 16);
        Mat g = make_mat(efmt, ff * ne, n_in), u = make_mat(efmt, ff * ne, n_in), sg = make_mat(W_Q8_0, ff, n_in), su = make_mat(W_Q8_0, ff, n_in);
        size_t dqs = (size_t)n_in * (efmt == W_Q8_0 ? ff : ff / 2), dss = (size_t)n_in * (efmt == W_Q8_0 ? ff / 32 * 2 : ff / 16);
        Mat d = make_mat(efmt, n_in * ne, ff), sd = make_mat(W_Q8_0, n_in, ff);
        auto x = randf(n_in), logits = randf(ne), sc2 = randf(ne, 0.1f);
        logits[5] = logits[9];  // a tie
        float *dx = dev(x), *dlog = dev(logits), *dsc = dev(sc2);
        // reference route: softmax + top-k on the host is not needed: run the exact path with the last-block router via fused_gemv? use route_topk kernels
        std::vector<float> outs[2], shs[2], xs2[2]; std::vector<int> idsr[2]; std::vector<float> wr[2];
        for (int exact = 0; exact < 2; exact++) {
            int32_t* ids; float* w; CK(hipMalloc(&ids, 64)); CK(hipMalloc(&w, 64));
            float* probs = dev(logits);
            if (exact) { softmax_rows(probs, 1, ne, 0, 0); route_topk(probs, 1, ne, nu, ids, w, 0); }
            float* out = dev(std::vector<float>((size_t)nu * ff, 0.f)); float* sh = dev(std::vector<float>(ff, 0.f));
            MoeGluP p{}; p.x = dx; p.gq = g.q; p.gs = g.s; p.uq = u.q; p.us = u.s; p.gscale2 = dsc; p.uscale2 = dsc; p.q_stride = qs; p.s_stride = ss;
            p.fmt = efmt; p.n_in = n_in; p.n_out = ff; p.n_expert = ne; p.n_used = nu; p.exact = exact; p.sh_gq = sg.q; p.sh_gs = sg.s; p.sh_uq = su.q; p.sh_us = su.s; p.sh_fmt = W_Q8_0; p.sh_n_out = ff;
            p.out = out; p.sh_out = sh; p.route_ids = ids;
            if (!exact) { p.logits = dlog; p.route_ids_out = ids; p.route_w_out = w; }
            moe_glu_fused(p, 0);
            outs[exact] = host(out, (size_t)nu * ff); shs[exact] = host(sh, ff); idsr[exact] = host((int*)ids, nu); wr[exact] = host(w, nu);
            auto resid = std::vector<float>(n_in, 1.0f); float* dres = dev(resid); float lg = 0.3f; float* dlg = dev(std::vector<float>(1, lg));
            MoeDownP q{}; q.g_all = out; q.g_shared = sh; q.q = d.q; q.s = d.s; q.scale2 = dsc; q.q_stride = dqs; q.s_stride = dss; q.fmt = efmt; q.n_in = ff; q.n_out = n_in; q.n_used = nu; q.exact = exact;
            q.sh_q = sd.q; q.sh_s = sd.s; q.sh_fmt = W_Q8_0; q.sh_n_in = ff; q.route_ids = ids; q.route_w = w; q.logit = dlg; q.x = dres;
            moe_down_fused(q, 0);
            xs2[exact] = host(dres, n_in);
        }
        char nm[128];
        bool same = idsr[0] == idsr[1];
        if (!same) g_bad++;
        printf("moe efmt=%d n_in=%d ff=%d route ids %s:", efmt, n_in, ff, same ? "same" : "DIFFERENT"); for (int i = 0; i < nu; i++) printf(" %d/%d", idsr[0][i], idsr[1][i]); printf("\n");
        snprintf(nm, sizeof nm, "moe efmt=%d n_in=%d ff=%d route weights", efmt, n_in, ff); report(nm, wr[0], wr[1]);
        snprintf(nm, sizeof nm, "moe efmt=%d n_in=%d ff=%d glu routed", efmt, n_in, ff); report(nm, outs[0], outs[1]);
        snprintf(nm, sizeof nm, "moe efmt=%d n_in=%d ff=%d glu shared", efmt, n_in, ff); report(nm, shs[0], shs[1]);
        snprintf(nm, sizeof nm, "moe efmt=%d n_in=%d ff=%d down+residual", efmt, n_in, ff); report(nm, xs2[0], xs2[1]);
    }
    // ---- attention: prep folded into the tile kernel against attn_prep + the plain tile kernel
    for (int hd : {64, 128, 256}) for (int n_pos : {1, 64, 65, 300}) {
        const int nh = hd == 256 ? 16 : 8, nkv = 2, kvd = nkv * hd, n_rot = hd / 4, half = n_rot / 2, cap = 512;
        auto qg = randf((size_t)nh * 2 * hd), kp = randf(kvd), vp = randf(kvd), qn = randf(hd, 0.5f), kn = randf(hd, 0.5f);
        std::vector<float> tab((size_t)cap * half * 2);
        for (int p = 0; p < cap; p++) for (int i = 0; i < half; i++) { double a = p * std::pow(1e6, -2.0 * i / n_rot); tab[((size_t)p * half + i) * 2] = (float)std::cos(a); tab[((size_t)p * half + i) * 2 + 1] = (float)std::sin(a); }
        std::vector<uint16_t> kslab((size_t)cap * kvd), vslab((size_t)cap * kvd);
        for (auto& x : kslab) x = f2h(std::normal_distribution<float>(0, 1)(rng));
        for (auto& x : vslab) x = f2h(std::normal_distribution<float>(0, 1)(rng));
        float *dqg = dev(qg), *dkp = dev(kp), *dvp = dev(vp), *dqn = dev(qn), *dkn = dev(kn); float2* dtab = (float2*)dev(tab);
        const int pos = n_pos - 1; int* dpos = dev(std::vector<int>{pos}); int* dnpos = dev(std::vector<int>{n_pos});
        const int n_split = attend_split_count(cap, 1, hd, nh / nkv);
        std::vector<float> outs[2]; std::vector<uint16_t> krows[2], vrows[2];
        for (int fused = 0; fused < 2; fused++) {
            uint16_t *dk = dev(kslab), *dv = dev(vslab);
            float* dq = dev(std::vector<float>((size_t)nh * hd, 0.f)); float* dout = dev(std::vector<float>((size_t)nh * hd, 0.f));
            float* scratch = dev(std::vector<float>((size_t)nh * n_split * (hd + 2), 0.f));
            AttnArgs a{dq, dk, dv, 1, kvd, 0, hd, nh, nkv, 1.0f / std::sqrt((float)hd), dnpos};
            const float* gate = dqg + hd;
            if (!fused) {
                AttnPrepP pp{}; pp.qg = dqg; pp.k = dkp; pp.v = dvp; pp.q_norm = dqn; pp.k_norm = dkn; pp.rope = dtab; pp.pos_dyn = dpos; pp.q = dq;
                pp.k_slab = dk; pp.v_slab = dv; pp.n_head = nh; pp.n_head_kv = nkv; pp.head_dim = hd; pp.n_rot = n_rot; pp.kv_dim = kvd; pp.exact = 0; pp.eps = 1e-6f;
                attn_prep(pp, 0);
                attend_split_gated(a, n_split, scratch, dout, gate, 2 * hd, 0);
            } else {
                TilePrepP tp{}; tp.qg = dqg; tp.kproj = dkp; tp.vproj = dvp; tp.q_norm = dqn; tp.k_norm = dkn; tp.rope = dtab; tp.n_rot = n_rot; tp.eps = 1e-6f; tp.k_slab = dk; tp.v_slab = dv;
                if (!attend_tile_prep_ok(a, tp)) { printf("attention prep hd=%d: fused form refused  MISMATCH\n", hd); g_bad++; break; }
                attend_split_gated_prep(a, tp, n_split, scratch, dout, gate, 2 * hd, 0);
            }
            outs[fused] = host(dout, (size_t)nh * hd);
            krows[fused] = host(dk + (size_t)pos * kvd, kvd); vrows[fused] = host(dv + (size_t)pos * kvd, kvd);
        }
        if (outs[1].empty()) continue;
        char nm[128];
        snprintf(nm, sizeof nm, "attention prep folded in, hd=%d n_pos=%d: output", hd, n_pos); report(nm, outs[1], outs[0]);
        int kd = 0, vd = 0;
        for (int i = 0; i < kvd; i++) { kd += std::abs((int)krows[0][i] - (int)krows[1][i]) > 1; vd += vrows[0][i] != vrows[1][i]; }
        printf("attention prep folded in, hd=%d n_pos=%d: new K row %d values off by more than one f16 step, new V row %d differ  %s\n", hd, n_pos, kd, vd, kd || vd ? "MISMATCH" : "ok");
        if (kd || vd) g_bad++;
    }
    printf("%d mismatches\n", g_bad);
    return g_bad ? 1 : 0;
}
