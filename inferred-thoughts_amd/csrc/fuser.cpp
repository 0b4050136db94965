// Rewrites the seam ops of one single-token pass into fused launches.
//
// The op sequence a qwen35moe forward issues per layer is fixed
// (/root/reference src/model/qwen35.rs:1006-1093, 1138-1328, 1587-1700), so each block
// is matched as a whole: op ids in order plus the pointer links between them
// (an op's output must be the next one's input).  A block that does not match
// exactly — a different model, a traced pass, an NVFP4 shared expert with second
// scales — is simply issued op by op.  A fused launch sits at the position of its
// block's first op; everything it replaces is dropped, except an activation
// quantization that some unfused op still reads.
#include <cstddef>
#include <cstdio>
#include <cstring>
#include <memory>
#include <cstdlib>
#include "backend.h"

using namespace itk;
using Op = it_hip::OpRec;

namespace {

struct Plan {
    it_hip* be;
    std::vector<Op>& ops;
    std::vector<char> consumed;
    // which stage of a layer a fused launch is (0: none of them), with its arguments: the chain pass below rebuilds
    // runs of them as one persistent kernel
    enum Stage { ST_NONE = 0, ST_GDN_IN, ST_GDN_CORE, ST_GDN_OUT, ST_ROUTER, ST_GLU, ST_DOWN, ST_ATTN_IN, ST_ATTEND, ST_ATTN_OUT };
    struct Launch {
        int fam;         // it_hip::Family, for the per-kernel timing
        uint64_t bytes;  // algorithmic bytes of the launch (weights + state it must move once)
        std::function<void(hipStream_t)> fn;
        int stage = ST_NONE;
        FusedGemvP gv{};
        GdnCoreP gc{};
        MoeGluP mg{};
        MoeDownP md{};
        AttnArgs aa{};        // ST_ATTEND
        TilePrepP tp{};
        const float* gate = nullptr;
        int gate_stride = 0;
        float* attn_out = nullptr;
    };
    std::vector<std::vector<Launch>> at;  // fused launches keyed by position
    Launch& add(size_t i, int fam, uint64_t bytes, std::function<void(hipStream_t)> fn) {
        at[i].push_back(Launch{fam, bytes, std::move(fn)});
        return at[i].back();
    }
    // buffers a block's chain form leaves unwritten, keyed by the block's position
    struct Skips {
        size_t pos;
        std::vector<const void*> bufs;
    };
    std::vector<Skips> gdn_skips, ffn_skips, attn_skips;
    Plan(it_hip* b, std::vector<Op>& o) : be(b), ops(o), consumed(o.size(), 0), at(o.size()) {}
    // slot of a position scalar in the pass's device array, -1 when the pointer is not one
    int dyn_index(const void* p) const {
        const int* q = (const int*)p;
        return q >= be->dyn_dev && q < be->dyn_dev + it_hip::DYN_CAP ? (int)(q - be->dyn_dev) : -1;
    }
    bool ids(size_t i, std::initializer_list<int> want) const {
        if (i + want.size() > ops.size()) return false;
        size_t k = i;
        for (int w : want)
            if (ops[k++].id != w) return false;
        return true;
    }
    void take(size_t i, size_t n) {
        for (size_t k = i; k < i + n; k++) consumed[k] = 1;
    }
};

bool quantized_fmt(int64_t f) { return f == W_Q8_0 || f == W_NVFP4; }

bool float_fmt(int64_t f) { return f == W_F32 || f == W_F16 || f == W_BF16; }

// bytes of `rows` repacked rows of n_in weights (Q8_0: 34 per 32, NVFP4: 9 per 16; unquantized rows as stored)
uint64_t rows_bytes(int fmt, uint64_t rows, uint64_t n_in) {
    if (fmt == W_F32) return rows * n_in * 4;
    if (fmt == W_F16 || fmt == W_BF16) return rows * n_in * 2;
    return fmt == W_NVFP4 ? rows * n_in * 9 / 16 : rows * n_in * 34 / 32;
}
uint64_t gemv_bytes(const FusedGemvP& p) {
    uint64_t b = (uint64_t)p.n_in * 4;
    for (int i = 0; i < p.n_mats; i++) b += rows_bytes(p.m[i].fmt, p.m[i].n_out, p.n_in) + (uint64_t)p.m[i].n_out * 4;
    return b;
}

// MATMUL `m` reads activation `x` (f32) whose Q8_0 form was produced by QUANT `q`, one token.
bool mm_reads(const Op& m, const void* x, const Op& q) {
    return m.id == OP_MATMUL && m.p[2] == x && m.p[3] == q.p[1] && m.p[4] == q.p[2] && m.i[3] == 1 &&
           quantized_fmt(m.i[0]) && m.i[1] == q.i[0];
}

// MATMUL `m` with unquantized weights (the router and ssm alpha / beta of real files are F32) reads the f32
// activation `x` itself, one token.  Only the fast kernels take such a matrix into a fused launch.
bool mm_reads_f32(const Op& m, const void* x, int64_t n_in, int exact) {
    return !exact && m.id == OP_MATMUL && m.p[2] == x && m.i[3] == 1 && float_fmt(m.i[0]) && m.i[1] == n_in;
}

FusedMat mat_of(const Op& m, int epi, float* out_override = nullptr) {
    FusedMat f{};
    f.q = (const uint8_t*)m.p[0];
    f.s = (const uint8_t*)m.p[1];
    f.out = out_override ? out_override : (float*)m.p[5];
    f.n_out = (int)m.i[2];
    f.fmt = (int)m.i[0];
    f.epi = epi;
    return f;
}

// GDN mixer: 18 ops -> fused_gemv (norm + qkv/z/alpha/beta + conv) + gdn_core + fused_gemv (ssm_out += x)
bool match_gdn(Plan& pl, size_t i, int exact) {
    if (!pl.ids(i, {OP_RMS, OP_QUANT, OP_MATMUL, OP_MATMUL, OP_MATMUL, OP_MATMUL, OP_CONV, OP_GATHER, OP_GATHER,
                    OP_GATHER, OP_L2, OP_L2, OP_DELTA, OP_RMS_HEADS, OP_EW, OP_QUANT, OP_MATMUL, OP_EW}))
        return false;
    auto& o = pl.ops;
    const Op &rms = o[i], &q1 = o[i + 1], &mqkv = o[i + 2], &mz = o[i + 3], &ma = o[i + 4], &mb = o[i + 5];
    const Op &conv = o[i + 6], &g0 = o[i + 7], &g1 = o[i + 8], &g2 = o[i + 9], &l0 = o[i + 10], &l1 = o[i + 11];
    const Op &dl = o[i + 12], &rh = o[i + 13], &sm = o[i + 14], &q2 = o[i + 15], &mo = o[i + 16], &add = o[i + 17];
    const void* normed = rms.p[2];
    if (rms.i[0] != 1 || q1.p[0] != normed || q1.i[0] != rms.i[1]) return false;
    if (!mm_reads(mqkv, normed, q1) || !mm_reads(mz, normed, q1)) return false;
    if (!mm_reads(ma, normed, q1) && !mm_reads_f32(ma, normed, rms.i[1], exact)) return false;
    if (!mm_reads(mb, normed, q1) && !mm_reads_f32(mb, normed, rms.i[1], exact)) return false;
    int64_t dk = dl.i[1], dv = dl.i[2], nk = dl.i[3], nv = dl.i[4];
    int64_t kdim = nk * dk, vdim = nv * dv, cdim = 2 * kdim + vdim;
    if (dl.i[0] != 1 || dk != dv || (dk != 64 && dk != 128)) return false;
    if (conv.i[0] != 4 || conv.i[2] != 1 || conv.i[1] != cdim || conv.p[1] != mqkv.p[5] || mqkv.i[2] != cdim) return false;
    const void* cv = conv.p[3];
    auto gather_is = [&](const Op& g, int64_t chunk, int64_t off) {
        return g.p[0] == cv && g.i[0] == chunk && g.i[1] == cdim && g.i[2] == off && g.i[3] == chunk;
    };
    if (!gather_is(g0, kdim, 0) || !gather_is(g1, kdim, kdim) || !gather_is(g2, vdim, 2 * kdim)) return false;
    if (l0.p[0] != g0.p[1] || l1.p[0] != g1.p[1] || l0.i[0] != dk || l1.i[0] != dk || l0.f[0] != l1.f[0]) return false;
    if (dl.p[0] != g0.p[1] || dl.p[1] != g1.p[1] || dl.p[2] != g2.p[1] || dl.p[3] != ma.p[5] || dl.p[4] != mb.p[5])
        return false;
    if (ma.i[2] != nv || mb.i[2] != nv || mz.i[2] != vdim) return false;
    if (rh.p[0] != dl.p[8] || rh.i[0] != dv || rh.i[1] != nv) return false;
    if (sm.i[0] != 0 || sm.p[0] != mz.p[5] || sm.p[1] != dl.p[8] || sm.i[1] != vdim) return false;
    const void* z = mz.p[5];
    if (q2.p[0] != z || q2.i[0] != vdim || !mm_reads(mo, z, q2)) return false;
    if (add.i[0] != 2 || add.p[1] != mo.p[5] || add.p[0] != rms.p[0] || add.i[1] != mo.i[2]) return false;

    FusedGemvP a{};
    a.x = (const float*)rms.p[0];
    a.norm_w = (const float*)rms.p[1];
    a.x_copy = (float*)normed;
    a.eps = rms.f[0];
    a.n_in = (int)rms.i[1];
    a.mode = 1;
    a.exact = exact;
    a.n_mats = 4;
    a.m[0] = mat_of(mqkv, 1, (float*)cv);
    a.m[1] = mat_of(mz, exact ? 0 : 3);  // fast mode stores silu(z) once here instead of in every block of ssm_out
    a.m[2] = mat_of(ma, 0);
    a.m[3] = mat_of(mb, 0);
    a.conv_state = (float*)conv.p[0];
    a.conv_w = (const float*)conv.p[2];
    if ((float_fmt(ma.i[0]) || float_fmt(mb.i[0])) && !fused_gemv_fast_takes(a)) return false;

    GdnCoreP c{};
    c.conv = (const float*)cv;
    c.alpha = (const float*)dl.p[3];
    c.beta = (const float*)dl.p[4];
    c.ssm_a = (const float*)dl.p[5];
    c.dt_bias = (const float*)dl.p[6];
    c.state = (float*)dl.p[7];
    c.core = (float*)dl.p[8];
    c.n_k_heads = (int)nk;
    c.n_v_heads = (int)nv;
    c.exact = exact;
    c.eps = l0.f[0];
    c.q_scale = 1.0f / sqrtf((float)dk);
    int dki = (int)dk;
    if (nv > 64) return false;

    // ssm_out reads silu(z) * rms_norm_heads(core): formed in the GEMV's prologue
    FusedGemvP b{};
    b.x = (const float*)dl.p[8];
    b.norm_w = (const float*)rh.p[1];
    b.gate = (const float*)z;
    b.eps = rh.f[0];
    b.n_in = (int)vdim;
    b.mode = exact ? 2 : 3;
    b.head_dim = (int)dv;
    b.exact = exact;
    b.n_mats = 1;
    b.m[0] = mat_of(mo, 2, (float*)rms.p[0]);

    pl.take(i, 18);
    {
        auto& la = pl.add(i, it_hip::FAM_FUSED_GEMV, gemv_bytes(a) + (uint64_t)cdim * 8 * 4, [=](hipStream_t s) { fused_gemv(a, s); });
        la.stage = Plan::ST_GDN_IN;
        la.gv = a;
    }
    {
        auto& lc = pl.add(i, it_hip::FAM_GDN_ROWS, (uint64_t)nv * dv * dk * 8 + (uint64_t)(cdim + vdim) * 4, [=](hipStream_t s) { gdn_core(c, dki, s); });
        lc.stage = dki == 128 ? Plan::ST_GDN_CORE : Plan::ST_NONE;
        lc.gc = c;
    }
    {
        auto& lb = pl.add(i, it_hip::FAM_FUSED_GEMV, gemv_bytes(b) + (uint64_t)vdim * 4, [=](hipStream_t s) { fused_gemv(b, s); });
        lb.stage = Plan::ST_GDN_OUT;
        lb.gv = b;
    }
    // what the chain form of this block does not write: the normed input, the conv output, silu(z), alpha, beta, the read-out
    pl.gdn_skips.push_back({i, {normed, cv, z, ma.p[5], mb.p[5], dl.p[8]}});
    return true;
}

// rms_norm [+ whole-row gather copy] + quantize + 1..4 matmuls on the same activation
bool match_norm_matmuls(Plan& pl, size_t i, int exact) {
    auto& o = pl.ops;
    if (i + 2 >= o.size() || o[i].id != OP_RMS || o[i].i[0] != 1) return false;
    size_t k = i + 1;
    const void* act = o[i].p[2];
    float* copy2 = nullptr;
    if (o[k].id == OP_GATHER && o[k].p[0] == act && o[k].i[0] == o[i].i[1] && o[k].i[2] == 0 &&
        o[k].i[3] == o[i].i[1]) {
        copy2 = (float*)o[k].p[1];
        act = o[k].p[1];
        k++;
    }
    if (k >= o.size() || o[k].id != OP_QUANT || o[k].p[0] != act || o[k].i[0] != o[i].i[1]) return false;
    const Op& q = o[k];
    size_t m0 = k + 1, n = 0;
    while (n < 4 && m0 + n < o.size() && mm_reads(o[m0 + n], act, q)) n++;
    if (n == 0) return false;
    FusedGemvP a{};
    a.x = (const float*)o[i].p[0];
    a.norm_w = (const float*)o[i].p[1];
    a.x_copy = (float*)o[i].p[2];
    a.x_copy2 = copy2;
    a.eps = o[i].f[0];
    a.n_in = (int)o[i].i[1];
    a.mode = 1;
    a.exact = exact;
    a.n_mats = (int)n;
    for (size_t j = 0; j < n; j++) a.m[j] = mat_of(o[m0 + j], 0);
    pl.take(i, m0 + n - i);
    pl.add(i, it_hip::FAM_FUSED_GEMV, gemv_bytes(a), [=](hipStream_t s) { fused_gemv(a, s); });
    return true;
}

// quantize + matmul + add_assign of the result into another buffer
bool match_matmul_residual(Plan& pl, size_t i, int exact) {
    auto& o = pl.ops;
    if (!pl.ids(i, {OP_QUANT, OP_MATMUL, OP_EW})) return false;
    const Op &q = o[i], &m = o[i + 1], &add = o[i + 2];
    if (!mm_reads(m, q.p[0], q) || add.i[0] != 2 || add.p[1] != m.p[5] || add.i[1] != m.i[2] || add.p[0] == q.p[0])
        return false;
    FusedGemvP b{};
    b.x = (const float*)q.p[0];
    b.n_in = (int)q.i[0];
    b.exact = exact;
    b.n_mats = 1;
    b.m[0] = mat_of(m, 2, (float*)add.p[0]);
    pl.take(i, 3);
    pl.add(i, it_hip::FAM_FUSED_GEMV, gemv_bytes(b), [=](hipStream_t s) { fused_gemv(b, s); });
    return true;
}

// last-row gather + final norm + LM head
bool match_final(Plan& pl, size_t i, int exact) {
    auto& o = pl.ops;
    if (!pl.ids(i, {OP_GATHER, OP_RMS, OP_QUANT, OP_MATMUL})) return false;
    const Op &g = o[i], &rms = o[i + 1], &q = o[i + 2], &m = o[i + 3];
    if (g.i[3] != g.i[0] || rms.p[0] != g.p[1] || rms.i[0] != 1 || rms.i[1] != g.i[0]) return false;
    if (q.p[0] != rms.p[2] || q.i[0] != rms.i[1] || !mm_reads(m, rms.p[2], q)) return false;
    FusedGemvP a{};
    a.x = (const float*)g.p[0] + g.i[2];
    a.norm_w = (const float*)rms.p[1];
    a.x_copy = (float*)rms.p[2];
    a.eps = rms.f[0];
    a.n_in = (int)rms.i[1];
    a.mode = 1;
    a.exact = exact;
    a.n_mats = 1;
    a.m[0] = mat_of(m, 0);
    pl.take(i, 4);
    pl.add(i, it_hip::FAM_LM_HEAD, gemv_bytes(a), [=](hipStream_t s) { fused_gemv(a, s); });
    return true;
}


// attention mixer: 18 ops -> fused_gemv (norm + wq/wk/wv) + attn_prep + split-K attend with the
// gate folded into its merge + fused_gemv (wo += x)
bool match_attn(Plan& pl, size_t i, int exact) {
    if (!pl.ids(i, {OP_RMS, OP_QUANT, OP_MATMUL, OP_GATHER, OP_GATHER, OP_MATMUL, OP_MATMUL, OP_RMS_HEADS, OP_RMS_HEADS,
                    OP_ROPE, OP_ROPE, OP_KVWRITE, OP_KVWRITE, OP_ATTEND, OP_EW, OP_QUANT, OP_MATMUL, OP_EW}))
        return false;
    auto& o = pl.ops;
    const Op &rms = o[i], &q1 = o[i + 1], &mq = o[i + 2], &gq = o[i + 3], &gg = o[i + 4], &mk = o[i + 5], &mv = o[i + 6];
    const Op &nq = o[i + 7], &nk = o[i + 8], &rq = o[i + 9], &rk = o[i + 10], &wk = o[i + 11], &wv = o[i + 12];
    const Op &at = o[i + 13], &sg = o[i + 14], &q2 = o[i + 15], &mo = o[i + 16], &add = o[i + 17];
    const void* normed = rms.p[2];
    if (rms.i[0] != 1 || q1.p[0] != normed || q1.i[0] != rms.i[1]) return false;
    if (!mm_reads(mq, normed, q1) || !mm_reads(mk, normed, q1) || !mm_reads(mv, normed, q1)) return false;
    if (at.i[0] != 1 || !at.p[3]) return false;  // one query row, graphed position
    int64_t hd = at.i[2], nh = at.i[3], nkv = at.i[4], kvd = at.i[1];
    const void* qg = mq.p[5];
    if (mq.i[2] != 2 * hd * nh || mk.i[2] != nkv * hd || mv.i[2] != nkv * hd || kvd != nkv * hd) return false;
    auto gather_is = [&](const Op& g, int64_t off) {
        return g.p[0] == qg && g.i[0] == hd && g.i[1] == 2 * hd && g.i[2] == off && g.i[3] == hd * nh;
    };
    if (!gather_is(gq, 0) || !gather_is(gg, hd)) return false;
    const void *qb = gq.p[1], *gb = gg.p[1], *kb = mk.p[5], *vb = mv.p[5];
    if (nq.p[0] != qb || nq.i[0] != hd || nq.i[1] != nh || nk.p[0] != kb || nk.i[0] != hd || nk.i[1] != nkv ||
        nq.f[0] != nk.f[0])
        return false;
    if (rq.p[0] != qb || rk.p[0] != kb || rq.p[1] != rk.p[1] || !rq.p[2] || !rk.p[2] || rq.i[1] != 1 || rk.i[1] != 1 ||
        rq.i[2] != hd || rk.i[2] != hd || rq.i[3] != rk.i[3] || rq.i[4] != nh || rk.i[4] != nkv)
        return false;
    if (wk.p[2] != kb || wv.p[2] != vb || !wk.p[1] || !wv.p[1] || wk.i[0] != kvd || wv.i[0] != kvd || wk.i[2] != kvd ||
        wv.i[2] != kvd || wk.p[0] != at.p[1] || wv.p[0] != at.p[2])
        return false;
    if (at.p[0] != qb) return false;
    // One position feeds the fused block's rotation, cache writes and context length.  The seam passes them
    // separately, so they are compared here (this pass's values) and again before every replay.
    const std::array<int, 4> slots = {pl.dyn_index(rq.p[2]), pl.dyn_index(wk.p[1]), pl.dyn_index(wv.p[1]), pl.dyn_index(at.p[3])};
    if (pl.dyn_index(rk.p[2]) < 0 || pl.be->dyn_host[pl.dyn_index(rk.p[2])] != pl.be->dyn_host[slots[0] < 0 ? 0 : slots[0]]) return false;
    if (!pl.be->attn_positions_agree({slots})) return false;
    const void* attn = at.p[5];
    if (sg.i[0] != 1 || sg.p[0] != attn || sg.p[1] != gb || sg.i[1] != hd * nh) return false;
    if (q2.p[0] != attn || q2.i[0] != hd * nh || !mm_reads(mo, attn, q2)) return false;
    if (add.i[0] != 2 || add.p[1] != mo.p[5] || add.p[0] != rms.p[0] || add.i[1] != mo.i[2]) return false;

    FusedGemvP a{};
    a.x = (const float*)rms.p[0];
    a.norm_w = (const float*)rms.p[1];
    a.x_copy = (float*)normed;
    a.eps = rms.f[0];
    a.n_in = (int)rms.i[1];
    a.mode = 1;
    a.exact = exact;
    a.n_mats = 3;
    a.m[0] = mat_of(mq, 0);
    a.m[1] = mat_of(mk, 0);
    a.m[2] = mat_of(mv, 0);

    AttnPrepP pp{};
    pp.qg = (const float*)qg;
    pp.k = (const float*)kb;
    pp.v = (const float*)vb;
    pp.q_norm = (const float*)nq.p[1];
    pp.k_norm = (const float*)nk.p[1];
    pp.rope = (const float2*)rq.p[1];
    pp.pos_dyn = (const int*)rq.p[2];
    pp.q = (float*)qb;
    pp.k_slab = (uint16_t*)wk.p[0];
    pp.v_slab = (uint16_t*)wv.p[0];
    pp.n_head = (int)nh;
    pp.n_head_kv = (int)nkv;
    pp.head_dim = (int)hd;
    pp.n_rot = (int)rq.i[3];
    pp.kv_dim = (int)kvd;
    pp.exact = exact;
    pp.eps = nq.f[0];

    AttnArgs aa{(const float*)qb, (const uint16_t*)at.p[1], (const uint16_t*)at.p[2], 1, (int)kvd, 0, (int)hd, (int)nh,
                (int)nkv, at.f[0], (const int*)at.p[3]};
    int n_split = (int)at.i[5];
    float* scratch = (float*)at.p[4];
    float* attn_out = (float*)attn;
    const float* gate = (const float*)qg + hd;
    int gate_stride = (int)(2 * hd);

    FusedGemvP b{};
    b.x = (const float*)attn;
    b.n_in = (int)(hd * nh);
    b.exact = exact;
    b.n_mats = 1;
    b.m[0] = mat_of(mo, 2, (float*)rms.p[0]);

    pl.take(i, 18);
    pl.be->fused_attn_slots.push_back(slots);
    it_hip* be = pl.be;
    // K and V rows of the live context, f16 (the position is the one this pass was recorded at)
    const uint64_t kv_bytes = (uint64_t)at.i[8] * kvd * 2 * 2;
    Plan::Launch& l_in = pl.add(i, it_hip::FAM_FUSED_GEMV, gemv_bytes(a), [=](hipStream_t s) { fused_gemv(a, s); });
    const size_t in_at = pl.at[i].size() - 1;
    (void)l_in;
    TilePrepP tp{};
    tp.qg = pp.qg;
    tp.kproj = pp.k;
    tp.vproj = pp.v;
    tp.q_norm = pp.q_norm;
    tp.k_norm = pp.k_norm;
    tp.rope = pp.rope;
    tp.n_rot = pp.n_rot;
    tp.eps = pp.eps;
    tp.k_slab = pp.k_slab;
    tp.v_slab = pp.v_slab;
    bool three = false;
    if (at.i[6] == 0 && attend_tile_prep_ok(aa, tp)) {
        // norm + rotation of q and of the new key, and the slab writes, happen inside the tile kernel
        Plan::Launch& l_at = pl.add(i, it_hip::FAM_ATTEND, kv_bytes + (uint64_t)(2 * hd * nh + 2 * kvd) * 4, [=](hipStream_t s) {
            if (!attend_split_gated_prep(aa, tp, n_split, scratch, attn_out, gate, gate_stride, s))
                be->fail("attend: the split-K kernels could not be launched");
        });
        l_at.stage = Plan::ST_ATTEND;
        l_at.aa = aa;
        l_at.tp = tp;
        l_at.gate = gate;
        l_at.gate_stride = gate_stride;
        l_at.attn_out = attn_out;
        three = true;
    } else if (at.i[6] == 0) {
        pl.add(i, it_hip::FAM_ATTN_PREP, (uint64_t)(2 * hd * nh + 2 * kvd) * 4 + kvd * 4, [=](hipStream_t s) { attn_prep(pp, s); });
        pl.add(i, it_hip::FAM_ATTEND, kv_bytes, [=](hipStream_t s) {
            if (!attend_split_gated(aa, n_split, scratch, attn_out, gate, gate_stride, s))
                be->fail("attend: the split-K kernels could not be launched");
        });
    } else {
        pl.add(i, it_hip::FAM_ATTN_PREP, (uint64_t)(2 * hd * nh + 2 * kvd) * 4 + kvd * 4, [=](hipStream_t s) { attn_prep(pp, s); });
        // the exact attention kernel and its gate stay as they are
        auto run_attend = at.run, run_gate = sg.run, run_gather_gate = gg.run;
        pl.add(i, it_hip::FAM_OTHER, 0, run_gather_gate);
        pl.add(i, it_hip::FAM_ATTEND, kv_bytes, run_attend);
        pl.add(i, it_hip::FAM_OTHER, 0, run_gate);
    }
    Plan::Launch& l_out = pl.add(i, it_hip::FAM_FUSED_GEMV, gemv_bytes(b), [=](hipStream_t s) { fused_gemv(b, s); });
    if (three) {   // the form whose in- and out-projection a layer chain may take over
        l_out.stage = Plan::ST_ATTN_OUT;
        l_out.gv = b;
        pl.at[i][in_at].stage = Plan::ST_ATTN_IN;
        pl.at[i][in_at].gv = a;
        pl.attn_skips.push_back({i, {normed}});
    }
    return true;
}

// routed FFN: 17 to 20 ops -> fused_gemv (norm + router + shared gate logit) + moe_glu_fused + moe_down_fused
bool match_ffn(Plan& pl, size_t i, int exact, unsigned* counter, unsigned long long* tally) {
    // With a quantized router the activation is quantized before the router matmul; with an unquantized one
    // (F32 in real files) the first reader of the quantized form is the expert gate/up product, after the route.
    // An NVFP4 file carries a second, per-tensor scale for each of the shared expert's matrices
    // (src/model/qwen35.rs:1669-1682): up to two SCALE ops follow the shared gate / up products and one the
    // shared down product.  The walk below takes the fixed ops in order and those three where they are present.
    auto& o = pl.ops;
    size_t k = i;
    auto take = [&](int id) -> const Op* { return k < o.size() && o[k].id == id ? &o[k++] : nullptr; };
    const Op *rms_p = take(OP_RMS), *ga_p = take(OP_GATHER);
    if (!rms_p || !ga_p) return false;
    const Op* q1_p = take(OP_QUANT);
    const bool q_first = q1_p != nullptr;
    if (!q_first && exact) return false;
    const Op *mr_p = take(OP_MATMUL), *ml_p = take(OP_MATMUL), *sm_p = take(OP_SOFTMAX), *rt_p = take(OP_ROUTE);
    if (!mr_p || !ml_p || !sm_p || !rt_p) return false;
    if (!q_first && !(q1_p = take(OP_QUANT))) return false;
    const Op *glu_p = take(OP_GLU), *q2_p = take(OP_QUANT), *ex_p = take(OP_EXPERTS), *sgm_p = take(OP_MATMUL), *sum_p = take(OP_MATMUL);
    if (!glu_p || !q2_p || !ex_p || !sgm_p || !sum_p) return false;
    float sh_scale[3] = {1.0f, 1.0f, 1.0f};   // gate, up, down
    bool has_up = false, has_gate = false;
    while (k < o.size() && o[k].id == OP_SCALE) {   // the up product is scaled first, then the gate product
        const Op& sc = o[k];
        if (!has_up && !has_gate && sc.p[0] == sum_p->p[5] && sc.i[0] == sum_p->i[2]) {
            sh_scale[1] = sc.f[0];
            has_up = true;
        } else if (!has_gate && sc.p[0] == sgm_p->p[5] && sc.i[0] == sgm_p->i[2]) {
            sh_scale[0] = sc.f[0];
            has_gate = true;
        } else {
            return false;
        }
        k++;
    }
    const Op *sil_p = take(OP_EW), *q3_p = take(OP_QUANT), *sdm_p = take(OP_MATMUL);
    if (!sil_p || !q3_p || !sdm_p) return false;
    if (k < o.size() && o[k].id == OP_SCALE) {
        const Op& sc = o[k];
        if (sc.p[0] != sdm_p->p[5] || sc.i[0] != sdm_p->i[2]) return false;
        sh_scale[2] = sc.f[0];
        k++;
    }
    const Op *fin_p = take(OP_FINISH), *add_p = take(OP_EW);
    if (!fin_p || !add_p) return false;
    const size_t n_ops = k - i;
    const Op &rms = *rms_p, &ga = *ga_p, &q1 = *q1_p, &mr = *mr_p, &ml = *ml_p, &sm = *sm_p, &rt = *rt_p;
    const Op &glu = *glu_p, &q2 = *q2_p, &ex = *ex_p, &sgm = *sgm_p, &sum_ = *sum_p, &sil = *sil_p;
    const Op &q3 = *q3_p, &sdm = *sdm_p, &fin = *fin_p, &add = *add_p;
    int64_t nd = rms.i[1];
    if (rms.i[0] != 1) return false;
    // experts placed through a table (a pool larger than its device tier) are read by the unfused kernels only
    if (glu.i[8] || ex.i[8]) return false;
    if (ga.p[0] != rms.p[2] || ga.i[0] != nd || ga.i[2] != 0 || ga.i[3] != nd) return false;
    const void* x = ga.p[1];
    if (q1.p[0] != x || q1.i[0] != nd || ml.i[2] != 1) return false;
    if (q_first ? !mm_reads(mr, x, q1) : !mm_reads_f32(mr, x, nd, exact)) return false;
    if (!mm_reads(ml, x, q1) && !mm_reads_f32(ml, x, nd, exact)) return false;
    int64_t ne = mr.i[2];
    const void* router = mr.p[5];
    if (sm.p[0] != router || sm.i[0] != 1 || sm.i[1] != ne) return false;
    if (rt.p[0] != router || rt.i[0] != 1 || rt.i[1] != ne) return false;
    int64_t nu = rt.i[2];
    if (nu > 16 || ne > nd || !counter) return false;
    if (glu.p[6] != rt.p[1] || glu.p[7] != q1.p[1] || glu.p[8] != q1.p[2] || glu.i[1] != nd || glu.i[3] != nu ||
        glu.i[4] != nu || !quantized_fmt(glu.i[0]))
        return false;
    int64_t ff = glu.i[2];
    const void* g_all = glu.p[9];
    if (q2.p[0] != g_all || q2.i[0] != nu * ff) return false;
    if (ex.p[3] != rt.p[1] || ex.p[4] != q2.p[1] || ex.p[5] != q2.p[2] || ex.i[1] != ff || ex.i[2] != nd ||
        ex.i[3] != nu || ex.i[5] != 0 || !quantized_fmt(ex.i[0]))
        return false;
    if (!mm_reads(sgm, x, q1) || !mm_reads(sum_, x, q1) || sgm.i[2] != sum_.i[2] || sgm.i[0] != sum_.i[0]) return false;
    int64_t sff = sgm.i[2];
    const void* e_gate = sgm.p[5];
    if (sil.i[0] != 0 || sil.p[0] != e_gate || sil.p[1] != sum_.p[5] || sil.i[1] != sff) return false;
    if (q3.p[0] != e_gate || q3.i[0] != sff || !mm_reads(sdm, e_gate, q3) || sdm.i[2] != nd) return false;
    if (fin.p[1] != ex.p[6] || fin.p[2] != rt.p[2] || fin.p[3] != sdm.p[5] || fin.p[4] != ml.p[5] || fin.i[0] != 0 ||
        fin.i[1] != nd || fin.i[2] != 1 || fin.i[3] != nu || fin.i[4] != 0)
        return false;
    if (add.i[0] != 2 || add.p[1] != fin.p[0] || add.p[0] != rms.p[0] || add.i[1] != nd) return false;

    FusedGemvP a{};
    a.x = (const float*)rms.p[0];
    a.norm_w = (const float*)rms.p[1];
    a.x_copy = (float*)rms.p[2];
    a.x_copy2 = (float*)x;
    a.eps = rms.f[0];
    a.n_in = (int)nd;
    a.mode = 1;
    a.exact = exact;
    a.n_mats = 2;
    a.m[0] = mat_of(mr, 0);
    a.m[1] = mat_of(ml, 0);
    // fast mode ranks the logits inside the expert kernel instead (no cross-block hand-off)
    a.route_counter = exact ? counter : nullptr;
    a.n_expert = (int)ne;
    a.n_used = (int)nu;
    a.route_ids = (int32_t*)rt.p[1];
    a.route_w = (float*)rt.p[2];
    if ((float_fmt(mr.i[0]) || float_fmt(ml.i[0])) && !fused_gemv_fast_takes(a)) return false;

    MoeGluP g{};
    g.x = (const float*)x;
    g.gq = (const uint8_t*)glu.p[0];
    g.gs = (const uint8_t*)glu.p[1];
    g.uq = (const uint8_t*)glu.p[2];
    g.us = (const uint8_t*)glu.p[3];
    g.gscale2 = (const float*)glu.p[4];
    g.uscale2 = (const float*)glu.p[5];
    g.q_stride = glu.i[6];
    g.s_stride = glu.i[7];
    g.fmt = (int)glu.i[0];
    g.n_in = (int)nd;
    g.n_out = (int)ff;
    g.n_expert = (int)ne;
    g.n_used = (int)nu;
    g.exact = exact;
    g.sh_gq = (const uint8_t*)sgm.p[0];
    g.sh_gs = (const uint8_t*)sgm.p[1];
    g.sh_uq = (const uint8_t*)sum_.p[0];
    g.sh_us = (const uint8_t*)sum_.p[1];
    g.sh_fmt = (int)sgm.i[0];
    g.sh_n_out = (int)sff;
    g.sh_gscale = sh_scale[0];
    g.sh_uscale = sh_scale[1];
    g.out = (float*)g_all;
    g.sh_out = (float*)e_gate;
    g.route_ids = (const int32_t*)rt.p[1];
    if (!exact) {
        g.logits = (const float*)router;
        g.route_ids_out = (int32_t*)rt.p[1];
        g.route_w_out = (float*)rt.p[2];
    }

    MoeDownP d{};
    d.g_all = (const float*)g_all;
    d.g_shared = (const float*)e_gate;
    d.q = (const uint8_t*)ex.p[0];
    d.s = (const uint8_t*)ex.p[1];
    d.scale2 = (const float*)ex.p[2];
    d.q_stride = ex.i[6];
    d.s_stride = ex.i[7];
    d.fmt = (int)ex.i[0];
    d.n_in = (int)ff;
    d.n_out = (int)nd;
    d.n_used = (int)nu;
    d.exact = exact;
    d.sh_q = (const uint8_t*)sdm.p[0];
    d.sh_s = (const uint8_t*)sdm.p[1];
    d.sh_fmt = (int)sdm.i[0];
    d.sh_n_in = (int)sff;
    d.sh_dscale = sh_scale[2];
    d.route_ids = (const int32_t*)rt.p[1];
    d.route_w = (const float*)rt.p[2];
    d.logit = (const float*)ml.p[5];
    d.x = (float*)rms.p[0];
    if (pl.be->count_reads_in_fused) {
        d.counts_gate = (uint32_t*)glu.p[10];
        d.counts_up = (uint32_t*)glu.p[11];
        d.counts_down = (uint32_t*)ex.p[7];
        d.tally = tally;
    }

    pl.take(i, n_ops);
    const uint64_t glu_b = 2 * rows_bytes(g.fmt, (uint64_t)nu * ff, nd) + 2 * rows_bytes(g.sh_fmt, sff, nd) + (uint64_t)nd * 4 +
                           (uint64_t)(nu * ff + sff) * 4;
    const uint64_t down_b = rows_bytes(d.fmt, (uint64_t)nu * nd, ff) + rows_bytes(d.sh_fmt, nd, sff) +
                            (uint64_t)(nu * ff + sff) * 4 + (uint64_t)nd * 8;
    {
        auto& la = pl.add(i, it_hip::FAM_FUSED_GEMV, gemv_bytes(a), [=](hipStream_t s) { fused_gemv(a, s); });
        la.stage = Plan::ST_ROUTER;
        la.gv = a;
    }
    {
        auto& lg = pl.add(i, it_hip::FAM_MOE_GLU, glu_b, [=](hipStream_t s) { moe_glu_fused(g, s); });
        lg.stage = Plan::ST_GLU;
        lg.mg = g;
    }
    {
        auto& ld = pl.add(i, it_hip::FAM_MOE_DOWN, down_b, [=](hipStream_t s) { moe_down_fused(d, s); });
        ld.stage = Plan::ST_DOWN;
        ld.md = d;
    }
    // what the chain form does not write: the normed input and its copy, the logits, the intermediates
    pl.ffn_skips.push_back({i, {rms.p[2], x, router, ml.p[5], g_all, e_gate}});
    return true;
}


// ---------------------------------------------------------------------------------- layer chains
// Runs of fused layer stages become one persistent kernel each (k_chain.hip): a Gated DeltaNet block's three launches
// followed by its routed FFN's three are one layer of a chain; an FFN whose mixer is not a Gated DeltaNet block (an
// attention layer's) may open a chain.  A run ends at anything else: an unfused op, another fused launch, a layer of
// another shape, the chain's capacity.
bool q8(const FusedMat& m, int n_out, int epi) { return m.fmt == W_Q8_0 && m.n_out == n_out && m.epi == epi; }
bool al16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

bool f32m(const FusedMat& m, int n_out, int epi) { return m.fmt == W_F32 && m.n_out == n_out && m.epi == epi; }

// rf: 1 when the small matrices (alpha / beta here, router / gate logit in the FFN) are F32, 0 when Q8_0
bool chain_mixer(const FusedGemvP& a, const GdnCoreP& c, const FusedGemvP& b, ChainMixer* m, int* rf) {
    if (a.exact || a.n_in != 2048 || a.mode != 1 || a.n_mats != 4 || a.route_counter) return false;
    if (!q8(a.m[0], 8192, 1) || !q8(a.m[1], 4096, 3)) return false;
    if (q8(a.m[2], 32, 0) && q8(a.m[3], 32, 0)) *rf = 0;
    else if (f32m(a.m[2], 32, 0) && f32m(a.m[3], 32, 0)) *rf = 1;
    else return false;
    if (c.n_k_heads != 16 || c.n_v_heads != 32 || c.exact) return false;
    if (b.n_in != 4096 || b.mode != 3 || b.head_dim != 128 || b.n_mats != 1 || !q8(b.m[0], 2048, 2) || b.m[0].out != a.x) return false;
    if (c.conv != a.m[0].out || c.alpha != a.m[2].out || c.beta != a.m[3].out || b.gate != a.m[1].out || b.x != c.core) return false;
    for (int i = 0; i < 4; i++)
        if (!al16(a.m[i].q) || (!(*rf && i >= 2) && !al16(a.m[i].s))) return false;
    if (!al16(b.m[0].q) || !al16(b.m[0].s) || !al16(a.norm_w) || !al16(a.conv_w) || !al16(c.state) || !al16(a.x)) return false;
    m->norm_w = a.norm_w;
    m->qkv_q = a.m[0].q; m->qkv_s = a.m[0].s;
    m->z_q = a.m[1].q; m->z_s = a.m[1].s;
    m->a_q = a.m[2].q; m->a_s = a.m[2].s;
    m->b_q = a.m[3].q; m->b_s = a.m[3].s;
    m->conv_state = a.conv_state;
    m->conv_w = a.conv_w;
    m->ssm_a = c.ssm_a;
    m->dt_bias = c.dt_bias;
    m->state = c.state;
    m->head_norm_w = b.norm_w;
    m->o_q = b.m[0].q; m->o_s = b.m[0].s;
    m->eps_norm = a.eps;
    m->eps_l2 = c.eps;
    m->eps_head = b.eps;
    m->q_scale = c.q_scale;
    return true;
}

bool chain_ffn(const FusedGemvP& r, const MoeGluP& g, const MoeDownP& d, ChainFfn* f, int* sh_fmt, int* rf) {
    if (r.exact || r.n_in != 2048 || r.mode != 1 || r.n_mats != 2 || r.route_counter) return false;
    if (q8(r.m[0], 512, 0) && q8(r.m[1], 1, 0)) *rf = 0;
    else if (f32m(r.m[0], 512, 0) && f32m(r.m[1], 1, 0)) *rf = 1;
    else return false;
    if (g.exact || g.fmt != W_NVFP4 || g.n_in != 2048 || g.n_out != 512 || g.n_expert != 512 || g.n_used != 10 || g.sh_n_out != 512) return false;
    if (g.sh_fmt != W_Q8_0 && g.sh_fmt != W_NVFP4) return false;
    if (!g.logits || g.logits != r.m[0].out || !g.route_ids_out || !g.route_w_out || g.x != r.x_copy2) return false;
    if (d.exact || d.fmt != W_NVFP4 || d.n_in != 512 || d.n_out != 2048 || d.n_used != 10 || d.sh_fmt != g.sh_fmt || d.sh_n_in != 512) return false;
    if (d.g_all != g.out || d.g_shared != g.sh_out || d.logit != r.m[1].out || d.x != r.x || d.route_ids != g.route_ids_out || d.route_w != g.route_w_out)
        return false;
    if (!*rf && (!r.m[0].s || !r.m[1].s || !al16(r.m[0].s) || !al16(r.m[1].s))) return false;
    const void* ptrs[] = {r.m[0].q, r.m[1].q, g.gq, g.gs, g.uq, g.us, g.sh_gq, g.sh_gs, g.sh_uq, g.sh_us, d.q, d.s, d.sh_q, d.sh_s, r.norm_w, r.x};
    for (const void* p : ptrs)
        if (!p || !al16(p)) return false;
    if (g.q_stride % 16 || g.s_stride % 16 || d.q_stride % 16 || d.s_stride % 16) return false;
    f->norm_w = r.norm_w;
    f->r_q = r.m[0].q; f->r_s = r.m[0].s;
    f->l_q = r.m[1].q; f->l_s = r.m[1].s;
    f->sg_q = g.sh_gq; f->sg_s = g.sh_gs; f->su_q = g.sh_uq; f->su_s = g.sh_us;
    f->sd_q = d.sh_q; f->sd_s = d.sh_s;
    f->eg_q = g.gq; f->eg_s = g.gs; f->eu_q = g.uq; f->eu_s = g.us; f->ed_q = d.q; f->ed_s = d.s;
    f->gscale2 = g.gscale2; f->uscale2 = g.uscale2; f->dscale2 = d.scale2;
    f->gu_q_stride = g.q_stride; f->gu_s_stride = g.s_stride; f->d_q_stride = d.q_stride; f->d_s_stride = d.s_stride;
    f->sh_gscale = g.sh_gscale; f->sh_uscale = g.sh_uscale; f->sh_dscale = d.sh_dscale;
    f->eps = r.eps;
    f->route_ids = g.route_ids_out;
    f->route_w = g.route_w_out;
    f->counts_gate = d.counts_gate; f->counts_up = d.counts_up; f->counts_down = d.counts_down;
    *sh_fmt = g.sh_fmt;
    return true;
}

bool chain_attn_out(const FusedGemvP& b, ChainMixer* m) {
    if (b.exact || b.mode != 0 || b.n_in != 4096 || b.n_mats != 1 || !q8(b.m[0], 2048, 2) || b.route_counter) return false;
    if (!al16(b.m[0].q) || !al16(b.m[0].s) || !al16(b.x) || !al16(b.m[0].out)) return false;
    *m = ChainMixer{};
    m->o_q = b.m[0].q;
    m->o_s = b.m[0].s;
    m->attn = b.x;
    return true;
}

bool chain_attn_in(const FusedGemvP& a, ChainTail* t) {
    if (a.exact || a.mode != 1 || a.n_in != 2048 || a.n_mats != 3 || a.route_counter) return false;
    if (!q8(a.m[0], 8192, 0) || !q8(a.m[1], 512, 0) || !q8(a.m[2], 512, 0)) return false;
    for (int i = 0; i < 3; i++)
        if (!al16(a.m[i].q) || !al16(a.m[i].s)) return false;
    if (!al16(a.norm_w)) return false;
    t->norm_w = a.norm_w;
    t->q_q = a.m[0].q; t->q_s = a.m[0].s;
    t->k_q = a.m[1].q; t->k_s = a.m[1].s;
    t->v_q = a.m[2].q; t->v_s = a.m[2].s;
    t->out_q = a.m[0].out; t->out_k = a.m[1].out; t->out_v = a.m[2].out;
    t->eps = a.eps;
    return true;
}

// a whole attention block as a chain layer: in-projection, attention launch and out-projection must be the shapes the
// chain's stages are written for and hang together (the attention reads what the in-projection writes and writes what
// the out-projection reads; the gate is the second half of every head's wq rows)
// Beyond this many positions the block stays between two chains: the chain's attention walks a range's keys 64 at a
// time in one block per (KV head, range) and is measured up to 30,000 positions; the split-K kernels between chains
// size their grid to the context
constexpr int CHAIN_ATTN_MAX_POS = 65536;
bool chain_attn(const Plan& pl, const FusedGemvP& in, const Plan::Launch& at, const FusedGemvP& out, ChainAttn* a, ChainMixer* m) {
    const int slot = pl.dyn_index(at.aa.n_pos_dyn);
    if (slot < 0 || pl.be->dyn_host[slot] > CHAIN_ATTN_MAX_POS) return false;
    ChainTail t{};
    ChainMixer mo{};
    if (!chain_attn_in(in, &t) || !chain_attn_out(out, &mo)) return false;
    const AttnArgs& aa = at.aa;
    const TilePrepP& tp = at.tp;
    if (aa.n_q != 1 || aa.n_head != 16 || aa.n_head_kv != 2 || aa.head_dim != 256 || aa.kv_dim != 512 || !aa.n_pos_dyn) return false;
    if (tp.qg != t.out_q || tp.kproj != t.out_k || tp.vproj != t.out_v || at.gate != tp.qg + 256 || at.gate_stride != 512) return false;
    if (at.attn_out != mo.attn || out.m[0].out != in.x) return false;
    if (tp.k_slab != aa.k || tp.v_slab != aa.v || !tp.q_norm || !tp.k_norm || !tp.rope) return false;
    if (tp.n_rot <= 0 || tp.n_rot > 256 || (tp.n_rot / 2) % 4 || ((tp.n_rot / 8) & (tp.n_rot / 8 - 1))) return false;
    if (!al16(tp.q_norm) || !al16(tp.k_norm) || !al16(tp.rope) || !al16(tp.k_slab) || !al16(tp.v_slab)) return false;
    *a = ChainAttn{};
    a->norm_w = t.norm_w;
    a->q_q = t.q_q; a->q_s = t.q_s; a->k_q = t.k_q; a->k_s = t.k_s; a->v_q = t.v_q; a->v_s = t.v_s;
    a->q_norm = tp.q_norm; a->k_norm = tp.k_norm;
    a->rope = tp.rope;
    a->k_slab = tp.k_slab; a->v_slab = tp.v_slab;
    a->n_pos = aa.n_pos_dyn;
    a->eps = t.eps; a->eps_head = tp.eps; a->scale = aa.scale;
    a->n_rot = tp.n_rot;
    *m = ChainMixer{};
    m->o_q = mo.o_q;
    m->o_s = mo.o_s;
    return true;
}

void build_chains(Plan& pl, unsigned long long* tally) {
    it_hip* be = pl.be;
    be->chain_launches = be->chain_layers = 0;
    if (!be->chain_enabled || be->exact || !layer_chain_fits()) return;
    enum Kind { U_GDN, U_FFN, U_ATTN_OUT, U_ATTN };
    struct Unit {
        size_t pos;
        Kind kind;
    };
    size_t tail_pos = 0;   // position of the attention block whose in-projection is cp's tail
    // (30 KB, nearly all of it the layer array: on the heap, and only the entries in use are cleared and copied)
    std::unique_ptr<ChainP, void (*)(void*)> cp_box((ChainP*)calloc(1, sizeof(ChainP)), free);
    ChainP& cp = *cp_box;
    int cp_touched = 0;   // entries of cp.layer written since they were last cleared
    auto layer_at = [&](int k) -> ChainLayer& {
        if (k + 1 > cp_touched) cp_touched = k + 1;
        return cp.layer[k];
    };
    const size_t cp_head = offsetof(ChainP, layer);
    std::vector<Unit> units;          // the blocks folded into cp so far
    bool mixer_open = false;          // the last layer of cp has its mixer and still waits for its FFN
    int chain_rf = -1;                // the small matrices of cp's layers: Q8_0 (0) or F32 (1); -1 while no layer says
    uint64_t bytes = 0;
    auto skips_of = [&](const std::vector<Plan::Skips>& v, size_t pos, std::vector<const void*>* out) {
        for (auto& sk : v)
            if (sk.pos == pos) out->insert(out->end(), sk.bufs.begin(), sk.bufs.end());
    };
    auto emit = [&]() {
        int n = cp.n_layers;
        size_t n_units = units.size();
        if (mixer_open) {   // a mixer without its FFN stays as it was
            n--;
            n_units--;
            cp.has_tail = 0;
        }
        if (n >= 1 && be->chain_acquire()) {
            cp.n_layers = n;
            cp.ll = be->chain.ll;
            cp.epoch = be->chain.epoch;
            cp.abort_flag = be->chain.abort_flag;
            cp.tally = be->count_reads_in_fused ? tally : nullptr;
            cp.spin_limit = be->chain_spin_limit;
            cp.rf = chain_rf > 0 ? 1 : 0;
            // (on the heap, shared by the copies a std::function makes of what it holds)
            std::shared_ptr<ChainP> launch((ChainP*)malloc(sizeof(ChainP)), free);
            memcpy((void*)launch.get(), (const void*)&cp, cp_head + (size_t)n * sizeof(ChainLayer));
            auto drop_stage = [&](size_t pos, int stage) {
                auto& v = pl.at[pos];
                for (size_t k = 0; k < v.size(); k++)
                    if (v[k].stage == stage) {
                        v.erase(v.begin() + (long)k);
                        break;
                    }
            };
            for (size_t u = 0; u < n_units; u++) {
                if (units[u].kind == U_ATTN_OUT) {
                    drop_stage(units[u].pos, Plan::ST_ATTN_OUT);   // the attention kernels before it stay where they are
                } else if (units[u].kind == U_ATTN) {
                    // nothing of the block is written but the cache rows and the residual stream
                    for (auto& l : pl.at[units[u].pos]) {
                        if (l.stage == Plan::ST_ATTN_IN)
                            for (int k = 0; k < 3; k++) be->fused_elided.push_back(l.gv.m[k].out);
                        if (l.stage == Plan::ST_ATTEND) be->fused_elided.push_back(l.attn_out);
                    }
                    pl.at[units[u].pos].clear();
                    skips_of(pl.attn_skips, units[u].pos, &be->fused_elided);
                } else {
                    pl.at[units[u].pos].clear();
                    skips_of(units[u].kind == U_GDN ? pl.gdn_skips : pl.ffn_skips, units[u].pos, &be->fused_elided);
                }
            }
            if (cp.has_tail) {
                drop_stage(tail_pos, Plan::ST_ATTN_IN);
                skips_of(pl.attn_skips, tail_pos, &be->fused_elided);
            }
            pl.add(units[0].pos, it_hip::FAM_CHAIN, bytes, [=](hipStream_t s) {
                if (!layer_chain(*launch, s)) be->fail("layer chain: the persistent kernel could not be launched");
            });
            be->chain_launches++;
            be->chain_layers += (uint64_t)n;
        }
        memset((void*)&cp, 0, cp_head + (size_t)cp_touched * sizeof(ChainLayer));
        cp_touched = 0;
        units.clear();
        mixer_open = false;
        bytes = 0;
        chain_rf = -1;
    };
    for (size_t i = 0; i < pl.ops.size(); i++) {
        auto& ls = pl.at[i];
        const bool is_gdn = ls.size() == 3 && ls[0].stage == Plan::ST_GDN_IN && ls[1].stage == Plan::ST_GDN_CORE && ls[2].stage == Plan::ST_GDN_OUT;
        const bool is_ffn = ls.size() == 3 && ls[0].stage == Plan::ST_ROUTER && ls[1].stage == Plan::ST_GLU && ls[2].stage == Plan::ST_DOWN;
        const bool is_attn = ls.size() == 3 && ls[0].stage == Plan::ST_ATTN_IN && ls[1].stage == Plan::ST_ATTEND && ls[2].stage == Plan::ST_ATTN_OUT;
        bool taken = false;
        if (is_attn && be->chain_attn_enabled) {
            // the whole block as a layer of the chain (its FFN follows)
            if (mixer_open || cp.n_layers >= be->chain_max_layers) emit();
            ChainAttn a{};
            ChainMixer m{};
            if (chain_attn(pl, ls[0].gv, ls[1], ls[2].gv, &a, &m) && (cp.n_layers == 0 || cp.x == ls[0].gv.x)) {
                layer_at(cp.n_layers).has_mixer = 3;
                layer_at(cp.n_layers).a = a;
                layer_at(cp.n_layers).m = m;
                cp.x = const_cast<float*>(ls[0].gv.x);
                cp.n_layers++;
                mixer_open = true;
                units.push_back({i, U_ATTN});
                bytes += ls[0].bytes + ls[1].bytes + ls[2].bytes;
                continue;
            }
        }
        if (is_attn) {
            // its in-projection closes the chain so far, its out-projection opens the next one; the attention kernels
            // between them stay launches of their own
            const FusedGemvP in = ls[0].gv, out = ls[2].gv;
            const uint64_t in_bytes = ls[0].bytes, out_bytes = ls[2].bytes;
            ChainTail t{};
            if (cp.n_layers >= 1 && !mixer_open && cp.x == in.x && chain_attn_in(in, &t)) {
                cp.has_tail = 1;
                cp.tail = t;
                tail_pos = i;
                bytes += in_bytes;
            }
            emit();
            ChainMixer m{};
            if (chain_attn_out(out, &m)) {
                layer_at(0).has_mixer = 2;
                layer_at(0).m = m;
                cp.x = out.m[0].out;
                cp.n_layers = 1;
                mixer_open = true;
                units.push_back({i, U_ATTN_OUT});
                bytes += out_bytes;
            }
            continue;
        }
        if (is_gdn) {
            if (mixer_open || cp.n_layers >= be->chain_max_layers) emit();
            ChainMixer m{};
            int rf = 0;
            if (chain_mixer(ls[0].gv, ls[1].gc, ls[2].gv, &m, &rf) && (cp.n_layers == 0 || cp.x == ls[0].gv.x) && (chain_rf < 0 || chain_rf == rf)) {
                chain_rf = rf;
                layer_at(cp.n_layers).has_mixer = 1;
                layer_at(cp.n_layers).m = m;
                cp.x = const_cast<float*>(ls[0].gv.x);
                cp.n_layers++;
                mixer_open = true;
                units.push_back({i, U_GDN});
                bytes += ls[0].bytes + ls[1].bytes + ls[2].bytes;
                taken = true;
            }
        } else if (is_ffn) {
            ChainFfn f{};
            int sh_fmt = 0;
            if (!mixer_open && cp.n_layers >= be->chain_max_layers) emit();
            int rf = 0;
            const bool fits = chain_ffn(ls[0].gv, ls[1].mg, ls[2].md, &f, &sh_fmt, &rf) && (chain_rf < 0 || chain_rf == rf) &&
                              (cp.n_layers == 0 || (cp.x == ls[0].gv.x && (cp.sh_fmt == sh_fmt || (cp.n_layers == 1 && mixer_open))));
            if (fits) {
                chain_rf = rf;
                if (!mixer_open) {
                    layer_at(cp.n_layers).has_mixer = 0;
                    cp.n_layers++;
                }
                layer_at(cp.n_layers - 1).f = f;
                cp.sh_fmt = sh_fmt;
                cp.x = const_cast<float*>(ls[0].gv.x);
                mixer_open = false;
                units.push_back({i, U_FFN});
                bytes += ls[0].bytes + ls[1].bytes + ls[2].bytes;
                taken = true;
            }
        }
        if (taken) continue;
        // anything that runs here ends the run: other fused launches, or an op issued as it is
        if (!ls.empty() || !pl.consumed[i]) emit();
    }
    emit();
}

bool references(const Op& op, const void* a, const void* b) {
    for (const void* p : op.p)
        if (p && (p == a || p == b)) return true;
    return false;
}

}  // namespace

// ---------------------------------------------------------------------------------- batch passes
// Two runs of elementwise ops of a Gated DeltaNet layer over a batch (src/model/qwen35.rs:1255-1315) have a one-kernel
// form in fast mode:
//   CONV, GATHER q, GATHER k, GATHER v, L2 q, L2 k      -> conv_split_l2 (the conv output and the unnormed q, k are
//                                                          not written: nothing else in the loop reads them)
//   RMS_HEADS core, EW silu_mul(z, core), QUANT z        -> gated_norm_silu_q8 (core is left unnormed)
// The ops are held back as they arrive and checked link by link (an op's input must be the run's own buffer).
// The routed FFN of a short batch (2..32 tokens; src/model/qwen35.rs:1630-1700) as a run:
//   SOFTMAX, ROUTE, [QUANT x], GLU, QUANT g, EXPERTS, MATMUL shared gate, MATMUL shared up, [SCALE]*, EW silu_mul,
//   QUANT, MATMUL shared down, [SCALE], FINISH
// Where the run stands follows from what is held; an op is accepted by its kind here, and the links between the ops
// (whose output feeds whom, the shapes) are checked once the run is complete: a run that fails there is issued op by op.
namespace {
constexpr int SMALL_FFN_MAX = 32;   // tokens (measured on the 512-expert top-10 layer: 176 against 232 us at 32, 271 against 298 at 48, behind from about 56 on)
enum FfnAt { F_ROUTE = 1, F_QX_OR_GLU, F_GLU, F_QG, F_EXPERTS, F_SG, F_SU, F_SCALE_OR_SILU, F_QS, F_SD, F_SCALE_OR_FINISH, F_FINISH };
int ffn_at(const std::vector<it_hip::OpRec>& held) {   // what may come next
    int at = F_ROUTE;
    for (size_t k = 1; k < held.size(); k++) {
        const int id = held[k].id;
        switch (at) {
            case F_ROUTE: at = F_QX_OR_GLU; break;
            case F_QX_OR_GLU: at = id == OP_QUANT ? F_GLU : F_QG; break;
            case F_GLU: at = F_QG; break;
            case F_QG: at = F_EXPERTS; break;
            case F_EXPERTS: at = F_SG; break;
            case F_SG: at = F_SU; break;
            case F_SU: at = F_SCALE_OR_SILU; break;
            case F_SCALE_OR_SILU: at = id == OP_SCALE ? F_SCALE_OR_SILU : F_QS; break;
            case F_QS: at = F_SD; break;
            case F_SD: at = F_SCALE_OR_FINISH; break;
            case F_SCALE_OR_FINISH: at = F_FINISH; break;
            default: break;
        }
    }
    return at;
}
}  // namespace

int it_hip::hold_step(const OpRec& r) const {
    const size_t n = held.size();
    if (n == 0) {
        if (r.id == OP_CONV && r.i[2] >= 64 && r.i[1] % 128 == 0) return 1;
        if (r.id == OP_RMS_HEADS && r.i[0] == 128 && r.i[1] >= 256) return 1;
        if (r.id == OP_SOFTMAX && r.i[0] >= 2 && r.i[0] <= SMALL_FFN_MAX && r.i[1] >= 16 && r.i[1] <= 2048 && !expert_cold_entries && small_ffn_enabled) return 1;
        return 0;
    }
    const OpRec& h0 = held[0];
    if (h0.id == OP_SOFTMAX) {
        switch (ffn_at(held)) {
            case F_ROUTE: return r.id == OP_ROUTE && r.p[0] == h0.p[0] && r.i[0] == h0.i[0] && r.i[1] == h0.i[1] && r.i[2] <= 16 ? 1 : 0;
            case F_QX_OR_GLU: return r.id == OP_QUANT || (r.id == OP_GLU && !r.i[8]) ? 1 : 0;
            case F_GLU: return r.id == OP_GLU && !r.i[8] ? 1 : 0;
            case F_QG: return r.id == OP_QUANT ? 1 : 0;
            case F_EXPERTS: return r.id == OP_EXPERTS && !r.i[8] ? 1 : 0;
            case F_SG:
            case F_SU:
            case F_SD: return r.id == OP_MATMUL ? 1 : 0;
            case F_SCALE_OR_SILU: return r.id == OP_SCALE || (r.id == OP_EW && r.i[0] == 0) ? 1 : 0;
            case F_QS: return r.id == OP_QUANT ? 1 : 0;
            case F_SCALE_OR_FINISH: return r.id == OP_SCALE ? 1 : r.id == OP_FINISH ? 2 : 0;
            case F_FINISH: return r.id == OP_FINISH ? 2 : 0;
        }
        return 0;
    }
    if (h0.id == OP_CONV) {
        const int64_t nc = h0.i[1], nt = h0.i[2];
        if (n <= 3) {
            if (r.id != OP_GATHER || r.p[0] != h0.p[3] || r.i[1] != nc) return 0;
            const int64_t kdim = n == 1 ? r.i[0] : held[1].i[0];
            if (kdim <= 0 || kdim % 128 || 2 * kdim >= nc) return 0;
            const int64_t chunk = n == 3 ? nc - 2 * kdim : kdim, off = (int64_t)(n - 1) * kdim;
            return r.i[0] == chunk && r.i[2] == off && r.i[3] == nt * chunk ? 1 : 0;
        }
        const OpRec& g = held[n - 3];   // n = 4: the q part, n = 5: the k part
        if (r.id != OP_L2 || r.p[0] != g.p[1] || r.i[0] != 128 || r.i[1] * 128 != nt * held[1].i[0]) return 0;
        if (n == 5 && r.f[0] != held[4].f[0]) return 0;
        return n == 5 ? 2 : 1;
    }
    if (h0.id == OP_RMS_HEADS) {
        if (n == 1) return r.id == OP_EW && r.i[0] == 0 && r.p[1] == h0.p[0] && r.i[1] == h0.i[1] * 128 ? 1 : 0;
        if (n == 2) return r.id == OP_QUANT && r.p[0] == held[1].p[0] && r.i[0] == held[1].i[1] ? 2 : 0;
    }
    return 0;
}

void it_hip::release_held() {
    auto ops = std::move(held);
    held.clear();
    for (auto& op : ops) {
        Span sp(this, op.fam, op.bytes);
        op.run(stream);
    }
    check(hipGetLastError(), "kernel launch");
}

// The complete FFN run of a short batch as two launches: gate / up with the route inside (every block ranks its
// token's logits; grid row = token), then down + combine.  False, with nothing launched, when a link or a shape is not
// what the kernels take.
bool it_hip::small_ffn(const std::vector<OpRec>& h) {
    size_t k = 0;
    auto take = [&](int id) -> const OpRec* { return k < h.size() && h[k].id == id ? &h[k++] : nullptr; };
    const OpRec *sm = take(OP_SOFTMAX), *rt = take(OP_ROUTE), *q1 = take(OP_QUANT), *glu = take(OP_GLU), *q2 = take(OP_QUANT);
    const OpRec *ex = take(OP_EXPERTS), *sgm = take(OP_MATMUL), *sum_ = take(OP_MATMUL);
    if (!sm || !rt || !glu || !q2 || !ex || !sgm || !sum_) return false;
    float sh_scale[3] = {1.0f, 1.0f, 1.0f};   // gate, up, down
    bool has_up = false, has_gate = false;
    while (k < h.size() && h[k].id == OP_SCALE) {   // the up product is scaled first, then the gate product
        const OpRec& sc = h[k];
        if (!has_up && !has_gate && sc.p[0] == sum_->p[5] && sc.i[0] == sum_->i[2] * sum_->i[3]) {
            sh_scale[1] = sc.f[0];
            has_up = true;
        } else if (!has_gate && sc.p[0] == sgm->p[5] && sc.i[0] == sgm->i[2] * sgm->i[3]) {
            sh_scale[0] = sc.f[0];
            has_gate = true;
        } else {
            return false;
        }
        k++;
    }
    const OpRec *sil = take(OP_EW), *q3 = take(OP_QUANT), *sdm = take(OP_MATMUL);
    if (!sil || !q3 || !sdm) return false;
    if (k < h.size() && h[k].id == OP_SCALE) {
        const OpRec& sc = h[k];
        if (sc.p[0] != sdm->p[5] || sc.i[0] != sdm->i[2] * sdm->i[3]) return false;
        sh_scale[2] = sc.f[0];
        k++;
    }
    const OpRec* fin = take(OP_FINISH);
    if (!fin || k != h.size()) return false;

    const int64_t nt = sm->i[0], ne = sm->i[1], nu = rt->i[2];
    const int64_t nd = glu->i[1], ff = glu->i[2], sff = sgm->i[2];
    const void* router = sm->p[0];
    const void* x = sgm->p[2];   // the f32 activation: the shared expert's products read the same rows as the routed ones
    if (nt < 2 || nt > SMALL_FFN_MAX || nu < 1 || nu > 16 || ne < nu) return false;
    if (q1 && (q1->p[0] != x || q1->i[0] != nt * nd)) return false;
    if (glu->p[6] != rt->p[1] || glu->p[7] != sgm->p[3] || glu->p[8] != sgm->p[4] || glu->i[3] != nt * nu || glu->i[4] != nu ||
        glu->i[5] != 1 || !quantized_fmt(glu->i[0]))
        return false;
    const void* g_all = glu->p[9];
    if (q2->p[0] != g_all || q2->i[0] != nt * nu * ff) return false;
    if (ex->p[3] != rt->p[1] || ex->p[4] != q2->p[1] || ex->p[5] != q2->p[2] || ex->i[1] != ff || ex->i[2] != nd || ex->i[3] != nt * nu ||
        ex->i[4] != nu || ex->i[5] != 0 || !quantized_fmt(ex->i[0]))
        return false;
    auto reads_x = [&](const OpRec& m) {
        return m.p[2] == x && m.p[3] == sgm->p[3] && m.p[4] == sgm->p[4] && m.i[1] == nd && m.i[3] == nt && quantized_fmt(m.i[0]);
    };
    if (!reads_x(*sgm) || !reads_x(*sum_) || sum_->i[2] != sff || sum_->i[0] != sgm->i[0]) return false;
    const void* e_gate = sgm->p[5];
    if (sil->i[0] != 0 || sil->p[0] != e_gate || sil->p[1] != sum_->p[5] || sil->i[1] != nt * sff) return false;
    if (q3->p[0] != e_gate || q3->i[0] != nt * sff) return false;
    if (sdm->p[2] != e_gate || sdm->p[3] != q3->p[1] || sdm->p[4] != q3->p[2] || sdm->i[1] != sff || sdm->i[2] != nd || sdm->i[3] != nt ||
        !quantized_fmt(sdm->i[0]))
        return false;
    if (fin->p[1] != ex->p[6] || fin->p[2] != rt->p[2] || fin->p[3] != sdm->p[5] || fin->i[1] != nd || fin->i[2] != nt || fin->i[3] != nu)
        return false;

    MoeGluP g{};
    g.x = (const float*)x;
    g.gq = (const uint8_t*)glu->p[0]; g.gs = (const uint8_t*)glu->p[1]; g.uq = (const uint8_t*)glu->p[2]; g.us = (const uint8_t*)glu->p[3];
    g.gscale2 = (const float*)glu->p[4]; g.uscale2 = (const float*)glu->p[5];
    g.q_stride = glu->i[6]; g.s_stride = glu->i[7];
    g.fmt = (int)glu->i[0]; g.n_in = (int)nd; g.n_out = (int)ff; g.n_expert = (int)ne; g.n_used = (int)nu;
    g.sh_gq = (const uint8_t*)sgm->p[0]; g.sh_gs = (const uint8_t*)sgm->p[1]; g.sh_uq = (const uint8_t*)sum_->p[0]; g.sh_us = (const uint8_t*)sum_->p[1];
    g.sh_fmt = (int)sgm->i[0]; g.sh_n_out = (int)sff;
    g.sh_gscale = sh_scale[0]; g.sh_uscale = sh_scale[1];
    g.out = (float*)g_all; g.sh_out = (float*)e_gate;
    g.logits = (const float*)router;
    g.route_ids_out = (int32_t*)rt->p[1]; g.route_w_out = (float*)rt->p[2];
    g.n_tok = (int)nt;
    MoeDownP d{};
    d.g_all = (const float*)g_all; d.g_shared = (const float*)e_gate;
    d.q = (const uint8_t*)ex->p[0]; d.s = (const uint8_t*)ex->p[1]; d.scale2 = (const float*)ex->p[2];
    d.q_stride = ex->i[6]; d.s_stride = ex->i[7];
    d.fmt = (int)ex->i[0]; d.n_in = (int)ff; d.n_out = (int)nd; d.n_used = (int)nu;
    d.sh_q = (const uint8_t*)sdm->p[0]; d.sh_s = (const uint8_t*)sdm->p[1]; d.sh_fmt = (int)sdm->i[0]; d.sh_n_in = (int)sff;
    d.sh_dscale = sh_scale[2];
    d.route_ids = (const int32_t*)rt->p[1]; d.route_w = (const float*)rt->p[2];
    d.logit = (const float*)fin->p[4] + fin->i[4];
    d.y = (float*)fin->p[0] + fin->i[0];
    d.x = d.y;
    d.n_tok = (int)nt;
    if (count_reads_in_fused) {
        d.counts_gate = (uint32_t*)glu->p[10];
        d.counts_up = (uint32_t*)glu->p[11];
        d.counts_down = (uint32_t*)ex->p[7];
        d.tally = expert_tally;
    }
    if (!moe_glu_fast(g, stream, true) || !moe_down_fast(d, stream, true)) return false;
    moe_glu_fast(g, stream);
    moe_down_fast(d, stream);
    // what the two launches do not write: the probabilities (the router buffer keeps its logits), the shared expert's
    // up product, the pairs' down products, and every quantized form of the run
    mark_elided({router, sum_->p[5], ex->p[6], sdm->p[5]});
    for (const OpRec* q : {q1, q2, q3})
        if (q)
            if (Act* a = act_by_dev(q->p[0])) a->q_valid = false;
    return true;
}

void it_hip::finish_held() {
    bool done = false;
    uint64_t bytes = 0;
    for (auto& op : held) bytes += op.bytes;
    if (held[0].id == OP_SOFTMAX) {
        {
            Span sp(this, FAM_MOE_GLU, bytes);
            done = small_ffn(held);
        }
        if (done) {
            held.clear();
            check(hipGetLastError(), "kernel launch");
        } else {
            release_held();
        }
        return;
    }
    {
        Span sp(this, held[0].fam, bytes);
        if (held[0].id == OP_CONV && held.size() == 6) {
            const OpRec &c = held[0], &gq = held[1], &gk = held[2], &gv = held[3], &l = held[4];
            done = conv_split_l2((float*)c.p[0], (const float*)c.p[1], (const float*)c.p[2], (int)c.i[0], (int)c.i[1], (int)c.i[2],
                                 (float*)gq.p[1], (float*)gk.p[1], (float*)gv.p[1], (int)gq.i[0], l.f[0], stream);
        } else if (held[0].id == OP_RMS_HEADS && held.size() == 3) {
            const OpRec &n = held[0], &e = held[1], &q = held[2];
            done = gated_norm_silu_q8((const float*)n.p[0], (const float*)n.p[1], (float*)e.p[0], (float*)q.p[1], (int8_t*)q.p[2],
                                      n.i[1], n.f[0], stream);
        }
    }
    if (done) {
        // the conv output (first run) and the normed read-out (second run: `core` keeps the delta rule's raw values) are
        // not what their ops would have left there
        mark_elided({held[0].id == OP_CONV ? held[0].p[3] : held[0].p[0]});
        held.clear();
        check(hipGetLastError(), "kernel launch");
    } else {
        release_held();
    }
}

void it_hip::run_fused(std::vector<OpRec>& ops) {
    Plan pl(this, ops);
    fused_attn_slots.clear();
    fused_elided.clear();
    chain_launches = chain_layers = 0;
    if (fuse_enabled) {
        for (size_t i = 0; i < ops.size(); i++) {
            if (pl.consumed[i]) continue;
            if (match_gdn(pl, i, exact)) continue;
            if (match_attn(pl, i, exact)) continue;
            if (match_ffn(pl, i, exact, route_counter, expert_tally)) continue;
            if (match_final(pl, i, exact)) continue;
            if (match_norm_matmuls(pl, i, exact)) continue;
            if (match_matmul_residual(pl, i, exact)) continue;
        }
        // a dropped quantization whose output an unfused op still reads is put back; a deferred pass is issued in
        // pieces, and a later piece (the expert products after the picks were read back) may read what this one
        // quantized, so there every quantization is kept
        for (size_t i = 0; i < ops.size(); i++) {
            if (!pl.consumed[i] || ops[i].id != OP_QUANT) continue;
            if (mode == Mode::Deferred && expert_cold_entries) {
                pl.consumed[i] = 0;
                continue;
            }
            for (size_t k = i + 1; k < ops.size(); k++) {
                if (pl.consumed[k]) continue;
                if (ops[k].id == OP_QUANT && ops[k].p[1] == ops[i].p[1]) break;  // re-quantized later
                if (references(ops[k], ops[i].p[1], ops[i].p[2])) {
                    pl.consumed[i] = 0;
                    break;
                }
            }
        }
    }
    if (fuse_enabled && !expert_cold_entries) build_chains(pl, expert_tally);
    uint64_t n = 0;
    for (size_t i = 0; i < ops.size(); i++) {
        for (auto& l : pl.at[i]) {
            Span sp(this, l.fam, l.bytes);
            l.fn(stream);
            n++;
        }
        if (!pl.consumed[i]) {
            Span sp(this, FAM_OTHER, 0);
            ops[i].run(stream);
            n++;
        }
    }
    fused_launches = n;
}
