"""Device time of the single-op configurations, measured through the C ABI one launch at a time.

Three workloads beside the whole-model run, each at the shapes the baseline names:

* the routed expert FFN (512 NVFP4 experts, hidden 2048, inter 512, top-10 + one shared expert) for
  1 / 8 / 64 / 512 tokens: softmax, top-k, gate/up with silu-mul, down, the shared expert, the combine;
* GQA decode attention (16 query heads, 2 KV heads, head_dim 256, f16 K and V) at contexts of
  1,024 / 8,192 / 32,000 positions;
* the Gated DeltaNet mixer core (16 key / 32 value heads, dk = dv = 128): causal conv (kernel 4) and the
  delta rule, one decode step and a 5,700-token batch.

Every figure is the sum of the HIP-event durations of the launches of one call sequence (the backend's
profile mode: an event before and after each launch on the launch stream), averaged over repetitions
that rotate over several copies of the large operands so that a repetition does not find them in the
caches.  Algorithmic bytes are the operands that must move once: the distinct experts a batch touches
(counted from the routing actually drawn), K and V up to the context, the recurrent state read and
written.  Weights and slabs are uploaded before the timed launches; uploads are not in the figures.
"""
from __future__ import annotations

import numpy as np

HBM_PEAK_GBS = 8000.0


def _bf16(x):
    u = x.astype(np.float32).view(np.uint32).astype(np.uint64)
    u = ((u + 0x7fff + ((u >> 16) & 1)) >> 16) << 16
    return u.astype(np.uint32).view(np.float32)


_POOL = {}


def _nvfp4(r, n_rows, n_in):
    """Rows of NVFP4 blocks (4 UE4M3 scale bytes + 32 nibble bytes per 64 elements): nibbles uniform over
    the 16 codes, scales the nearest code to |N(0,1)| (never 0x00 or 0x7f).  Blocks are drawn with
    replacement from a pool of 2^18 blocks built that way (a 300 MB tensor in a second instead of six)."""
    if "blocks" not in _POOL:
        n_pool = 1 << 18
        pool = np.empty((n_pool, 36), np.uint8)
        pool[:, 4:] = r.integers(0, 256, (n_pool, 32), dtype=np.uint8)
        codes = np.arange(1, 0x7f)
        exp = (codes >> 3) & 0xf
        man = (codes & 7).astype(np.float64)
        vals = np.where(exp == 0, man * 2.0 ** -9, (1 + man / 8) * 2.0 ** (exp - 7.0))  # ascending in the code
        mid = (vals[1:] + vals[:-1]) / 2
        mags = np.abs(r.standard_normal((n_pool, 4)))
        pool[:, :4] = codes[np.searchsorted(mid, mags)].astype(np.uint8)
        _POOL["blocks"] = pool
    pool = _POOL["blocks"]
    n_blocks = n_rows * n_in // 64
    return pool[r.integers(0, pool.shape[0], n_blocks)].reshape(-1)


def _timed(be, fn, reps):
    """Sum of the event-timed launch durations of fn(i), averaged over reps calls: (ms per call, launches per call)."""
    be.profile_begin()
    for i in range(reps):
        fn(i)
    rows = be.profile_end()
    err = be.take_error()
    if err:
        raise RuntimeError(f"device error in a single-op run: {err}")
    return sum(r["ms"] for r in rows) / reps, sum(r["launches"] for r in rows) / reps, rows


def _line(bytes_, ms, launches, **extra):
    gbs = bytes_ / 1e9 / (ms / 1e3)
    d = dict(algorithmic_mb=round(bytes_ / 1e6, 2), us=round(ms * 1e3, 1), ops=round(launches, 1),
             gb_s=round(gbs, 1), hbm_frac=round(gbs / HBM_PEAK_GBS, 4))
    d.update(extra)
    return d


def expert_ffn(ih, be, seed=0, tokens=(1, 2, 8, 16, 64, 512), n_expert=512, n_used=10, nd=2048, ff=512):
    r = np.random.default_rng(seed)
    gate, up, down = _nvfp4(r, n_expert * ff, nd), _nvfp4(r, n_expert * ff, nd), _nvfp4(r, n_expert * nd, ff)
    sh_gate, sh_up, sh_down = _nvfp4(r, ff, nd), _nvfp4(r, ff, nd), _nvfp4(r, nd, ff)
    scales = [(r.random(n_expert).astype(np.float32) * 0.01 + 0.002) for _ in range(3)]
    eg = ih.experts(gate, ih.NVFP4, nd, ff, n_expert, scales[0])
    eu = ih.experts(up, ih.NVFP4, nd, ff, n_expert, scales[1])
    ed = ih.experts(down, ih.NVFP4, ff, nd, n_expert, scales[2])
    wg, wu, wd = ih.weights(sh_gate, ih.NVFP4, nd, ff), ih.weights(sh_up, ih.NVFP4, nd, ff), ih.weights(sh_down, ih.NVFP4, ff, nd)
    expert_bytes = 3 * ff * nd // 64 * 36
    out = {}
    for T in tokens:
        reps = 12 if T <= 64 else 6
        # a fresh routing and activation per repetition: a small batch must not find its ten experts cached
        # (one more set for the untimed first call)
        xs = [_bf16(r.standard_normal(T * nd).astype(np.float32)) for _ in range(reps + 1)]
        logits = [r.standard_normal((T, n_expert)).astype(np.float32) for _ in range(reps + 1)]
        distinct = [len(np.unique(np.argsort(-l, axis=1)[:, :n_used])) for l in logits[:reps]]
        pairs = T * n_used
        probs = [l.reshape(-1).copy() for l in logits]
        g_all, u_all = np.zeros(pairs * ff, np.float32), np.zeros(pairs * ff, np.float32)
        o_all = np.zeros(pairs * nd, np.float32)
        s_gate, s_up, s_out = np.zeros(T * ff, np.float32), np.zeros(T * ff, np.float32), np.zeros(T * nd, np.float32)
        y, sh_logit = np.zeros(T * nd, np.float32), np.zeros(T, np.float32)
        held = xs + probs + [g_all, u_all, o_all, s_gate, s_up, s_out, y, sh_logit]
        for a in held:
            be.host_wrote(a)  # a fresh buffer may sit at an address the backend has seen before

        def once(i):
            # inside a pass of T tokens, as the model loop issues it: a short batch (2..32 tokens) is then held back and
            # issued as two launches (gate / up with the route inside, down + combine)
            be.begin_pass(T)
            be.softmax(probs[i], n_expert)
            route = be.route(probs[i], n_expert, n_used)
            be.moe_glu(eg, eu, route, xs[i], g_all, u_all)
            be.matmul_experts(ed, route, g_all, o_all)
            be.matmul(wg, xs[i], s_gate)
            be.matmul(wu, xs[i], s_up)
            be.silu_mul(s_gate, s_up)
            be.matmul(wd, s_gate, s_out)
            be.moe_finish(y, 0, nd, o_all, route, s_out, sh_logit, 0)
            be.end_pass()

        once(reps)  # weights become resident, buffers are sized
        # the inputs of the timed repetitions resident in device memory before the clock starts (each goes through the
        # backend once: its mirrors exist and are current, so no pass stops to allocate or upload)
        for i in range(reps):
            be.matmul(wg, xs[i], s_gate)    # (a product through the backend: the quantized form's buffers exist as well)
            be.scale(probs[i], 1.0)
        once(reps)  # once more with every buffer in place: the launches of the timed passes have all run before
        be.sync()
        ms, launches, _ = _timed(be, once, reps)
        bytes_ = (np.mean(distinct) + 1) * expert_bytes + 2 * T * nd * 4
        out[str(T)] = _line(bytes_, ms, launches, experts_touched=round(float(np.mean(distinct)), 1))
        for a in held:
            be.release(a)
    be.drop_mirrors()
    return out


def expert_ffn_fused_decode(ih, seed=0, n_expert=512, n_used=10, nd=2048, ff=512, reps=16):
    """Config 2's one-token point through the path a decode pass takes: the routed FFN issued as the model loop issues
    it (norm, router + shared-gate logit, softmax, top-k, experts' gate/up, down, shared expert, combine, residual)
    inside a single-token pass, which the backend fuses into three launches (router GEMV; gate/up with the in-kernel
    top-10; down + combine + residual) and replays as a graph.  Timed like the other points: the fused launches
    issued one by one between HIP events.  Bytes: ten routed experts + the shared one + the router matrix."""
    from inferred_hip import F32  # noqa: F401  (the package is the caller's)
    r = np.random.default_rng(seed + 3)
    be = ih.Hip(exact=False)
    try:
        def q8(n_out, n_in, gain):
            w = (r.standard_normal((n_out, n_in)) * (gain / np.sqrt(n_in))).astype(np.float32).reshape(-1, 32)
            d = np.abs(w).max(1) / 127.0
            q = np.where(d[:, None] > 0, np.rint(w / np.maximum(d, 1e-30)[:, None]), 0).astype(np.int8)
            blk = np.zeros((w.shape[0], 34), np.uint8)
            blk[:, :2] = d.astype(np.float16).view(np.uint8).reshape(-1, 2)
            blk[:, 2:] = q.view(np.uint8)
            return blk.reshape(-1)
        gate, up, down = _nvfp4(r, n_expert * ff, nd), _nvfp4(r, n_expert * ff, nd), _nvfp4(r, n_expert * nd, ff)
        scales = [(r.random(n_expert).astype(np.float32) * 0.01 + 0.002) for _ in range(3)]
        eg = ih.experts(gate, ih.NVFP4, nd, ff, n_expert, scales[0])
        eu = ih.experts(up, ih.NVFP4, nd, ff, n_expert, scales[1])
        ed = ih.experts(down, ih.NVFP4, ff, nd, n_expert, scales[2])
        router_b, logit_b = q8(n_expert, nd, 3.0), q8(1, nd, 1.0)
        sg_b, su_b, sd_b = q8(ff, nd, 1.5), q8(ff, nd, 1.5), q8(nd, ff, 2.0)
        wr, wl = ih.weights(router_b, ih.Q8_0, nd, n_expert), ih.weights(logit_b, ih.Q8_0, nd, 1)
        wg, wu, wd = ih.weights(sg_b, ih.Q8_0, nd, ff), ih.weights(su_b, ih.Q8_0, nd, ff), ih.weights(sd_b, ih.Q8_0, ff, nd)
        norm_w = np.ones(nd, np.float32)
        z = lambda n: np.zeros(n, np.float32)
        x, normed, e_in, router, logit = z(nd), z(nd), z(nd), z(n_expert), z(1)
        g_all, u_all, o_all, e_gate, e_up, e_out, ffn = z(n_used * ff), z(n_used * ff), z(n_used * nd), z(ff), z(ff), z(nd), z(nd)
        xs = [r.standard_normal(nd).astype(np.float32) for _ in range(reps + 3)]

        def once(i):
            x[:] = xs[i]
            be.begin_pass(1); be.host_wrote(x)
            be.rms_norm(x, norm_w, 1e-6, normed)
            be.gather_chunks(normed, nd, nd, 0, e_in)
            be.matmul_pair(wr, wl, e_in, router, logit)
            be.softmax(router, n_expert)
            route = be.route(router, n_expert, n_used)
            be.moe_glu(eg, eu, route, e_in, g_all, u_all)
            be.matmul_experts(ed, route, g_all, o_all)
            be.matmul(wg, e_in, e_gate); be.matmul(wu, e_in, e_up)
            be.silu_mul(e_gate, e_up)
            be.matmul(wd, e_gate, e_out)
            be.moe_finish(ffn, 0, nd, o_all, route, e_out, logit, 0)
            be.add_assign(x, ffn)
            be.end_pass()

        for i in range(3):
            once(reps + i)       # eager, eager, captured
        be.sync()
        st = be.graph_stats()
        ms, launches, _ = _timed(be, once, reps)
        expert_bytes = 3 * ff * nd // 64 * 36
        bytes_ = n_used * expert_bytes + 3 * ff * nd // 32 * 34 + (n_expert + 1) * nd // 32 * 34 + 2 * nd * 4
        return _line(bytes_, ms, launches, fused_launches=st["graph_kernels"], experts_touched=n_used,
                     note="the decode path: router GEMV, gate/up with the in-kernel top-10, down + combine; "
                          "Q8_0 router and shared expert as in the headline model")
    finally:
        be.close()


def attention_decode(ih, be, seed=0, contexts=(1024, 8192, 32000), n_head=16, n_head_kv=2, hd=256):
    r = np.random.default_rng(seed + 1)
    kv_dim = n_head_kv * hd
    out = {}
    for ctx in contexts:
        slabs = max(4, min(16, (400 << 20) // (ctx * kv_dim * 4)))  # beyond the 256 MB last-level cache, or 16 copies
        reps = 2 * slabs
        ks = [r.standard_normal(ctx * kv_dim).astype(np.float16).view(np.uint16) for _ in range(slabs)]
        vs = [r.standard_normal(ctx * kv_dim).astype(np.float16).view(np.uint16) for _ in range(slabs)]
        q = _bf16(r.standard_normal(n_head * hd).astype(np.float32))
        o = np.zeros(n_head * hd, np.float32)
        scale = float(1.0 / np.sqrt(np.float32(hd)))

        def once(i):
            be.attend(q, ks[i % slabs], vs[i % slabs], kv_dim, ctx, hd, n_head, n_head_kv, scale, o)

        for i in range(slabs):
            once(i)  # slabs become resident
        be.sync()
        ms, launches, _ = _timed(be, once, reps)
        out[str(ctx)] = _line(2 * ctx * kv_dim * 2, ms, launches, kv_copies=slabs)
        be.drop_mirrors()
    return out


def delta_net(ih, be, seed=0, n_k=16, n_v=32, dk=128, dv=128, kernel=4, prefill=5700):
    r = np.random.default_rng(seed + 2)
    kdim, vdim = n_k * dk, n_v * dv
    cdim = 2 * kdim + vdim

    def l2n(x):
        x = x.reshape(-1, dk)
        return _bf16((x / np.linalg.norm(x, axis=1, keepdims=True)).astype(np.float32).reshape(-1))

    ssm_a, dt = -np.ones(n_v, np.float32), np.zeros(n_v, np.float32)
    conv_w = r.standard_normal(cdim * kernel).astype(np.float32) * 0.3
    out = {}
    for name, T, copies in (("decode", 1, 8), (f"prefill_{prefill}", prefill, 2)):
        reps = 2 * copies if T == 1 else 4
        states = [(r.standard_normal(n_v * dk * dv) * 0.1).astype(np.float32) for _ in range(copies)]
        cstates = [r.standard_normal(cdim * (kernel - 1)).astype(np.float32) for _ in range(copies)]
        qkv = _bf16(r.standard_normal(T * cdim).astype(np.float32))
        conv_out = np.zeros(T * cdim, np.float32)
        q, k = l2n(r.standard_normal(T * kdim)), l2n(r.standard_normal(T * kdim))
        v = _bf16(r.standard_normal(T * vdim).astype(np.float32))
        alpha, beta = r.standard_normal(T * n_v).astype(np.float32), r.standard_normal(T * n_v).astype(np.float32)
        o = np.zeros(T * vdim, np.float32)

        def conv(i):
            be.ssm_conv(cstates[i % copies], qkv, conv_w, kernel, conv_out)

        def rule(i):
            be.delta_rule(q, k, v, alpha, beta, ssm_a, dt, dk, dv, n_k, n_v, states[i % copies], o)

        for i in range(copies):
            conv(i); rule(i)
        be.sync()
        ms_c, l_c, _ = _timed(be, conv, reps)
        ms_r, l_r, _ = _timed(be, rule, reps)
        state_bytes = 2 * n_v * dk * dv * 4
        out[name] = {
            "ssm_conv": _line(2 * T * cdim * 4 + 2 * cdim * (kernel - 1) * 4 + cdim * kernel * 4, ms_c, l_c),
            "delta_rule": _line(state_bytes + T * (2 * kdim + 2 * vdim + 2 * n_v) * 4, ms_r, l_r),
        }
        if T > 1:
            chunk_macs = 3 * 64 * dk * dv + 64 * 64 * dv + 64 * 64 * dk
            flops = 2 * chunk_macs * n_v * (T / 64)
            out[name]["delta_rule"]["fp32_mfma_tflops"] = round(flops / (ms_r / 1e3) / 1e12, 1)
        be.drop_mirrors()
    return out


def run(ih, seed=0, exact=False, ffn_tokens=None):
    """All three workloads on a backend of their own (no pass recording: every op launches as it is called).
    ffn_tokens: only the expert FFN, at these token counts (for a kernel trace of one point of the sweep)."""
    be = ih.Hip(exact=exact, graph=False, fuse=False)
    # the expert FFN runs inside passes of T tokens on a backend that may hold a short batch's ops back (a single-token
    # pass still launches op by op: no graph)
    be_ffn = ih.Hip(exact=exact, graph=False)
    try:
        if ffn_tokens:
            return {"expert_ffn_nvfp4_512x10": expert_ffn(ih, be_ffn, seed, tokens=tuple(ffn_tokens))}
        return {"timing": "sum of per-launch HIP-event durations of one call sequence (each launch carries about "
                          "2 us of event overhead); operands rotated over copies so that they come from HBM",
                "expert_ffn_nvfp4_512x10": expert_ffn(ih, be_ffn, seed),
                "expert_ffn_nvfp4_512x10_one_token_fused": None if exact else expert_ffn_fused_decode(ih, seed),
                "attention_decode_16q_2kv_hd256": attention_decode(ih, be, seed),
                "gated_delta_net_16k_32v_128": delta_net(ih, be, seed)}
    finally:
        be.close()
        be_ffn.close()
