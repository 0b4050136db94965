"""The fused fast-mode decode kernels (what bench.py's decode leg runs) against the CPU oracle, block by block.

A single-token pass of a qwen35moe layer is issued op by op through the C ABI, exactly as the host loop issues
it (/root/reference src/model/qwen35.rs:1138-1223 attention, :1232-1328 gated delta net, :1587-1700 routed FFN,
:1113-1121 the output head).  The backend runs the first two passes eagerly (unfused fast kernels), captures the
third into a HIP graph of FUSED launches and replays that graph afterwards, so five passes exercise both forms;
every pass is compared with the same op sequence composed from the oracle's ops on identical inputs at config
5's layer shapes (hidden 2048; GDN 16 key / 32 value heads of 128; attention 16 query / 2 kv heads of 256 at a
context of 5,800; 512 NVFP4 experts top-10 of 512 rows + a Q8_0 shared expert; vocabulary 151,936).

Compared per pass: the block's contribution to the residual stream (x_out - x_in; the weights are drawn so that
it is O(1)), the new recurrent state and conv window, and the new K / V rows.  Tolerance: rel/abs 1e-3 per entry, the absolute part scaled down when
the whole vector is small (fast mode sums in wave order and takes exp on the transcendental unit;
the integer block dots are the oracle's).
"""
import numpy as np
import pytest

from util import close, f16_bits, q8_0_weights, rng, worst

pytestmark = pytest.mark.gpu

ND, EPS = 2048, 1e-6
PASSES = 5          # 2 eager + 1 captured + 2 replayed


def nvfp4_rows(r, n_out, n_in):
    """NVFP4 rows with every nibble code and scale codes of 0.125 .. 0.94 (exponent fields 5..7), drawn directly
    (util.nvfp4_weights ranks |N(0,1)| against all codes, too slow for 512 experts)."""
    n_blocks = n_out * n_in // 64
    out = np.zeros((n_blocks, 36), np.uint8)
    out[:, 4:] = r.integers(0, 256, (n_blocks, 32), dtype=np.uint8)
    out[:, :4] = r.integers(0x28, 0x40, (n_blocks, 4), dtype=np.uint8)
    return out.reshape(-1)


class Both:
    """One set of host buffers per backend and the two libraries' argument structs over the same weight bytes."""

    def __init__(self, hip, orc):
        import inferred_hip as ih
        from oracle import binding as ob
        self.hip, self.orc, self.ih, self.ob = hip, orc, ih, ob
        self.keep = []

    def w(self, data, ty, n_in, n_out):
        self.keep.append(data)
        return self.ih.weights(data, ty, n_in, n_out), self.ob.weights(data, ty, n_in, n_out)

    def e(self, data, ty, n_in, n_out, n_expert, scale):
        self.keep += [data, scale]
        return (self.ih.experts(data, ty, n_in, n_out, n_expert, scale),
                self.ob.experts(data, ty, n_in, n_out, n_expert, scale))

    def q8(self, r, n_out, n_in, gain=1.0):
        return self.w(q8_0_weights(self.orc, r, n_out, n_in, std=gain / np.sqrt(n_in)), self.ih.Q8_0, n_in, n_out)


def bufs(**sizes):
    """Two identical sets of zeroed f32 buffers: [0] for the HIP backend (stable addresses), [1] for the oracle."""
    return [{k: np.zeros(n, np.float32) for k, n in sizes.items()} for _ in range(2)]


@pytest.fixture()
def pair():
    import inferred_hip as ih
    from oracle import binding as ob
    hip = ih.Hip(exact=False, chain=False)      # the per-stage fused kernels; tests/test_gpu_chain.py covers their chain form
    both = Both(hip, ob.Oracle(threads=8))
    yield both
    err = hip.take_error()
    hip.close()
    assert err is None, err


def fused_graph_ran(hip, kernels):
    g = hip.graph_stats()
    assert g["captures"] == 1 and g["aborts"] == 0, g
    assert g["replays"] == PASSES - 2, g
    assert g["graph_kernels"] == kernels, g       # the block's seam ops became this many fused launches


# --------------------------------------------------------------------------------------------- gated delta net
def test_gdn_block(pair):
    hip, orc = pair.hip, pair.orc
    NK, NV, DK = 16, 32, 128
    kdim, vdim = NK * DK, NV * DK
    cdim = 2 * kdim + vdim
    r = rng(101)
    wqkv, wz = pair.q8(r, cdim, ND, 2.0), pair.q8(r, vdim, ND, 2.0)
    wa, wb, wo = pair.q8(r, NV, ND, 2.0), pair.q8(r, NV, ND, 2.0), pair.q8(r, ND, vdim, 4.0)
    norm_w = (0.5 + r.random(ND)).astype(np.float32); ssm_norm = (0.5 + r.random(DK)).astype(np.float32)
    conv_w = (r.standard_normal(cdim * 4) * 0.5).astype(np.float32)
    ssm_a = (-np.exp(r.standard_normal(NV) * 0.5)).astype(np.float32); dt = (r.standard_normal(NV) * 0.5).astype(np.float32)
    B = bufs(x=ND, normed=ND, qkv=cdim, z=vdim, alpha=NV, beta=NV, convo=cdim, q=kdim, k=kdim, v=vdim, core=vdim,
             mixed=ND, conv_state=cdim * 3, ssm=NV * DK * DK)
    for b in B:
        b["conv_state"][:] = (rng(5).standard_normal(cdim * 3) * 0.5).astype(np.float32)
        b["ssm"][:] = (rng(6).standard_normal(NV * DK * DK) * 0.05).astype(np.float32)

    def block(ops, i, b):
        W = lambda t: t[i]
        ops.rms_norm(b["x"], norm_w, EPS, b["normed"])
        ops.matmul(W(wqkv), b["normed"], b["qkv"]); ops.matmul(W(wz), b["normed"], b["z"])
        ops.matmul_pair(W(wa), W(wb), b["normed"], b["alpha"], b["beta"])
        ops.ssm_conv(b["conv_state"], b["qkv"], conv_w, 4, b["convo"])
        ops.gather_chunks(b["convo"], kdim, cdim, 0, b["q"]); ops.gather_chunks(b["convo"], kdim, cdim, kdim, b["k"])
        ops.gather_chunks(b["convo"], vdim, cdim, 2 * kdim, b["v"])
        ops.l2_norm_heads(b["q"], DK, EPS); ops.l2_norm_heads(b["k"], DK, EPS)
        ops.delta_rule(b["q"], b["k"], b["v"], b["alpha"], b["beta"], ssm_a, dt, DK, DK, NK, NV, b["ssm"], b["core"])
        ops.rms_norm_heads(b["core"], ssm_norm, DK, EPS)
        ops.silu_mul(b["z"], b["core"])
        ops.matmul(W(wo), b["z"], b["mixed"])
        ops.add_assign(b["x"], b["mixed"])

    for p in range(PASSES):
        x0 = rng(200 + p).standard_normal(ND).astype(np.float32)
        B[0]["x"][:] = x0; B[1]["x"][:] = x0
        print(f"gdn block pass {p}", flush=True)
        hip.begin_pass(1); hip.host_wrote(B[0]["x"]); block(hip, 0, B[0]); hip.end_pass()
        hip.host_needs(B[0]["x"]); hip.read_state(B[0]["ssm"]); hip.read_state(B[0]["conv_state"])
        hip.raise_if_error()
        block(orc, 1, B[1])
        got, want = B[0]["x"] - x0, B[1]["x"].astype(np.float64) - x0
        assert np.abs(want).max() > 0.3                      # the contribution is not hidden under the residual
        assert close(got, want), (p, worst(got, want))
        assert close(B[0]["ssm"], B[1]["ssm"]), (p, worst(B[0]["ssm"], B[1]["ssm"]))
        assert close(B[0]["conv_state"], B[1]["conv_state"]), p
    fused_graph_ran(hip, 3)      # in-proj + conv, delta rule, gated norm + out-proj + residual


# --------------------------------------------------------------------------------------------- attention
def test_attention_block(pair):
    hip, orc = pair.hip, pair.orc
    NH, NKV, HD, NROT, THETA, NCTX, POS0 = 16, 2, 256, 64, 1e7, 8192, 5800
    qd, kd = NH * HD, NKV * HD
    r = rng(102)
    wq, wk, wv, wo = pair.q8(r, 2 * qd, ND, 2.0), pair.q8(r, kd, ND, 2.0), pair.q8(r, kd, ND, 2.0), pair.q8(r, ND, qd, 8.0)
    norm_w = (0.5 + r.random(ND)).astype(np.float32)
    qn = (0.5 + r.random(HD)).astype(np.float32); kn = (0.5 + r.random(HD)).astype(np.float32)
    B = bufs(x=ND, normed=ND, qg=2 * qd, q=qd, g=qd, k=kd, v=kd, attn=qd, mixed=ND)
    k0 = f16_bits(r.standard_normal(NCTX * kd)); v0 = f16_bits(r.standard_normal(NCTX * kd))
    k0[POS0 * kd:] = 0; v0[POS0 * kd:] = 0
    slabs = [dict(k=k0.copy(), v=v0.copy()) for _ in range(2)]
    sc = float(1.0 / np.sqrt(np.float32(HD)))

    def block(ops, i, b, s, pos, rope_pos=None):
        rope_pos = pos if rope_pos is None else rope_pos
        W = lambda t: t[i]
        ops.rms_norm(b["x"], norm_w, EPS, b["normed"])
        ops.matmul(W(wq), b["normed"], b["qg"])
        ops.gather_chunks(b["qg"], HD, 2 * HD, 0, b["q"]); ops.gather_chunks(b["qg"], HD, 2 * HD, HD, b["g"])
        ops.matmul(W(wk), b["normed"], b["k"]); ops.matmul(W(wv), b["normed"], b["v"])
        ops.rms_norm_heads(b["q"], qn, HD, EPS); ops.rms_norm_heads(b["k"], kn, HD, EPS)
        ops.rope_neox(b["q"], rope_pos, HD, NROT, NH, THETA); ops.rope_neox(b["k"], rope_pos, HD, NROT, NKV, THETA)
        ops.kv_write(s["k"], pos * kd, b["k"]); ops.kv_write(s["v"], pos * kd, b["v"])
        ops.attend(b["q"], s["k"], s["v"], kd, pos + 1, HD, NH, NKV, sc, b["attn"])
        ops.sigmoid_mul(b["attn"], b["g"])
        ops.matmul(W(wo), b["attn"], b["mixed"])
        ops.add_assign(b["x"], b["mixed"])

    for p in range(PASSES):
        pos = POS0 + p
        x0 = rng(300 + p).standard_normal(ND).astype(np.float32)
        B[0]["x"][:] = x0; B[1]["x"][:] = x0
        print(f"attention block pass {p} at position {pos}", flush=True)
        hip.begin_pass(1); hip.host_wrote(B[0]["x"]); block(hip, 0, B[0], slabs[0], pos); hip.end_pass()
        hip.host_needs(B[0]["x"]); hip.read_kv(slabs[0]["k"]); hip.read_kv(slabs[0]["v"])
        hip.raise_if_error()
        block(orc, 1, B[1], slabs[1], pos)
        # The gated attention output (the buffer the out-projection reads; the fused kernels leave it in place) against
        # the oracle's: split-K in wave order with the probabilities rounded to f16 for the matrix cores.
        hip.host_needs(B[0]["attn"])
        assert close(B[0]["attn"], B[1]["attn"]), (p, worst(B[0]["attn"], B[1]["attn"]))
        # The out-projection + residual against the oracle's matmul of the SAME attention vector: the Q8_0 rounding
        # of that vector is a step function, so a 1e-4 difference in it moves the product by ~1e-3 of its size in the
        # oracle as well; on identical inputs the kernel is held to the 1e-3 bound ...
        mixed_of_got = np.zeros(ND, np.float32)
        orc.matmul(wo[1], B[0]["attn"], mixed_of_got)
        got, want = B[0]["x"] - x0, B[1]["x"].astype(np.float64) - x0
        assert np.abs(want).max() > 0.3
        assert close(got, mixed_of_got), (p, worst(got, mixed_of_got))
        # ... and end to end, through the rounding step, to 1e-2
        assert close(got, want, 1e-2), (p, worst(got, want))
        for t in "kv":
            a = slabs[0][t].view(np.float16).astype(np.float32); b = slabs[1][t].view(np.float16).astype(np.float32)
            assert np.array_equal(a[:POS0 * kd], b[:POS0 * kd]) and not a[(pos + 1) * kd:].any()  # only new rows moved
            assert close(a[POS0 * kd:(pos + 1) * kd], b[POS0 * kd:(pos + 1) * kd], 2e-3), (p, t)   # one f16 step
    fused_graph_ran(hip, 3)      # q/k/v projections, attention with norm + rope + cache write folded in, out-proj
    # The fused kernel takes ONE position for the rotation, the cache row and the context length; the seam passes
    # them separately.  A pass whose rotation position differs from its cache row (same op sequence, so the graph's
    # signature still matches) must not be replayed with the graph's single position: it runs op by op.
    pos = POS0 + PASSES
    x0 = rng(399).standard_normal(ND).astype(np.float32)
    B[0]["x"][:] = x0; B[1]["x"][:] = x0
    hip.begin_pass(1); hip.host_wrote(B[0]["x"]); block(hip, 0, B[0], slabs[0], pos, rope_pos=pos + 7); hip.end_pass()
    hip.host_needs(B[0]["x"]); hip.host_needs(B[0]["attn"]); hip.read_kv(slabs[0]["k"]); hip.raise_if_error()
    block(orc, 1, B[1], slabs[1], pos, rope_pos=pos + 7)
    assert hip.graph_stats()["aborts"] == 1
    assert close(B[0]["attn"], B[1]["attn"]), worst(B[0]["attn"], B[1]["attn"])
    a = slabs[0]["k"].view(np.float16).astype(np.float32); b = slabs[1]["k"].view(np.float16).astype(np.float32)
    assert close(a[pos * kd:(pos + 1) * kd], b[pos * kd:(pos + 1) * kd], 2e-3)


# --------------------------------------------------------------------------------------------- routed FFN
@pytest.mark.parametrize("shared", ["q8_0", "nvfp4_scaled"])
def test_ffn_block_512_experts(pair, shared):
    """shared = nvfp4_scaled: the shared expert as an NVFP4 file stores it, three NVFP4 matrices with a second scale
    each, applied by SCALE ops after the products (qwen35.rs:1669-1682); the fused kernels take the scales as scalars."""
    hip, orc, ih = pair.hip, pair.orc, pair.ih
    NE, NU, FF, SFF = 512, 10, 512, 512
    r = rng(103)
    router = pair.q8(r, NE, ND, 3.0)                   # logits of a few units: a peaked but not one-hot softmax
    sh_inp = pair.q8(r, 1, ND, 1.0)
    g_s = (0.5 + r.random(NE)).astype(np.float32) / 54.0; u_s = (0.5 + r.random(NE)).astype(np.float32) / 54.0
    d_s = (0.5 + r.random(NE)).astype(np.float32) / 27.0
    gate = pair.e(nvfp4_rows(r, NE * FF, ND), ih.NVFP4, ND, FF, NE, g_s)
    up = pair.e(nvfp4_rows(r, NE * FF, ND), ih.NVFP4, ND, FF, NE, u_s)
    down = pair.e(nvfp4_rows(r, NE * ND, FF), ih.NVFP4, FF, ND, NE, d_s)
    if shared == "q8_0":
        sg, su, sd = pair.q8(r, SFF, ND, 1.5), pair.q8(r, SFF, ND, 1.5), pair.q8(r, ND, SFF, 2.0)
        s_g = s_u = s_d = None
    else:
        sg, su = pair.w(nvfp4_rows(r, SFF, ND), ih.NVFP4, ND, SFF), pair.w(nvfp4_rows(r, SFF, ND), ih.NVFP4, ND, SFF)
        sd = pair.w(nvfp4_rows(r, ND, SFF), ih.NVFP4, SFF, ND)
        s_g, s_u, s_d = float(0.7 / 54.0), float(1.3 / 54.0), float(1.1 / 27.0)
    norm_w = (0.5 + r.random(ND)).astype(np.float32)
    B = bufs(x=ND, normed=ND, e_in=ND, router=NE, logit=1, g_all=NU * FF, u_all=NU * FF, o_all=NU * ND, e_gate=SFF,
             e_up=SFF, e_out=ND, ffn_out=ND)

    def block(ops, i, b, is_hip):
        W = lambda t: t[i]
        ops.rms_norm(b["x"], norm_w, EPS, b["normed"])
        ops.gather_chunks(b["normed"], ND, ND, 0, b["e_in"])
        ops.matmul_pair(W(router), W(sh_inp), b["e_in"], b["router"], b["logit"])
        ops.softmax(b["router"], NE)
        if is_hip:
            route = ops.route(b["router"], NE, NU)
            ops.moe_glu(W(gate), W(up), route, b["e_in"], b["g_all"], b["u_all"])
            ops.matmul_experts(W(down), route, b["g_all"], b["o_all"])
        else:
            ids, w = ops.route(b["router"], NE, NU)
            ops.moe_glu(W(gate), W(up), ids, NU, b["e_in"], b["g_all"], b["u_all"])
            ops.matmul_experts(W(down), ids, NU, b["g_all"], b["o_all"])
        ops.matmul(W(sg), b["e_in"], b["e_gate"]); ops.matmul(W(su), b["e_in"], b["e_up"])
        if s_u is not None:
            ops.scale(b["e_up"], s_u); ops.scale(b["e_gate"], s_g)
        ops.silu_mul(b["e_gate"], b["e_up"])
        ops.matmul(W(sd), b["e_gate"], b["e_out"])
        if s_d is not None:
            ops.scale(b["e_out"], s_d)
        if is_hip:
            ops.moe_finish(b["ffn_out"], 0, ND, b["o_all"], route, b["e_out"], b["logit"], 0)
        else:
            ops.moe_finish(b["ffn_out"], 0, ND, b["o_all"], w, NU, b["e_out"], b["logit"], 0)
        ops.add_assign(b["x"], b["ffn_out"])
        return None if is_hip else (ids, w)

    for p in range(PASSES):
        x0 = rng(400 + p).standard_normal(ND).astype(np.float32)
        B[0]["x"][:] = x0; B[1]["x"][:] = x0
        print(f"ffn block pass {p}", flush=True)
        hip.begin_pass(1); hip.host_wrote(B[0]["x"]); block(hip, 0, B[0], True); hip.end_pass()
        hip.host_needs(B[0]["x"]); hip.raise_if_error()
        ids, w = block(orc, 1, B[1], False)
        assert len(set(ids.tolist())) == NU and w.min() > 1e-3     # ten distinct experts that all count
        # Stage 1: the ten experts' silu(gate) * up rows, in pick order, and the shared expert's (the buffers the down
        # kernel reads).  A different pick by the in-kernel router would put another expert's row here.
        hip.host_needs(B[0]["g_all"]); hip.host_needs(B[0]["e_gate"])
        for name in ("g_all", "e_gate"):
            assert close(B[0][name], B[1][name]), (p, name, worst(B[0][name], B[1][name]))
        # Stage 2: down products, weighted sum, shared expert's sigmoid gate and the residual, against the oracle's ops
        # applied to the SAME intermediates (their Q8_0 rounding is a step function: a last-bit difference in one of
        # the 5,632 values can move a step, and with it the sum, by ~1e-3 of its size in the oracle as well) ...
        o_all = np.zeros(NU * ND, np.float32); e_out = np.zeros(ND, np.float32); ffn = np.zeros(ND, np.float32)
        orc.matmul_experts(down[1], ids, NU, B[0]["g_all"], o_all)
        orc.matmul(sd[1], B[0]["e_gate"], e_out)
        if s_d is not None:
            orc.scale(e_out, s_d)
        orc.moe_finish(ffn, 0, ND, o_all, w, NU, e_out, B[1]["logit"], 0)
        got, want = B[0]["x"] - x0, B[1]["x"].astype(np.float64) - x0
        assert np.abs(want).max() > 0.3
        assert close(got, ffn), (p, worst(got, ffn))
        # ... and end to end, through the rounding step, to 1e-2
        assert close(got, want, 1e-2), (p, worst(got, want))
    fused_graph_ran(hip, 3)      # router + shared logit, experts' gate/up with the in-kernel top-10, down + combine
    st = hip.expert_stats()
    assert st.resident == 3 * NE and st.oversubscribed == 0


# --------------------------------------------------------------------------------------------- output head
def test_output_head(pair):
    hip, orc = pair.hip, pair.orc
    NV = 151936
    r = rng(104)
    out_w = pair.q8(r, NV, ND, 1.0)
    norm_w = (0.5 + r.random(ND)).astype(np.float32)
    B = bufs(x=ND, last=ND, final=ND, logits=NV)

    def block(ops, i, b):
        ops.gather_chunks(b["x"], ND, ND, 0, b["last"])
        ops.rms_norm(b["last"], norm_w, EPS, b["final"])
        ops.matmul(out_w[i], b["final"], b["logits"])

    for p in range(PASSES):
        x0 = rng(500 + p).standard_normal(ND).astype(np.float32)
        B[0]["x"][:] = x0; B[1]["x"][:] = x0
        print(f"output head pass {p}", flush=True)
        hip.begin_pass(1); hip.host_wrote(B[0]["x"]); block(hip, 0, B[0]); hip.end_pass()
        hip.host_needs(B[0]["logits"]); hip.raise_if_error()
        block(orc, 1, B[1])
        assert close(B[0]["logits"], B[1]["logits"]), (p, worst(B[0]["logits"], B[1]["logits"]))
        top = int(np.argmax(B[1]["logits"]))
        margin = np.partition(B[1]["logits"], -2)[-2:]
        if margin[1] - margin[0] > 1e-3 * max(1.0, abs(margin[1])):
            assert hip.argmax(B[0]["logits"]) == top == orc.argmax(B[1]["logits"])
    g = hip.graph_stats()
    assert g["captures"] == 1 and g["graph_kernels"] == 1, g
