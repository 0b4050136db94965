"""The layer chain (runs of decode layers as ONE persistent kernel, k_chain.hip) against the CPU oracle.

Whole layers of a single-token pass are issued op by op through the C ABI exactly as the host loop issues them
(/root/reference src/model/qwen35.rs:1232-1328 gated delta net, :1587-1700 routed FFN).  The backend runs the first
two passes eagerly, captures the third into a HIP graph and replays it; at capture the fuser folds every run of
(Gated DeltaNet block, routed FFN) layers, optionally opened by an FFN whose mixer is not one, into one persistent
kernel.  Shapes are config 5's (hidden 2048; 16 key / 32 value heads of 128; 512 NVFP4 experts top-10 of 512 rows +
a Q8_0 or NVFP4 shared expert).

Compared per pass with the same op sequence composed from the oracle's ops on identical inputs:
  * the layers' contribution to the residual stream, end to end: |error| <= 2e-3 * max(|value|, rms of the vector).
    Between the blocks of a layer every activation is quantized to Q8_0, a step function: fast mode's last-bit
    differences (sums in wave order, exp on the transcendental unit) move a step in roughly every other vector, and
    one moved step shifts every output of the block by ~2e-4 of the vector's scale, in the oracle as in the kernel, so
    the bound is against the vector's scale rather than each entry's own size (measured: 1e-6 of the scale when no
    step moves, 1.4e-5 when one does; tests/test_gpu_fused_fast.py holds each block on its own to 1e-3 per entry
    by splitting it at the quantization, which a chain cannot be: its intermediates never leave the kernel);
  * every layer's recurrent state and conv window to 1e-3 per entry;
  * the routed experts of every layer, exactly (read from the expert cache's device-side read counters);
and with the per-stage fused kernels (the same arithmetic, six launches a layer) to the same bounds.
"""
import os

import numpy as np
import pytest

from test_gpu_fused_fast import Both, bufs, nvfp4_rows, ND, EPS
from util import close, f16_bits, rng, worst

pytestmark = pytest.mark.gpu

NK, NV, DK = 16, 32, 128
KDIM, VDIM = NK * DK, NV * DK
CDIM = 2 * KDIM + VDIM
NE, NU, FF, SFF = 512, 10, 512, 512
PASSES = 5


def near(got, want, tol=2e-3):
    """|got - want| <= tol * max(|want_i|, rms(want)): a bound against the vector's scale."""
    want = np.asarray(want, np.float64)
    floor = float(np.sqrt((want ** 2).mean())) if want.size else 0.0
    return bool(np.all(np.abs(np.asarray(got, np.float64) - want) <= tol * np.maximum(np.abs(want), floor)))


def far(got, want):
    """largest error as a multiple of the bound at tol = 1"""
    want = np.asarray(want, np.float64)
    floor = float(np.sqrt((want ** 2).mean())) if want.size else 0.0
    return float((np.abs(np.asarray(got, np.float64) - want) / np.maximum(np.maximum(np.abs(want), floor), 1e-300)).max())


class Layers:
    """Weights of `n` layers over shared expert tensors (one set of 512 experts serves every layer: 0.9 GB)."""

    def __init__(self, pair, n, shared, seed=7, small_f32=False, mute_ffn=False):
        """small_f32: the router, the shared expert's gate-logit row and ssm alpha / beta as F32 matrices, as real files
        of this model keep them (/root/reference src/model/qwen35.rs:1626, :1273: `matmul_pair` on unquantized weights
        reads the f32 activation itself), instead of Q8_0."""
        ih = pair.ih
        r = rng(seed)
        self.pair, self.n, self.shared = pair, n, shared

        def small(n_out, gain):
            if not small_f32:
                return pair.q8(r, n_out, ND, gain)
            w = (r.standard_normal(n_out * ND) * (gain / np.sqrt(ND))).astype(np.float32)
            return pair.w(w.view(np.uint8), ih.F32, ND, n_out)
        g_s = (0.5 + r.random(NE)).astype(np.float32) / 54.0
        u_s = (0.5 + r.random(NE)).astype(np.float32) / 54.0
        d_s = (0.5 + r.random(NE)).astype(np.float32) / 108.0
        if mute_ffn:   # second scales of zero on every down product: the FFN runs and adds nothing (NVFP4 shared expert)
            d_s[:] = 0.0
        self.gate_raw = nvfp4_rows(r, NE * FF, ND)
        self.gate = pair.e(self.gate_raw, ih.NVFP4, ND, FF, NE, g_s)
        self.up = pair.e(nvfp4_rows(r, NE * FF, ND), ih.NVFP4, ND, FF, NE, u_s)
        self.down = pair.e(nvfp4_rows(r, NE * ND, FF), ih.NVFP4, FF, ND, NE, d_s)
        self.L = []
        for _ in range(n):
            d = {}
            d["wqkv"], d["wz"] = pair.q8(r, CDIM, ND, 2.0), pair.q8(r, VDIM, ND, 2.0)
            d["wa"], d["wb"], d["wo"] = small(NV, 2.0), small(NV, 2.0), pair.q8(r, ND, VDIM, 1.0)
            d["norm"] = (0.5 + r.random(ND)).astype(np.float32)
            d["ssm_norm"] = (0.5 + r.random(DK)).astype(np.float32)
            d["conv_w"] = (r.standard_normal(CDIM * 4) * 0.5).astype(np.float32)
            d["ssm_a"] = (-np.exp(r.standard_normal(NV) * 0.5)).astype(np.float32)
            d["dt"] = (r.standard_normal(NV) * 0.5).astype(np.float32)
            d["router"], d["sh_inp"] = small(NE, 3.0), small(1, 1.0)
            if shared == "q8_0":
                d["sg"], d["su"], d["sd"] = pair.q8(r, SFF, ND, 1.0), pair.q8(r, SFF, ND, 1.0), pair.q8(r, ND, SFF, 1.0)
                d["s"] = None
            else:
                d["sg"] = pair.w(nvfp4_rows(r, SFF, ND), ih.NVFP4, ND, SFF)
                d["su"] = pair.w(nvfp4_rows(r, SFF, ND), ih.NVFP4, ND, SFF)
                d["sd"] = pair.w(nvfp4_rows(r, ND, SFF), ih.NVFP4, SFF, ND)
                d["s"] = (float(0.7 / 54.0), float(1.3 / 54.0), 0.0 if mute_ffn else float(1.1 / 27.0))
            d["ffn_norm"] = (0.5 + r.random(ND)).astype(np.float32)
            self.L.append(d)

    def buffers(self):
        """Per backend: one residual stream, per-layer scratch and state."""
        out = []
        for _ in range(2):
            per = {"x": np.zeros(ND, np.float32), "layers": []}
            for li in range(self.n):
                b = bufs(normed=ND, qkv=CDIM, z=VDIM, alpha=NV, beta=NV, convo=CDIM, q=KDIM, k=KDIM, v=VDIM, core=VDIM,
                         mixed=ND, conv_state=CDIM * 3, ssm=NV * DK * DK, fnormed=ND, e_in=ND, router=NE, logit=1,
                         g_all=NU * FF, u_all=NU * FF, o_all=NU * ND, e_gate=SFF, e_up=SFF, e_out=ND, ffn_out=ND)[0]
                b["conv_state"][:] = (rng(50 + li).standard_normal(CDIM * 3) * 0.5).astype(np.float32)
                b["ssm"][:] = (rng(60 + li).standard_normal(NV * DK * DK) * 0.05).astype(np.float32)
                per["layers"].append(b)
            out.append(per)
        return out

    def gdn(self, ops, i, d, b, x):
        W = lambda t: t[i]
        ops.rms_norm(x, d["norm"], EPS, b["normed"])
        ops.matmul(W(d["wqkv"]), b["normed"], b["qkv"]); ops.matmul(W(d["wz"]), b["normed"], b["z"])
        ops.matmul_pair(W(d["wa"]), W(d["wb"]), b["normed"], b["alpha"], b["beta"])
        ops.ssm_conv(b["conv_state"], b["qkv"], d["conv_w"], 4, b["convo"])
        ops.gather_chunks(b["convo"], KDIM, CDIM, 0, b["q"]); ops.gather_chunks(b["convo"], KDIM, CDIM, KDIM, b["k"])
        ops.gather_chunks(b["convo"], VDIM, CDIM, 2 * KDIM, b["v"])
        ops.l2_norm_heads(b["q"], DK, EPS); ops.l2_norm_heads(b["k"], DK, EPS)
        ops.delta_rule(b["q"], b["k"], b["v"], b["alpha"], b["beta"], d["ssm_a"], d["dt"], DK, DK, NK, NV, b["ssm"], b["core"])
        ops.rms_norm_heads(b["core"], d["ssm_norm"], DK, EPS)
        ops.silu_mul(b["z"], b["core"])
        ops.matmul(W(d["wo"]), b["z"], b["mixed"])
        ops.add_assign(x, b["mixed"])

    def ffn(self, ops, i, d, b, x, is_hip):
        W = lambda t: t[i]
        ops.rms_norm(x, d["ffn_norm"], EPS, b["fnormed"])
        ops.gather_chunks(b["fnormed"], ND, ND, 0, b["e_in"])
        ops.matmul_pair(W(d["router"]), W(d["sh_inp"]), b["e_in"], b["router"], b["logit"])
        ops.softmax(b["router"], NE)
        ids = None
        if is_hip:
            route = ops.route(b["router"], NE, NU)
            ops.moe_glu(W(self.gate), W(self.up), route, b["e_in"], b["g_all"], b["u_all"])
            ops.matmul_experts(W(self.down), route, b["g_all"], b["o_all"])
        else:
            ids, w = ops.route(b["router"], NE, NU)
            ops.moe_glu(W(self.gate), W(self.up), ids, NU, b["e_in"], b["g_all"], b["u_all"])
            ops.matmul_experts(W(self.down), ids, NU, b["g_all"], b["o_all"])
        ops.matmul(W(d["sg"]), b["e_in"], b["e_gate"]); ops.matmul(W(d["su"]), b["e_in"], b["e_up"])
        if d["s"] is not None:
            ops.scale(b["e_up"], d["s"][1]); ops.scale(b["e_gate"], d["s"][0])
        ops.silu_mul(b["e_gate"], b["e_up"])
        ops.matmul(W(d["sd"]), b["e_gate"], b["e_out"])
        if d["s"] is not None:
            ops.scale(b["e_out"], d["s"][2])
        if is_hip:
            ops.moe_finish(b["ffn_out"], 0, ND, b["o_all"], route, b["e_out"], b["logit"], 0)
        else:
            ops.moe_finish(b["ffn_out"], 0, ND, b["o_all"], w, NU, b["e_out"], b["logit"], 0)
        ops.add_assign(x, b["ffn_out"])
        return ids

    def run(self, ops, i, B, is_hip, first_mixer=True):
        """One pass over the layers; first_mixer False: the first layer contributes its FFN only (as the FFN of a layer
        whose mixer is an attention block would open a chain)."""
        picked = []
        for li, d in enumerate(self.L):
            if li > 0 or first_mixer:
                self.gdn(ops, i, d, B["layers"][li], B["x"])
            picked.append(self.ffn(ops, i, d, B["layers"][li], B["x"], is_hip))
        return picked


def make_pair(chain=True):
    import inferred_hip as ih
    from oracle import binding as ob
    hip = ih.Hip(exact=False, chain=chain)
    return Both(hip, ob.Oracle(threads=8))


def hip_pass(hip, layers, B, x0, first_mixer=True):
    B["x"][:] = x0
    hip.begin_pass(1); hip.host_wrote(B["x"]); layers.run(hip, 0, B, True, first_mixer); hip.end_pass()
    hip.host_needs(B["x"])
    for li, b in enumerate(B["layers"]):
        if li > 0 or first_mixer:
            hip.read_state(b["ssm"]); hip.read_state(b["conv_state"])
    hip.raise_if_error()


@pytest.mark.parametrize("shared,first_mixer,small_f32", [("q8_0", True, False), ("nvfp4_scaled", True, False), ("q8_0", False, False),
                                                         ("nvfp4_scaled", True, True), ("q8_0", False, True)])
def test_layers_as_one_kernel(shared, first_mixer, small_f32):
    """small_f32 with an NVFP4 shared expert is the layout of a real NVFP4 file of this model.  Those cases run ONE layer
    (a chain of one) and the oracle goes on from the kernel's recurrent state after every pass: fast mode's f32 rows
    differ from the oracle's serial sums by about 4e-6, which now and then moves one Q8_0 step of an activation the other
    way, and the NVFP4-scaled FFN behind it multiplies that to 2-3 % of the scale for that pass (measured the same with
    every op issued eagerly, so not a property of the chain).  At most one of the passes may be off like that, and by no
    more than 5 %; the picks, the state and every other pass are held to the usual bound.  The hand-offs between layers
    are the same code whatever the small matrices' format: the Q8_0 cases and the comparison with the per-stage kernels
    below cover them."""
    n_layers = 1 if small_f32 else 2
    stepped = 0
    pair = make_pair()
    hip, orc = pair.hip, pair.orc
    try:
        layers = Layers(pair, n_layers, shared, small_f32=small_f32)
        B = layers.buffers()
        counts_before = np.zeros(NE, np.int64)
        for p in range(PASSES):
            x0 = rng(700 + p).standard_normal(ND).astype(np.float32)
            print(f"chain {shared} first_mixer={first_mixer} pass {p}", flush=True)
            hip_pass(hip, layers, B[0], x0, first_mixer)
            B[1]["x"][:] = x0
            picked = layers.run(orc, 1, B[1], False, first_mixer)
            got, want = B[0]["x"] - x0, B[1]["x"].astype(np.float64) - x0
            assert np.abs(want).max() > 0.3
            if small_f32 and not near(got, want) and far(got, want) < 0.05:
                stepped += 1
                assert stepped <= 1, (p, far(got, want))
            else:
                assert near(got, want), (p, far(got, want))
            for li in range(n_layers):
                if li == 0 and not first_mixer:
                    continue
                a, b = B[0]["layers"][li], B[1]["layers"][li]
                assert close(a["ssm"], b["ssm"]), (p, li, worst(a["ssm"], b["ssm"]))
                assert close(a["conv_state"], b["conv_state"]), (p, li, worst(a["conv_state"], b["conv_state"]))
            # the picks of both layers, from the device-side read counters of the gate tensor
            counts = hip.expert_counts(layers.gate_raw, NE).astype(np.int64)
            want_counts = np.zeros(NE, np.int64)
            for ids in picked:
                assert len(set(ids.tolist())) == NU
                np.add.at(want_counts, ids.astype(np.int64), 1)
            assert np.array_equal(counts - counts_before, want_counts), (p, np.flatnonzero(counts - counts_before != want_counts))
            counts_before = counts
            if small_f32:   # each pass compared on its own: the oracle goes on from the kernel's recurrent state
                for li in range(n_layers):
                    for name in ("ssm", "conv_state"):
                        B[1]["layers"][li][name][:] = B[0]["layers"][li][name]
        g, c = hip.graph_stats(), hip.chain_stats()
        assert g["captures"] == 1 and g["aborts"] == 0 and g["replays"] == PASSES - 2, g
        assert g["graph_kernels"] == 1 and c["chains"] == 1 and c["layers"] == n_layers and c["enabled"], (g, c)
        # what the chain no longer writes is refused to the host instead of handed over stale
        hip.host_needs(B[0]["layers"][n_layers - 1]["g_all"])
        err = hip.take_error()
        assert err is not None and "fused kernel" in err, err
    finally:
        err = hip.take_error()
        hip.close()
    assert err is None, err


@pytest.mark.parametrize("shared,small_f32", [("q8_0", False), ("nvfp4_scaled", True)])
def test_chain_against_the_per_stage_kernels(shared, small_f32):
    """The same three layers through the chain and through the six launches a layer it replaces (the second case is the
    layout of a real NVFP4 file: F32 router, gate-logit and alpha / beta matrices, NVFP4 shared expert with scales).
    The two differ by a few 1e-7 (other summation orders in the delta rule and the norms).  Both are deterministic, so
    the comparison is too; should a change to a kernel move this to a few per cent with equal picks, look for an
    activation that sits within 1e-7 of a Q8_0 rounding boundary in this data before looking for a bug (seed 11 has
    one in pass 2 with the F32 layout), and try another seed."""
    outs = []
    for chain in (True, False):
        pair = make_pair(chain)
        hip = pair.hip
        try:
            layers = Layers(pair, 3, shared, seed=12 if small_f32 else 11, small_f32=small_f32)
            B = layers.buffers()[0]
            xs = []
            for p in range(PASSES):
                x0 = rng(900 + p).standard_normal(ND).astype(np.float32)
                print(f"chain={chain} pass {p}", flush=True)
                hip_pass(hip, layers, B, x0)
                xs.append(B["x"].copy())
            c = hip.chain_stats()
            assert (c["chains"], c["layers"]) == ((1, 3) if chain else (0, 0)), c
            assert hip.graph_stats()["graph_kernels"] == (1 if chain else 18)
            outs.append((xs, [b["ssm"].copy() for b in B["layers"]], [b["conv_state"].copy() for b in B["layers"]],
                         hip.expert_counts(layers.gate_raw, NE).copy()))
        finally:
            err = hip.take_error()
            hip.close()
        assert err is None, err
    (xa, sa, ca, na), (xb, sb, cb, nb) = outs
    for p in range(PASSES):
        assert near(xa[p], xb[p]), (p, far(xa[p], xb[p]))
    for li in range(3):
        assert close(sa[li], sb[li]), (li, worst(sa[li], sb[li]))
        assert close(ca[li], cb[li]), (li, worst(ca[li], cb[li]))
    assert np.array_equal(na, nb)


def test_a_wait_that_gives_up_is_an_error_not_a_hang():
    """With the bound on a hand-off wait forced down to one poll from the host, every block of the chain gives up at
    its first wait and the kernel drains: the pass's results are void, the sticky error says so, the chains are
    switched off for the backend, and the next passes run on the per-stage kernels."""
    os.environ["INFERRED_HIP_CHAIN_SPINS"] = "1"
    try:
        pair = make_pair()
    finally:
        del os.environ["INFERRED_HIP_CHAIN_SPINS"]
    hip, orc = pair.hip, pair.orc
    try:
        assert hip.chain_stats()["spin_limit"] == 1
        layers = Layers(pair, 2, "q8_0", seed=13)
        B = layers.buffers()
        for p in range(2):          # eager passes
            hip_pass(hip, layers, B[0], rng(40 + p).standard_normal(ND).astype(np.float32))
        x0 = rng(42).standard_normal(ND).astype(np.float32)
        B[0]["x"][:] = x0
        print("the pass whose chain gives up", flush=True)
        hip.begin_pass(1); hip.host_wrote(B[0]["x"]); layers.run(hip, 0, B[0], True); hip.end_pass()
        hip.sync()
        err = hip.take_error()
        assert err is not None and "layer chain" in err, err
        assert not hip.chain_stats()["enabled"]
        # the backend keeps working without chains: with the oracle's state on both sides again, the next pass agrees
        # with it, and the passes after that (recorded into a new graph of per-stage kernels) raise nothing
        for li in range(2):
            for name in ("ssm", "conv_state"):
                B[0]["layers"][li][name][:] = B[1]["layers"][li][name]
        hip.forget_state()          # the host copies are the state again: uploaded at their next use
        x0 = rng(45).standard_normal(ND).astype(np.float32)
        print("after the error, pass 0", flush=True)
        hip_pass(hip, layers, B[0], x0)
        B[1]["x"][:] = x0
        layers.run(orc, 1, B[1], False)
        got, want = B[0]["x"] - x0, B[1]["x"].astype(np.float64) - x0
        assert near(got, want), far(got, want)
        for p in range(1, 4):
            print(f"after the error, pass {p}", flush=True)
            hip_pass(hip, layers, B[0], rng(45 + p).standard_normal(ND).astype(np.float32))
            assert np.all(np.isfinite(B[0]["x"]))
        assert hip.graph_stats()["graph_kernels"] == 12
        assert hip.chain_stats()["chains"] == 0
    finally:
        err = hip.take_error()
        hip.close()
    assert err is None, err


@pytest.mark.parametrize("pos0", [5800, 40, 12000, 8189])
def test_the_attention_mixer_inside_a_chain_against_the_oracle(pos0):
    """One attention layer whose FFN adds nothing (second scales of zero on every down product), so that the pass's
    change of the residual stream IS the mixer's output: in-projection, head norms, rotation, the new cache rows,
    attention over the context in 128 key ranges, merge, sigmoid gate, out-projection, all stages of the persistent
    kernel.  Held to the oracle at 2e-3 of the vector's scale and the new K / V rows at 2e-3 of the row's, five
    positions each: a context of 5,800 (a range is 46 keys: one tile), of 40 (fewer keys than ranges: most blocks have
    none), of 12,000 (a range is 94 keys: two tiles with the running maximum carried across) and of 8,189 (a range grows
    from 64 keys, one full tile, to 65: a second tile of one key)."""
    NH, NKV, AHD, NROT, THETA, NCTX = 16, 2, 256, 64, 1e7, 12288
    qd, kd = NH * AHD, NKV * AHD
    sc = float(1.0 / np.sqrt(np.float32(AHD)))
    pair = make_pair(True)
    hip, orc = pair.hip, pair.orc
    try:
        layers = Layers(pair, 1, "nvfp4_scaled", seed=31, mute_ffn=True)
        r = rng(32)
        wq, wk, wv = pair.q8(r, 2 * qd, ND, 2.0), pair.q8(r, kd, ND, 2.0), pair.q8(r, kd, ND, 2.0)
        wo = pair.q8(r, ND, qd, 2.0)
        anorm = (0.5 + r.random(ND)).astype(np.float32)
        qn = (0.5 + r.random(AHD)).astype(np.float32); kn = (0.5 + r.random(AHD)).astype(np.float32)
        # keys with a spread of lengths, so that the probabilities are not flat and a few keys carry most of a head's weight
        k0 = f16_bits(r.standard_normal(NCTX * kd) * np.repeat(np.exp(r.standard_normal(NCTX * NKV) * 0.7), AHD))
        v0 = f16_bits(r.standard_normal(NCTX * kd))
        k0[pos0 * kd:] = 0; v0[pos0 * kd:] = 0
        slabs = [dict(k=k0.copy(), v=v0.copy()) for _ in range(2)]
        A = bufs(normed=ND, qg=2 * qd, q=qd, g=qd, k=kd, v=kd, attn=qd, mixed=ND)
        B = layers.buffers()

        def run(ops, i, is_hip, pos):
            W = lambda t: t[i]
            b, s, x = A[i], slabs[i], B[i]["x"]
            ops.rms_norm(x, anorm, EPS, b["normed"])
            ops.matmul(W(wq), b["normed"], b["qg"])
            ops.gather_chunks(b["qg"], AHD, 2 * AHD, 0, b["q"]); ops.gather_chunks(b["qg"], AHD, 2 * AHD, AHD, b["g"])
            ops.matmul(W(wk), b["normed"], b["k"]); ops.matmul(W(wv), b["normed"], b["v"])
            ops.rms_norm_heads(b["q"], qn, AHD, EPS); ops.rms_norm_heads(b["k"], kn, AHD, EPS)
            ops.rope_neox(b["q"], pos, AHD, NROT, NH, THETA); ops.rope_neox(b["k"], pos, AHD, NROT, NKV, THETA)
            ops.kv_write(s["k"], pos * kd, b["k"]); ops.kv_write(s["v"], pos * kd, b["v"])
            ops.attend(b["q"], s["k"], s["v"], kd, pos + 1, AHD, NH, NKV, sc, b["attn"])
            ops.sigmoid_mul(b["attn"], b["g"])
            ops.matmul(W(wo), b["attn"], b["mixed"])
            ops.add_assign(x, b["mixed"])
            layers.ffn(ops, i, layers.L[0], B[i]["layers"][0], x, is_hip)

        # Position 8,192 is where the rotation table doubles (an allocation: the recorded graph is dropped, that pass and
        # the next run op by op, the one after is recorded again); the context that crosses it runs three passes more,
        # so that ranges of 65 keys (a full tile and a tile of one key) go through the chain as well
        crossing = pos0 < 8192 <= pos0 + PASSES
        n_pass = PASSES + 3 if crossing else PASSES
        op_by_op = {0, 1} | ({8192 - pos0, 8193 - pos0} if crossing else set())
        for p in range(n_pass):
            pos = pos0 + p
            x0 = rng(850 + p).standard_normal(ND).astype(np.float32)
            print(f"attention mixer in the chain, pass {p} at position {pos}", flush=True)
            B[0]["x"][:] = x0
            hip.begin_pass(1); hip.host_wrote(B[0]["x"]); run(hip, 0, True, pos); hip.end_pass()
            hip.host_needs(B[0]["x"]); hip.read_kv(slabs[0]["k"]); hip.read_kv(slabs[0]["v"])
            hip.raise_if_error()
            B[1]["x"][:] = x0
            run(orc, 1, False, pos)
            got, want = B[0]["x"] - x0, B[1]["x"].astype(np.float64) - x0
            assert np.abs(want).max() > 0.05
            # (the passes issued op by op, before there is a chain: their attention rounds the probabilities to f16 for
            # the matrix cores and is held to 5e-3; the chain's takes them as exact f16 pairs)
            assert near(got, want, 5e-3 if p in op_by_op else 2e-3), (p, far(got, want))
            print(f"  pass {p}: {far(got, want):.3g} of the scale", flush=True)
            for t in "kv":
                a = slabs[0][t].view(np.float16).astype(np.float32); b = slabs[1][t].view(np.float16).astype(np.float32)
                assert np.array_equal(a[:pos0 * kd], b[:pos0 * kd]) and not a[(pos + 1) * kd:].any()
                assert near(a[pos * kd:(pos + 1) * kd], b[pos * kd:(pos + 1) * kd]), (p, t)
                slabs[1][t][pos * kd:(pos + 1) * kd] = slabs[0][t][pos * kd:(pos + 1) * kd]
        g, c = hip.graph_stats(), hip.chain_stats()
        if crossing:
            assert g["captures"] == 2 and g["aborts"] == 1, g
        else:
            assert g["captures"] == 1 and g["aborts"] == 0 and g["replays"] == PASSES - 2, g
        assert c["chains"] == 1 and c["layers"] == 1 and g["graph_kernels"] == 1, (g, c)
    finally:
        err = hip.take_error()
        hip.close()
    assert err is None, err


@pytest.mark.parametrize("attn_in_chain", [True, False])
def test_an_attention_layer_between_chains(attn_in_chain, monkeypatch):
    """layer 0 (Gated DeltaNet + FFN), layer 1 (attention + FFN), layer 2 (Gated DeltaNet + FFN) in one pass.  With the
    attention mixer inside the chain (in-projection, head norms, rotation, cache rows, attention over 128 key ranges,
    merge + gate, out-projection as stages of the persistent kernel) the pass is ONE kernel.  With that switched off
    (INFERRED_HIP_NO_CHAIN_ATTN=1) the attention layer's in-projection is the last stage of the first chain and its
    out-projection the first stage of the second; norm + rotation + cache write + split-K attention stay the launch
    between them: three kernels in all.

    Held to the per-stage kernels (the same passes on a backend with the chains switched off) at the bounds of the
    module: the residual stream, both recurrent states, the new K / V rows, the picks.  Held to the oracle where a
    chain's output reaches the host before the attention output is quantized: layer 0's state (1e-3) and the new K / V
    rows, which are the first chain's last stage (2e-3 of the row's scale).  Behind that point the comparison with the
    oracle is a gross one (0.15 of the vector's scale: a missing or doubled term fails it, see below): the attention
    output is a mean over 5800 rows and small against its own Q8_0 step, fast mode's 1e-4 relative difference in it
    moves tens of steps in the oracle's favour or the kernel's, and the two blocks behind multiply what that leaves
    (measured with every op issued eagerly, so not a property of the chain: 1.6e-4 of the scale behind the
    out-projection, 1.1e-2 behind the next FFN, 5e-2 at the end)."""
    NH, NKV, AHD, NROT, THETA, NCTX, POS0 = 16, 2, 256, 64, 1e7, 8192, 5800
    qd, kd = NH * AHD, NKV * AHD
    sc = float(1.0 / np.sqrt(np.float32(AHD)))
    outs = []
    if attn_in_chain:
        monkeypatch.delenv("INFERRED_HIP_NO_CHAIN_ATTN", raising=False)
    else:
        monkeypatch.setenv("INFERRED_HIP_NO_CHAIN_ATTN", "1")
    for chain in (True, False):
        pair = make_pair(chain)
        hip, orc = pair.hip, pair.orc
        try:
            layers = Layers(pair, 3, "q8_0", seed=21)
            r = rng(22)
            wq, wk, wv = pair.q8(r, 2 * qd, ND, 2.0), pair.q8(r, kd, ND, 2.0), pair.q8(r, kd, ND, 2.0)
            wo = pair.q8(r, ND, qd, 2.0)
            anorm = (0.5 + r.random(ND)).astype(np.float32)
            qn = (0.5 + r.random(AHD)).astype(np.float32); kn = (0.5 + r.random(AHD)).astype(np.float32)
            k0 = f16_bits(r.standard_normal(NCTX * kd)); v0 = f16_bits(r.standard_normal(NCTX * kd))
            k0[POS0 * kd:] = 0; v0[POS0 * kd:] = 0
            slabs = [dict(k=k0.copy(), v=v0.copy()) for _ in range(2)]
            A = bufs(normed=ND, qg=2 * qd, q=qd, g=qd, k=kd, v=kd, attn=qd, mixed=ND)
            B = layers.buffers()

            def attention(ops, i, b, s, x, pos):
                W = lambda t: t[i]
                ops.rms_norm(x, anorm, EPS, b["normed"])
                ops.matmul(W(wq), b["normed"], b["qg"])
                ops.gather_chunks(b["qg"], AHD, 2 * AHD, 0, b["q"]); ops.gather_chunks(b["qg"], AHD, 2 * AHD, AHD, b["g"])
                ops.matmul(W(wk), b["normed"], b["k"]); ops.matmul(W(wv), b["normed"], b["v"])
                ops.rms_norm_heads(b["q"], qn, AHD, EPS); ops.rms_norm_heads(b["k"], kn, AHD, EPS)
                ops.rope_neox(b["q"], pos, AHD, NROT, NH, THETA); ops.rope_neox(b["k"], pos, AHD, NROT, NKV, THETA)
                ops.kv_write(s["k"], pos * kd, b["k"]); ops.kv_write(s["v"], pos * kd, b["v"])
                ops.attend(b["q"], s["k"], s["v"], kd, pos + 1, AHD, NH, NKV, sc, b["attn"])
                ops.sigmoid_mul(b["attn"], b["g"])
                ops.matmul(W(wo), b["attn"], b["mixed"])
                ops.add_assign(x, b["mixed"])

            def run(ops, i, is_hip, pos):
                Bi, L = B[i], layers.L
                layers.gdn(ops, i, L[0], Bi["layers"][0], Bi["x"]); layers.ffn(ops, i, L[0], Bi["layers"][0], Bi["x"], is_hip)
                attention(ops, i, A[i], slabs[i], Bi["x"], pos)
                layers.ffn(ops, i, L[1], Bi["layers"][1], Bi["x"], is_hip)
                layers.gdn(ops, i, L[2], Bi["layers"][2], Bi["x"]); layers.ffn(ops, i, L[2], Bi["layers"][2], Bi["x"], is_hip)

            xs = []
            for p in range(PASSES):
                pos = POS0 + p
                x0 = rng(800 + p).standard_normal(ND).astype(np.float32)
                print(f"chains around an attention layer (chain={chain}), pass {p} at position {pos}", flush=True)
                B[0]["x"][:] = x0
                hip.begin_pass(1); hip.host_wrote(B[0]["x"]); run(hip, 0, True, pos); hip.end_pass()
                hip.host_needs(B[0]["x"]); hip.read_kv(slabs[0]["k"]); hip.read_kv(slabs[0]["v"])
                for li in (0, 2):
                    hip.read_state(B[0]["layers"][li]["ssm"]); hip.read_state(B[0]["layers"][li]["conv_state"])
                hip.raise_if_error()
                xs.append(B[0]["x"] - x0)
                if not chain:
                    continue
                B[1]["x"][:] = x0
                run(orc, 1, False, pos)
                want = B[1]["x"].astype(np.float64) - x0
                assert np.abs(want).max() > 0.3
                assert near(xs[-1], want, 0.15), (p, far(xs[-1], want))
                a, b = B[0]["layers"][0], B[1]["layers"][0]
                assert close(a["ssm"], b["ssm"]), (p, worst(a["ssm"], b["ssm"]))
                assert close(a["conv_state"], b["conv_state"]), (p, worst(a["conv_state"], b["conv_state"]))
                for t in "kv":
                    a = slabs[0][t].view(np.float16).astype(np.float32); b = slabs[1][t].view(np.float16).astype(np.float32)
                    assert np.array_equal(a[:POS0 * kd], b[:POS0 * kd]) and not a[(pos + 1) * kd:].any()
                    assert near(a[pos * kd:(pos + 1) * kd], b[pos * kd:(pos + 1) * kd]), (p, t)
                    # the oracle goes on from the kernel's rows, so that the next position attends over the same cache
                    slabs[1][t][pos * kd:(pos + 1) * kd] = slabs[0][t][pos * kd:(pos + 1) * kd]
                for li in (0, 2):       # and from the kernel's state, so that each pass is compared on its own
                    for name in ("ssm", "conv_state"):
                        B[1]["layers"][li][name][:] = B[0]["layers"][li][name]
            g, c = hip.graph_stats(), hip.chain_stats()
            assert g["captures"] == 1 and g["aborts"] == 0 and g["replays"] == PASSES - 2, g
            if chain and attn_in_chain:
                assert c["chains"] == 1 and c["layers"] == 3 and g["graph_kernels"] == 1, (g, c)
            elif chain:
                assert c["chains"] == 2 and c["layers"] == 3 and g["graph_kernels"] == 3, (g, c)
            else:
                assert c["chains"] == 0, c
            outs.append((xs, [B[0]["layers"][li][n].copy() for li in (0, 2) for n in ("ssm", "conv_state")],
                         [slabs[0][t][POS0 * kd:(POS0 + PASSES) * kd].view(np.float16).astype(np.float32) for t in "kv"],
                         hip.expert_counts(layers.gate_raw, NE).copy()))
        finally:
            err = hip.take_error()
            hip.close()
        assert err is None, err
    (xa, sa, ka, na), (xb, sb, kb, nb) = outs
    for a, b in zip(ka, kb):
        assert near(a, b), far(a, b)
    if attn_in_chain:
        # The chain's attention takes the probabilities as exact f16 pairs, the per-stage kernel rounds the probabilities to f16 for the matrix
        # cores: 1e-4 of the attention output, which the quantization in front of the out-projection and the two blocks
        # behind turn into per cent (the docstring's measurement).  What is in front of the attention is held as
        # everywhere (layer 0's state, the new K / V rows above); what is behind it grossly here, and sharply in
        # test_the_attention_mixer_inside_a_chain_against_the_oracle.
        for p in range(PASSES):
            assert near(xa[p], xb[p], 0.15), (p, far(xa[p], xb[p]))
        for a, b in zip(sa[:2], sb[:2]):
            assert close(a, b), worst(a, b)
        return
    for p in range(PASSES):
        assert near(xa[p], xb[p]), (p, far(xa[p], xb[p]))
    for a, b in zip(sa, sb):
        assert close(a, b), worst(a, b)
    assert np.array_equal(na, nb)
