"""The routed FFN of a short batch (2..32 tokens) in fast mode, against the CPU oracle's separate ops.

A batch pass issues the block op by op (/root/reference src/model/qwen35.rs:1587-1700: rms_norm, gather, router +
shared-gate logit, softmax, route, the picks' gate / up, their down products, the shared expert, moe_finish, the
residual).  From the softmax on the backend holds the ops back and, once the run is complete, issues it as two launches
whose grid rows are the tokens: gate / up with the route inside, then down + combine.  Shapes are config 2's / config
5's layer: 512 NVFP4 experts top-10, 2048 -> 512 -> 2048, a Q8_0 or an NVFP4 shared expert (the second with its three
per-tensor scales).

Compared with the oracle per pass: the FFN's output row by row, |error| <= 2e-3 * max(|value|, rms of the row) (the
two Q8_0 re-quantizations inside the block are step functions of fast mode's last bits: the bound is against the row's
scale, as for the layer chain); the picks of every token exactly (the expert cache's device-side read counters); and the
same pass with the run switched off (INFERRED_HIP_NO_SMALL_FFN) to the same bounds.  The number of launches says that
the run was taken: 2 instead of 12 behind the router product.
"""
import os

import numpy as np
import pytest

from test_gpu_chain import Layers, make_pair, near, far, ND, NE, NU, FF, SFF, EPS
from util import rng

pytestmark = pytest.mark.gpu


def ffn_batch(layers, ops, i, d, b, x, n, is_hip):
    """Layers.ffn over n rows (the reference's moe_batch)."""
    W = lambda t: t[i]
    ops.rms_norm(x, d["ffn_norm"], EPS, b["fnormed"])
    ops.gather_chunks(b["fnormed"], n * ND, n * ND, 0, b["e_in"])
    ops.matmul_pair(W(d["router"]), W(d["sh_inp"]), b["e_in"], b["router"], b["logit"])
    ops.softmax(b["router"], NE)
    ids = None
    if is_hip:
        route = ops.route(b["router"], NE, NU)
        ops.moe_glu(W(layers.gate), W(layers.up), route, b["e_in"], b["g_all"], b["u_all"])
        ops.matmul_experts(W(layers.down), route, b["g_all"], b["o_all"])
    else:
        ids, w = ops.route(b["router"], NE, NU)
        ops.moe_glu(W(layers.gate), W(layers.up), ids, NU, b["e_in"], b["g_all"], b["u_all"])
        ops.matmul_experts(W(layers.down), ids, NU, b["g_all"], b["o_all"])
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


def buffers(n):
    z = lambda k: np.zeros(k, np.float32)
    return [dict(x=z(n * ND), fnormed=z(n * ND), e_in=z(n * ND), router=z(n * NE), logit=z(n), g_all=z(n * NU * FF),
                 u_all=z(n * NU * FF), o_all=z(n * NU * ND), e_gate=z(n * SFF), e_up=z(n * SFF), e_out=z(n * ND),
                 ffn_out=z(n * ND)) for _ in range(2)]


@pytest.mark.parametrize("shared", ["q8_0", "nvfp4_scaled"])
def test_short_batch_ffn_as_two_launches(shared):
    outs = {}
    for fused in (True, False):
        if not fused:
            os.environ["INFERRED_HIP_NO_SMALL_FFN"] = "1"
        try:
            pair = make_pair()
        finally:
            os.environ.pop("INFERRED_HIP_NO_SMALL_FFN", None)
        hip, orc = pair.hip, pair.orc
        try:
            layers = Layers(pair, 1, shared, seed=31)
            d = layers.L[0]
            counts_before = np.zeros(NE, np.int64)
            for n in (2, 8, 32, 16):
                B = buffers(n)
                for rep in range(2):      # the first pass of a size sizes the mirrors (which ends a held run)
                    x0 = rng(300 + 7 * n + rep).standard_normal(n * ND).astype(np.float32)
                    print(f"short batch: shared={shared} fused={fused} n={n} pass {rep}", flush=True)
                    B[0]["x"][:] = x0
                    hip.begin_pass(n); hip.host_wrote(B[0]["x"])
                    if rep:
                        hip.profile_begin()
                    ffn_batch(layers, hip, 0, d, B[0], B[0]["x"], n, True)
                    rows = hip.profile_end() if rep else None
                    hip.end_pass()
                    hip.host_needs(B[0]["x"])
                    hip.raise_if_error()
                    B[1]["x"][:] = x0
                    ids = ffn_batch(layers, orc, 1, d, B[1], B[1]["x"], n, False)
                    got, want = (B[0]["x"] - x0).reshape(n, ND), (B[1]["x"].astype(np.float64) - x0).reshape(n, ND)
                    for t in range(n):
                        assert np.abs(want[t]).max() > 0.3
                        assert near(got[t], want[t]), (n, rep, t, far(got[t], want[t]))
                    counts = hip.expert_counts(layers.gate_raw, NE).astype(np.int64)
                    want_counts = np.zeros(NE, np.int64)
                    np.add.at(want_counts, np.asarray(ids, np.int64).reshape(-1), 1)
                    assert np.array_equal(counts - counts_before, want_counts), (n, rep)
                    counts_before = counts
                    if rep:
                        launches = sum(r["launches"] for r in rows)
                        # norm (+ quantization), gather, router pair; then the run: 2 launches, or 12 and more
                        assert (launches <= 8) == fused, (fused, launches, [(r["name"], r["launches"]) for r in rows])
                        outs[(fused, n)] = got.copy()
            if fused:
                # what the run does not write is refused to the host instead of handed over stale
                hip.host_needs(B[0]["o_all"])
                err = hip.take_error()
                assert err is not None and "fused kernel" in err, err
        finally:
            err = hip.take_error()
            hip.close()
        assert err is None, err
    for n in (2, 8, 16, 32):
        a, b = outs[(True, n)], outs[(False, n)]
        for t in range(n):
            assert near(a[t], b[t]), (n, t, far(a[t], b[t]))
