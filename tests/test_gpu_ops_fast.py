"""Fast mode (the mode bench.py measures) op by op against the CPU oracle, through the C ABI.

Fast mode keeps the oracle's integer dots and scale products but sums in wave order, runs
attention split over the context and the delta rule with rows split over lanes, so results are
held to rel/abs 1e-3 of the oracle rather than to the bit.  Shapes are the single-op
configurations of the baseline: GQA decode attention (16 q heads, 2 kv heads, head_dim 256,
contexts 1024 / 8192 / 32000, q and the result rounded to bf16), the Gated DeltaNet layer
(16 key / 32 value heads, dk = dv = 128, one decode step and a multi-token batch) and the
NVFP4 expert matmuls, plus the tiny configuration's shapes.
"""
import numpy as np
import pytest

from util import bf16_round, f16_bits, nvfp4_weights, q8_0_weights, rng

pytestmark = pytest.mark.gpu

# The NVFP4 matrix-core kernels against the oracle: every entry to 2e-5 of its row's largest (the weights are exact in
# f16, the Q8_0 activations an f16 pair of 22 bits, sums in f32 in tile order: what is left is the order of the sums,
# which is absolute in the row's scale, not relative to an entry that cancels to nearly nothing).
ROW_TOL = 2e-5


@pytest.fixture(scope="module")
def hip():
    import inferred_hip as ih
    be = ih.Hip(exact=False)
    yield be
    err = be.take_error()
    be.close()
    assert err is None, err


@pytest.fixture(scope="module")
def orc():
    from oracle import binding as ob
    o = ob.Oracle(threads=8)
    return o


def fresh(hip):
    hip.drop_mirrors()
    hip.begin_pass(1)


def close(a, b, tol=1e-3):
    """rel/abs: |a - b| <= tol * max(1, |b|) elementwise."""
    return np.all(np.abs(a - b) <= tol * np.maximum(1.0, np.abs(b)))


def l2n(x, hd):
    x = x.reshape(-1, hd)
    return (x / np.linalg.norm(x, axis=1, keepdims=True)).astype(np.float32).reshape(-1)


@pytest.mark.parametrize("n_q,n_pos,hd,nh,nkv", [(1, 1024, 256, 16, 2), (1, 8192, 256, 16, 2), (1, 32000, 256, 16, 2),
                                                  (1, 63, 64, 8, 2), (1, 200, 128, 8, 1), (5, 300, 256, 16, 2),
                                                  # the few-query kernel's edges: one key, fewer keys than a group of
                                                  # 16, a query that sees a single position, every group size it takes,
                                                  # more key ranges than the 256 splits (two tiles per block)
                                                  (1, 1, 256, 16, 2), (1, 5, 64, 8, 2), (1, 16, 128, 8, 8), (1, 17, 256, 16, 2),
                                                  (5, 5, 256, 16, 2), (16, 16, 64, 8, 2), (3, 129, 128, 4, 2), (2, 700, 64, 2, 2),
                                                  (1, 20000, 64, 8, 2), (4, 33000, 128, 8, 1),
                                                  (16, 300, 256, 16, 2),
                                                  # more than 16 queries: one pass over the keys on the f16 matrix cores
                                                  # (whole prompt; a batch at an offset; ragged last query tile; one
                                                  # to sixteen query heads per KV head)
                                                  (40, 700, 64, 8, 2), (17, 17, 256, 16, 2), (64, 64, 64, 8, 2),
                                                  (300, 300, 256, 16, 2), (100, 450, 128, 8, 1), (130, 130, 128, 4, 4),
                                                  (33, 1000, 256, 16, 2), (70, 70, 64, 16, 1), (1500, 1500, 256, 16, 2)])
def test_attend_split(hip, orc, n_q, n_pos, hd, nh, nkv):
    fresh(hip)
    r = rng(31)
    kv_dim = nkv * hd
    q = bf16_round(r.standard_normal(n_q * nh * hd).astype(np.float32))
    k = f16_bits(r.standard_normal(n_pos * kv_dim)); v = f16_bits(r.standard_normal(n_pos * kv_dim))
    a, b = np.zeros(n_q * nh * hd, np.float32), np.zeros(n_q * nh * hd, np.float32)
    sc = 1.0 / np.sqrt(np.float32(hd))
    hip.attend(q, k, v, kv_dim, n_pos, hd, nh, nkv, sc, a); hip.host_needs(a)
    orc.attend(q, k, v, kv_dim, n_pos, hd, nh, nkv, sc, b)
    hip.raise_if_error()
    assert close(a, b), np.abs(a - b).max()
    assert close(bf16_round(a), bf16_round(b), 8e-3)     # one bf16 step at most after rounding the result


# up to 63 tokens: rows split over lanes, token by token; 64 and more: chunks of 64 on fp32 MFMA (ragged last chunk,
# one chunk, the baseline's 5,700-token prefill)
@pytest.mark.parametrize("n_tok,dk,nk,nv", [(1, 128, 16, 32), (64, 128, 16, 32), (65, 128, 16, 32), (380, 128, 16, 32),
                                            (2048, 128, 16, 32), (5700, 128, 16, 32), (1, 64, 4, 8), (37, 64, 4, 8),
                                            (63, 128, 16, 32), (127, 64, 4, 8), (200, 64, 4, 8)])
def test_delta_rule_fast(hip, orc, n_tok, dk, nk, nv):
    fresh(hip)
    r = rng(32)
    dv = dk
    q = l2n(bf16_round(r.standard_normal(n_tok * nk * dk)), dk); k = l2n(bf16_round(r.standard_normal(n_tok * nk * dk)), dk)
    v = bf16_round(r.standard_normal(n_tok * nv * dv).astype(np.float32))
    alpha = r.standard_normal(n_tok * nv).astype(np.float32); alpha[0] = 25.0
    beta = r.standard_normal(n_tok * nv).astype(np.float32)
    ssm_a = -np.ones(nv, np.float32); dt = np.zeros(nv, np.float32)      # g = -softplus(alpha), as config 4 states it
    sa = (r.standard_normal(nv * dk * dv) * 0.1).astype(np.float32); sb = sa.copy()
    a, b = np.zeros(n_tok * nv * dv, np.float32), np.zeros(n_tok * nv * dv, np.float32)
    hip.delta_rule(q, k, v, alpha, beta, ssm_a, dt, dk, dv, nk, nv, sa, a); hip.host_needs(a); hip.read_state(sa)
    orc.delta_rule(q, k, v, alpha, beta, ssm_a, dt, dk, dv, nk, nv, sb, b)
    hip.raise_if_error()
    assert close(a, b), np.abs(a - b).max()
    assert close(sa, sb), np.abs(sa - sb).max()


def test_delta_rule_fast_state_carries_over_calls(hip, orc):
    """Three calls in a row on one state (chunked, token by token, chunked) equal the oracle's."""
    fresh(hip)
    r = rng(34)
    dk = dv = 128; nk, nv = 16, 32
    ssm_a = -(0.5 + r.random(nv)).astype(np.float32); dt = (r.standard_normal(nv) * 0.3).astype(np.float32)
    sa = (r.standard_normal(nv * dk * dv) * 0.1).astype(np.float32); sb = sa.copy()
    for n_tok in (150, 9, 70):
        q = l2n(r.standard_normal(n_tok * nk * dk).astype(np.float32), dk); k = l2n(r.standard_normal(n_tok * nk * dk).astype(np.float32), dk)
        v = r.standard_normal(n_tok * nv * dv).astype(np.float32)
        alpha = r.standard_normal(n_tok * nv).astype(np.float32); beta = r.standard_normal(n_tok * nv).astype(np.float32)
        a, b = np.zeros(n_tok * nv * dv, np.float32), np.zeros(n_tok * nv * dv, np.float32)
        hip.begin_pass(n_tok)
        hip.delta_rule(q, k, v, alpha, beta, ssm_a, dt, dk, dv, nk, nv, sa, a); hip.host_needs(a)
        orc.delta_rule(q, k, v, alpha, beta, ssm_a, dt, dk, dv, nk, nv, sb, b)
        hip.raise_if_error()
        assert close(a, b), (n_tok, np.abs(a - b).max())
    hip.read_state(sa)
    assert close(sa, sb), np.abs(sa - sb).max()


# NVFP4 expert matmuls over a batch: pairs grouped by expert and multiplied on the f16 matrix cores (weights exact
# in f16, activations as an f16 hi/lo pair).  Tiles of 1..4 token groups, an expert with more than one tile,
# experts with no pair at all, ragged row counts.
@pytest.mark.parametrize("n_tok,n_expert,n_used,nd,ff", [(48, 64, 10, 2048, 512), (200, 16, 4, 512, 256),
                                                         (600, 64, 10, 2048, 512), (700, 16, 4, 512, 256),
                                                         (33, 512, 10, 2048, 512), (90, 8, 2, 256, 192),
                                                         # the baseline's single-op expert FFN: 512 experts top-10,
                                                         # hidden 2048, inter 512, token sweep (1 token: test_gpu_ops)
                                                         (1, 512, 10, 2048, 512), (8, 512, 10, 2048, 512), (64, 512, 10, 2048, 512),
                                                         (512, 512, 10, 2048, 512)])
def test_moe_stage_fast_nvfp4(hip, orc, n_tok, n_expert, n_used, nd, ff):
    import inferred_hip as ih
    from oracle import binding as ob
    fresh(hip)
    hip.begin_pass(n_tok)
    r = rng(40)
    mk = lambda rows, n_in: nvfp4_weights(r, rows, n_in)
    code = ih.NVFP4
    scales = [(r.random(n_expert).astype(np.float32) * 0.01 + 0.002) for _ in range(3)]
    gate, up, down = mk(n_expert * ff, nd), mk(n_expert * ff, nd), mk(n_expert * nd, ff)
    # token magnitudes over four decades (a Q8_0 block scale is an f16: the gate/up products must stay below 8e6)
    x = (r.standard_normal(n_tok * nd) * np.repeat(10.0 ** r.uniform(-2.5, 1.5, n_tok), nd)).astype(np.float32)
    ids = np.stack([r.permutation(n_expert)[:n_used] for _ in range(n_tok)]).astype(np.uint32).reshape(-1)
    w = r.random(n_tok * n_used).astype(np.float32)
    pairs = n_tok * n_used
    route = ih.Hip.host_route(ids, w, n_used)
    ga, gb = np.zeros(pairs * ff, np.float32), np.zeros(pairs * ff, np.float32)
    sa, sb = np.zeros(pairs * ff, np.float32), np.zeros(pairs * ff, np.float32)
    hip.moe_glu(ih.experts(gate, code, nd, ff, n_expert, scales[0]), ih.experts(up, code, nd, ff, n_expert, scales[1]),
                route, x, ga, sa)
    orc.moe_glu(ob.experts(gate, code, nd, ff, n_expert, scales[0]), ob.experts(up, code, nd, ff, n_expert, scales[1]),
                ids, n_used, x, gb, sb)
    hip.host_needs(ga); hip.raise_if_error()
    scale = np.repeat(np.abs(gb.reshape(pairs, ff)).max(axis=1) + 1e-30, ff)
    assert np.all(np.abs(ga - gb) <= ROW_TOL * scale), (np.abs(ga - gb) / scale).max()
    oa, obuf = np.zeros(pairs * nd, np.float32), np.zeros(pairs * nd, np.float32)
    hip.matmul_experts(ih.experts(down, code, ff, nd, n_expert, scales[2]), route, gb, oa)
    orc.matmul_experts(ob.experts(down, code, ff, nd, n_expert, scales[2]), ids, n_used, gb, obuf)
    hip.host_needs(oa); hip.raise_if_error()
    assert np.isfinite(obuf).all()
    scale = np.repeat(np.abs(obuf.reshape(pairs, nd)).max(axis=1) + 1e-30, nd)
    assert np.all(np.abs(oa - obuf) <= ROW_TOL * scale), (np.abs(oa - obuf) / scale).max()


# A dense NVFP4 matrix over a batch (the shared expert of an NVFP4 file during prefill): from 513 tokens on it runs as
# a one-expert batch on the f16 tile kernel; below that, and in exact mode, one GEMV per token.  Ragged token counts,
# a row count that is not a multiple of the tile, the baseline's shared-expert shapes at the baseline's prompt length.
@pytest.mark.parametrize("n_in,n_out,n", [(2048, 512, 129), (2048, 512, 512), (2048, 512, 513), (512, 2048, 700),
                                          (512, 260, 641), (2048, 512, 5700), (512, 2048, 5700)])
def test_matmul_nvfp4_batched_fast(hip, orc, n_in, n_out, n):
    import inferred_hip as ih
    from oracle import binding as ob
    fresh(hip)
    hip.begin_pass(n)
    r = rng(43)
    wb = nvfp4_weights(r, n_out, n_in)
    x = (r.standard_normal(n * n_in) * np.repeat(10.0 ** r.uniform(-2.0, 1.0, n), n_in)).astype(np.float32)
    a = np.zeros(n * n_out, np.float32); b = np.zeros_like(a)
    hip.matmul(ih.weights(wb, ih.NVFP4, n_in, n_out), x, a); hip.host_needs(a)
    orc.matmul(ob.weights(wb, ih.NVFP4, n_in, n_out), x, b)
    hip.raise_if_error()
    assert np.isfinite(b).all()
    scale = np.repeat(np.abs(b.reshape(n, n_out)).max(axis=1) + 1e-30, n_out)
    assert np.all(np.abs(a - b) <= ROW_TOL * scale), (np.abs(a - b) / scale).max()
    # a second call in the same pass (the shared expert's up after its gate) reuses the token grouping
    a2 = np.zeros_like(a)
    hip.matmul(ih.weights(wb, ih.NVFP4, n_in, n_out), x, a2); hip.host_needs(a2)
    hip.raise_if_error()
    assert np.array_equal(a, a2)


def test_nvfp4_tiles_keep_subnormal_and_extreme_scales(hip, orc):
    """The f16 tile kernel takes an e4m3 scale code straight into an f16's bit fields (times 2^-8, the magnitudes
    carry the factor back): the subnormal codes 1..7, the largest code 0x7e and the not-a-number code 0x7f (zero in
    the CPU path) must come out as the CPU path has them."""
    import inferred_hip as ih
    from oracle import binding as ob
    fresh(hip)
    n_in, n_out, n = 512, 256, 600
    hip.begin_pass(n)
    r = rng(44)
    wb = nvfp4_weights(r, n_out, n_in).reshape(-1, 36)
    kinds = r.integers(0, 4, wb.shape[0])
    wb[kinds == 0, :4] = r.integers(1, 8, (int((kinds == 0).sum()), 4), dtype=np.uint8)        # subnormal scales
    wb[kinds == 1, :4] = 0x7e                                                                   # 448
    wb[kinds == 2, :4] = r.choice(np.array([0x7f, 0x00, 0x08], np.uint8), (int((kinds == 2).sum()), 4))
    wb = wb.reshape(-1).copy()
    # every row of one run is made of subnormal-scale blocks only: nothing larger hides a flushed scale
    sub = nvfp4_weights(r, n_out, n_in).reshape(-1, 36)
    sub[:, :4] = r.integers(1, 8, (sub.shape[0], 4), dtype=np.uint8)
    sub = sub.reshape(-1).copy()
    x = r.standard_normal(n * n_in).astype(np.float32)
    for w_bytes in (wb, sub):
        a = np.zeros(n * n_out, np.float32); b = np.zeros_like(a)
        hip.matmul(ih.weights(w_bytes, ih.NVFP4, n_in, n_out), x, a); hip.host_needs(a)
        orc.matmul(ob.weights(w_bytes, ih.NVFP4, n_in, n_out), x, b)
        hip.raise_if_error()
        assert np.isfinite(b).all() and np.abs(b).max() > 0
        scale = np.repeat(np.abs(b.reshape(n, n_out)).max(axis=1) + 1e-30, n_out)
        assert np.all(np.abs(a - b) <= ROW_TOL * scale), (np.abs(a - b) / scale).max()


# unquantized weights (the router and ssm alpha / beta of real files are F32): wave-split row sums for up to 16
# tokens, LDS-tiled products for more (64 x 64 tiles; 128 x 128 for 1,024 tokens and 256 rows on: the router over a prefill pass)
@pytest.mark.parametrize("ty", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("n_in,n_out,n", [(2048, 512, 1), (2048, 32, 1), (2048, 1, 5), (512, 16, 16), (2048, 512, 100),
                                          (512, 70, 17), (2048, 33, 300), (2048, 513, 1100), (512, 300, 1024)])
def test_matmul_float_types_fast(hip, orc, ty, n_in, n_out, n):
    import inferred_hip as ih
    from oracle import binding as ob
    fresh(hip)
    hip.begin_pass(n)
    r = rng(41)
    w = r.standard_normal((n_out, n_in)).astype(np.float32)
    if ty == "f32":
        wb, code = w.view(np.uint8).reshape(-1).copy(), ih.F32
    elif ty == "f16":
        wb, code = w.astype(np.float16).view(np.uint8).reshape(-1).copy(), ih.F16
    else:
        wb, code = (w.view(np.uint32) >> 16).astype(np.uint16).view(np.uint8).reshape(-1).copy(), ih.BF16
    x = r.standard_normal(n * n_in).astype(np.float32)
    a = np.zeros(n * n_out, np.float32); b = np.zeros_like(a)
    hip.matmul(ih.weights(wb, code, n_in, n_out), x, a); hip.host_needs(a)
    orc.matmul(ob.weights(wb, code, n_in, n_out), x, b)
    hip.raise_if_error()
    assert np.all(np.abs(a - b) <= 1e-3 * np.maximum(np.abs(b), np.sqrt(n_in))), np.abs(a - b).max()
    assert np.abs(a - b).max() <= 2e-4 * np.sqrt(n_in)     # f32 rounding of a different sum order, no more


@pytest.mark.parametrize("n_in,n_a,n_b,n", [(2048, 513, 1, 1100), (2048, 32, 32, 300), (512, 70, 3, 17), (2048, 513, 1, 16)])
def test_matmul_pair_float_batch(hip, orc, n_in, n_a, n_b, n):
    """Two F32 matrices read with one batch of activations (the router with the shared-gate logit, ssm alpha with beta,
    of a real file during prefill): above 16 tokens one launch serves both; rows of the second matrix follow the
    first's inside the tiles, each matrix keeps its own output."""
    import inferred_hip as ih
    from oracle import binding as ob
    fresh(hip)
    hip.begin_pass(n)
    r = rng(43)
    wa = r.standard_normal((n_a, n_in)).astype(np.float32).view(np.uint8).reshape(-1).copy()
    wb = r.standard_normal((n_b, n_in)).astype(np.float32).view(np.uint8).reshape(-1).copy()
    x = r.standard_normal(n * n_in).astype(np.float32)
    oa, ob_ = np.zeros(n * n_a, np.float32), np.zeros(n * n_b, np.float32)
    ra, rb = np.zeros_like(oa), np.zeros_like(ob_)
    hip.matmul_pair(ih.weights(wa, ih.F32, n_in, n_a), ih.weights(wb, ih.F32, n_in, n_b), x, oa, ob_)
    hip.host_needs(oa); hip.host_needs(ob_)
    orc.matmul(ob.weights(wa, ih.F32, n_in, n_a), x, ra)
    orc.matmul(ob.weights(wb, ih.F32, n_in, n_b), x, rb)
    hip.raise_if_error()
    for got, want in ((oa, ra), (ob_, rb)):
        assert np.abs(got - want).max() <= 2e-4 * np.sqrt(n_in)


@pytest.mark.parametrize("n,nd", [(1, 2048), (33, 2048), (3, 512)])
def test_rms_norm_fast(hip, orc, n, nd):
    fresh(hip)
    r = rng(33)
    x = r.standard_normal(n * nd).astype(np.float32) * 3
    w = r.standard_normal(nd).astype(np.float32)
    a, b = np.zeros_like(x), np.zeros_like(x)
    hip.rms_norm(x, w, 1e-6, a); hip.host_needs(a)
    orc.rms_norm(x, w, 1e-6, b)
    assert close(a, b, 1e-5)


@pytest.mark.parametrize("heads,hd", [(8, 64), (300, 64), (1000 * 16 + 3, 128), (257, 256), (40 * 32, 128)])
def test_head_norms_fast(hip, orc, heads, hd):
    """rms and l2 norms over heads: batches of 256 heads and more take a wave per head with the sum of
    squares added across lanes; the f64 sum only changes its order, so results stay within a few ulp."""
    fresh(hip)
    r = rng(31)
    x = (r.standard_normal(heads * hd) * 3).astype(np.float32)
    w = r.standard_normal(hd).astype(np.float32)
    a, b = x.copy(), x.copy()
    hip.rms_norm_heads(a, w, hd, 1e-6); hip.host_needs(a)
    orc.rms_norm_heads(b, w, hd, 1e-6)
    assert np.all(np.abs(a - b) <= 1e-6 * np.maximum(1.0, np.abs(b)))
    a, b = x.copy(), x.copy()
    a[:hd] = 0; b[:hd] = 0  # the eps clamp
    fresh(hip)
    hip.l2_norm_heads(a, hd, 1e-6); hip.host_needs(a)
    orc.l2_norm_heads(b, hd, 1e-6)
    assert np.all(np.abs(a - b) <= 1e-6 * np.maximum(1.0, np.abs(b)))
