"""Expert matmuls of a small batch in fast mode against the CPU oracle, through the C ABI.

From 1.25 pairs per expert on, fast mode sorts the (token, pick) pairs by expert.  NVFP4 experts then run tiles of 16
pairs on the f16 matrix cores (k_gemm_f16s.hip: weights exact in f16, activations as an f16 hi + lo pair) up to 48 pairs
per expert; Q8_0 experts, and shapes that kernel does not take, stream every touched expert's rows once and multiply by
the integer dots of the CPU path (k_moe_rows.hip) until the int8 tiles pay.  Only the f32 summation order (and the 2^-22
of the split) differs from the oracle, so the bound is 2e-5 of the row's largest output, fifty times tighter than the
mode's 1e-3.  Covered: NVFP4 and Q8_0; the gate/up pair with silu and a single matrix; rows of 8 .. 128 units; experts
with no pair, with one pair, with more than one tile; a ragged row count; the activation row per token and per pair;
the dense form (shared expert, 2 .. 512 tokens).
"""
import numpy as np
import pytest

from util import nvfp4_weights, q8_0_weights, rng

pytestmark = pytest.mark.gpu
TOL = 2e-5


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
    return ob.Oracle(threads=8)


def fresh(hip, n):
    hip.drop_mirrors()
    hip.begin_pass(n)


def row_close(a, b, n_rows, tol=TOL):
    a = a.reshape(n_rows, -1); b = b.reshape(n_rows, -1)
    scale = np.abs(b).max(axis=1, keepdims=True) + 1e-30
    err = np.abs(a - b) / scale
    return bool(np.all(err <= tol)), float(err.max())


def make(r, orc, fmt, rows, n_in):
    import inferred_hip as ih
    if fmt == ih.NVFP4:
        return nvfp4_weights(r, rows, n_in)
    return q8_0_weights(orc, r, rows, n_in, std=0.05)


@pytest.mark.parametrize("fmt_name", ["nvfp4", "q8_0"])
@pytest.mark.parametrize("n_tok,n_expert,n_used,nd,ff", [
    (8, 512, 10, 2048, 512),      # the baseline's expert FFN at 8 tokens: below 1.25 pairs per expert, one GEMV per pair
    (64, 512, 10, 2048, 512),     # ... at 64 tokens: 16-pair tiles (NVFP4), rows streamed once (Q8_0)
    (40, 16, 4, 512, 256),        # 20 pairs on each of 8 experts: two tiles per expert; Q8_0 on the int8 tiles
    (40, 64, 4, 512, 256),        # 2.5 pairs per expert: Q8_0 on the row kernel, 16 and 8 lanes per row
    (20, 32, 4, 1024, 100),       # a ragged row count (100 rows); 32 lanes per row
    (24, 16, 2, 4096, 64),        # rows of 128 units (two passes of 64 lanes), 3 pairs per expert
    (33, 8, 1, 4096, 64),         # top-1
    (100, 64, 10, 256, 2048),     # 15.6 pairs per expert
    (150, 32, 10, 512, 256),      # 47 pairs per expert on average (94 on the busy half): just below the switch to the 128-pair tiles
])
def test_expert_rows_glu_and_down(hip, orc, fmt_name, n_tok, n_expert, n_used, nd, ff):
    import inferred_hip as ih
    from oracle import binding as ob
    code = ih.NVFP4 if fmt_name == "nvfp4" else ih.Q8_0
    fresh(hip, n_tok)
    r = rng(71)
    scales = [(r.random(n_expert).astype(np.float32) * 0.01 + 0.002) for _ in range(3)] if code == ih.NVFP4 else [None] * 3
    gate, up = make(r, orc, code, n_expert * ff, nd), make(r, orc, code, n_expert * ff, nd)
    x = (r.standard_normal(n_tok * nd) * np.repeat(10.0 ** r.uniform(-2.0, 1.0, n_tok), nd)).astype(np.float32)
    # a skewed draw: half of the experts take all the pairs, the others none
    pref = r.permutation(n_expert)
    ids = np.stack([pref[np.sort(r.choice(max(n_used, n_expert // 2), n_used, replace=False))] for _ in range(n_tok)])
    ids = ids.astype(np.uint32).reshape(-1)
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
    assert np.isfinite(gb).all()
    ok, worst = row_close(ga, gb, pairs, 1e-4)   # silu through the hardware exponential
    assert ok, worst
    if ff % 64:
        return   # the down matrix would have rows that are not whole blocks
    down = make(r, orc, code, n_expert * nd, ff)
    oa, obuf = np.zeros(pairs * nd, np.float32), np.zeros(pairs * nd, np.float32)
    hip.matmul_experts(ih.experts(down, code, ff, nd, n_expert, scales[2]), route, gb, oa)      # one row per pair
    orc.matmul_experts(ob.experts(down, code, ff, nd, n_expert, scales[2]), ids, n_used, gb, obuf)
    hip.host_needs(oa); hip.raise_if_error()
    ok, worst = row_close(oa, obuf, pairs)
    assert ok, worst
    # the same matrix over one row per token (the gate/up products' addressing without the silu)
    single = make(r, orc, code, n_expert * ff, nd)
    ta, tb = np.zeros(pairs * ff, np.float32), np.zeros(pairs * ff, np.float32)
    hip.matmul_experts(ih.experts(single, code, nd, ff, n_expert, scales[0]), route, x, ta)
    orc.matmul_experts(ob.experts(single, code, nd, ff, n_expert, scales[0]), ids, n_used, x, tb)
    hip.host_needs(ta); hip.raise_if_error()
    ok, worst = row_close(ta, tb, pairs)
    assert ok, worst


@pytest.mark.parametrize("fmt_name,n_in,n_out,n", [("nvfp4", 2048, 512, 8), ("nvfp4", 2048, 512, 128), ("nvfp4", 2048, 512, 200),
                                                   ("nvfp4", 512, 2048, 129), ("nvfp4", 2048, 512, 512), ("nvfp4", 256, 100, 130),
                                                   ("nvfp4", 4096, 64, 131), ("q8_0", 2048, 512, 2), ("q8_0", 512, 2048, 9)])
def test_dense_rows(hip, orc, fmt_name, n_in, n_out, n):
    """A dense quantized matrix over a short batch: NVFP4 from 128 to 512 tokens runs on the row kernel, eight or sixteen
    tokens per pass over the rows (ragged token and row counts included); shorter batches and Q8_0 below the 16 tokens
    of its matrix-core kernel are one GEMV per token."""
    import inferred_hip as ih
    from oracle import binding as ob
    code = ih.NVFP4 if fmt_name == "nvfp4" else ih.Q8_0
    fresh(hip, n)
    r = rng(72)
    wb = make(r, orc, code, n_out, n_in)
    x = (r.standard_normal(n * n_in) * np.repeat(10.0 ** r.uniform(-2.0, 1.0, n), n_in)).astype(np.float32)
    a = np.zeros(n * n_out, np.float32); b = np.zeros_like(a)
    hip.matmul(ih.weights(wb, code, n_in, n_out), x, a); hip.host_needs(a)
    orc.matmul(ob.weights(wb, code, n_in, n_out), x, b)
    hip.raise_if_error()
    assert np.isfinite(b).all()
    ok, worst = row_close(a, b, n)
    assert ok, worst
