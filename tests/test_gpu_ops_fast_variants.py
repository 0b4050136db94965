"""Fast mode (the mode bench.py measures) op by op against the CPU oracle: the variants that only long batches select.

tests/test_gpu_ops_fast.py covers attention, the delta rule, the NVFP4 expert products, unquantized matmuls and the
head norms.  Here are the rest of the seam ops at the sizes where the backend switches to its fast-mode kernels in a
prefill pass: the four-per-lane silu / sigmoid products with the exponential on the transcendental unit (65,536
elements and more), the row softmax, the chunked causal conv (64 tokens and more), the four-per-lane routed-FFN
combine (16 tokens and more), Q8_0 dense products (GEMV and int8 matrix-core tiles), matmul_pair, and the routed
FFN with Q8_0 experts.  Bound: rel/abs 1e-3 (util.bound); the observed error is printed by a failing assert.
"""
import numpy as np
import pytest

from util import close, q8_0_weights, rng, worst

pytestmark = pytest.mark.gpu


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


def fresh(hip, n=1):
    hip.drop_mirrors()
    hip.begin_pass(n)


@pytest.mark.parametrize("n", [65536, 65536 + 4, 1 << 20, 5700 * 4096])
def test_silu_and_sigmoid_products(hip, orc, n):
    r = rng(8)
    g = (r.standard_normal(n) * 5).astype(np.float32); u = r.standard_normal(n).astype(np.float32)
    g[:6] = [0.0, -0.0, 88.0, -88.0, 20.0, -104.0]            # saturation on both sides, signed zero
    for name in ["silu_mul", "sigmoid_mul"]:
        a, b = g.copy(), g.copy()
        fresh(hip, 64)
        getattr(hip, name)(a, u); hip.host_needs(a)
        getattr(orc, name)(b, u)
        hip.raise_if_error()
        assert np.isfinite(a).all()
        assert close(a, b, 1e-5), (name, worst(a, b))          # one or two ulps of the exponential


@pytest.mark.parametrize("n,row", [(1, 16), (1, 512), (9, 512), (700, 512), (64, 16), (33, 1000)])
def test_softmax(hip, orc, n, row):
    fresh(hip, n)
    x = rng(7).standard_normal(n * row).astype(np.float32) * 4
    x[0] = 80.0
    a, b = x.copy(), x.copy()
    hip.softmax(a, row); hip.host_needs(a)
    orc.softmax(b, row)
    hip.raise_if_error()
    assert close(a, b, 1e-5), worst(a, b)
    assert np.allclose(a.reshape(n, row).sum(1), 1.0, atol=1e-5)


@pytest.mark.parametrize("n_tok,nc,kernel", [(64, 8192, 4), (70, 1024, 4), (130, 8192, 4), (5700, 8192, 4), (97, 512, 2),
                                              (64, 512, 3), (81, 1028, 5)])
def test_ssm_conv(hip, orc, n_tok, nc, kernel):
    fresh(hip, n_tok)
    r = rng(11)
    sa = r.standard_normal(nc * (kernel - 1)).astype(np.float32); sb = sa.copy()
    x = r.standard_normal(n_tok * nc).astype(np.float32)
    w = r.standard_normal(nc * kernel).astype(np.float32)
    a, b = np.zeros_like(x), np.zeros_like(x)
    hip.ssm_conv(sa, x, w, kernel, a); hip.host_needs(a); hip.read_state(sa)
    orc.ssm_conv(sb, x, w, kernel, b)
    hip.raise_if_error()
    assert close(a, b, 1e-5), worst(a, b)
    assert np.array_equal(sa, sb)                              # the window is a copy of the last inputs


@pytest.mark.parametrize("n_tok,n_used,nd", [(20, 8, 512), (33, 5, 256), (16, 10, 2048), (40, 4, 516), (600, 10, 2048)])
def test_moe_finish(hip, orc, n_tok, n_used, nd):
    import inferred_hip as ih
    fresh(hip, n_tok)
    r = rng(21)
    rows = r.standard_normal(n_tok * n_used * nd).astype(np.float32)
    ids = np.zeros(n_tok * n_used, np.uint32); w = r.random(n_tok * n_used).astype(np.float32)
    shared = r.standard_normal(n_tok * nd).astype(np.float32); logit = (r.standard_normal(n_tok + 2) * 4).astype(np.float32)
    fa, fb = np.zeros(n_tok * nd + 8, np.float32), np.zeros(n_tok * nd + 8, np.float32)
    hip.moe_finish(fa, 8, nd, rows, ih.Hip.host_route(ids, w, n_used), shared, logit, 2); hip.host_needs(fa)
    orc.moe_finish(fb, 8, nd, rows, w, n_used, shared, logit, 2)
    hip.raise_if_error()
    assert close(fa, fb, 1e-5), worst(fa, fb)


@pytest.mark.parametrize("n_in,n_out,n", [(512, 1024, 1), (512, 16, 1), (512, 1, 3), (2048, 8192, 1), (4096, 2048, 1),
                                            (2048, 512, 7), (2048, 2048, 16), (2048, 1000, 37), (4096, 512, 380),
                                            (256, 33, 200), (2048, 8, 64), (2048, 12352, 600)])
def test_matmul_q8_0(hip, orc, n_in, n_out, n):
    import inferred_hip as ih
    from oracle import binding as ob
    fresh(hip, n)
    r = rng(3)
    wb = q8_0_weights(orc, r, n_out, n_in)
    x = r.standard_normal(n * n_in).astype(np.float32)
    a = np.zeros(n * n_out, np.float32); b = np.zeros_like(a)
    hip.matmul(ih.weights(wb, ih.Q8_0, n_in, n_out), x, a); hip.host_needs(a)
    orc.matmul(ob.weights(wb, ob.Q8_0, n_in, n_out), x, b)
    hip.raise_if_error()
    assert close(a, b, 1e-5), worst(a, b)


@pytest.mark.parametrize("ty", ["q8_0", "f32"])
@pytest.mark.parametrize("n_in,n_a,n_b,n", [(2048, 512, 1, 1), (2048, 512, 1, 5), (2048, 32, 32, 1), (2048, 32, 32, 70),
                                              (512, 16, 1, 3)])
def test_matmul_pair(hip, orc, ty, n_in, n_a, n_b, n):
    """The router + shared-gate logit pair and the ssm alpha / beta pair, quantized (this build's config 5) and F32
    (what real files keep them in), one token and a batch."""
    import inferred_hip as ih
    from oracle import binding as ob
    fresh(hip, n)
    r = rng(33)

    def mk(rows):
        if ty == "q8_0":
            return q8_0_weights(orc, r, rows, n_in, std=1.0 / np.sqrt(n_in)), ih.Q8_0
        return (r.standard_normal((rows, n_in)) / np.sqrt(n_in)).astype(np.float32).view(np.uint8).reshape(-1).copy(), ih.F32
    (wa, code), (wb, _) = mk(n_a), mk(n_b)
    x = r.standard_normal(n * n_in).astype(np.float32)
    oa, ob_ = np.zeros(n * n_a, np.float32), np.zeros(n * n_b, np.float32)
    ra, rb = np.zeros_like(oa), np.zeros_like(ob_)
    hip.matmul_pair(ih.weights(wa, code, n_in, n_a), ih.weights(wb, code, n_in, n_b), x, oa, ob_)
    hip.host_needs(oa); hip.host_needs(ob_)
    orc.matmul_pair(ob.weights(wa, code, n_in, n_a), ob.weights(wb, code, n_in, n_b), x, ra, rb)
    hip.raise_if_error()
    assert close(oa, ra, 1e-4), worst(oa, ra)
    assert close(ob_, rb, 1e-4), worst(ob_, rb)


@pytest.mark.parametrize("n_tok,n_expert,n_used,nd,ff", [(1, 16, 4, 512, 256), (6, 16, 4, 512, 256), (1, 64, 10, 2048, 512),
                                                         (37, 16, 4, 512, 256), (200, 16, 4, 512, 256),
                                                         (48, 64, 10, 2048, 512), (600, 16, 4, 512, 256)])
def test_moe_stage_q8_0(hip, orc, n_tok, n_expert, n_used, nd, ff):
    """moe_glu + matmul_experts(down) + moe_finish with Q8_0 experts (config 1's format) in fast mode."""
    import inferred_hip as ih
    from oracle import binding as ob
    fresh(hip, n_tok)
    r = rng(15)
    mk = lambda rows, n_in: q8_0_weights(orc, r, rows, n_in, std=1.0 / np.sqrt(n_in))
    gate, up, down = mk(n_expert * ff, nd), mk(n_expert * ff, nd), mk(n_expert * nd, ff)
    x = r.standard_normal(n_tok * nd).astype(np.float32)
    ids = np.stack([r.permutation(n_expert)[:n_used] for _ in range(n_tok)]).astype(np.uint32).reshape(-1)
    w = r.random(n_tok * n_used).astype(np.float32)
    pairs = n_tok * n_used
    route = ih.Hip.host_route(ids, w, n_used)
    E = lambda lib, d, a, b: lib.experts(d, ih.Q8_0, a, b, n_expert)
    ga, gb = np.zeros(pairs * ff, np.float32), np.zeros(pairs * ff, np.float32)
    sa, sb = np.zeros_like(ga), np.zeros_like(gb)
    hip.moe_glu(E(ih, gate, nd, ff), E(ih, up, nd, ff), route, x, ga, sa)
    orc.moe_glu(E(ob, gate, nd, ff), E(ob, up, nd, ff), ids, n_used, x, gb, sb)
    hip.host_needs(ga); hip.raise_if_error()
    assert close(ga, gb, 1e-5), worst(ga, gb)
    oa, obuf = np.zeros(pairs * nd, np.float32), np.zeros(pairs * nd, np.float32)
    hip.matmul_experts(E(ih, down, ff, nd), route, gb, oa)         # the oracle's intermediates: identical inputs
    orc.matmul_experts(E(ob, down, ff, nd), ids, n_used, gb, obuf)
    hip.host_needs(oa); hip.raise_if_error()
    assert close(oa, obuf, 1e-5), worst(oa, obuf)
    shared = r.standard_normal(n_tok * nd).astype(np.float32); logit = r.standard_normal(n_tok).astype(np.float32)
    fa, fb = np.zeros(n_tok * nd, np.float32), np.zeros(n_tok * nd, np.float32)
    hip.moe_finish(fa, 0, nd, obuf, route, shared, logit, 0); hip.host_needs(fa)
    orc.moe_finish(fb, 0, nd, obuf, w, n_used, shared, logit, 0)
    hip.raise_if_error()
    assert close(fa, fb, 1e-5), worst(fa, fb)
