"""Every seam op on the MI355X against the CPU oracle, through the C ABI.

Exact mode: bit-identical.  Inputs are seeded; shapes cover the tiny (T) and the
35B-A3B (B) configurations, batch sizes 1 and >1, and the edge cases the reference's
own device tests plant (tests/cuda_ops.rs:236-371, 863-942, 1273-1391, 6012-6109).
"""
import numpy as np
import pytest

from util import assert_bits_equal, f16_bits, nvfp4_weights, q8_0_weights, rng

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip():
    import inferred_hip as ih
    be = ih.Hip(exact=True)
    yield be
    err = be.take_error()
    be.close()
    assert err is None, err


@pytest.fixture(scope="module")
def orc():
    from oracle import binding as ob
    return ob.Oracle(threads=1)


def fresh(hip):
    hip.drop_mirrors()
    hip.begin_pass(1)


@pytest.mark.parametrize("n,nd", [(1, 512), (5, 512), (1, 2048), (33, 2048)])
def test_rms_norm(hip, orc, n, nd):
    fresh(hip)
    r = rng(1)
    x = r.standard_normal(n * nd).astype(np.float32) * 3
    w = r.standard_normal(nd).astype(np.float32)
    a, b = np.zeros_like(x), np.zeros_like(x)
    hip.rms_norm(x, w, 1e-6, a); hip.host_needs(a)
    orc.rms_norm(x, w, 1e-6, b)
    assert_bits_equal(a, b, "rms_norm")


@pytest.mark.parametrize("heads,hd", [(8, 64), (3 * 16, 256), (7 * 32, 128)])
def test_rms_norm_heads_and_l2(hip, orc, heads, hd):
    fresh(hip)
    r = rng(2)
    x = r.standard_normal(heads * hd).astype(np.float32)
    w = r.standard_normal(hd).astype(np.float32)
    a, b = x.copy(), x.copy()
    hip.rms_norm_heads(a, w, hd, 1e-6); hip.host_needs(a)
    orc.rms_norm_heads(b, w, hd, 1e-6)
    assert_bits_equal(a, b, "rms_norm_heads")
    a, b = x.copy(), x.copy()
    a[:hd] = 0; b[:hd] = 0  # the eps clamp
    hip.host_wrote(a)
    hip.l2_norm_heads(a, hd, 1e-6); hip.host_needs(a)
    orc.l2_norm_heads(b, hd, 1e-6)
    assert_bits_equal(a, b, "l2_norm_heads")


@pytest.mark.parametrize("n_in,n_out,n", [(512, 1024, 1), (512, 16, 1), (512, 1, 3), (2048, 8192, 1),
                                            (4096, 2048, 1), (2048, 512, 7), (256, 512, 4),
                                            # 16 tokens and more take the int8 matrix-core kernel: ragged rows and tokens
                                            (2048, 2048, 16), (2048, 1000, 37), (4096, 512, 380), (512, 1024, 129),
                                            (256, 33, 200), (2048, 8, 64)])
def test_matmul_q8_0(hip, orc, n_in, n_out, n):
    import inferred_hip as ih
    from oracle import binding as ob
    fresh(hip)
    r = rng(3)
    wb = q8_0_weights(orc, r, n_out, n_in)
    x = r.standard_normal(n * n_in).astype(np.float32)
    a = np.zeros(n * n_out, np.float32); b = np.zeros_like(a)
    hip.matmul(ih.weights(wb, ih.Q8_0, n_in, n_out), x, a); hip.host_needs(a)
    orc.matmul(ob.weights(wb, ob.Q8_0, n_in, n_out), x, b)
    hip.raise_if_error()
    assert_bits_equal(a, b, "matmul q8_0")


@pytest.mark.parametrize("n_in,n_out,n", [(2048, 512, 1), (512, 2048, 1), (2048, 1024, 5), (64, 64, 2)])
def test_matmul_nvfp4(hip, orc, n_in, n_out, n):
    import inferred_hip as ih
    from oracle import binding as ob
    fresh(hip)
    r = rng(4)
    wb = nvfp4_weights(r, n_out, n_in)
    x = r.standard_normal(n * n_in).astype(np.float32)
    a = np.zeros(n * n_out, np.float32); b = np.zeros_like(a)
    hip.matmul(ih.weights(wb, ih.NVFP4, n_in, n_out), x, a); hip.host_needs(a)
    orc.matmul(ob.weights(wb, ob.NVFP4, n_in, n_out), x, b)
    hip.raise_if_error()
    assert_bits_equal(a, b, "matmul nvfp4")


@pytest.mark.parametrize("ty", ["f32", "f16", "bf16"])
def test_matmul_float_types(hip, orc, ty):
    import inferred_hip as ih
    from oracle import binding as ob
    fresh(hip)
    r = rng(5)
    n_in, n_out, n = 512, 16, 3
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
    assert_bits_equal(a, b, f"matmul {ty}")


def test_rope(hip, orc):
    fresh(hip)
    r = rng(6)
    for (n, hd, n_rot, nh, pos, theta) in [(1, 64, 16, 8, 0, 1e6), (4, 64, 16, 2, 95, 1e6), (3, 256, 64, 16, 5699, 1e7),
                                           (2, 64, 64, 2, 7, 1e4)]:
        x = r.standard_normal(n * hd * nh).astype(np.float32)
        a, b = x.copy(), x.copy()
        hip.host_wrote(a)
        hip.rope_neox(a, pos, hd, n_rot, nh, theta); hip.host_needs(a)
        orc.rope_neox(b, pos, hd, n_rot, nh, theta)
        assert_bits_equal(a, b, "rope_neox")


@pytest.mark.parametrize("n,row", [(1, 16), (5, 16), (1, 512), (9, 512)])
def test_softmax(hip, orc, n, row):
    fresh(hip)
    x = rng(7).standard_normal(n * row).astype(np.float32) * 4
    x[0] = 80.0  # large input stays finite (naive.rs:1091-1104)
    a, b = x.copy(), x.copy()
    hip.softmax(a, row); hip.host_needs(a)
    orc.softmax(b, row)
    assert_bits_equal(a, b, "softmax")


@pytest.mark.parametrize("n", [4096 + 3, 65536, 65536 + 4])  # the long ones take four elements per lane
def test_elementwise(hip, orc, n):
    fresh(hip)
    r = rng(8)
    g = (r.standard_normal(n) * 5).astype(np.float32); u = r.standard_normal(n).astype(np.float32)
    for name in ["silu_mul", "sigmoid_mul", "add_assign"]:
        a, b = g.copy(), g.copy()
        fresh(hip)  # numpy may hand a new buffer an address the backend has mirrored before
        getattr(hip, name)(a, u); hip.host_needs(a)
        getattr(orc, name)(b, u)
        assert_bits_equal(a, b, name)
    a, b = g.copy(), g.copy()
    fresh(hip)
    hip.scale(a, 0.37); hip.host_needs(a); orc.scale(b, 0.37)
    assert_bits_equal(a, b, "scale")
    a, b = g.copy(), g.copy()
    fresh(hip)
    hip.add_scaled(a, u, -1.7); hip.host_needs(a); orc.add_scaled(b, u, -1.7)
    assert_bits_equal(a, b, "add_scaled")
    logit = np.array([0.3], np.float32)
    a, b = g.copy(), g.copy()
    fresh(hip)
    hip.add_scaled_sigmoid(a, u, logit); hip.host_needs(a); orc.add_scaled_sigmoid(b, u, logit)
    assert_bits_equal(a, b, "add_scaled_sigmoid")
    rows = r.standard_normal(4 * 512).astype(np.float32); sc = r.random(4).astype(np.float32)
    a, b = np.zeros(512, np.float32), np.zeros(512, np.float32)
    fresh(hip)
    hip.add_scaled_rows(a, rows, sc); hip.host_needs(a); orc.add_scaled_rows(b, rows, sc)
    assert_bits_equal(a, b, "add_scaled_rows")


def test_gather_scatter(hip, orc):
    fresh(hip)
    src = rng(9).standard_normal(3 * 8 * 128).astype(np.float32)
    a, b = np.zeros(3 * 8 * 64, np.float32), np.zeros(3 * 8 * 64, np.float32)
    hip.gather_chunks(src, 64, 128, 64, a); hip.host_needs(a)
    orc.gather_chunks(src, 64, 128, 64, b)
    assert_bits_equal(a, b, "gather_chunks")
    da, db = np.ones(3 * 8 * 128, np.float32), np.ones(3 * 8 * 128, np.float32)
    hip.scatter_chunks(a, 64, 128, 64, da); hip.host_needs(da)
    orc.scatter_chunks(b, 64, 128, 64, db)
    assert_bits_equal(da, db, "scatter_chunks")
    # long batches move 16 bytes per lane: a slice of every row, as the model cuts q, k, v and gates apart
    for rows, chunk, stride, offset in [(300, 256, 1024, 512), (64, 512, 516, 4), (200, 128, 1024, 130)]:
        fresh(hip)
        src = rng(10).standard_normal(rows * stride).astype(np.float32)
        a, b = np.zeros(rows * chunk, np.float32), np.zeros(rows * chunk, np.float32)
        hip.gather_chunks(src, chunk, stride, offset, a); hip.host_needs(a)
        orc.gather_chunks(src, chunk, stride, offset, b)
        assert_bits_equal(a, b, f"gather_chunks {rows}x{chunk}")


def test_kv_write(hip, orc):
    fresh(hip)
    src = (rng(10).standard_normal(3 * 128) * 100).astype(np.float32)
    src[:4] = [65504.0, 65520.0, 1e-8, -6.1e-5]
    a, b = np.zeros(16 * 128, np.uint16), np.zeros(16 * 128, np.uint16)
    hip.kv_write(a, 5 * 128, src); hip.read_kv(a)
    orc.kv_write(b, 5 * 128, src)
    assert np.array_equal(a, b)


@pytest.mark.parametrize("n_tok,nc,kernel", [(1, 1024, 4), (6, 1024, 4), (1, 8192, 4), (3, 8192, 4),
                                              # token chunks, and from 64 tokens on four channels per lane
                                              (40, 1024, 4), (70, 1024, 4), (130, 8192, 4), (97, 512, 2), (64, 512, 3),
                                              (81, 1028, 5), (66, 1022, 4)])
def test_ssm_conv(hip, orc, n_tok, nc, kernel):
    fresh(hip)
    r = rng(11)
    sa = r.standard_normal(nc * (kernel - 1)).astype(np.float32); sb = sa.copy()
    x = r.standard_normal(n_tok * nc).astype(np.float32)
    w = r.standard_normal(nc * kernel).astype(np.float32)
    a, b = np.zeros_like(x), np.zeros_like(x)
    hip.ssm_conv(sa, x, w, kernel, a); hip.host_needs(a); hip.read_state(sa)
    orc.ssm_conv(sb, x, w, kernel, b)
    assert_bits_equal(a, b, "ssm_conv out")
    assert_bits_equal(sa, sb, "ssm_conv state")


def l2n(x, hd):
    x = x.reshape(-1, hd)
    return (x / np.linalg.norm(x, axis=1, keepdims=True)).astype(np.float32).reshape(-1)


@pytest.mark.parametrize("n_tok,dk,nk,nv", [(1, 64, 4, 8), (5, 64, 4, 8), (1, 128, 16, 32), (3, 128, 16, 32)])
def test_delta_rule(hip, orc, n_tok, dk, nk, nv):
    fresh(hip)
    r = rng(12)
    dv = dk
    q = l2n(r.standard_normal(n_tok * nk * dk), dk); k = l2n(r.standard_normal(n_tok * nk * dk), dk)
    v = r.standard_normal(n_tok * nv * dv).astype(np.float32)
    alpha = r.standard_normal(n_tok * nv).astype(np.float32); alpha[0] = 25.0  # the softplus cutoff
    beta = r.standard_normal(n_tok * nv).astype(np.float32)
    ssm_a = -np.exp(r.standard_normal(nv)).astype(np.float32); dt = r.standard_normal(nv).astype(np.float32)
    sa = (r.standard_normal(nv * dk * dv) * 0.1).astype(np.float32); sb = sa.copy()
    a, b = np.zeros(n_tok * nv * dv, np.float32), np.zeros(n_tok * nv * dv, np.float32)
    hip.delta_rule(q, k, v, alpha, beta, ssm_a, dt, dk, dv, nk, nv, sa, a); hip.host_needs(a); hip.read_state(sa)
    orc.delta_rule(q, k, v, alpha, beta, ssm_a, dt, dk, dv, nk, nv, sb, b)
    hip.raise_if_error()
    assert_bits_equal(a, b, "delta_rule out")
    assert_bits_equal(sa, sb, "delta_rule state")


@pytest.mark.parametrize("n_q,n_pos,hd,nh,nkv", [(1, 1, 64, 8, 2), (1, 96, 64, 8, 2), (7, 40, 64, 8, 2),
                                                  (1, 300, 256, 16, 2), (3, 130, 256, 16, 2)])
def test_attend_exact(hip, orc, n_q, n_pos, hd, nh, nkv):
    fresh(hip)
    r = rng(13)
    kv_dim = nkv * hd
    q = r.standard_normal(n_q * nh * hd).astype(np.float32)
    k = f16_bits(r.standard_normal((n_pos + 3) * kv_dim)); v = f16_bits(r.standard_normal((n_pos + 3) * kv_dim))
    a, b = np.zeros(n_q * nh * hd, np.float32), np.zeros(n_q * nh * hd, np.float32)
    sc = 1.0 / np.sqrt(np.float32(hd))
    hip.attend(q, k, v, kv_dim, n_pos, hd, nh, nkv, sc, a); hip.host_needs(a)
    orc.attend(q, k, v, kv_dim, n_pos, hd, nh, nkv, sc, b)
    hip.raise_if_error()
    assert_bits_equal(a, b, "attend")


def planted_probs(r, n_tok, n_expert):
    p = r.random((n_tok, n_expert)).astype(np.float32)
    p /= p.sum(1, keepdims=True)
    return p


@pytest.mark.parametrize("n_tok,n_expert,n_used", [(1, 16, 4), (9, 16, 4), (1, 512, 10), (5, 512, 10), (2, 256, 8),
                                                     (301, 512, 10), (70, 1000, 16), (33, 100, 5)])
def test_route(hip, orc, n_tok, n_expert, n_used):
    import ctypes as C
    fresh(hip)
    r = rng(14)
    p = planted_probs(r, n_tok, n_expert)
    p[0, 3] = p[0, 7] = p[0].max() * 1.5        # a planted tie resolves to the lower id
    if n_tok > 1:
        p[1, :] = 1.0 / n_expert                 # all equal => 0..n_used
    if n_tok > 2:
        p[2, :] = 1e-7                           # below the 6.1e-5 clamp
    p = p.reshape(-1).copy()
    route = hip.route(p, n_expert, n_used)
    ids_o, w_o = orc.route(p, n_expert, n_used)
    # consume the device route through moe_finish with identity rows to read the weights back
    n = 4
    rows = np.zeros(n_tok * n_used * n, np.float32)
    for t in range(n_tok):
        for e in range(n_used):
            rows[(t * n_used + e) * n:(t * n_used + e + 1) * n] = [1.0 if e == j else 0.0 for j in range(n)]
    shared = np.zeros(n_tok * n, np.float32); logit = np.zeros(n_tok, np.float32)
    out = np.zeros(n_tok * n, np.float32)
    hip.moe_finish(out, 0, n, rows, route, shared, logit, 0); hip.host_needs(out)
    hip.raise_if_error()
    assert_bits_equal(out.reshape(n_tok, n), w_o.reshape(n_tok, n_used)[:, :n], "route weights")
    # ids: a one-hot expert matmul reads them back exactly
    import inferred_hip as ih
    from oracle import binding as ob
    n_in, n_out = 64, 64
    wb = q8_0_weights(orc, r, n_expert * n_out, n_in, std=1.0)
    x = r.standard_normal(n_tok * n_in).astype(np.float32)
    a = np.zeros(n_tok * n_used * n_out, np.float32); b = np.zeros_like(a)
    hip.matmul_experts(ih.experts(wb, ih.Q8_0, n_in, n_out, n_expert), route, x, a); hip.host_needs(a)
    orc.matmul_experts(ob.experts(wb, ob.Q8_0, n_in, n_out, n_expert), ids_o, n_used, x, b)
    hip.raise_if_error()
    assert_bits_equal(a, b, "experts chosen by the device route")
    if n_tok > 1:
        assert list(ids_o.reshape(n_tok, n_used)[1]) == list(range(n_used))
    assert ids_o[0] == 3


@pytest.mark.parametrize("fmt", ["q8_0", "nvfp4"])
@pytest.mark.parametrize("n_tok,n_expert,n_used,nd,ff", [(1, 16, 4, 512, 256), (6, 16, 4, 512, 256),
                                                         (1, 64, 10, 2048, 512), (3, 64, 10, 2048, 512),
                                                         # 32 pairs and more: expert-grouped tiles on the matrix cores
                                                         (37, 16, 4, 512, 256), (200, 16, 4, 512, 256),
                                                         (48, 64, 10, 2048, 512)])
def test_moe_stage(hip, orc, fmt, n_tok, n_expert, n_used, nd, ff):
    """moe_glu + matmul_experts(down) + moe_finish, host route, against the oracle's defaults."""
    import inferred_hip as ih
    from oracle import binding as ob
    fresh(hip)
    r = rng(15)
    if fmt == "q8_0":
        mk = lambda rows, n_in: q8_0_weights(orc, r, rows, n_in)
        code, scales = ih.Q8_0, [None, None, None]
    else:
        mk = lambda rows, n_in: nvfp4_weights(r, rows, n_in)
        code = ih.NVFP4
        scales = [(r.random(n_expert).astype(np.float32) * 0.01 + 0.002) for _ in range(3)]
    gate, up, down = mk(n_expert * ff, nd), mk(n_expert * ff, nd), mk(n_expert * nd, ff)
    x = r.standard_normal(n_tok * nd).astype(np.float32)
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
    assert_bits_equal(ga, gb, "moe_glu")
    oa, obuf = np.zeros(pairs * nd, np.float32), np.zeros(pairs * nd, np.float32)
    hip.matmul_experts(ih.experts(down, code, ff, nd, n_expert, scales[2]), route, ga, oa)
    orc.matmul_experts(ob.experts(down, code, ff, nd, n_expert, scales[2]), ids, n_used, gb, obuf)
    hip.host_needs(oa); hip.raise_if_error()
    assert_bits_equal(oa, obuf, "matmul_experts(down)")
    shared = r.standard_normal(n_tok * nd).astype(np.float32); logit = r.standard_normal(n_tok).astype(np.float32)
    fa, fb = np.zeros(n_tok * nd, np.float32), np.zeros(n_tok * nd, np.float32)
    hip.moe_finish(fa, 0, nd, oa, route, shared, logit, 0); hip.host_needs(fa)
    orc.moe_finish(fb, 0, nd, obuf, w, n_used, shared, logit, 0)
    assert_bits_equal(fa, fb, "moe_finish")


@pytest.mark.parametrize("n_tok,n_used,nd", [(20, 8, 512), (33, 5, 256), (16, 10, 2048), (40, 4, 516), (15, 8, 512)])
def test_moe_finish_batches(hip, orc, n_tok, n_used, nd):
    """The weighted sum of the picks' rows plus the gated shared expert, in pick order, for the batch shapes
    that take four outputs per lane and the ones that do not."""
    import inferred_hip as ih
    fresh(hip)
    r = rng(21)
    rows = r.standard_normal(n_tok * n_used * nd).astype(np.float32)
    ids = np.zeros(n_tok * n_used, np.uint32); w = r.random(n_tok * n_used).astype(np.float32)
    shared = r.standard_normal(n_tok * nd).astype(np.float32); logit = r.standard_normal(n_tok + 2).astype(np.float32)
    fa, fb = np.zeros(n_tok * nd + 8, np.float32), np.zeros(n_tok * nd + 8, np.float32)
    hip.moe_finish(fa, 8, nd, rows, ih.Hip.host_route(ids, w, n_used), shared, logit, 2); hip.host_needs(fa)
    orc.moe_finish(fb, 8, nd, rows, w, n_used, shared, logit, 2)
    assert_bits_equal(fa, fb, "moe_finish")


def test_quantized_activation_cache_is_invalidated(hip, orc):
    """A second matmul on a rewritten buffer must re-quantize it (residency.rs:40-56)."""
    import inferred_hip as ih
    from oracle import binding as ob
    fresh(hip)
    r = rng(16)
    wb = q8_0_weights(orc, r, 64, 512)
    x = r.standard_normal(512).astype(np.float32)
    a = np.zeros(64, np.float32); b = np.zeros(64, np.float32)
    W = ih.weights(wb, ih.Q8_0, 512, 64)
    hip.matmul(W, x, a)
    hip.scale(x, 3.0)            # device-side write
    hip.matmul(W, x, a); hip.host_needs(a)
    x2 = x.copy(); orc.scale(x2, 3.0)
    orc.matmul(ob.weights(wb, ob.Q8_0, 512, 64), x2, b)
    assert_bits_equal(a, b, "matmul after an in-place write")
    x[:] = r.standard_normal(512).astype(np.float32); hip.host_wrote(x)
    hip.matmul(W, x, a); hip.host_needs(a)
    orc.matmul(ob.weights(wb, ob.Q8_0, 512, 64), x, b)
    assert_bits_equal(a, b, "matmul after host_wrote")


def test_argmax_ties_to_lower_index(hip, orc):
    fresh(hip)
    x = rng(17).standard_normal(151936).astype(np.float32)
    x[100000] = x[777] = 9.5
    assert hip.argmax(x) == 777 == orc.argmax(x)
    x[:] = 1.0; hip.host_wrote(x)
    assert hip.argmax(x) == 0


def test_empty_inputs_launch_nothing(hip, orc):
    """Zero tokens / zero elements: every op returns without an error and without a launch, as the reference's
    loops over empty slices do (ops/naive.rs walks `chunks_exact` of empty slices; ops/cuda/ops/mod.rs:91-110 checks
    shapes before any launch)."""
    import inferred_hip as ih
    fresh(hip)
    r = rng(5)
    e = np.zeros(0, np.float32)
    e2 = np.zeros(0, np.float32)
    before = hip.launch_count()
    hip.rms_norm(e, np.ones(512, np.float32), 1e-6, e2)
    hip.rms_norm_heads(e, np.ones(64, np.float32), 64, 1e-6)
    hip.l2_norm_heads(e, 64, 1e-6)
    hip.softmax(e, 16)
    hip.silu_mul(e, e2)
    hip.sigmoid_mul(e, e2)
    hip.add_assign(e, e2)
    hip.scale(e, 2.0)
    hip.rope_neox(e, 0, 64, 16, 8, 1e6)
    w = ih.weights(q8_0_weights(orc, r, 32, 512), ih.Q8_0, 512, 32)
    hip.matmul(w, e, e2)
    state = np.zeros(1024 * 3, np.float32)
    s0 = state.copy()
    hip.ssm_conv(state, e, np.ones(1024 * 4, np.float32), 4, e2)
    assert hip.take_error() is None
    assert hip.launch_count() == before
    hip.host_needs(state)
    assert np.array_equal(state, s0)


def test_shape_errors_are_sticky_not_fatal(hip):
    """A bad shape records an error and launches nothing (ops/cuda/ops/mod.rs:91-110)."""
    x = np.zeros(100, np.float32); w = np.zeros(64, np.float32); out = np.zeros(100, np.float32)
    hip.rms_norm(x, w, 1e-6, out)
    assert "rms_norm" in (hip.take_error() or "")
    assert hip.take_error() is None


def test_mfma_ceilings_are_measured(hip):
    """The back-to-back MFMA loop gives a rate for every instruction kind; the rates sit below the published
    dense peaks (5 POP/s int8, 2.5 PFLOP/s f16, 157.3 TFLOP/s fp32 with some slack for clocks above nominal)
    and above a tenth of them, and the 64-deep int8 instruction is not slower than the 32-deep one."""
    import inferred_hip as ih
    peak = {"int8_16x16x64": 5000e12, "int8_16x16x32": 5000e12, "f16_32x32x16": 2500e12, "f16_16x16x32": 2500e12,
            "f32_16x16x4": 157.3e12}
    got = {k: hip.mfma_ceiling(k, 4000) for k in ih.Hip.MFMA_KINDS}
    for k, v in got.items():
        assert 0.1 * peak[k] < v < 1.25 * peak[k], (k, v)
    assert got["int8_16x16x64"] >= 0.95 * got["int8_16x16x32"]
    with pytest.raises(KeyError):
        hip.mfma_ceiling("f64_16x16x4")
