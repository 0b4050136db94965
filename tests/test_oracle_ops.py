"""Closed forms and invariants that pin each oracle op independently of its own formula.

Each case is chosen so a plausible mistake (dropped term, wrong sign or index, transposed
operand, wrong grouping) fails it.  Sources of the cases: the reference's unit tests in
src/ops/naive.rs:863-1472 and tests/cuda_ops.rs:1204-1391.
"""
import numpy as np
import pytest

from oracle import binding as ob
from util import f16_bits, nvfp4_weights, q8_0_weights, rng


@pytest.fixture(scope="module")
def orc():
    return ob.Oracle(threads=1)


def test_rms_norm_three_four(orc):
    x = np.array([3, 4], np.float32); w = np.ones(2, np.float32); out = np.zeros(2, np.float32)
    orc.rms_norm(x, w, 0.0, out)
    assert np.allclose(out, np.array([3, 4]) / np.sqrt(12.5), rtol=1e-7)
    orc.rms_norm(x, np.zeros(2, np.float32), 0.0, out)
    assert (out == 0).all()
    # rows are independent
    x2 = np.array([3, 4, 30, 40], np.float32); o2 = np.zeros(4, np.float32)
    orc.rms_norm(x2, w, 0.0, o2)
    assert np.allclose(o2[:2], o2[2:])


def test_rms_norm_matches_float64_and_uses_f64_accumulation(orc):
    r = rng(0)
    x = r.standard_normal(4096).astype(np.float32) * 7; w = r.standard_normal(4096).astype(np.float32)
    out = np.zeros_like(x)
    orc.rms_norm(x, w, 1e-6, out)
    sq = (x * x).astype(np.float64)          # f32 square, f64 accumulate
    scale = np.float32(1.0) / np.sqrt(np.float32(sq.sum() / 4096) + np.float32(1e-6), dtype=np.float32)
    assert np.array_equal(out, x * scale * w)


def test_l2_norm(orc):
    x = np.array([3, 4, 0, 0], np.float32)
    orc.l2_norm_heads(x, 2, 1e-6)
    assert np.allclose(x[:2], [0.6, 0.8], rtol=1e-7)
    assert (x[2:] == 0).all()               # eps clamps the norm: 0 / eps, not NaN
    y = np.array([1e-9, 0], np.float32)
    orc.l2_norm_heads(y, 2, 1e-6)
    assert np.isclose(y[0], 1e-3)           # scaled by 1/eps, not normalised to 1


def test_rope(orc):
    r = rng(1)
    x = r.standard_normal(2 * 64).astype(np.float32); x0 = x.copy()
    orc.rope_neox(x, 0, 64, 16, 2, 1e6)
    assert np.array_equal(x, x0)            # position 0 is the identity
    # one radian on the first pair, NEOX pairing (i, i + n_rot/2)
    v = np.zeros(8, np.float32); v[0] = 1.0
    orc.rope_neox(v, 1, 8, 4, 1, 10000.0)
    assert np.isclose(v[0], np.cos(1.0)) and np.isclose(v[2], np.sin(1.0)) and v[1] == 0
    # pair norms are preserved, the tail past n_rot passes through, row t rotates at pos + t
    y = r.standard_normal(3 * 2 * 64).astype(np.float32); y0 = y.copy()
    orc.rope_neox(y, 17, 64, 16, 2, 1e6)
    a, b = y0.reshape(3, 2, 64), y.reshape(3, 2, 64)
    assert np.array_equal(a[..., 16:], b[..., 16:])
    assert np.allclose(a[..., :8] ** 2 + a[..., 8:16] ** 2, b[..., :8] ** 2 + b[..., 8:16] ** 2, rtol=1e-5)
    z = y0.reshape(3, 2, 64)[2:].copy().reshape(-1)
    orc.rope_neox(z, 19, 64, 16, 2, 1e6)
    assert np.array_equal(z, b[2].reshape(-1))
    freq = 1e6 ** (-2.0 * 3 / 16)
    assert np.isclose(b[1, 0, 3], a[1, 0, 3] * np.cos(18 * freq) - a[1, 0, 11] * np.sin(18 * freq), rtol=1e-5)


def test_softmax(orc):
    x = np.array([1000.0, 1000.0, -1000.0, 0, 1, 2], np.float32)
    orc.softmax(x, 3)
    assert np.allclose(x[:3], [0.5, 0.5, 0.0])
    e = np.exp(np.array([0, 1, 2.0])); assert np.allclose(x[3:], e / e.sum(), rtol=1e-6)


def test_conv_tap_order_and_state_advance(orc):
    # naive.rs:1139-1159: state oldest-first; taps 1,2,3 on history 1,2,3 and 4 on the token
    state = np.array([1, 2, 3], np.float32); w = np.array([1, 10, 100, 1000], np.float32)
    x = np.array([4], np.float32); out = np.zeros(1, np.float32)
    orc.ssm_conv(state, x, w, 4, out)
    s = 1 + 20 + 300 + 4000.0
    assert np.isclose(out[0], s / (1 + np.exp(-s)))
    assert list(state) == [2, 3, 4]
    # batch == sequential calls
    r = rng(2)
    st1 = r.standard_normal(6).astype(np.float32); st2 = st1.copy()
    wt = r.standard_normal(8).astype(np.float32); xs = r.standard_normal(10).astype(np.float32)
    o1 = np.zeros(10, np.float32); o2 = np.zeros(10, np.float32)
    orc.ssm_conv(st1, xs, wt, 4, o1)
    for t in range(5):
        orc.ssm_conv(st2, xs[2 * t:2 * t + 2].copy(), wt, 4, o2[2 * t:2 * t + 2])
    assert np.array_equal(o1, o2) and np.array_equal(st1, st2)


def delta(orc, q, k, v, alpha, beta, ssm_a, dt, dk, dv, nk, nv, state):
    out = np.zeros(v.size, np.float32)
    orc.delta_rule(q.astype(np.float32), k.astype(np.float32), v.astype(np.float32), np.float32(alpha),
                   np.float32(beta), np.float32(ssm_a), np.float32(dt), dk, dv, nk, nv, state, out)
    return out


def test_delta_rule_closed_forms(orc):
    dk = dv = 4
    k = np.array([1, 0, 0, 0.0]); q = k.copy(); v = np.array([2, 4, 6, 8.0])
    z = np.zeros(1)
    # ssm_a = 0 => g = 1; beta = +40 => sigmoid = 1: an exact associative write, read back / sqrt(dk)
    st = np.zeros(16, np.float32)
    out = delta(orc, q, k, v, z, np.array([40.0]), z, z, dk, dv, 1, 1, st)
    assert np.allclose(out, v / 2)
    assert np.allclose(st.reshape(4, 4)[:, 0], v) and np.count_nonzero(st) == 4   # state is [value][key]
    # writing the same key again corrects rather than accumulates
    out2 = delta(orc, q, k, v, z, np.array([40.0]), z, z, dk, dv, 1, 1, st)
    assert np.allclose(out2, v / 2) and np.allclose(st.reshape(4, 4)[:, 0], v)
    # forget: softplus(0) * ssm_a with ssm_a = -ln2/ln2... choose g = 0.5 exactly: softplus(0) = ln 2, ssm_a = -1
    st = np.zeros(16, np.float32); st.reshape(4, 4)[:, 0] = v
    out3 = delta(orc, q, np.zeros(4), np.zeros(4), z, np.array([-40.0]), np.array([-1.0]), z, dk, dv, 1, 1, st)
    assert np.allclose(st.reshape(4, 4)[:, 0], v * 0.5, rtol=1e-6) and np.allclose(out3, v * 0.25, rtol=1e-6)
    # beta = 0 logit => half the correction
    st = np.zeros(16, np.float32)
    delta(orc, q, k, v, z, z, z, z, dk, dv, 1, 1, st)
    assert np.allclose(st.reshape(4, 4)[:, 0], v * 0.5)
    # softplus cutoff: a > 20 uses a itself
    st = np.ones(16, np.float32)
    delta(orc, np.zeros(4), np.zeros(4), np.zeros(4), np.array([30.0]), z, np.array([-0.01]), z, dk, dv, 1, 1, st)
    assert np.allclose(st, np.exp(-0.3), rtol=1e-6)


def test_delta_rule_head_grouping_is_modulo(orc):
    # ops/mod.rs:404-413: value head h reads key head h % n_k_heads => [0,1,0,1]
    dk = dv = 2; nk, nv = 2, 4
    k = np.array([1, 0, 0, 1.0]); q = k.copy()     # key head 0 = e0, key head 1 = e1
    v = np.arange(1, 9.0)
    st = np.zeros(nv * 4, np.float32)
    z4 = np.zeros(4)
    delta(orc, q, k, v, z4, np.full(4, 40.0), z4, z4, dk, dv, nk, nv, st)
    s = st.reshape(nv, dv, dk)
    for h in range(nv):
        col = h % nk
        assert np.allclose(s[h][:, col], v[2 * h:2 * h + 2]) and np.allclose(s[h][:, 1 - col], 0)


def test_delta_rule_matches_float64_recurrence(orc):
    r = rng(3)
    dk = dv = 16; nk, nv, T = 2, 4, 6
    q = r.standard_normal((T, nk, dk)); k = r.standard_normal((T, nk, dk))
    q /= np.linalg.norm(q, axis=-1, keepdims=True); k /= np.linalg.norm(k, axis=-1, keepdims=True)
    v = r.standard_normal((T, nv, dv)); al = r.standard_normal((T, nv)); be = r.standard_normal((T, nv))
    a = -np.exp(r.standard_normal(nv)); dt = r.standard_normal(nv)
    st = (r.standard_normal(nv * dv * dk) * 0.1).astype(np.float32)
    S = st.astype(np.float64).reshape(nv, dv, dk).copy()
    out = delta(orc, q.reshape(-1), k.reshape(-1), v.reshape(-1), al.reshape(-1), be.reshape(-1), a, dt, dk, dv, nk, nv, st)
    ref = np.zeros((T, nv, dv))
    for t in range(T):
        for h in range(nv):
            kh = h % nk
            g = np.exp(np.log1p(np.exp(al[t, h] + dt[h])) * a[h]); b = 1 / (1 + np.exp(-be[t, h]))
            S[h] *= g
            d = b * (v[t, h] - S[h] @ k[t, kh])
            S[h] += np.outer(d, k[t, kh])
            ref[t, h] = S[h] @ q[t, kh] / np.sqrt(dk)
    assert np.allclose(out.reshape(T, nv, dv), ref, rtol=2e-5, atol=2e-6)
    assert np.allclose(st.reshape(nv, dv, dk), S, rtol=2e-5, atol=2e-6)


def attend(orc, q, k, v, kv_dim, n_pos, hd, nh, nkv):
    out = np.zeros(q.size, np.float32)
    orc.attend(q.astype(np.float32), f16_bits(k), f16_bits(v), kv_dim, n_pos, hd, nh, nkv,
               np.float32(1 / np.sqrt(hd)), out)
    return out


def test_attend_special_cases(orc):
    r = rng(4)
    hd, nh, nkv = 8, 4, 2
    kv_dim = nkv * hd
    q = r.standard_normal(nh * hd); k = r.standard_normal(5 * kv_dim); v = r.standard_normal(5 * kv_dim)
    v16 = v.astype(np.float16).astype(np.float32).reshape(5, nkv, hd)
    # one position: the output is that position's V row of the head's kv group (division grouping)
    o = attend(orc, q, k, v, kv_dim, 1, hd, nh, nkv).reshape(nh, hd)
    for h in range(nh):
        assert np.allclose(o[h], v16[0, h // 2])
    # all-equal scores: the mean of V
    o = attend(orc, np.zeros(nh * hd), k, v, kv_dim, 5, hd, nh, nkv).reshape(nh, hd)
    assert np.allclose(o[3], v16[:, 1].mean(0), rtol=1e-6)


def test_attend_matches_float64_and_is_causal(orc):
    r = rng(5)
    hd, nh, nkv, n_pos, n_q = 16, 4, 2, 11, 3
    kv_dim = nkv * hd
    q = r.standard_normal((n_q, nh, hd)); k = r.standard_normal((n_pos, nkv, hd)); v = r.standard_normal((n_pos, nkv, hd))
    k16 = k.astype(np.float16).astype(np.float64); v16 = v.astype(np.float16).astype(np.float64)
    o = attend(orc, q.reshape(-1), k.reshape(-1), v.reshape(-1), kv_dim, n_pos, hd, nh, nkv).reshape(n_q, nh, hd)
    for t in range(n_q):
        npos_t = n_pos - n_q + 1 + t
        for h in range(nh):
            s = k16[:npos_t, h // 2] @ q[t, h].astype(np.float32).astype(np.float64) / np.sqrt(hd)
            p = np.exp(s - s.max()); p /= p.sum()
            assert np.allclose(o[t, h], p @ v16[:npos_t, h // 2], rtol=1e-5, atol=1e-6)


def test_q8_0_matmul_is_the_integer_dot_of_the_quantized_activation(orc):
    r = rng(6)
    n_in, n_out = 256, 8
    wb = q8_0_weights(orc, r, n_out, n_in, std=1.0)
    x = r.standard_normal(n_in).astype(np.float32)
    out = np.zeros(n_out, np.float32)
    orc.matmul(ob.weights(wb, ob.Q8_0, n_in, n_out), x, out)
    blocks = wb.reshape(n_out, n_in // 32, 34)
    dw = blocks[:, :, :2].copy().view(np.float16).astype(np.float32)[..., 0]
    qw = blocks[:, :, 2:].view(np.int8).astype(np.int64)
    xb = x.reshape(-1, 32)
    d = np.abs(xb).max(1) / np.float32(127)
    dx = d.astype(np.float16).astype(np.float32)
    qx = np.where(d[:, None] > 0, np.sign(xb) * np.floor(np.abs(xb * (np.float32(1) / d)[:, None]) + 0.5), 0).astype(np.int64)
    for j in range(n_out):
        acc = np.float32(0)
        for b in range(n_in // 32):
            acc = np.float32(acc + np.float32(int((qw[j, b] * qx[b]).sum())) * np.float32(dw[j, b] * dx[b]))
        assert out[j] == acc
    # and it differs from exact f32 arithmetic by the quantization error only
    wf = orc.dequantize(ob.Q8_0, wb, n_in * n_out).reshape(n_out, n_in)
    assert np.allclose(out, wf @ x, atol=0.25) and not np.array_equal(out, (wf @ x).astype(np.float32))


def test_nvfp4_matmul_against_dequantized_float64(orc):
    r = rng(7)
    n_in, n_out = 256, 6
    wb = nvfp4_weights(r, n_out, n_in)
    x = r.standard_normal(n_in).astype(np.float32)
    out = np.zeros(n_out, np.float32)
    orc.matmul(ob.weights(wb, ob.NVFP4, n_in, n_out), x, out)
    wf = orc.dequantize(ob.NVFP4, wb, n_in * n_out).reshape(n_out, n_in).astype(np.float64)
    sc, q = orc.quantize_q8_0(x)
    xq = (q.reshape(-1, 32) * sc[:, None]).reshape(-1).astype(np.float64)   # the Q8_0 activation the dot sees
    assert np.allclose(out, wf @ xq, rtol=1e-5, atol=1e-4)


def host_route_rule(p, n_used):
    # the rule transcribed at tests/cuda_ops.rs:1204-1227
    ids = []
    for _ in range(n_used):
        best = None
        for e in range(len(p)):
            if e in ids:
                continue
            if best is None or p[e] > p[best]:
                best = e
        ids.append(best)
    s = np.float32(0)
    for e in ids:
        s = np.float32(s + p[e])
    return ids, [np.float32(p[e] / max(s, np.float32(6.103515625e-5))) for e in ids]


def test_route_cases(orc):
    r = rng(8)
    cases = []
    p = r.random(16).astype(np.float32); p[3] = p[7] = 2.0; cases.append((p, 4))       # planted tie
    cases.append((np.full(16, 1 / 16, np.float32), 4))                                   # all equal => 0..n_used
    cases.append((np.full(16, 1e-7, np.float32), 4))                                     # below the clamp
    cases.append((np.arange(16, 0, -1, dtype=np.float32) / 136, 4))                      # descending
    cases.append((np.arange(1, 17, dtype=np.float32) / 136, 4))                          # ascending
    q = r.random(512).astype(np.float32); q /= q.sum(); cases.append((q, 10))            # top-10 of 512
    for p, n_used in cases:
        ids, w = orc.route(p.copy(), p.size, n_used)
        eids, ew = host_route_rule(p, n_used)
        assert list(ids) == eids
        assert np.array_equal(w, np.array(ew, np.float32))
    ids, w = orc.route(cases[0][0].copy(), 16, 4); assert list(ids[:2]) == [3, 7]
    ids, w = orc.route(cases[1][0].copy(), 16, 4); assert list(ids) == [0, 1, 2, 3] and np.allclose(w, 0.25)
    ids, w = orc.route(cases[2][0].copy(), 16, 4); assert np.allclose(w, 1e-7 / 6.103515625e-5)
    # descending probability order within a token; weights sum to 1 above the clamp
    ids, w = orc.route(cases[5][0].copy(), 512, 10)
    assert np.all(np.diff(cases[5][0][ids]) <= 0) and np.isclose(w.sum(), 1.0, rtol=1e-6)


def test_matmul_experts_row_selection_and_scale(orc):
    r = rng(9)
    n_in, n_out, n_expert, n_used, n_tok = 64, 32, 8, 2, 3
    wb = q8_0_weights(orc, r, n_expert * n_out, n_in, std=1.0)
    scale = (r.random(n_expert) + 0.5).astype(np.float32)
    ids = np.array([5, 1, 0, 7, 3, 3], np.uint32)
    stride = n_out * n_in // 32 * 34

    def single(e, x):
        o = np.zeros(n_out, np.float32)
        one = wb[int(e) * stride:(int(e) + 1) * stride].copy()   # kept alive across the call
        orc.matmul(ob.weights(one, ob.Q8_0, n_in, n_out), np.ascontiguousarray(x), o)
        return o * scale[e]
    E = ob.experts(wb, ob.Q8_0, n_in, n_out, n_expert, scale)
    # one row per token: pick i reads row i // n_used (ops/mod.rs:1069-1078)
    x_tok = r.standard_normal(n_tok * n_in).astype(np.float32)
    out = np.zeros(ids.size * n_out, np.float32)
    orc.matmul_experts(E, ids, n_used, x_tok, out)
    for i, e in enumerate(ids):
        assert np.array_equal(out[i * n_out:(i + 1) * n_out], single(e, x_tok[(i // n_used) * n_in:(i // n_used + 1) * n_in]))
    # one row per pick
    x_pick = r.standard_normal(ids.size * n_in).astype(np.float32)
    orc.matmul_experts(E, ids, n_used, x_pick, out)
    for i, e in enumerate(ids):
        assert np.array_equal(out[i * n_out:(i + 1) * n_out], single(e, x_pick[i * n_in:(i + 1) * n_in]))
    # a single shared row
    x_one = r.standard_normal(n_in).astype(np.float32)
    orc.matmul_experts(E, ids, n_used, x_one, out)
    assert np.array_equal(out[4 * n_out:5 * n_out], single(3, x_one))


def test_moe_finish_and_argmax(orc):
    n, n_used, n_tok = 4, 2, 2
    rows = np.arange(n_tok * n_used * n, dtype=np.float32)
    w = np.array([0.25, 0.75, 0.5, 0.5], np.float32)
    shared = np.ones(n_tok * n, np.float32); logit = np.array([9.0, 0.0, -50.0], np.float32)
    out = np.full(3 * n, -1, np.float32)
    orc.moe_finish(out, n, n, rows, w, n_used, shared, logit, 1)     # rows start at `at`, logits at logit_at
    assert (out[:n] == -1).all()
    assert np.allclose(out[n:2 * n], 0.25 * rows[0:4] + 0.75 * rows[4:8] + 0.5)
    assert np.allclose(out[2 * n:], 0.5 * rows[8:12] + 0.5 * rows[12:16] + 0.0, atol=1e-6)
    assert orc.argmax(np.array([1, 5, 5, 2], np.float32)) == 1       # first strict maximum
    assert orc.argmax(np.array([7, 7, 7], np.float32)) == 0


def test_threaded_backend_is_bit_identical(orc):
    r = rng(10)
    wb = q8_0_weights(orc, r, 512, 512); x = r.standard_normal(5 * 512).astype(np.float32)
    o1 = np.zeros(5 * 512, np.float32); o2 = np.zeros_like(o1)
    W = ob.weights(wb, ob.Q8_0, 512, 512)
    orc.matmul(W, x, o1)
    q = r.standard_normal(3 * 4 * 16).astype(np.float32); k = f16_bits(r.standard_normal(100 * 32)); v = f16_bits(r.standard_normal(100 * 32))
    a1 = np.zeros(q.size, np.float32); a2 = np.zeros_like(a1)
    orc.attend(q, k, v, 32, 100, 16, 4, 2, 0.25, a1)
    for threads in (2, 3, 5, 8):
        orc.set_threads(threads)
        orc.matmul(W, x, o2); orc.attend(q, k, v, 32, 100, 16, 4, 2, 0.25, a2)
        assert np.array_equal(o1, o2) and np.array_equal(a1, a2)
    orc.set_threads(1)


# ---- hand values for the small ops: each case is built so that a swapped operand, a dropped offset or a
# ---- wrong stride gives a different number

def test_silu_mul_and_sigmoid_mul_operand_roles(orc):
    ln3 = np.float32(np.log(3.0))
    # silu_mul(gate, up): gate <- gate / (1 + e^-gate) * up (src/ops/naive.rs:317-327; sigmoid(ln 3) = 3/4)
    gate = np.array([ln3, 0.0, -ln3, 2.0], np.float32); up = np.array([2.0, 5.0, 4.0, 0.0], np.float32)
    g = gate.copy(); u0 = up.copy()
    orc.silu_mul(g, up)
    assert np.allclose(g, [ln3 * 0.75 * 2.0, 0.0, -ln3 * 0.25 * 4.0, 0.0], rtol=1e-6, atol=0)
    assert np.array_equal(up, u0)                       # `up` is read only
    # with the roles swapped element 0 would be 2 * sigmoid(2) * ln 3 = 1.935, not 1.648
    assert abs(g[0] - 1.6479184) < 1e-6
    # sigmoid_mul(x, g): x <- x * sigmoid(g) (naive.rs:339-345)
    x = np.array([8.0, -4.0, 1.0], np.float32); gg = np.array([ln3, -ln3, 0.0], np.float32)
    g0 = gg.copy()
    orc.sigmoid_mul(x, gg)
    assert np.allclose(x, [6.0, -1.0, 0.5], rtol=1e-6) and np.array_equal(gg, g0)


def test_scale_and_the_add_scaled_family(orc):
    a = np.array([1.0, 2.0, 3.0], np.float32)
    orc.scale(a, 0.5)
    assert np.array_equal(a, [0.5, 1.0, 1.5])
    b = np.array([10.0, 20.0, 30.0], np.float32)
    orc.add_scaled(a, b, 0.25)                          # a += b * s (ops/mod.rs:1265-1270)
    assert np.array_equal(a, [3.0, 6.0, 9.0]) and np.array_equal(b, [10.0, 20.0, 30.0])
    # add_scaled_rows WRITES acc = sum_e scales[e] * rows[e * n + j] (ops/mod.rs:1228-1238): the old contents go
    acc = np.array([100.0, 100.0], np.float32)
    rows = np.array([1.0, 2.0, 10.0, 20.0, 100.0, 200.0], np.float32)     # three rows of two
    orc.add_scaled_rows(acc, rows, np.array([1.0, 0.5, 0.25], np.float32))
    assert np.array_equal(acc, [1.0 + 5.0 + 25.0, 2.0 + 10.0 + 50.0])
    # add_scaled_sigmoid: acc += b * sigmoid(logit[0]) (ops/mod.rs:1250-1253); only the first logit counts
    acc = np.array([1.0, 1.0], np.float32)
    orc.add_scaled_sigmoid(acc, np.array([4.0, 8.0], np.float32), np.array([np.log(3.0), -30.0], np.float32))
    assert np.allclose(acc, [4.0, 7.0], rtol=1e-6)
    a = np.array([1.0, 2.0], np.float32)
    orc.add_assign(a, np.array([0.5, -2.0], np.float32))
    assert np.array_equal(a, [1.5, 0.0])


def test_gather_and_scatter_chunks_with_offset_and_stride(orc):
    src = np.arange(20, dtype=np.float32)
    out = np.full(6, -1, np.float32)
    orc.gather_chunks(src, 2, 7, 3, out)                # chunk c reads src[c * 7 + 3 ..][:2] (naive.rs:220-232)
    assert np.array_equal(out, [3, 4, 10, 11, 17, 18])
    # the attention split: q and gate interleaved per head with stride 2 * head_dim (qwen35.rs:1176-1177)
    qg = np.arange(16, dtype=np.float32)                # two heads of [q q q q | g g g g]
    q = np.zeros(8, np.float32); g = np.zeros(8, np.float32)
    orc.gather_chunks(qg, 4, 8, 0, q); orc.gather_chunks(qg, 4, 8, 4, g)
    assert np.array_equal(q, [0, 1, 2, 3, 8, 9, 10, 11]) and np.array_equal(g, [4, 5, 6, 7, 12, 13, 14, 15])
    dst = np.full(12, -1, np.float32)
    orc.scatter_chunks(np.array([1, 2, 3, 4], np.float32), 2, 5, 1, dst)  # block i -> dst[1 + i * 5 ..][:2]
    assert np.array_equal(dst, [-1, 1, 2, -1, -1, -1, 3, 4, -1, -1, -1, -1])


def test_rms_norm_heads_normalizes_each_head_by_its_own_mean_square(orc):
    # three heads of four with very different magnitudes and a per-dimension weight: a kernel that normalized the
    # whole row, or indexed the weight by the flat position, gives other numbers
    w = np.array([1.0, 2.0, 0.5, -1.0], np.float32)
    x = np.array([3, 4, 0, 0,   30, 40, 0, 0,   0, 0, 0, 6], np.float32)
    orc.rms_norm_heads(x, w, 4, 0.0)
    # head 0: mean square 25/4 -> scale 0.4; head 1: 2500/4 -> 0.04; head 2: 36/4 -> 1/3
    want = np.array([1.2, 3.2, 0, 0,   1.2, 3.2, 0, 0,   0, 0, 0, -2.0], np.float32)
    assert np.allclose(x, want, rtol=1e-6, atol=0)
    # against float64 on random heads, eps inside the root
    r = rng(21)
    x = r.standard_normal(5 * 64).astype(np.float32) * np.repeat(10.0 ** np.arange(5), 64).astype(np.float32)
    w = r.standard_normal(64).astype(np.float32)
    ref = (x.reshape(5, 64).astype(np.float64) / np.sqrt((x.reshape(5, 64).astype(np.float64) ** 2).mean(1, keepdims=True) + 1e-6) * w).reshape(-1)
    orc.rms_norm_heads(x, w, 64, 1e-6)
    assert np.allclose(x, ref, rtol=2e-6, atol=0)


def test_kv_write_lands_at_the_offset_as_round_to_nearest_even_f16(orc):
    slab = np.full(16, 0x1234, np.uint16)
    src = np.array([1.0, -2.5, 65520.0, 1e-8, 1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11], np.float32)
    orc.kv_write(slab, 5, src)                          # slab[5 + i] = f16(src[i]) (ops/mod.rs:1421-1425)
    assert (slab[:5] == 0x1234).all() and (slab[11:] == 0x1234).all()
    # 65520 is the midpoint above f16's largest finite value: overflow to infinity; 1e-8 is below half the smallest
    # subnormal: zero; 1 + 2^-11 is a tie that goes to the even mantissa (1.0), 1 + 3 * 2^-11 to 1 + 2^-9
    assert list(slab[5:11]) == [0x3c00, 0xc100, 0x7c00, 0x0000, 0x3c00, 0x3c02]
    with np.errstate(over="ignore"):
        assert np.array_equal(slab[5:11], src.astype(np.float16).view(np.uint16))


def test_moe_glu_is_two_expert_products_and_a_silu_mul(orc):
    r = rng(22)
    n_in, ff, n_expert, n_used, n_tok = 64, 32, 6, 2, 3
    gate = q8_0_weights(orc, r, n_expert * ff, n_in, std=1.0); up = q8_0_weights(orc, r, n_expert * ff, n_in, std=1.0)
    gs = (r.random(n_expert) + 0.5).astype(np.float32); us = (r.random(n_expert) + 0.5).astype(np.float32)
    G = ob.experts(gate, ob.Q8_0, n_in, ff, n_expert, gs); U = ob.experts(up, ob.Q8_0, n_in, ff, n_expert, us)
    ids = np.array([4, 0, 5, 5, 1, 2], np.uint32)
    x = r.standard_normal(n_tok * n_in).astype(np.float32)
    out = np.zeros(ids.size * ff, np.float32); scratch = np.zeros_like(out)
    orc.moe_glu(G, U, ids, n_used, x, out, scratch)
    a = np.zeros_like(out); b = np.zeros_like(out)
    orc.matmul_experts(G, ids, n_used, x, a); orc.matmul_experts(U, ids, n_used, x, b)
    orc.silu_mul(a, b)                                  # ops/mod.rs:1105-1117: gate product, up product, silu_mul
    assert np.array_equal(out.view(np.uint32), a.view(np.uint32))
    # and against float64 from the dequantized weights and the Q8_0-rounded activation: the per-expert scales sit
    # between the dot and the silu (ops/mod.rs:1082-1086)
    sc, q = orc.quantize_q8_0(x)
    xq = (q.reshape(-1, 32).astype(np.float64) * sc[:, None]).reshape(n_tok, n_in)
    gw = orc.dequantize(ob.Q8_0, gate, n_expert * ff * n_in).reshape(n_expert, ff, n_in).astype(np.float64)
    uw = orc.dequantize(ob.Q8_0, up, n_expert * ff * n_in).reshape(n_expert, ff, n_in).astype(np.float64)
    for i, e in enumerate(ids):
        g = gw[e] @ xq[i // n_used] * gs[e]; u = uw[e] @ xq[i // n_used] * us[e]
        assert np.allclose(out[i * ff:(i + 1) * ff], g / (1 + np.exp(-g)) * u, rtol=2e-5, atol=1e-5)
