"""Runs of elementwise ops that a batch pass issues as one kernel in fast mode, against the CPU oracle's separate ops.

A Gated DeltaNet layer over a batch (/root/reference src/model/qwen35.rs:1255-1315) calls ssm_conv, three gather_chunks
(the q, k and v parts of the conv output) and two l2_norm_heads in a row, and later rms_norm_heads on the delta rule's
output, silu_mul with the gate, and a matmul that first quantizes its input.  The backend holds such a run back until
it is complete and then launches one kernel for it; a run that breaks off (another op, a host read, the end of the pass)
is issued op by op.  Both ways must give the oracle's values (rel/abs 1e-3; the arithmetic per element is that of the
separate fast kernels, so the observed error is a few ulps), and the conv state must advance the same way.
"""
import numpy as np
import pytest

from util import close, q8_0_weights, rng, worst

pytestmark = pytest.mark.gpu

KD, VD, HD, EPS = 512, 1024, 128, 1e-6      # 4 key heads and 8 value heads of 128; the conv runs over 2 * KD + VD channels
NC = 2 * KD + VD


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


def conv_run(ops, bufs, n, taps, upto):
    """ssm_conv, then up to three gathers and two l2 norms (upto = how many of those five follow the conv)."""
    ops.ssm_conv(bufs["state"], bufs["x"], taps, 4, bufs["conv"])
    steps = [lambda: ops.gather_chunks(bufs["conv"], KD, NC, 0, bufs["q"]),
             lambda: ops.gather_chunks(bufs["conv"], KD, NC, KD, bufs["k"]),
             lambda: ops.gather_chunks(bufs["conv"], VD, NC, 2 * KD, bufs["v"]),
             lambda: ops.l2_norm_heads(bufs["q"], HD, EPS),
             lambda: ops.l2_norm_heads(bufs["k"], HD, EPS)]
    for s in steps[:upto]:
        s()


@pytest.mark.parametrize("n,upto", [(64, 5), (300, 5), (1000, 5), (300, 3), (300, 4), (300, 1), (40, 5)])
def test_conv_split_and_l2(hip, orc, n, upto):
    """upto = 5 is the whole run (one kernel from 64 tokens on; 40 tokens is below the chunked conv's size); shorter
    runs end at the host read and are issued op by op, the conv output included."""
    r = rng(21)
    taps = (r.standard_normal(NC * 4) * 0.5).astype(np.float32)
    state0 = r.standard_normal(NC * 3).astype(np.float32)
    x = (r.standard_normal(n * NC) * 2).astype(np.float32)
    B = [{"state": state0.copy(), "x": x.copy(), "conv": np.zeros(n * NC, np.float32), "q": np.zeros(n * KD, np.float32),
          "k": np.zeros(n * KD, np.float32), "v": np.zeros(n * VD, np.float32)} for _ in range(2)]
    hip.drop_mirrors()
    for rep in range(2):                               # twice: the conv state carries over
        hip.begin_pass(n)
        hip.host_wrote(B[0]["x"])
        conv_run(hip, B[0], n, taps, upto)
        names = ["q", "k", "v"][:min(upto, 3)] + (["conv"] if upto < 5 else [])
        for name in names:
            hip.host_needs(B[0][name])
        hip.end_pass()
        hip.raise_if_error()
        conv_run(orc, B[1], n, taps, upto)
        for name in names:
            assert close(B[0][name], B[1][name], 1e-5), (rep, name, worst(B[0][name], B[1][name]))
    hip.begin_pass(1); hip.read_state(B[0]["state"]); hip.end_pass()
    assert close(B[0]["state"], B[1]["state"], 0.0), "conv state"


@pytest.mark.parametrize("n,with_matmul", [(64, True), (700, True), (700, False), (16, True)])
def test_gated_norm_silu_and_quantized_product(hip, orc, n, with_matmul):
    """rms_norm_heads(core), silu_mul(z, core), then the out-projection (which quantizes z): one kernel for the norm,
    the product and the Q8_0 form from 256 heads on (n = 16 has 128: issued op by op); without the matmul the run
    ends at the host read after two ops."""
    import inferred_hip as ih
    from oracle import binding as ob
    r = rng(22)
    w = (0.5 + r.random(HD)).astype(np.float32)
    core0 = (r.standard_normal(n * VD) * np.repeat(10.0 ** r.uniform(-2, 1, n * VD // HD), HD)).astype(np.float32)
    z0 = (r.standard_normal(n * VD) * 3).astype(np.float32)
    wo = q8_0_weights(orc, r, 256, VD, std=0.05)
    B = [{"core": core0.copy(), "z": z0.copy(), "out": np.zeros(n * 256, np.float32)} for _ in range(2)]
    hip.drop_mirrors()
    hip.begin_pass(n)
    hip.host_wrote(B[0]["core"]); hip.host_wrote(B[0]["z"])
    hip.rms_norm_heads(B[0]["core"], w, HD, EPS)
    hip.silu_mul(B[0]["z"], B[0]["core"])
    if with_matmul:
        hip.matmul(ih.weights(wo, ih.Q8_0, VD, 256), B[0]["z"], B[0]["out"])
        hip.host_needs(B[0]["out"])
    hip.host_needs(B[0]["z"])
    hip.end_pass()
    hip.raise_if_error()
    orc.rms_norm_heads(B[1]["core"], w, HD, EPS)
    orc.silu_mul(B[1]["z"], B[1]["core"])
    assert close(B[0]["z"], B[1]["z"], 1e-5), worst(B[0]["z"], B[1]["z"])
    if with_matmul:
        # The product, against the oracle's product of the SAME z (the backend's): Q8_0 rounding is a step function, so a
        # z that differs in its last bits moves a few quants by one and the sums with them; given equal inputs the
        # quantization and the integer dots are the oracle's, and only the f32 additions round differently.
        orc.matmul(ob.weights(wo, ih.Q8_0, VD, 256), B[0]["z"], B[1]["out"])
        assert close(B[0]["out"], B[1]["out"], 1e-5), worst(B[0]["out"], B[1]["out"])


def test_what_a_one_kernel_run_leaves_unwritten_is_refused_not_handed_over_stale():
    """The one-kernel forms skip two buffers of the seam: the conv output (conv + split + l2) and the normed read-out
    (`core` keeps the delta rule's raw values behind gated norm + silu-mul + quantize).  A host read of either after a
    completed run raises the sticky error; a traced pass, whose read lands inside the run, still gets the op's value
    (the run is then issued op by op: covered above)."""
    import inferred_hip as ih
    be = ih.Hip(exact=False)
    try:
        DK, n = HD, 256
        kdim, vdim, cdim = KD, VD, NC
        r = rng(91)
        qkv = r.standard_normal(n * cdim).astype(np.float32)
        conv_w = (r.standard_normal(cdim * 4) * 0.5).astype(np.float32)
        state = np.zeros(cdim * 3, np.float32)
        convo = np.zeros(n * cdim, np.float32)
        q, k, v = np.zeros(n * kdim, np.float32), np.zeros(n * kdim, np.float32), np.zeros(n * vdim, np.float32)
        for rep in range(2):       # the first pass sizes the device mirrors (which ends a held run): the second holds
            be.begin_pass(n)
            be.host_wrote(qkv)
            be.ssm_conv(state, qkv, conv_w, 4, convo)
            be.gather_chunks(convo, kdim, cdim, 0, q); be.gather_chunks(convo, kdim, cdim, kdim, k)
            be.gather_chunks(convo, vdim, cdim, 2 * kdim, v)
            be.l2_norm_heads(q, DK, 1e-6); be.l2_norm_heads(k, DK, 1e-6)
            be.end_pass()
        be.host_needs(q)
        assert be.take_error() is None and np.abs(q).max() > 0          # what the run does write is there
        be.host_needs(convo)
        err = be.take_error()
        assert err is not None and "fused kernel" in err, err
    finally:
        be.take_error()
        be.close()
