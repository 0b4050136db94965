"""The CPU oracle against the reference's own golden vectors (copied data files under
tests/golden/) and against independent implementations (numpy, torch, libm).

Fixture formats: ITFX (/root/reference tests/dequantize.rs:32-68) holds raw block bytes and
llama.cpp's dequantized f32; ITDP (tests/kquant_dots.rs:57-109) holds real NVFP4 weight rows,
an f32 activation, ggml's own Q8_0 bytes for it, and ggml's vec_dot results.
"""
import ctypes
import struct

import numpy as np
import pytest

from oracle import binding as ob


@pytest.fixture(scope="module")
def orc():
    return ob.Oracle(threads=1)


def load_itfx(path):
    b = path.read_bytes()
    assert b[:4] == b"ITFX" and struct.unpack_from("<I", b, 4)[0] == 1
    ty, n, raw_len, name_len = struct.unpack_from("<IQQI", b, 8)
    p = 8 + 24
    name = b[p:p + name_len].decode(); p += name_len
    raw = np.frombuffer(b, np.uint8, raw_len, p).copy(); p += raw_len
    ref = np.frombuffer(b, np.float32, n, p).copy()
    return name, ty, raw, ref


def load_itdp(path):
    b = path.read_bytes()
    assert b[:4] == b"ITDP" and struct.unpack_from("<I", b, 4)[0] == 1
    ty, n, rows, name_len = struct.unpack_from("<IQQI", b, 8)
    p = 8 + 24
    name = b[p:p + name_len].decode(); p += name_len
    (w_len,) = struct.unpack_from("<Q", b, p); p += 8
    weights = np.frombuffer(b, np.uint8, w_len, p).copy(); p += w_len
    act = np.frombuffer(b, np.float32, n, p).copy(); p += 4 * n
    (q_len,) = struct.unpack_from("<Q", b, p); p += 8
    q8 = np.frombuffer(b, np.uint8, q_len, p).copy(); p += q_len
    generic = np.frombuffer(b, np.float32, rows, p).copy(); p += 4 * rows
    dispatch = np.frombuffer(b, np.float32, rows, p).copy()
    return dict(name=name, ty=ty, n=n, rows=rows, weights=weights, act=act, q8=q8, generic=generic, dispatch=dispatch)


@pytest.mark.parametrize("fname", ["q8_0_Qwen3-0.6B-Q8_0.gguf.itfx", "q8_0_Qwen_Qwen3.6-35B-A3B-IQ4_XS.gguf.itfx",
                                   "f16_edge_cases.itfx", "f32_Qwen3-0.6B-Q8_0.gguf.itfx",
                                   "f32_Qwen_Qwen3.6-35B-A3B-IQ4_XS.gguf.itfx"])
def test_dequantize_matches_llama_cpp_bitwise(orc, golden_dir, fname):
    name, ty, raw, ref = load_itfx(golden_dir / fname)
    got = orc.dequantize(ty, raw, ref.size)
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32)), name


def test_nvfp4_dot_and_q8_0_activation_match_ggml_bitwise(orc, golden_dir):
    f = load_itdp(golden_dir / "dot_nvfp4_Qwen3.6-35B-A3B-NVFP4-Q8_0.gguf.itdp")
    assert f["ty"] == ob.NVFP4 and f["n"] == 2048 and f["rows"] == 64
    # a3: ggml's quantize_row_q8_0_ref bytes
    assert np.array_equal(orc.q8_0_blocks(f["act"]), f["q8"])
    # a5: ggml's vec_dot_nvfp4_q8_0 per row; through the dot and through matmul
    sc, q = orc.quantize_q8_0(f["act"])
    row_bytes = f["n"] // 64 * 36
    L = ob.lib()
    for j in range(f["rows"]):
        row = f["weights"][j * row_bytes:(j + 1) * row_bytes]
        got = np.float32(L.orc_dot_nvfp4_q8_0(row.ctypes.data, f["n"], sc.ctypes.data, q.ctypes.data))
        assert got.view(np.uint32) == f["generic"][j:j + 1].view(np.uint32)[0], j
    out = np.zeros(f["rows"], np.float32)
    orc.matmul(ob.weights(f["weights"], ob.NVFP4, f["n"], f["rows"]), f["act"], out)
    assert np.array_equal(out.view(np.uint32), f["generic"].view(np.uint32))
    assert np.array_equal(f["generic"].view(np.uint32), f["dispatch"].view(np.uint32))


def test_f16_decode_exhaustive_against_numpy():
    L = ob.lib()
    h = np.arange(65536, dtype=np.uint16)
    want = h.view(np.float16).astype(np.float32)
    got = np.array([L.orc_c_f16_to_f32(int(v)) for v in h], np.float32)
    nan = np.isnan(want)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))
    assert np.isnan(got[nan]).all()


def test_bf16_decode_exhaustive_against_the_bit_shift():
    """bf16 is the top half of an f32 (/root/reference src/quant/half.rs:61-63): all 65,536 codes."""
    L = ob.lib()
    h = np.arange(65536, dtype=np.uint32)
    want = (h << 16).astype(np.uint32).view(np.float32)
    got = np.array([L.orc_c_bf16_to_f32(int(v)) for v in h], np.float32)
    nan = np.isnan(want)          # (a signalling NaN is quieted on its way back through the C float return)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))
    assert np.isnan(got[nan]).all()


@pytest.mark.parametrize("ty,np_ty", [("f32", np.float32), ("f16", np.float16), ("bf16", None)])
def test_matmul_on_unquantized_rows_is_the_serial_f32_fold_of_the_widened_weights(orc, ty, np_ty):
    """F32 / F16 / BF16 rows (/root/reference src/ops/naive.rs:843-861): each output is the serial f32 sum of
    widened weight times activation from zero, checked bit for bit against that fold written in numpy, and against
    the float64 product of the widened weights (a wrong widening, a transposed operand or a dropped row would be far
    outside it)."""
    r = np.random.default_rng(17)
    n_in, n_out, n_tok = 96, 7, 3
    w32 = (r.standard_normal((n_out, n_in)) * 0.5).astype(np.float32)
    if ty == "bf16":
        bits = (w32.view(np.uint32) >> 16).astype(np.uint16)          # truncation picks representable values
        wide = (bits.astype(np.uint32) << 16).view(np.float32)
        raw, code = bits.view(np.uint8).reshape(-1).copy(), ob.BF16
    elif ty == "f16":
        half = w32.astype(np.float16)
        wide = half.astype(np.float32)
        raw, code = half.view(np.uint8).reshape(-1).copy(), ob.F16
    else:
        wide = w32
        raw, code = w32.view(np.uint8).reshape(-1).copy(), ob.F32
    x = r.standard_normal(n_tok * n_in).astype(np.float32)
    out = np.zeros(n_tok * n_out, np.float32)
    orc.matmul(ob.weights(raw, code, n_in, n_out), x, out)
    want = np.zeros((n_tok, n_out), np.float32)
    for t in range(n_tok):
        for j in range(n_out):
            acc = np.float32(0.0)
            for i in range(n_in):
                acc = np.float32(acc + np.float32(wide[j, i] * x[t * n_in + i]))
            want[t, j] = acc
    assert np.array_equal(out.view(np.uint32), want.reshape(-1).view(np.uint32))
    f64 = x.reshape(n_tok, n_in).astype(np.float64) @ wide.astype(np.float64).T
    assert np.allclose(out.reshape(n_tok, n_out), f64, rtol=0, atol=1e-4)


def test_f32_to_f16_round_to_nearest_even_against_numpy():
    L = ob.lib()
    r = np.random.default_rng(0)
    xs = np.concatenate([
        (r.standard_normal(20000) * 10.0 ** r.uniform(-9, 5, 20000)).astype(np.float32),
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9, -1e9, np.inf, -np.inf, 5.96e-8, 2.98e-8, 2.981e-8,
                  6.1e-5, 6.097e-5, 1.0009765625, 1.00048828125, 1.001464843750], np.float32),
        # every midpoint between adjacent normal halves in one binade
        (np.arange(1024, dtype=np.float32) * 2 + 1) / 2048 + 1.0])
    with np.errstate(over="ignore"):
        want = xs.astype(np.float16).view(np.uint16)
    got = np.array([L.orc_c_f32_to_f16(float(v)) for v in xs], np.uint16)
    assert np.array_equal(got, want)


def test_ue4m3_all_codes_against_torch_float8():
    torch = pytest.importorskip("torch")
    L = ob.lib()
    codes = torch.arange(0, 0x7f, dtype=torch.uint8)
    want = codes.view(torch.float8_e4m3fn).float().numpy() * 0.5   # halved (quant/mod.rs:271-284)
    got = np.array([L.orc_c_ue4m3_to_f32(int(c)) for c in range(0x7f)], np.float32)
    assert np.array_equal(got, want.astype(np.float32))
    assert L.orc_c_ue4m3_to_f32(0x7f) == 0.0 and L.orc_c_ue4m3_to_f32(0) == 0.0
    # bit 7 is not examined
    assert all(L.orc_c_ue4m3_to_f32(c | 0x80) == L.orc_c_ue4m3_to_f32(c) for c in range(1, 0x7f))


def test_nvfp4_block_decodes_split_nibbles(orc):
    # quant/mod.rs:549-566: byte j of sub-block s carries element j (low nibble) and j + 8 (high)
    blk = np.zeros(36, np.uint8)
    blk[:4] = 0x38                      # 1.0 in E4M3 -> 0.5 halved; doubled table => code value
    blk[4] = 0x21                       # elem 0 = code 1 (0.5), elem 8 = code 2 (1.0)
    blk[4 + 8 + 7] = 0xf9               # sub-block 1: elem 7 = code 9 (-0.5), elem 15 = code 15 (-6)
    y = orc.dequantize(ob.NVFP4, blk, 64)
    assert y[0] == 0.5 and y[8] == 1.0 and y[16 + 7] == -0.5 and y[16 + 15] == -6.0
    assert np.count_nonzero(y) == 4


def test_expf_logf_against_libm_and_float64(orc):
    L = ob.lib()
    libm = ctypes.CDLL("libm.so.6")
    libm.expf.restype = libm.logf.restype = ctypes.c_float
    libm.expf.argtypes = libm.logf.argtypes = [ctypes.c_float]
    r = np.random.default_rng(1)
    xs = np.concatenate([r.uniform(-104, 89, 40000), r.standard_normal(40000) * 5, [0.0, -0.0, 88.7, -103.9, 20.0]]).astype(np.float32)
    mism = 0
    for x in xs:
        a, b = np.float32(L.orc_c_expf(float(x))), np.float32(libm.expf(float(x)))
        mism += a.view(np.uint32) != b.view(np.uint32)
        ref = np.exp(np.float64(x))
        if 1e-37 < ref < 3e38:
            assert abs(float(a) - ref) <= 1.0 * np.spacing(np.float32(ref)), x
    # libm's x86-64 FMA variant differs from the portable evaluation on two inputs in 2^32
    assert mism <= 1
    ps = np.abs(np.concatenate([r.standard_normal(40000) * 10.0 ** r.uniform(-30, 30, 40000), [1.0, 1.0 + 2 ** -23, 1e-40]])).astype(np.float32)
    ps = ps[ps > 0]
    for x in ps:
        a, b = np.float32(L.orc_c_logf(float(x))), np.float32(libm.logf(float(x)))
        assert a.view(np.uint32) == b.view(np.uint32), x
    assert L.orc_c_expf(float("-inf")) == 0.0 and L.orc_c_expf(1000.0) == float("inf")
