"""Shared helpers for the parity tests: seeded inputs in the formats the seam carries."""
import numpy as np


def rng(seed):
    return np.random.default_rng(seed)


def q8_0_weights(oracle, r, n_out, n_in, std=0.02):
    """Rows of N(0, std) quantized to Q8_0 with the oracle's own quantizer (ggml's rule)."""
    w = (r.standard_normal((n_out, n_in)) * std).astype(np.float32)
    return oracle.q8_0_blocks(w.reshape(-1)).copy()


def nvfp4_weights(r, n_out, n_in):
    """NVFP4 rows as BASELINE config 2 draws them: nibbles uniform over the 16 codes, UE4M3
    scale bytes from |N(0,1)| (nearest code, never 0x00/0x7f)."""
    n_blocks = n_out * n_in // 64
    out = np.zeros((n_blocks, 36), np.uint8)
    out[:, 4:] = r.integers(0, 256, (n_blocks, 32), dtype=np.uint8)
    codes = np.arange(1, 0x7f)
    exp = (codes >> 3) & 0xf
    man = (codes & 7).astype(np.float64)
    vals = np.where(exp == 0, man * 2.0 ** -9, (1 + man / 8) * 2.0 ** (exp - 7.0))
    mags = np.abs(r.standard_normal((n_blocks, 4)))
    idx = np.abs(mags[..., None] - vals[None, None, :]).argmin(-1)
    out[:, :4] = codes[idx].astype(np.uint8)
    return out.reshape(-1).copy()


def bf16_round(x):
    """f32 -> nearest-even bf16 -> f32 (the single-op configs feed bf16 activations)."""
    u = x.astype(np.float32).view(np.uint32).astype(np.uint64)
    u = ((u + 0x7fff + ((u >> 16) & 1)) >> 16) << 16
    return u.astype(np.uint32).view(np.float32)


def f16_bits(x):
    return x.astype(np.float16).view(np.uint16)


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def assert_bits_equal(a, b, what=""):
    a, b = bits(a), bits(b)
    if not np.array_equal(a, b):
        bad = np.flatnonzero(a != b)
        raise AssertionError(f"{what}: {bad.size} of {a.size} values differ bitwise; first at {bad[0]}: "
                             f"{a.view(np.float32)[bad[0]]!r} vs {b.view(np.float32)[bad[0]]!r}")
