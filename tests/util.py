"""Shared helpers for the parity tests: seeded inputs in the formats the seam carries."""
import numpy as np


def rng(seed):
    return np.random.default_rng(seed)


def q8_0_weights(oracle, r, n_out, n_in, std=0.02):
    """Rows of N(0, std) quantized to Q8_0 with the oracle's own quantizer (ggml's rule)."""
    w = (r.standard_normal((n_out, n_in)) * std).astype(np.float32)
    return oracle.q8_0_blocks(w.reshape(-1)).copy()


def nvfp4_weights(r, n_out, n_in):
    """NVFP4 rows as benchmark configuration 2 draws them: nibbles uniform over the 16 codes, UE4M3
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


class Hiprt:
    """The few HIP runtime calls a test needs to hold device memory of its own (hipMalloc, copies, free), through
    ctypes on the runtime the product library is linked against, so a test of an entry point that takes device
    pointers needs nothing but the library under test."""

    def __init__(self):
        import ctypes as C
        import inferred_hip as ih
        ih.lib()                                  # maps libamdhip64 into the process
        self.C = C
        self.rt = C.CDLL("libamdhip64.so")
        self.rt.hipMalloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t]
        self.rt.hipFree.argtypes = [C.c_void_p]
        self.rt.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
        self.rt.hipMemset.argtypes = [C.c_void_p, C.c_int, C.c_size_t]
        self.rt.hipGetErrorString.restype = C.c_char_p
        self.rt.hipGetErrorString.argtypes = [C.c_int]
        self.held = []

    def check(self, rc, what):
        if rc != 0:
            raise RuntimeError(f"{what}: {self.rt.hipGetErrorString(rc).decode()}")

    def last_error(self):
        rc = self.rt.hipGetLastError()
        return None if rc == 0 else self.rt.hipGetErrorString(rc).decode()

    def upload(self, a):
        """Device copy of a contiguous numpy array; returns the device address."""
        p = self.C.c_void_p()
        self.check(self.rt.hipMalloc(self.C.byref(p), max(a.nbytes, 16)), "hipMalloc")
        self.held.append(p.value)
        self.check(self.rt.hipMemcpy(p, a.ctypes.data, a.nbytes, 1), "hipMemcpy(host to device)")
        return p.value

    def filled(self, nbytes, byte):
        p = self.C.c_void_p()
        self.check(self.rt.hipMalloc(self.C.byref(p), max(nbytes, 16)), "hipMalloc")
        self.held.append(p.value)
        self.check(self.rt.hipMemset(p, byte, nbytes), "hipMemset")
        return p.value

    def download(self, dev, like):
        out = np.empty_like(like)
        self.check(self.rt.hipDeviceSynchronize(), "hipDeviceSynchronize")
        self.check(self.rt.hipMemcpy(out.ctypes.data, dev, out.nbytes, 2), "hipMemcpy(device to host)")
        return out

    def mem_free(self):
        """free device memory in bytes (hipMemGetInfo)"""
        C = self.C
        free, total = C.c_size_t(0), C.c_size_t(0)
        self.check(self.rt.hipMemGetInfo(C.byref(free), C.byref(total)), "hipMemGetInfo")
        return int(free.value)

    def free_all(self):
        for p in self.held:
            self.rt.hipFree(p)
        self.held = []


def bound(b, tol):
    """The rel/abs bound of the fast-mode tests: tol * |b_i|, with an absolute floor of tol * min(1, largest |b|) for
    entries near zero (never looser than tol * max(1, |b_i|))."""
    b = np.abs(np.asarray(b, np.float64))
    top = float(b.max()) if b.size else 0.0
    return tol * np.maximum(b, min(1.0, top))


def close(a, b, tol=1e-3):
    return bool(np.all(np.abs(np.asarray(a, np.float64) - b) <= bound(b, tol)))


def worst(a, b):
    """largest error as a multiple of the bound at tol = 1 (1e-3 means: exactly at a 1e-3 limit)"""
    if np.asarray(b).size == 0:
        return 0.0
    return float((np.abs(np.asarray(a, np.float64) - b) / np.maximum(bound(b, 1.0), 1e-300)).max())
