"""it_hip_attend_noalloc (the entry point that allocates nothing) against it_hip_attend, through the C ABI.

Device memory is held with plain hipMalloc calls (util.Hiprt); the fixed scratch inside the library is shared by every call on
the GPU, so the test calls twice in a row, the second time with a smaller input, and checks both results: a
kernel that relied on the scratch starting clean, or on the first call's sizes, fails the second check.
The bar is bit-identity: the two entry points run the same kernels with the same split count."""
import numpy as np
import pytest

import inferred_hip as ih
from util import Hiprt, rng, f16_bits, assert_bits_equal

pytestmark = pytest.mark.gpu


def _case(hip, orc, rt, n_q, n_pos, slab_pos, hd, nh, nkv, seed):
    hip.drop_mirrors()   # numpy may hand this case the previous case's addresses: forget their device copies
    hip.begin_pass(1)
    r = rng(seed)
    kv_dim = nkv * hd
    q = r.standard_normal(n_q * nh * hd).astype(np.float32)
    k = f16_bits(r.standard_normal(slab_pos * kv_dim)); v = f16_bits(r.standard_normal(slab_pos * kv_dim))
    sc = float(1.0 / np.sqrt(np.float32(hd)))
    want = np.zeros(n_q * nh * hd, np.float32)
    hip.attend(q, k, v, kv_dim, n_pos, hd, nh, nkv, sc, want); hip.host_needs(want)
    hip.raise_if_error()
    ref = np.zeros_like(want)
    orc.attend(q, k, v, kv_dim, n_pos, hd, nh, nkv, sc, ref)
    # the existing entry point itself is within rel/abs 1e-3 of the CPU oracle on these inputs
    assert np.all(np.abs(want - ref) <= 1e-3 * np.maximum(1.0, np.abs(ref))), np.abs(want - ref).max()
    dq, dk, dv = rt.upload(q), rt.upload(k), rt.upload(v)
    dout = rt.filled(q.nbytes, 0xff)            # every float a NaN until the kernels write it
    rc, msg = ih.attend_noalloc(dq, q.size, dk, dv, k.size, kv_dim, n_pos, hd, nh, nkv, sc, dout, q.size, stream=0)
    assert rc == 0, msg
    got = rt.download(dout, want)
    rt.free_all()
    return want, got


@pytest.mark.parametrize("hd,nh,nkv,first,second", [
    (256, 16, 2, (1, 6000, 8192), (1, 700, 1024)),     # config 5's decode step, then a shorter context
    (256, 16, 2, (4, 1500, 2048), (1, 1, 64)),         # a short verify batch, then a single key
    (64, 8, 2, (3, 900, 1024), (2, 130, 256)),         # the tiny model's heads
    (96, 8, 4, (2, 500, 512), (1, 129, 256)),          # a head size the matrix-core kernel does not take
])
def test_two_calls_in_a_row_match_it_hip_attend(hd, nh, nkv, first, second):
    from oracle import binding as ob
    orc = ob.Oracle(threads=8)
    hip = ih.Hip(exact=False)
    rt = Hiprt()
    try:
        for i, (n_q, n_pos, slab_pos) in enumerate((first, second)):
            print(f"attend_noalloc case hd={hd} nh={nh} nkv={nkv} n_q={n_q} n_pos={n_pos}", flush=True)
            want, got = _case(hip, orc, rt, n_q, n_pos, slab_pos, hd, nh, nkv, seed=40 + i)
            assert np.isfinite(got).all()
            assert_bits_equal(got, want, f"attend_noalloc call {i + 1}")
    finally:
        rt.free_all()
        hip.close()


def test_refuses_what_the_fixed_scratch_cannot_hold():
    hd, nh, nkv, n_q, n_pos = 256, 16, 2, 16, 8192   # 16 rows x 16 heads x 128 splits x 258 floats = 33.8 MB
    rt = Hiprt()
    try:
        n, n_kv = n_q * nh * hd, n_pos * nkv * hd
        q, kv, out = rt.filled(n * 4, 0), rt.filled(n_kv * 2, 0), rt.filled(n * 4, 0)
        rc, msg = ih.attend_noalloc(q, n, kv, kv, n_kv, nkv * hd, n_pos, hd, nh, nkv, 0.0625, out, n)
        assert rc == 2 and "too large" in msg
        rc, msg = ih.attend_noalloc(q, n, kv, kv, n_kv, nkv * hd, n_pos + 1, hd, nh, nkv, 0.0625, out, n)
        assert rc == 1 and "n_pos" in msg
    finally:
        rt.free_all()


def test_a_warm_call_leaves_free_device_memory_as_it_was():
    """The property the entry point exists for: nothing is allocated.  After one call (the scratch address is looked
    up, the kernels are loaded), hipMemGetInfo reads the same before and after further calls."""
    hd, nh, nkv, n_q, n_pos, slab = 256, 16, 2, 1, 3000, 4096
    rt = Hiprt()
    try:
        r = rng(77)
        q = r.standard_normal(n_q * nh * hd).astype(np.float32)
        k = f16_bits(r.standard_normal(slab * nkv * hd)); v = f16_bits(r.standard_normal(slab * nkv * hd))
        dq, dk, dv, dout = rt.upload(q), rt.upload(k), rt.upload(v), rt.filled(q.nbytes, 0xff)
        call = lambda: ih.attend_noalloc(dq, q.size, dk, dv, k.size, nkv * hd, n_pos, hd, nh, nkv, 0.0625, dout, q.size, stream=0)
        rc, msg = call()
        assert rc == 0, msg
        rt.check(rt.rt.hipDeviceSynchronize(), "hipDeviceSynchronize")
        before = rt.mem_free()
        for _ in range(3):
            rc, msg = call()
            assert rc == 0, msg
        rt.check(rt.rt.hipDeviceSynchronize(), "hipDeviceSynchronize")
        assert rt.mem_free() == before
    finally:
        rt.free_all()


_FIRST_CALL = r"""
import sys
sys.path.insert(0, {tests!r}); sys.path.insert(0, {pkg!r}); sys.path.insert(0, {root!r})
import numpy as np
import inferred_hip as ih
from util import Hiprt, rng, f16_bits
hd, nh, nkv, n_q, n_pos, slab = 256, 16, 2, 1, 2500, 4096
rt = Hiprt()
r = rng(78)
q = r.standard_normal(n_q * nh * hd).astype(np.float32)
k = f16_bits(r.standard_normal(slab * nkv * hd)); v = f16_bits(r.standard_normal(slab * nkv * hd))
dq, dk, dv, dout = rt.upload(q), rt.upload(k), rt.upload(v), rt.filled(q.nbytes, 0xff)
# no backend exists yet in this process: the call itself looks the scratch up
rc, msg = ih.attend_noalloc(dq, q.size, dk, dv, k.size, nkv * hd, n_pos, hd, nh, nkv, 0.0625, dout, q.size, stream=0)
assert rc == 0, msg
got = rt.download(dout, q)
hip = ih.Hip(exact=False)
hip.begin_pass(1)
want = np.zeros_like(q)
hip.attend(q, k, v, nkv * hd, n_pos, hd, nh, nkv, 0.0625, want); hip.host_needs(want)
hip.raise_if_error()
assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), np.abs(got - want).max()
hip.close(); rt.free_all()
print("FIRST CALL OK")
"""


def test_the_first_call_of_a_process_needs_no_backend():
    """In a process that has created no backend, the entry point resolves its scratch on its first call (that call is
    not one to make under graph capture: the header says so) and gives it_hip_attend's bits."""
    import subprocess
    import sys
    from pathlib import Path
    root = Path(__file__).resolve().parent.parent
    code = _FIRST_CALL.format(tests=str(root / "tests"), pkg=str(root / "inferred-thoughts_amd"), root=str(root))
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0 and "FIRST CALL OK" in out.stdout, out.stdout[-2000:] + out.stderr[-2000:]
