"""Runs the native check of the fast single-token kernels (tests/native/fast_kernels_check.hip).

The fused fast kernels are only reachable through a captured model pass, where whole-model chaos hides
per-kernel error; the native program calls their launchers directly beside the order-preserving kernels
(the ones the bit-exact model tests pin to the oracle) on identical inputs.
"""
import subprocess
from pathlib import Path

import pytest

BIN = Path(__file__).resolve().parent / "native" / "fast_kernels_check"


@pytest.mark.gpu
def test_fast_kernels_match_order_preserving_kernels():
    assert BIN.exists(), f"{BIN} is not built: run make -C inferred-thoughts_amd/csrc"
    r = subprocess.run([str(BIN)], capture_output=True, text=True, timeout=300)
    bad = [l for l in r.stdout.splitlines() if "MISMATCH" in l or "DIFFERENT" in l]
    assert r.returncode == 0 and not bad, "\n".join(bad[:20]) + r.stderr[-2000:]
    assert r.stdout.count(" ok") > 400
