"""The reference's own C++ front end driving this backend (built where the reference is mounted)."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BINARY = os.path.join(ROOT, "oracle", "_ref", "frontend_dropin")


def test_reference_front_end_runs_on_this_backend():
    """tests/frontend_dropin.cpp: each expression evaluated by Tannic's front end on Host (its CPU kernels)
    and on Device (the HIP backend through the cuda:: adapter), compared with its own allclose."""
    if not os.path.exists(BINARY):
        pytest.skip("oracle/_ref/frontend_dropin is not built (needs /root/reference at build time)")
    proc = subprocess.run([BINARY], capture_output=True, text=True, timeout=110)
    print(proc.stdout)
    print(proc.stderr)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert "0 of" in proc.stdout
