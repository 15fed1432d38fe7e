"""The reference's own C++ front end driving this backend (built where the reference is mounted)."""
import os
import subprocess

import numpy as np
import pytest

import tannic_amd as ta
from tannic_amd import serialization

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BINARY = os.path.join(ROOT, "oracle", "_ref", "frontend_dropin")


def test_reference_front_end_runs_on_this_backend(tmp_path):
    """tests/frontend_dropin.cpp: each expression evaluated by Tannic's front end on Host (its CPU kernels)
    and on Device (the HIP backend through the cuda:: adapter), compared with its own allclose.  The program also reads
    a tensor file written here by the Python writer and writes one that the Python reader takes back (the file layout
    of include/tannic/serialization.hpp:26-66 from both sides)."""
    if not os.path.exists(BINARY):
        pytest.skip("oracle/_ref/frontend_dropin is not built (needs /root/reference at build time)")
    serialization.save(ta.tensor(0.5 * np.arange(24).reshape(2, 3, 4), ta.float32), tmp_path / "from_python.tannic")
    proc = subprocess.run([BINARY, str(tmp_path)], capture_output=True, text=True, timeout=110)
    print(proc.stdout)
    print(proc.stderr)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert "0 of" in proc.stdout and "a file written by the Python writer" in proc.stdout
    theirs = serialization.load(tmp_path / "from_cpp.tannic")
    assert theirs.dtype is ta.float32 and tuple(theirs.shape) == (8, 64, 32)
    values = theirs.numpy()
    assert np.isfinite(values).all() and 0.5 < np.abs(values).mean() < 1.5 and np.abs(values).max() <= 2.0   # 0.5 * uniform[-4, 4)
