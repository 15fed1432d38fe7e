"""Link-time proof of the drop-in: the reference's front end, compiled with its CUDA macro against the
adapter headers, links with adapter.cpp and the device library without an unresolved symbol."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REFERENCE = "/root/reference"


@pytest.mark.skipif(not os.path.isdir(os.path.join(REFERENCE, "src")), reason="the reference is not mounted here")
def test_front_end_links_against_the_adapter():
    proc = subprocess.run(["make", "-C", os.path.join(ROOT, "oracle"), "-j8", "_ref/frontend_dropin"], capture_output=True, text=True)
    assert proc.returncode == 0, proc.stdout[-3000:] + proc.stderr[-3000:]
    binary = os.path.join(ROOT, "oracle", "_ref", "frontend_dropin")
    undefined = subprocess.run(["nm", "-u", "-C", binary], capture_output=True, text=True).stdout
    needed = [l.split()[-1] for l in undefined.splitlines() if "tannic_hip_" in l]
    assert "tannic_hip_gemm" in needed and "tannic_hip_allocate" in needed   # resolved by libtannic_hip.so at load time
    assert "cuda::" not in undefined   # every cuda:: function the front end names is defined by the adapter
