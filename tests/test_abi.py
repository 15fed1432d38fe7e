"""The C-ABI library builds, loads and exports every symbol the header declares.
No compute call is made here (no GPU needed)."""
import ctypes as C
import os
import re
import subprocess

import tannic_amd as ta
from tannic_amd import abi, backend

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "tannic_hip.h")


def declared_symbols():
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    return sorted(set(re.findall(r"\b(tannic_hip_\w+)\s*\(", text)))


def test_header_and_bindings_agree():
    assert declared_symbols() == sorted(backend.exported_symbols())


def test_library_exports_every_declared_symbol():
    assert os.path.exists(ta.LIBRARY_PATH), "build the library first: python -m tannic_amd.build"
    out = subprocess.run(["nm", "-D", "--defined-only", ta.LIBRARY_PATH], check=True, capture_output=True, text=True).stdout
    exported = set(re.findall(r"\bT (tannic_hip_\w+)", out))
    missing = [s for s in declared_symbols() if s not in exported]
    assert not missing, missing


def test_library_loads_and_reports_its_target():
    lib = ta.library()
    assert lib.arch() == b"gfx950"
    assert lib.last_error() in (b"", None) or isinstance(lib.last_error(), bytes)


def test_header_compiles_as_c_and_layout_matches():
    src = ('#include "tannic_hip.h"\n#include <stdio.h>\n#include <stddef.h>\n'
           'int main(void){printf("%zu %zu %zu %zu %zu %zu\\n", sizeof(tannic_tensor_t), offsetof(tannic_tensor_t, strides),'
           ' offsetof(tannic_tensor_t, dtype), offsetof(tannic_tensor_t, size), sizeof(tannic_scalar_t), sizeof(tannic_stream_t));return 0;}\n')
    exe = "/tmp/tannic_hip_header_check"
    subprocess.run(["gcc", "-std=c11", "-I", os.path.join(ROOT, "include"), "-x", "c", "-", "-o", exe], input=src, text=True, check=True)
    got = subprocess.run([exe], check=True, capture_output=True, text=True).stdout.split()
    assert got == ["176", "80", "144", "160", "16", "8"]
    assert C.sizeof(abi.tensor_t) == 176


def test_missing_library_fails_loudly(tmp_path):
    import pytest
    with pytest.raises(ta.BackendError):
        backend.DeviceLibrary(str(tmp_path / "libtannic_hip.so"))


def test_host_operands_without_registered_functions_raise():
    import numpy as np
    import pytest
    previous = ta.ops._host_functions
    ta.ops.set_host_functions(None)
    try:
        x = ta.tensor(np.ones(3), ta.float32)
        with pytest.raises(ta.BackendError):
            ta.ops.exp(x)
    finally:
        ta.ops.set_host_functions(previous)
