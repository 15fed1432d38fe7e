"""The decoder layer written with the reference's own C++ front end (tests/frontend_decoder_layer.cpp), run on the device.

`check`: reduced size, float32 — Device against the front end's Host evaluation (the reference's CPU kernels), the
one-pass nodes against the composed form, a recording replayed.  `full`: hidden 4096, 32/8 heads, FFN 14336, 512
positions, bfloat16 — the program writes its inputs, parameters and results; the same layer is then evaluated from those
files by the Python harness (whose every stage tests/test_gpu_decoder_layer_full_size.py holds against the CPU checker)
and the two results are compared bit for bit: both front ends issue the same backend calls on the same bytes.
"""
import json
import os
import subprocess

import numpy as np
import pytest

import tannic_amd as ta
from tannic_amd import decoder_layer as dl
from tannic_amd import ops

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BINARY = os.path.join(ROOT, "oracle", "_ref", "frontend_decoder_layer")
GOLDEN = os.path.join(ROOT, "tests", "golden", "decoder_layer_front_end_samples.json")


def run(*args, timeout=110):
    if not os.path.exists(BINARY):
        pytest.skip("oracle/_ref/frontend_decoder_layer is not built (needs /root/reference at build time)")
    proc = subprocess.run([BINARY, *args], capture_output=True, text=True, timeout=timeout)
    print(proc.stdout)
    print(proc.stderr)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert "0 checks failed" in proc.stdout
    return proc.stdout


def test_reduced_layer_device_against_the_front_ends_host_evaluation():
    out = run("check")
    assert out.count(" ok") >= 5


def test_full_size_layer_through_the_cpp_front_end(tmp_path, device):
    out = run("full", str(tmp_path), "10")
    times = json.loads([line for line in out.splitlines() if line.startswith("{")][-1])
    assert 0 < times["composed_replay_us"] < 5000 and 0 < times["one_pass_replay_us"] < 5000
    s = dl.LayerShape()
    seq = 512
    shapes = dict(dl.weight_shapes(s), x=(1, seq, s.hidden), cos=(seq, s.head_dim // 2), sin=(seq, s.head_dim // 2), mask=(seq, seq))
    t = {}
    for name, shape in shapes.items():
        bits = np.fromfile(tmp_path / f"{name}.bin", dtype=np.uint16).reshape(shape)
        t[name] = ta.Tensor(ta.bfloat16, shape).initialize(device)
        t[name].write_raw(bits)
    one = ta.tensor(np.ones(1), ta.bfloat16, device)
    w = {name: t[name] for name in dl.weight_shapes(s)}
    composed = dl.forward(s, w, t["x"], t["cos"], t["sin"], t["mask"], one).storage()
    from_cpp = np.fromfile(tmp_path / "composed.bin", dtype=np.uint16).reshape(composed.shape)
    np.testing.assert_array_equal(from_cpp, composed, err_msg="composed layer: C++ front end against the Python harness")
    w["w13"] = ops.concatenate(w["w1"], w["w3"], 0)
    one_pass = dl.forward_fused(s, w, t["x"], t["cos"], t["sin"], t["mask"]).storage()
    from_cpp_one_pass = np.fromfile(tmp_path / "one_pass.bin", dtype=np.uint16).reshape(one_pass.shape)
    np.testing.assert_array_equal(from_cpp_one_pass, one_pass, err_msg="one-pass layer: C++ front end against the Python harness")
    values = ta.types.bfloat16_bits_to_float32(from_cpp).astype(np.float64)
    assert np.isfinite(values).all() and 0.5 < values.std() < 5
    # values of an earlier run on an MI355X, kept as data: the inputs are a pure function of the program's seeds
    if os.path.exists(GOLDEN):
        golden = json.load(open(GOLDEN))
        flat = values.reshape(-1)
        got = flat[np.array(golden["index"])]
        # summation order inside a product may differ between tile choices: a few roundings of the output type
        np.testing.assert_allclose(got, np.array(golden["composed"]), rtol=2 ** -5, atol=0.05)
    if os.environ.get("TANNIC_WRITE_GOLDEN"):
        index = [int(i) for i in np.linspace(0, values.size - 1, 64).astype(np.int64)]
        json.dump({"what": "64 evenly spaced outputs of the composed full-size layer of tests/frontend_decoder_layer.cpp (bfloat16 widened)",
                   "index": index, "composed": [float(v) for v in values.reshape(-1)[index]]}, open(os.environ["TANNIC_WRITE_GOLDEN"], "w"), indent=0)
