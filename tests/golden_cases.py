"""Runs the reference's own test vectors (tests/golden/reference_vectors.json)
through ``tannic_amd.ops`` in a chosen environment."""
import json
import math
import os

import numpy as np

import tannic_amd as ta
from tannic_amd import ops, types

HERE = os.path.dirname(os.path.abspath(__file__))
CASES = json.load(open(os.path.join(HERE, "golden", "reference_vectors.json")))["cases"]
TENSOR_CASES = [c for c in CASES if c["inputs"]]

LIBM = {
    "log": np.log, "exp": np.exp, "sqrt": np.sqrt, "sin": np.sin, "cos": np.cos, "tan": np.tan,
    "sinh": np.sinh, "cosh": np.cosh, "tanh": np.tanh,
}


def build(spec, env):
    dtype = types.BY_NAME[spec["dtype"]]
    t = ta.tensor(np.array(spec["data"], dtype=np.float64).reshape(spec["shape"]), dtype, env)
    if "transpose" in spec:
        t = t.transpose(*spec["transpose"])
    if "expand" in spec:
        t = t.expand(*spec["expand"])
    if "permute" in spec:
        t = t.permute(*spec["permute"])
    return t


def expected_of(case):
    if case.get("expected") is not None:
        e = case["expected"]
        return np.array(e["data"], dtype=np.float64).reshape(e["shape"])
    x = np.array(case["inputs"][0]["data"], dtype=np.float32).reshape(case["inputs"][0]["shape"])
    expr = case["expected_expr"]
    if expr == "pow":
        y = np.array(case["inputs"][1]["data"], dtype=np.float32).reshape(case["inputs"][1]["shape"])
        with np.errstate(over="ignore"):
            return np.power(x, y).astype(np.float32)
    if expr == "rsqrt":
        eps = np.float32(case["eps"])
        return (np.float32(1.0) / np.sqrt(x + eps)).astype(np.float32)
    return LIBM[expr](x).astype(np.float32)


def run(case, env):
    """Evaluates the case with its operands placed in ``env``; returns a numpy array."""
    op = case["op"]
    ins = [build(s, env) for s in case["inputs"]]
    if op == "matmul":
        out = ops.matmul(*ins)
    elif op == "conv2d":
        bias = ins[2] if len(ins) == 3 else None
        out = ops.convolve2d(ins[0], ins[1], bias, stride=tuple(case["stride"]), padding=tuple(case["padding"]))
    elif op in ("add", "sub", "mul", "pow"):
        out = getattr(ops, op)(*ins)
    elif op == "complex_mul":
        out = ops.realify(ops.mul(ops.complexify(ins[0]), ops.complexify(ins[1])))
    elif op == "mul_add":
        out = ops.add(ops.mul(ins[0], ins[1]), ins[2])
    elif op == "rsqrt":
        out = ops.rsqrt(ins[0], case["eps"])
    elif op in ("sum", "mean", "argmax", "argmin"):
        out = getattr(ops, op)(ins[0], case["axis"], case.get("keepdim", False))
    elif op == "mean_sq":
        out = ops.mean(ops.mul(ins[0], ins[0]), case["axis"])
    elif op == "conv1d":
        out = ops.convolve1d(ins[0], ins[1], case["stride"], case["padding"])
    elif op == "concat":
        out = ops.concatenate(ins[0], ins[1], case["axis"])
    elif op == "outer":
        out = ops.outer(ins[0], ins[1])
    elif op == "repeat":
        out = ops.repeat(ins[0], case["repeats"], case["axis"])
    elif op == "assign_rows":
        first, last = case["rows"]
        ops.copy_into(ins[0][first:last], ins[1])
        out = ins[0]
    elif op == "complex_roundtrip":
        out = ops.realify(ops.complexify(ins[0]))
    elif op == "polar":
        out = ops.realify(ops.polar(ins[0], ins[1]))
    else:
        out = getattr(ops, op)(ins[0])
    return out.numpy()


def tolerance(case):
    # the reference's tests use allclose with rtol 1e-5 / atol 1e-8 unless they say otherwise
    return case.get("rtol", 1e-5), case.get("atol", 1e-8)
