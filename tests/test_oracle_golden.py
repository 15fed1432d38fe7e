"""The CPU checker against every vector the reference's own tests hold for the path."""
import math

import numpy as np
import pytest

import golden_cases
import support
import tannic_amd as ta
from tannic_amd import ops, types


@pytest.mark.parametrize("case", golden_cases.TENSOR_CASES, ids=lambda c: c["name"])
def test_oracle_matches_reference_vectors(oracle, case):
    got = golden_cases.run(case, ta.Host())
    want = golden_cases.expected_of(case)
    rtol, atol = golden_cases.tolerance(case)
    support.assert_close(got, want, rtol, atol, case["name"])


@pytest.mark.parametrize("case", golden_cases.TENSOR_CASES, ids=lambda c: c["name"])
def test_real_reference_matches_its_vectors(reference, case):
    """Same vectors through the real reference build: checks the harness, not the oracle."""
    with support.use_functions(reference):
        got = golden_cases.run(case, ta.Host())
    rtol, atol = golden_cases.tolerance(case)
    support.assert_close(got, golden_cases.expected_of(case), rtol, atol, case["name"])


def _case(name):
    return next(c for c in golden_cases.CASES if c["name"] == name)


def test_llama_freq_cis(oracle):
    """polar(ones, position * exp(-2*d*scale)) against the table of tests/cpu/test-complex.cpp:93-108."""
    c = _case("llama_freq_cis")
    dim, seq = c["model_dimension"], c["sequence_length"]
    scale = math.log(c["theta"]) / dim
    phi = np.array([[p * math.exp(-2 * d * scale) for d in range(dim // 2)] for p in range(seq)])
    rho = np.ones_like(phi)
    z = ops.polar(ta.tensor(rho, ta.float64), ta.tensor(phi, ta.float64))
    got = ops.realify(z).numpy()
    want = np.array(c["expected"]["data"]).reshape(c["expected"]["shape"])
    support.assert_close(got, want, c["rtol"], c["atol"], "freq_cis")


def _value(v):
    return float(v) if isinstance(v, str) else v


def test_scalar_half_conversion_bits():
    for value, bits in _case("half_bits")["pairs"]:
        assert ops.float_to_half_bits(_value(value)) == bits, value


def test_scalar_bfloat_conversion_bits():
    for value, bits in _case("bhalf_bits")["pairs"]:
        assert int.from_bytes(ops.scalar_bytes(_value(value), ta.bfloat16), "little") == bits, value


def test_native_16bit_accumulation_known_answers(oracle):
    """fp16 accumulation in the reference saturates: 4096 ones sum to 2048; the mixed
    f16 x f32 entry (fp32 accumulator) gives 4096."""
    n = _case("native_f16_dot_of_ones")["length"]
    x = support.host_tensor(np.ones((1, n)), ta.float16)
    try:
        oracle.set_accumulate(False)
        assert ops.matmul(x, x.transpose()).numpy()[0, 0] == _case("native_f16_dot_of_ones")["expected_value"]
        assert ops.sum(x, -1).numpy()[0] == _case("native_f16_sum_of_ones")["expected_value"]
    finally:
        oracle.set_accumulate(True)
    y = support.host_tensor(np.ones((n, 1)), ta.float32)
    assert ops.matmul(x, y).numpy()[0, 0] == _case("mixed_f16_f32_dot_of_ones")["expected_value"]
    assert ops.matmul(x, x.transpose()).numpy()[0, 0] == 4096.0
