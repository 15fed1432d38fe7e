"""One decoder layer composed from the operators: the device against the CPU checker (fp32-accumulating mode).

Every elementwise step rounds once from fp32 on both sides; products and row sums add in a different order, so
results differ by bf16 roundings that the normalisations pass on.  The bar is a fraction of the output's spread."""
import numpy as np
import pytest

import support
import tannic_amd as ta
from tannic_amd import decoder_layer as dl

pytestmark = pytest.mark.gpu


def build(s, seq, dtype, env, seed):
    w = {}
    for i, (name, shape) in enumerate(dl.weight_shapes(s).items()):
        if name.startswith("g"):
            values = np.ones(shape)
        else:
            values = support.normal(seed, 10 + i, shape, 0.02 if dtype is not ta.float32 else 0.02)
        w[name] = ta.tensor(values, dtype, env)
    x = ta.tensor(support.normal(seed, 1, (1, seq, s.hidden), 1.0), dtype, env)
    cos, sin = dl.rotary_tables(s, seq, dtype, env)
    mask = dl.causal_mask(seq, dtype, env)
    one = ta.tensor(np.ones(1), dtype, env)
    return w, x, cos, sin, mask, one


@pytest.mark.parametrize("dtype,bar", [(ta.float32, 2e-4), (ta.bfloat16, 0.06)], ids=["float32", "bfloat16"])
def test_small_layer_matches_the_checker(device, oracle, dtype, bar):
    s = dl.LayerShape(hidden=256, heads=4, kv_heads=2, head_dim=64, ffn=512)
    seq = 40
    host = build(s, seq, dtype, ta.Host(), 3)
    dev = build(s, seq, dtype, device, 3)
    with support.use_functions(oracle):
        want = dl.forward(s, *host).numpy().astype(np.float64)
    got = dl.forward(s, *dev).numpy().astype(np.float64)
    assert got.shape == want.shape == (1, seq, s.hidden)
    assert np.isfinite(got).all()
    spread = want.std()
    assert np.abs(got - want).max() <= bar * spread, (np.abs(got - want).max(), spread)


def test_layer_is_causal(device):
    """Changing a later position must not change earlier outputs."""
    s = dl.LayerShape(hidden=128, heads=4, kv_heads=2, head_dim=32, ffn=256)
    seq = 16
    w, x, cos, sin, mask, one = build(s, seq, ta.float32, device, 4)
    a = dl.forward(s, w, x, cos, sin, mask, one).numpy()
    xv = x.numpy().copy()
    xv[0, 10:] += 1.0
    b = dl.forward(s, w, ta.tensor(xv, ta.float32, device), cos, sin, mask, one).numpy()
    np.testing.assert_array_equal(a[0, :10], b[0, :10])
    assert np.abs(a[0, 10:] - b[0, 10:]).max() > 1e-3


@pytest.mark.parametrize("dtype,bar", [(ta.float32, 2e-4), (ta.bfloat16, 0.06)], ids=["float32", "bfloat16"])
def test_one_pass_operators_give_the_same_layer(device, oracle, dtype, bar):
    """The layer written with rms_norm / rope / softmax / swiglu against the checker's evaluation of the chains."""
    s = dl.LayerShape(hidden=256, heads=4, kv_heads=2, head_dim=64, ffn=512)
    seq = 40
    host = build(s, seq, dtype, ta.Host(), 5)
    w, x, cos, sin, mask, one = build(s, seq, dtype, device, 5)
    with support.use_functions(oracle):
        want = dl.forward(s, *host).numpy().astype(np.float64)
    got = dl.forward_fused(s, w, x, cos, sin, mask).numpy().astype(np.float64)
    assert got.shape == want.shape and np.isfinite(got).all()
    assert np.abs(got - want).max() <= bar * want.std(), (np.abs(got - want).max(), want.std())
    # with q/k/v and gate/up as one product each: the same arithmetic per output element, so the same bits
    packed = dl.forward_fused(s, dl.pack_weights(w), x, cos, sin, mask).numpy().astype(np.float64)
    assert np.abs(packed - want).max() <= bar * want.std()
    if dtype is ta.float32:
        np.testing.assert_allclose(packed, got, rtol=1e-5, atol=1e-6)
