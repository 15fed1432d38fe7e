"""The decoder-layer composition against a textbook numpy implementation (float64), on the host.

This pins the composition itself — the rotary pairing, the interleaved repetition of KV heads, the softmax
written without a division, SiLU written with rsqrt — independently of any device."""
import numpy as np

import support
import tannic_amd as ta
from tannic_amd import decoder_layer as dl


def numpy_layer(s, w, x, seq):
    def rms(v, g):
        return v / np.sqrt((v * v).mean(-1, keepdims=True) + s.eps) * g

    def rope(t):                       # t: [heads, seq, d]; pairs (2i, 2i+1)
        inv = s.theta ** (-np.arange(0, s.head_dim, 2, dtype=np.float64) / s.head_dim)
        ang = np.outer(np.arange(seq), inv)
        even, odd = t[..., 0::2], t[..., 1::2]
        out = np.empty_like(t)
        out[..., 0::2] = even * np.cos(ang) - odd * np.sin(ang)
        out[..., 1::2] = even * np.sin(ang) + odd * np.cos(ang)
        return out

    xn = rms(x[0], w["g1"])
    q = (xn @ w["wq"].T).reshape(seq, s.heads, s.head_dim).transpose(1, 0, 2)
    k = (xn @ w["wk"].T).reshape(seq, s.kv_heads, s.head_dim).transpose(1, 0, 2)
    v = (xn @ w["wv"].T).reshape(seq, s.kv_heads, s.head_dim).transpose(1, 0, 2)
    q, k = rope(q), rope(k)
    group = s.heads // s.kv_heads
    k, v = np.repeat(k, group, axis=0), np.repeat(v, group, axis=0)
    scores = q @ k.transpose(0, 2, 1) / np.sqrt(s.head_dim)
    scores = np.where(np.tril(np.ones((seq, seq), dtype=bool)), scores, -np.inf)
    p = np.exp(scores - scores.max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)
    o = (p @ v).transpose(1, 0, 2).reshape(seq, s.heads * s.head_dim)
    h = x[0] + o @ w["wo"].T
    hn = rms(h, w["g2"])
    g = hn @ w["w1"].T
    y = (g / (1.0 + np.exp(-g)) * (hn @ w["w3"].T)) @ w["w2"].T
    return (h + y)[None]


def test_composition_is_a_llama_layer(oracle):
    s = dl.LayerShape(hidden=96, heads=6, kv_heads=2, head_dim=16, ffn=160)
    seq = 12
    values = {}
    for i, (name, shape) in enumerate(dl.weight_shapes(s).items()):
        values[name] = support.uniform(5, 20 + i, shape, 0.5, 1.5) if name.startswith("g") else support.normal(5, 20 + i, shape, 0.08)
    x = support.normal(5, 1, (1, seq, s.hidden), 1.0)
    f32 = {k: v.astype(np.float32).astype(np.float64) for k, v in values.items()}
    x32 = x.astype(np.float32).astype(np.float64)
    want = numpy_layer(s, f32, x32, seq)
    env = ta.Host()
    w = {k: ta.tensor(v, ta.float32, env) for k, v in values.items()}
    cos, sin = dl.rotary_tables(s, seq, ta.float32, env)
    with support.use_functions(oracle):
        got = dl.forward(s, w, ta.tensor(x, ta.float32, env), cos, sin, dl.causal_mask(seq, ta.float32, env), ta.tensor(np.ones(1), ta.float32, env)).numpy()
    np.testing.assert_allclose(got, want, rtol=2e-4, atol=2e-4)
    assert dl.flop_count(s, seq) == 2 * (seq * s.hidden * 160 + seq * 96 * s.hidden + 2 * s.heads * seq * seq * s.head_dim + 3 * seq * s.hidden * s.ffn)
