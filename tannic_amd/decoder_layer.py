"""One Llama-3 decoder layer written with the front end's operators only — the caller's side of the
boundary for the decoder-layer workload (hidden 4096, 32 heads, 8 KV heads, head size 128, SwiGLU FFN 14336).

Every step is an expression a Tannic program can write today: there is no division, no cast and no
softmax in the front end, so the reciprocal of a sum is ``rsqrt(s) * rsqrt(s)``, the rotary embedding is
the real-valued form on stride-2 slices (complex tensors exist only in fp32/fp64, ``include/tannic/complex.hpp:53-58``)
and the causal mask is a host-built table added to the scores.  Each operator call is one backend call with
its own destination, exactly as ``Callback`` issues them (``include/tannic/callback.hpp:46-178``); the only
operator without a reference twin is the row maximum of the softmax (``ops.max``).
"""
import math

import numpy as np

from . import ops, types
from .tensor import Tensor, tensor


class LayerShape:
    def __init__(self, hidden=4096, heads=32, kv_heads=8, head_dim=128, ffn=14336, eps=1e-5, theta=500000.0):
        self.hidden, self.heads, self.kv_heads, self.head_dim, self.ffn = hidden, heads, kv_heads, head_dim, ffn
        self.eps, self.theta = eps, theta


def weight_shapes(s):
    """name -> shape of the layer's parameters (projection weights are [out, in], as ``nn.Linear`` keeps them)."""
    return {
        "wq": (s.heads * s.head_dim, s.hidden), "wk": (s.kv_heads * s.head_dim, s.hidden), "wv": (s.kv_heads * s.head_dim, s.hidden),
        "wo": (s.hidden, s.heads * s.head_dim), "w1": (s.ffn, s.hidden), "w3": (s.ffn, s.hidden), "w2": (s.hidden, s.ffn),
        "g1": (s.hidden,), "g2": (s.hidden,),
    }


def rotary_tables(s, seq, dtype, env):
    """cos/sin of position * theta^(-2i/d), [seq, head_dim/2], rounded to ``dtype``."""
    inv = s.theta ** (-np.arange(0, s.head_dim, 2, dtype=np.float64) / s.head_dim)
    ang = np.outer(np.arange(seq, dtype=np.float64), inv)
    return tensor(np.cos(ang), dtype, env), tensor(np.sin(ang), dtype, env)


def causal_mask(seq, dtype, env):
    """0 on and below the diagonal, -inf above it."""
    m = np.where(np.tril(np.ones((seq, seq), dtype=bool)), 0.0, -np.inf)
    return tensor(m, dtype, env)


def rms_norm(x, gain, eps):
    ms = ops.mean(ops.mul(x, x), -1, True)
    return ops.mul(ops.mul(x, ops.rsqrt(ms, eps)), gain)


def rope(q, cos, sin):
    """q: [1, heads, seq, head_dim] (any strides).  Pairs (2i, 2i+1) are rotated by the position's angle."""
    qc = ops.repack(q)
    b, h, n, d = qc.shape
    q5 = qc.view(b, h, n, d // 2, 2)
    even, odd = q5[..., 0], q5[..., 1]
    re = ops.sub(ops.mul(even, cos), ops.mul(odd, sin))
    im = ops.add(ops.mul(even, sin), ops.mul(odd, cos))
    out = Tensor(qc.dtype, qc.shape).initialize(qc.environment)
    o5 = out.view(b, h, n, d // 2, 2)
    ops.copy_into(o5[..., 0], re)
    ops.copy_into(o5[..., 1], im)
    return out


def softmax_rows(scores):
    m = ops.max(scores, -1, True)
    e = ops.exp(ops.sub(scores, m))
    r = ops.rsqrt(ops.sum(e, -1, True))
    return ops.mul(ops.mul(e, r), r)


def silu(g, one):
    sg = ops.rsqrt(ops.add(ops.exp(ops.neg(g)), one))     # sigmoid(g) = sg * sg
    return ops.mul(ops.mul(g, sg), sg)


def pack_weights(w):
    """Adds the row-wise concatenations ``wqkv = [wq; wk; wv]`` and ``w13 = [w1; w3]`` to the parameter dictionary, so
    that the projections sharing an input are one product each (done once, when the parameters are loaded)."""
    packed = dict(w)
    packed["wqkv"] = ops.concatenate(ops.concatenate(w["wq"], w["wk"], 0), w["wv"], 0)
    packed["w13"] = ops.concatenate(w["w1"], w["w3"], 0)
    return packed


def split_heads(t, heads):
    """``[1, seq, heads * d]`` with unit stride along the last axis (a column slice included) seen as ``[1, heads, seq, d]``."""
    b, seq, width = t.shape
    d = width // heads
    return t._view((b, seq, heads, d), (t.strides[0], t.strides[1], d, 1)).transpose(1, 2)


def _keep(trace, **stages):
    """Records intermediate tensors by name when a caller asked for them (tests check every stage by itself)."""
    if trace is not None:
        trace.update(stages)


def forward_fused(s, w, x, cos, sin, mask, trace=None):
    """The same layer with the device library's one-pass operators (``ops.rms_norm``, ``ops.rope``, ``ops.softmax``,
    ``ops.swiglu``) in place of the chains; these have no counterpart in the reference's front end.  With the
    concatenated parameters of ``pack_weights`` the q/k/v and the gate/up projections are one product each and their
    parts are column slices of its result.  ``trace``: a dictionary that receives the intermediate tensors."""
    _, seq, _ = x.shape
    nq, nkv = s.heads * s.head_dim, s.kv_heads * s.head_dim
    xn = ops.rms_norm(x, w["g1"], s.eps)
    if "wqkv" in w:
        qkv = ops.matmul(xn, w["wqkv"].transpose())
        q, k, v = qkv[..., 0:nq], qkv[..., nq:nq + nkv], qkv[..., nq + nkv:nq + 2 * nkv]
    else:
        q, k, v = (ops.matmul(xn, w[name].transpose()) for name in ("wq", "wk", "wv"))
    _keep(trace, xn=xn, q=q, k=k, v=v)
    q, k, v = split_heads(q, s.heads), split_heads(k, s.kv_heads), split_heads(v, s.kv_heads)
    q, k = ops.rope(q, cos, sin), ops.rope(k, cos, sin)
    _keep(trace, q_rot=q, k_rot=k)
    group = s.heads // s.kv_heads
    k, v = ops.repeat(k, group, 1), ops.repeat(v, group, 1)
    scores = ops.matmul(q, k.transpose(-1, -2))
    p = ops.softmax(scores, mask, 1.0 / math.sqrt(s.head_dim))
    pv = ops.matmul(p, v)
    o = ops.repack(pv.transpose(1, 2)).view(1, seq, s.heads * s.head_dim)
    h = ops.add(x, ops.matmul(o, w["wo"].transpose()))
    hn = ops.rms_norm(h, w["g2"], s.eps)
    if "w13" in w:
        both = ops.matmul(hn, w["w13"].transpose())
        gate, up = both[..., 0:s.ffn], both[..., s.ffn:2 * s.ffn]
    else:
        gate, up = ops.matmul(hn, w["w1"].transpose()), ops.matmul(hn, w["w3"].transpose())
    act = ops.swiglu(gate, up)
    y = ops.matmul(act, w["w2"].transpose())
    out = ops.add(h, y)
    _keep(trace, k_all=k, v_all=v, scores=scores, p=p, pv=pv, o=o, h=h, hn=hn, gate=gate, up=up, act=act, y=y, out=out)
    return out


def forward(s, w, x, cos, sin, mask, one, trace=None):
    """x: [1, seq, hidden].  Returns the layer's output, same shape and dtype.  ``trace``: a dictionary that receives
    the intermediate tensors."""
    _, seq, _ = x.shape
    xn = rms_norm(x, w["g1"], s.eps)
    q = ops.matmul(xn, w["wq"].transpose())
    k = ops.matmul(xn, w["wk"].transpose())
    v = ops.matmul(xn, w["wv"].transpose())
    _keep(trace, xn=xn, q=q, k=k, v=v)
    q = q.view(1, seq, s.heads, s.head_dim).transpose(1, 2)
    k = k.view(1, seq, s.kv_heads, s.head_dim).transpose(1, 2)
    v = v.view(1, seq, s.kv_heads, s.head_dim).transpose(1, 2)
    q, k = rope(q, cos, sin), rope(k, cos, sin)
    _keep(trace, q_rot=q, k_rot=k)
    group = s.heads // s.kv_heads
    k, v = ops.repeat(k, group, 1), ops.repeat(v, group, 1)
    scores = ops.scale(ops.matmul(q, k.transpose(-1, -2)), 1.0 / math.sqrt(s.head_dim))
    p = softmax_rows(ops.add(scores, mask))
    pv = ops.matmul(p, v)
    o = ops.repack(pv.transpose(1, 2)).view(1, seq, s.heads * s.head_dim)
    h = ops.add(x, ops.matmul(o, w["wo"].transpose()))
    hn = rms_norm(h, w["g2"], s.eps)
    gate = ops.matmul(hn, w["w1"].transpose())
    up = ops.matmul(hn, w["w3"].transpose())
    act = ops.mul(silu(gate, one), up)
    y = ops.matmul(act, w["w2"].transpose())
    out = ops.add(h, y)
    _keep(trace, k_all=k, v_all=v, scores=scores, p=p, pv=pv, o=o, h=h, hn=hn, gate=gate, up=up, act=act, y=y, out=out)
    return out


def flop_count(s, seq):
    """Multiply-adds of the layer's matrix products, times two."""
    proj = seq * s.hidden * (s.heads + 2 * s.kv_heads) * s.head_dim + seq * s.heads * s.head_dim * s.hidden
    attn = 2 * s.heads * seq * seq * s.head_dim
    ffn = 3 * seq * s.hidden * s.ffn
    return 2 * (proj + attn + ffn)
