"""A plain, slow implementation of the Bugidra design in float64 numpy, one function per mechanism.

Everything is written from the design's equations and shares no code with the package: whole
sequences at once, no cache, no batching.  ``forward`` takes a config.json dictionary and the
tensors by their file names.

Notation: ``x`` [T, W] residual stream of one sequence, ``h`` a normed input, ``eps`` the norm's
constant, ``t`` the tensors by file name, ``p`` the prefix of a mixer's tensors.  Linear weights are
``[out, in]`` and applied as ``h @ W.T``.
"""
from __future__ import annotations

import math

import numpy as np


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rms_norm(x, w, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis, times ``w`` unless it is None."""
    y = x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)
    return y if w is None else y * w


def dynamic_tanh(x, t, name):
    """tanh(alpha x) * w + b: a norm that computes no statistics."""
    return np.tanh(float(t[name + ".alpha"]) * x) * t[name] + t[name + ".b"]


# ---------------------------------------------------------------- rotations
def rotary_frequencies(rot):
    """The ladder base^(-2i/dims), blended towards base^(-2i/dims) / factor for the slow dims when the
    config has a ``scaling`` section; returns (frequencies [dims/2], factor on cos and sin)."""
    dims, base = rot["dims"], float(rot["base"])
    f = np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)])
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, original = float(sc["factor"]), float(sc["original"])

    def turn(n):       # the (fractional) index whose wave makes n turns over the original length
        return dims * math.log(original / (2.0 * math.pi * n)) / (2.0 * math.log(base))

    lo = max(math.floor(turn(float(sc["fast"]))), 0)
    hi = min(math.ceil(turn(float(sc["slow"]))), dims - 1)
    ramp = np.clip((np.arange(dims // 2) - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate(x, positions, rot, layout):
    """x [T, heads, dim]: the first ``dims`` values of every head turned by position * frequency.
    ``layout`` "half": value i pairs with i + dims/2; "interleaved": 2i pairs with 2i + 1."""
    dims = rot["dims"]
    f, mag = rotary_frequencies(rot)
    a = np.asarray(positions, dtype=np.float64)[:, None] * f[None, :]      # [T, dims/2]
    c, s = (np.cos(a) * mag)[:, None, :], (np.sin(a) * mag)[:, None, :]
    y = x.copy()
    if layout == "half":
        u, v = x[..., :dims // 2], x[..., dims // 2:dims]
        y[..., :dims // 2] = u * c - v * s
        y[..., dims // 2:dims] = v * c + u * s
    else:
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        y[..., 0:dims:2] = u * c - v * s
        y[..., 1:dims:2] = v * c + u * s
    return y


# ---------------------------------------------------------------- softmax attention
def causal_softmax_attention(q, k, v, scale, softcap=None):
    """q [T, H, D], k [T, G, D], v [T, G, Dv]; query head h reads key/value head h // (H / G);
    token i sees j <= i; optional cap * tanh(score / cap) before the softmax."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        if softcap is not None:
            s = softcap * np.tanh(s / softcap)
        s = np.where(np.tril(np.ones((T, T), dtype=bool)), s, -np.inf)
        pr = np.exp(s - s.max(axis=1, keepdims=True))
        out[:, h] = (pr / pr.sum(axis=1, keepdims=True)) @ v[:, g]
    return out


def attention_mixer(h, t, p, m, eps, shared):
    """Queries and keys normed over the whole projection, interleaved rotation, capped scores, values
    blended with the first such layer's, a sigmoid gate on the heads' outputs."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rms_norm(h @ t[p + "q"].T, t[p + "q.norm"], eps).reshape(T, H, D)
    k = rms_norm(h @ t[p + "k"].T, t[p + "k.norm"], eps).reshape(T, G, D)
    v = (h @ t[p + "v"].T).reshape(T, G, Dv)
    pos = np.arange(T)
    if m.get("rot"):
        q, k = rotate(q, pos, m["rot"], "interleaved"), rotate(k, pos, m["rot"], "interleaved")
    if m.get("v_mix"):
        if "v_first" in shared:
            lam = float(t[p + "vmix"])
            v = (1.0 - lam) * v + lam * shared["v_first"]
        else:
            shared["v_first"] = v
    o = causal_softmax_attention(q, k, v, m["scale"], m.get("softcap"))
    o = o.reshape(T, H * Dv) * sigmoid(h @ t[p + "g"].T)
    return o @ t[p + "o"].T


def rotated_attention(h, t, p, m, eps):
    """The softmax half of a side-by-side mixer: half-split rotation (with its frequency blend), then
    every head of q and k divided by its root mean square."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ t[p + "q"].T).reshape(T, H, D)
    k = (h @ t[p + "k"].T).reshape(T, G, D)
    v = (h @ t[p + "v"].T).reshape(T, G, Dv)
    pos = np.arange(T)
    if m.get("rot"):
        q, k = rotate(q, pos, m["rot"], "half"), rotate(k, pos, m["rot"], "half")
    q, k = rms_norm(q, None, eps), rms_norm(k, None, eps)
    o = causal_softmax_attention(q, k, v, m["scale"])
    return o.reshape(T, H * Dv) @ t[p + "o"].T


# ---------------------------------------------------------------- recurrences
def retention(h, t, p, m, eps):
    """Linear attention with a fixed decay per head: S <- decay S + k v^T, o = S^T q."""
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ t[p + "q"].T).reshape(T, H, D)
    k = (h @ t[p + "k"].T).reshape(T, H, D)
    v = (h @ t[p + "v"].T).reshape(T, H, Dv)
    pos = np.arange(T)
    if m.get("rot"):
        q, k = rotate(q, pos, m["rot"], "half"), rotate(k, pos, m["rot"], "half")
    k = k * D ** -0.5
    o = np.zeros((T, H, Dv))
    for a in range(H):
        S = np.zeros((D, Dv))
        for i in range(T):
            S = float(m["decay"][a]) * S + np.outer(k[i, a], v[i, a])
            o[i, a] = S.T @ q[i, a]
    o = rms_norm(o, None, eps).reshape(T, H * Dv) * silu(h @ t[p + "g"].T)
    return o @ t[p + "o"].T


def side_by_side(h, t, p, m, eps):
    """Half the sum of both halves, each normed over the model width with its own gain."""
    left = rms_norm(rotated_attention(h, t, p + "left.", m["left"], eps), t[p + "left.out"], eps)
    right = rms_norm(retention(h, t, p + "right.", m["right"], eps), t[p + "right.out"], eps)
    return 0.5 * (left + right)


def short_convolution(x, w):
    """x [T, C], w [C, taps]: y[i] = sum_j w[:, taps - 1 - j] x[i - j], zeros before the start."""
    T, taps = x.shape[0], w.shape[1]
    y = np.zeros_like(x)
    for j in range(min(taps, T)):
        y[j:] += x[:T - j] * w[:, taps - 1 - j]
    return y


def gated_delta(h, t, p, m, eps):
    """The gated delta rule: S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(short_convolution(h @ t[p + "q"].T, t[p + "q.conv"])).reshape(T, G, D)
    k = silu(short_convolution(h @ t[p + "k"].T, t[p + "k.conv"])).reshape(T, G, D)
    v = silu(short_convolution(h @ t[p + "v"].T, t[p + "v.conv"])).reshape(T, H, Dv)
    q = q / np.sqrt((q * q).sum(-1, keepdims=True) + 1e-6) * D ** -0.5
    k = k / np.sqrt((k * k).sum(-1, keepdims=True) + 1e-6)
    beta = sigmoid(h @ t[p + "b"].T)                                         # [T, H]
    g = np.exp(-np.exp(t[p + "A_log"]) * softplus(h @ t[p + "a"].T + t[p + "dt_bias"]))
    o = np.zeros((T, H, Dv))
    for a in range(H):
        c = a // (H // G)
        S = np.zeros((D, Dv))
        for i in range(T):
            S = g[i, a] * S
            u = beta[i, a] * (v[i, a] - S.T @ k[i, c])
            S = S + np.outer(k[i, c], u)
            o[i, a] = S.T @ q[i, c]
    o = rms_norm(o, t[p + "norm"], eps).reshape(T, H * Dv) * silu(h @ t[p + "g"].T)
    return o @ t[p + "o"].T


# ---------------------------------------------------------------- the model
def feed_forward(h, t, p):
    return (gelu_tanh(h @ t[p + "gate"].T) * (h @ t[p + "up"].T)) @ t[p + "down"].T


def forward(config, t, tokens, return_layers=False):
    """Logits [T, vocab] of one sequence from its first token; with ``return_layers`` also the stream
    after every layer."""
    t = {k: np.asarray(v, dtype=np.float64) for k, v in t.items()}
    eps = config["norm"]["eps"]
    x = t["embed"][np.asarray(tokens)] * config["embedding"]["scale"]
    shared, after = {}, []
    for i, layer in enumerate(config["layers"]):
        p = f"l{i}."
        h = dynamic_tanh(x, t, p + "norm1")
        kind, m = layer["type"], layer["mixer"]
        if kind == "attention":
            x = x + attention_mixer(h, t, p + "mix.", m, eps, shared)
        elif kind == "parallel":
            x = x + side_by_side(h, t, p + "mix.", m, eps)
        elif kind == "delta":
            x = x + gated_delta(h, t, p + "mix.", m, eps)
        else:
            raise ValueError(kind)
        if layer.get("mlp") is not None:
            x = x + feed_forward(dynamic_tanh(x, t, p + "norm2"), t, p + "mlp.")
        after.append(x.copy())
    logits = dynamic_tanh(x, t, "final.norm") @ t["head"].T
    return (logits, np.stack(after)) if return_layers else logits
