"""A plain, slow implementation of the Kuvidra design in float64 numpy, one function per mechanism.

Everything is written from the design's equations and shares no code with the package: whole
sequences at once, no cache, no batching.  ``forward`` takes a config.json dictionary and the
tensors by their file names.

Notation: ``x`` [T, W] residual stream of one sequence, ``h`` a normed input, ``eps`` the norm's
constant.  Linear weights are ``[out, in]`` and applied as ``h @ W.T``.
"""
from __future__ import annotations

import math

import numpy as np


def rms_norm(x, w, eps):
    """x / sqrt(mean(x^2) + eps) * w over the last axis (``w`` None: no gain)."""
    y = x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)
    return y if w is None else y * w


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def gelu_erf(z):
    erf = np.vectorize(math.erf)
    return 0.5 * z * (1.0 + erf(z / math.sqrt(2.0)))


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def log_sigmoid(z):
    return -np.logaddexp(0.0, -z)


# ---------------------------------------------------------------- mixers
def latent_attention(h, t, prefix, mixer, eps):
    """Causal softmax attention whose keys and values are both expanded from one normed latent per
    token; queries pass through a normed latent of their own; every head's output is gated by a
    sigmoid of the mixer's input."""
    H, D, Dv = mixer["heads"], mixer["dim"], mixer["vdim"]
    T = h.shape[0]
    cq = rms_norm(h @ t[prefix + "dq"].T, t[prefix + "dq.norm"], eps)
    q = (cq @ t[prefix + "uq"].T).reshape(T, H, D)
    c = rms_norm(h @ t[prefix + "dkv"].T, t[prefix + "dkv.norm"], eps)
    k = (c @ t[prefix + "uk"].T).reshape(T, H, D)
    v = (c @ t[prefix + "uv"].T).reshape(T, H, Dv)
    gate = sigmoid(h @ t[prefix + "g"].T)                              # [T, H]
    out = np.zeros((T, H, Dv))
    for i in range(T):
        s = np.einsum("hd,jhd->hj", q[i], k[:i + 1]) * mixer["scale"]
        p = np.exp(s - s.max(axis=1, keepdims=True))
        p /= p.sum(axis=1, keepdims=True)
        out[i] = np.einsum("hj,jhv->hv", p, v[:i + 1])
    out *= gate[:, :, None]
    return out.reshape(T, H * Dv) @ t[prefix + "o"].T


def mlstm(h, t, prefix, mixer, eps):
    """Matrix memory with exponential gating, token by token.  Per head: a log input gate and a log
    forget gate (both soft-capped), a running maximum m that starts at 0, the memory S [D, Dv] and
    the normaliser n [D], both from zero."""
    H, D, Dv, cap = mixer["heads"], mixer["dim"], mixer["vdim"], mixer["gate_cap"]
    T = h.shape[0]
    q = (h @ t[prefix + "q"].T).reshape(T, H, D) * D ** -0.5
    k = (h @ t[prefix + "k"].T).reshape(T, H, D)
    v = (h @ t[prefix + "v"].T).reshape(T, H, Dv)
    gi = cap * np.tanh((h @ t[prefix + "i"].T + t[prefix + "i.b"]) / cap)
    gf = log_sigmoid(cap * np.tanh((h @ t[prefix + "f"].T + t[prefix + "f.b"]) / cap))
    out = np.zeros((T, H, Dv))
    for a in range(H):
        S, n, m = np.zeros((D, Dv)), np.zeros(D), 0.0
        for i in range(T):
            m_new = max(gf[i, a] + m, gi[i, a])
            keep, take = math.exp(gf[i, a] + m - m_new), math.exp(gi[i, a] - m_new)
            S = keep * S + take * np.outer(k[i, a], v[i, a])
            n = keep * n + take * k[i, a]
            m = m_new
            out[i, a] = (S.T @ q[i, a]) / (max(abs(n @ q[i, a]), math.exp(-m)) + 1e-6)
    out = rms_norm(out, None, eps).reshape(T, H * Dv) * t[prefix + "norm"]
    out = out * sigmoid(h @ t[prefix + "g"].T)
    return out @ t[prefix + "o"].T


# ---------------------------------------------------------------- feed-forwards
def dense_ff(h, t, prefix):
    return gelu_erf(h @ t[prefix + "up"].T) @ t[prefix + "down"].T


def gated_expert(h, t, prefix):
    return (silu(h @ t[prefix + "gate"].T) * (h @ t[prefix + "up"].T)) @ t[prefix + "down"].T


def moe_ff(h, t, prefix, mlp):
    """Sigmoid router, the ``top`` largest scores, not renormalised; the score scales the expert's
    INPUT.  A shared expert, gated per token, is added."""
    T = h.shape[0]
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    s = sigmoid(h @ t[prefix + "router"].T)
    out = np.zeros((T, t[prefix + "e0.down"].shape[0]))
    for i in range(T):
        chosen = sorted(range(E), key=lambda e: (-s[i, e], e))[:top]
        for e in chosen:
            out[i] += gated_expert(s[i, e] * h[i:i + 1], t, f"{prefix}e{e}.")[0]
    if mlp.get("shared"):
        out += sigmoid(h @ t[prefix + "shared.sg"].T) * gated_expert(h, t, prefix + "shared.")
    return out


# ---------------------------------------------------------------- the model
def run_order(config):
    """``[(layer, pass number or None, first of its pass)]`` in the order the layers run."""
    L = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return [(l, None, False) for l in range(L)]
    order = [(l, None, False) for l in range(loop["start"])]
    for p in range(loop["times"]):
        order += [(l, p, l == loop["start"]) for l in range(loop["start"], loop["stop"])]
    return order + [(l, None, False) for l in range(loop["stop"], L)]


def layer(x, t, l, spec, eps):
    h = rms_norm(x, t[f"l{l}.norm1"], eps)
    mix = {"latent_attention": latent_attention, "mlstm": mlstm}[spec["type"]]
    d = mix(h, t, f"l{l}.mix.", spec["mixer"], eps)
    mlp = spec.get("mlp")
    if mlp:
        d = d + (dense_ff(h, t, f"l{l}.mlp.") if mlp["kind"] == "dense" else moe_ff(h, t, f"l{l}.mlp.", mlp))
    return x + d


def forward(config, tensors, tokens, return_layers=False):
    """Logits [T, vocab] of one sequence (and the residual stream after every layer run)."""
    t = {k: np.asarray(v, dtype=np.float64) for k, v in tensors.items()}
    eps = config["norm"]["eps"]
    x = t["embed"][np.asarray(tokens)]
    x0 = x
    after = []
    for l, p, first in run_order(config):
        if first:
            x = np.concatenate([x, x0], axis=1) @ t["loop.in"].T + t["loop.step"][p]
        x = layer(x, t, l, config["layers"][l], eps)
        after.append(x)
    logits = rms_norm(x, t["final.norm"], eps) @ t["embed"].T
    return (logits, np.stack(after)) if return_layers else logits
