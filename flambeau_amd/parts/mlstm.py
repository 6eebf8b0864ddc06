"""The matrix memory of xLSTM (mLSTM) as a mixer with a state per request.

With h the mixer's input, per head: q = W_q h / sqrt(dim), k = W_k h, v = W_v h, a log input gate
i = cap * tanh((W_i h + b_i) / cap) and a log forget gate f = logsigmoid(cap * tanh((W_f h + b_f) / cap)).
The memory S [dim, vdim] and the normaliser n [dim] start at zero, the running maximum m at 0:
    m' = max(f + m, i);  S <- exp(f + m - m') S + exp(i - m') k v^T;  n likewise with k alone;
    o = S^T q / (max(|n . q|, exp(-m')) + 1e-6).
Every head's o is divided by its root mean square, the heads side by side are multiplied by a gain
and by sigmoid(W_g h), then projected.  All six projections of h are one joined product with 32-bit
results; gates, state and the walk are 32-bit; the state lives in the request's slot
(``StateSpec``), so a prompt may be cut anywhere.
"""
from __future__ import annotations

import torch

from ..config.base import ConfigError
from ..kernels import ops
from .base import MIXERS, Mixer, Product, StateSpec, TensorSpec


@MIXERS.register("mlstm")
class MLstm(Mixer):
    graph_safe = False          # a step run twice advances the state twice
    replayable = True

    def __init__(self, hidden_size: int, n_heads: int, head_dim: int, value_dim: int, gate_cap: float, eps: float):
        if head_dim > ops.mlstm_max_dim():
            raise ConfigError(f"mlstm: 'dim' {head_dim} is beyond what the kernel takes ({ops.mlstm_max_dim()})")
        self.hidden_size, self.n_heads, self.head_dim, self.value_dim = hidden_size, n_heads, head_dim, value_dim
        self.gate_cap, self.eps = float(gate_cap), float(eps)

    def cache_spec(self):
        return StateSpec((self.n_heads, ops.mlstm_state_floats(self.head_dim, self.value_dim)), torch.float32)

    def signature_group(self):
        return ("mlstm",)

    def step_signature(self, batch):
        return ()

    def tensors(self):
        W, H, D, Dv = self.hidden_size, self.n_heads, self.head_dim, self.value_dim
        return {"q.weight": TensorSpec((H * D, W)), "k.weight": TensorSpec((H * D, W)), "v.weight": TensorSpec((H * Dv, W)),
                "g.weight": TensorSpec((H * Dv, W)), "o.weight": TensorSpec((W, H * Dv)),
                "norm.weight": TensorSpec((H * Dv,), "vector32"),
                "i.weight": TensorSpec((H, W)), "i.bias": TensorSpec((H,), "vector32", init="normal"),
                "f.weight": TensorSpec((H, W)), "f.bias": TensorSpec((H,), "vector32", init="normal")}

    def bind(self, weights, rt):
        self.rt = rt
        H, D, Dv = self.n_heads, self.head_dim, self.value_dim
        self.w_in = rt.prepare_weight(torch.cat([weights[k + ".weight"] for k in ("q", "k", "v", "g", "i", "f")], dim=0).contiguous())
        self.cols = (0, H * D, 2 * H * D, 2 * H * D + 2 * H * Dv, 2 * H * D + 2 * H * Dv + H)     # q, k, v, i, f
        self.gate_col = 2 * H * D + H * Dv
        self.bias_i, self.bias_f = weights["i.bias"], weights["f.bias"]
        self.norm = weights["norm.weight"]
        self.w_o = rt.prepare_weight(weights["o.weight"])

    def forward(self, x, step, cache):
        rt, n = self.rt, x.shape[0]
        H, D, Dv = self.n_heads, self.head_dim, self.value_dim
        proj = rt.buffer("ml_proj", n, self.w_in.rows, torch.float32)
        rt.gemm(x, self.w_in, proj)
        hidden = rt.buffer("ml_hidden", n, H * Dv, torch.float32)
        factors = rt.buffer("ml_factors", n, 3 * H, torch.float32)
        ops.mlstm_scan(proj, self.cols, self.bias_i, self.bias_f, self.gate_cap, D ** -0.5, cache.state,
                       step.seq_q_start, step.seq_q_len, step.seq_slots, hidden, factors, H, D, Dv)
        out = rt.buffer("ml_out", n, H * Dv)
        ops.headnorm_gate(hidden, self.norm, proj, self.gate_col, out, H, self.eps)
        return Product(out, self.w_o)
