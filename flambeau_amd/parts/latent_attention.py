"""Attention whose keys and values are both made from one cached latent per token.

With h the mixer's input: the queries pass through a normed latent, c_q = Norm(W_dq h), q = W_uq c_q;
the token's cached row is c = Norm(W_dkv h); head a has k = W_uk,a c and v = W_uv,a c, the score
(q_a . k_j) * scale over the keys j <= i, an ordinary softmax, and its output is multiplied by
sigmoid((W_g h)_a) before the output projection.  There is no position encoding.

Only c is cached (``PagedRowSpec``).  Since k and v are linear in c, the key expansion is applied to
the query instead (qa = W_uk,a^T q_a, then qa . c_j = q_a . k_j) and the value expansion to the
weighted sum of the rows (W_uv,a sum_j p_j c_j): no key or value is ever made for a cached token,
and the same kernels serve whole prompts, portions and single tokens.  This step's rows are stored
before attention runs.  The three projections of h (dq, dkv, g) are one joined product; scores,
softmax, the weighted sum and both small products per head are 32-bit.
"""
from __future__ import annotations

import torch

from ..config.base import ConfigError
from ..kernels import latent_attention as _kernels  # noqa: F401  (registers this mixer's kernel set)
from ..kernels import ops
from .base import MIXERS, Mixer, PagedRowSpec, Product, TensorSpec


@MIXERS.register("latent_attention")
class LatentAttention(Mixer):
    graph_safe = True
    replayable = True

    def __init__(self, hidden_size: int, n_heads: int, head_dim: int, value_dim: int, q_rank: int, kv_rank: int,
                 scale: float, eps: float, window: int = 0, gated: bool = True):
        if kv_rank > ops.latent_max_width():
            raise ConfigError(f"latent_attention: 'kv_rank' {kv_rank} is beyond what the kernel takes ({ops.latent_max_width()})")
        self.hidden_size, self.n_heads, self.head_dim, self.value_dim = hidden_size, n_heads, head_dim, value_dim
        self.q_rank, self.kv_rank = q_rank, kv_rank
        self.scale, self.eps, self.window, self.gated = float(scale), float(eps), int(window or 0), bool(gated)

    def cache_spec(self):
        return PagedRowSpec(self.kv_rank, self.window)

    def signature_group(self):
        return ("latent_attention", self.n_heads)

    def step_signature(self, batch):
        """Into how many parts the kernels deal the keys: all that this mixer decides from the contexts' lengths."""
        return self.kernels.signature(batch, self.n_heads)

    @classmethod
    def step_metadata_for(cls, batch, mixers):
        """The work lists the kernels of the mixers' runtime want for the batch."""
        return mixers[0].kernels.metadata(batch, mixers) if mixers else {}

    def tensors(self):
        W, H, D, Dv, Rq, R = self.hidden_size, self.n_heads, self.head_dim, self.value_dim, self.q_rank, self.kv_rank
        t = {"dq.weight": TensorSpec((Rq, W)), "dq_norm.weight": TensorSpec((Rq,), "vector32"),
             "uq.weight": TensorSpec((H * D, Rq)),
             "dkv.weight": TensorSpec((R, W)), "dkv_norm.weight": TensorSpec((R,), "vector32"),
             "uk.weight": TensorSpec((H * D, R)), "uv.weight": TensorSpec((H * Dv, R)),
             "o.weight": TensorSpec((W, H * Dv))}
        if self.gated:
            t["g.weight"] = TensorSpec((H, W))
        return t

    def bind(self, weights, rt):
        self.rt = rt
        joined = [weights["dq.weight"], weights["dkv.weight"]] + ([weights["g.weight"]] if self.gated else [])
        self.w_low = rt.prepare_weight(torch.cat(joined, dim=0).contiguous())
        self.dq_norm, self.dkv_norm = weights["dq_norm.weight"], weights["dkv_norm.weight"]
        self.w_uq = rt.prepare_weight(weights["uq.weight"])
        self.kernels = rt.kernels("latent_attention")
        self.expansions = self.kernels.prepare(weights["uk.weight"], weights["uv.weight"], self.n_heads)
        self.w_o = rt.prepare_weight(weights["o.weight"])

    def forward(self, x, step, cache):
        rt, n = self.rt, x.shape[0]
        H, D, Dv, Rq, R = self.n_heads, self.head_dim, self.value_dim, self.q_rank, self.kv_rank
        table = step.block_tables[cache.group]
        low = rt.buffer("la_low", n, self.w_low.rows, torch.float32)
        rt.gemm(x, self.w_low, low)
        cq = rt.buffer("la_cq", n, Rq)
        ops.norm_slice(low, 0, Rq, self.dq_norm, self.eps, cq)
        if cache.writes:
            ops.norm_slice_to_pages(low, Rq, R, self.dkv_norm, self.eps, cache.kv, step.positions, step.tok_seq, table)
        q = rt.buffer("la_q", n, H * D, torch.float32)
        rt.gemm(cq, self.w_uq, q)
        out = rt.buffer("la_out", n, H * Dv)
        self.kernels.attend(q, self.expansions, cache.kv, step, table, self.scale, self.window,
                            low if self.gated else None, Rq + R, out)
        return Product(out, self.w_o)
