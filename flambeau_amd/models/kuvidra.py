"""Kuvidra as a description of parts.

A decoder of parallel layers (one norm feeds the mixer and the feed-forward, both are added to the
stream) whose mixers are attention over a cached latent (``latent_attention``) or the mLSTM
recurrence (``mlstm``), whose feed-forwards are an ungated gelu layer, routed experts with a gated
shared expert, or none, and in which a stretch of layers runs several times with the same weights:
before each pass the stream re-enters through ``stream_reentry`` (x <- W_in [x ; embedding] + b_pass).
Every pass has caches of its own, which is what run-order entries give.  The output head is the
embedding table.  Tensor names: ``embed``, ``final.norm``, ``loop.in``, ``loop.step`` and, per layer
``l<i>.``, ``norm1``, ``mix.*`` and ``mlp.*``.
"""
from __future__ import annotations

from ..config.kuvidra import DenseMlpConfig, KuvidraConfig, LatentAttentionConfig, MLstmConfig, MoeMlpConfig
from ..parts import PartSpec
from ..registry import register_architecture
from .decoder import LayerSpec, ModelSpec, RunEntry


def _mixer(cfg: KuvidraConfig, m, p: str):
    """The mixer's ``PartSpec`` and the file names of its tensors."""
    if isinstance(m, LatentAttentionConfig):
        spec = PartSpec("latent_attention", dict(hidden_size=cfg.width, n_heads=m.heads, head_dim=m.dim, value_dim=m.vdim,
                                                 q_rank=m.q_rank, kv_rank=m.kv_rank, scale=m.scale, eps=cfg.eps))
        names = {"dq.weight": "dq", "dq_norm.weight": "dq.norm", "uq.weight": "uq", "dkv.weight": "dkv",
                 "dkv_norm.weight": "dkv.norm", "uk.weight": "uk", "uv.weight": "uv", "g.weight": "g", "o.weight": "o"}
    elif isinstance(m, MLstmConfig):
        spec = PartSpec("mlstm", dict(hidden_size=cfg.width, n_heads=m.heads, head_dim=m.dim, value_dim=m.vdim,
                                      gate_cap=m.gate_cap, eps=cfg.eps))
        names = {"q.weight": "q", "k.weight": "k", "v.weight": "v", "g.weight": "g", "o.weight": "o", "norm.weight": "norm",
                 "i.weight": "i", "i.bias": "i.b", "f.weight": "f", "f.bias": "f.b"}
    else:
        raise TypeError(f"no mixer for {m!r}")
    return spec, {"mixer." + k: p + "mix." + v for k, v in names.items()}


def _feed_forward(cfg: KuvidraConfig, f, p: str):
    if f is None:
        return None, {}
    if isinstance(f, DenseMlpConfig):
        spec = PartSpec("mlp", dict(hidden_size=cfg.width, intermediate_size=f.ff, activation="gelu"))
        names = {"up.weight": "up", "down.weight": "down"}
    elif isinstance(f, MoeMlpConfig):
        spec = PartSpec("routed_experts", dict(hidden_size=cfg.width, n_experts=f.experts, top=f.top, expert_size=f.expert_ff,
                                               shared_size=f.shared_ff, scoring="sigmoid", renormalise=False,
                                               weight_on="input", shared_gate=True))
        names = {"router.weight": "router"}
        for e in range(f.experts):
            names.update({f"e{e}.{k}.weight": f"e{e}.{k}" for k in ("gate", "up", "down")})
        if f.shared_ff is not None:
            names.update({f"shared.{k}.weight": f"shared.{k}" for k in ("gate", "up", "down", "sg")})
    else:
        raise TypeError(f"no feed-forward for {f!r}")
    return spec, {"ffn." + k: p + "mlp." + v for k, v in names.items()}


def kuvidra_spec(cfg: KuvidraConfig) -> ModelSpec:
    norm = PartSpec("rmsnorm", dict(hidden_size=cfg.width, eps=cfg.eps))
    layers = []
    for l, layer in enumerate(cfg.layers):
        p = f"l{l}."
        mixer, names = _mixer(cfg, layer.mixer, p)
        ffn, ffn_names = _feed_forward(cfg, layer.mlp, p)
        names.update(ffn_names)
        names["norm.weight"] = p + "norm1"
        layers.append(LayerSpec(PartSpec("parallel", dict(mixer=mixer, feed_forward=ffn, norm=norm)), names))
    order = [RunEntry(l) for l in range(len(cfg.layers))]
    if cfg.loop is not None:
        lp = cfg.loop
        reentry = len(layers)
        layers.append(LayerSpec(PartSpec("stream_reentry", dict(hidden_size=cfg.width, times=lp.times)),
                                {"in.weight": "loop.in", "step.weight": "loop.step"}))
        looped = []
        for _ in range(lp.times):
            looped += [RunEntry(reentry)] + [RunEntry(l) for l in range(lp.start, lp.stop)]
        order = order[:lp.start] + looped + order[lp.stop:]
    return ModelSpec(
        architecture=cfg.architecture,
        hidden_size=cfg.width,
        vocab_size=cfg.vocab_size,
        max_position=cfg.max_position_embeddings,
        layers=layers,
        run_order=order,
        final_norm=norm,
        names={"embedding.weight": "embed", "final_norm.weight": "final.norm"},
        tied_head=True,
        eos_token_id=cfg.eos_token_id,
        eos_token_ids=(cfg.eos_token_id,) if cfg.eos_token_id is not None else (),
        keeps_embedding=cfg.loop is not None,
    )


register_architecture("Kuvidra", KuvidraConfig, kuvidra_spec)
