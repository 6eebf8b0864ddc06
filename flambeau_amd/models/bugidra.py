"""Bugidra as a description of parts.

A pre-norm decoder whose norms are Dynamic Tanh (``dynamic_tanh``), whose embedding is multiplied by a
constant, whose feed-forward is gated with the tanh form of gelu (``gated_mlp``) or absent, and whose
mixers are, layer by layer as config.json lists them:

* ``attention``: ``normed_gqa_attention`` with a norm over the whole projection of q and of k, the
  interleaved rotation, capped scores, values blended with those of the first such layer, and a sigmoid
  gate on the heads' outputs;
* ``parallel``: ``side_by_side`` of a ``normed_gqa_attention`` (split-half rotation with a stretched
  ladder of frequencies, every head of q and k divided by its root mean square afterwards) and a
  ``retention``, each normed over the width with its own gain, half of each;
* ``delta``: ``gated_delta`` behind short convolutions.

Tensor names: ``embed``, ``head``, ``final.norm`` (+ ``.alpha``, ``.b``) and per layer ``l<i>.``:
``norm1``, ``norm2``, ``mix.*``, ``mlp.*``.
"""
from __future__ import annotations

from ..config.bugidra import BugidraConfig, DeltaConfig, RetentionConfig, SideBySideConfig, SoftmaxAttentionConfig
from ..parts import PartSpec
from ..registry import register_architecture
from .decoder import LayerSpec, ModelSpec, RunEntry

VALUE_MIX_KEY = "bugidra_first_values"


def _position(rot, dim: int, layout: str) -> PartSpec:
    if rot is None:
        return PartSpec("none", {})
    params = dict(head_dim=dim, theta=rot.base, rotated_dims=rot.dims)
    if rot.scaling is not None:
        sc = rot.scaling
        return PartSpec("rope_blended", dict(params, factor=sc.factor, original=sc.original, fast=sc.fast, slow=sc.slow, layout=layout))
    return PartSpec("rope_neox" if layout == "half" else "rope_interleaved", params)


def _gated_attention(cfg: BugidraConfig, m: SoftmaxAttentionConfig, first_mix: bool):
    spec = PartSpec("normed_gqa_attention", dict(
        hidden_size=cfg.width, n_heads=m.heads, n_kv_heads=m.kv_heads, head_dim=m.dim, value_dim=m.vdim, scale=m.scale,
        position=_position(m.rot, m.dim, "interleaved"), qk_norm="projection", eps=cfg.eps, softcap=m.softcap,
        value_mix=(("source" if first_mix else "blend") if m.v_mix else None), value_mix_key=VALUE_MIX_KEY, gate="sigmoid"))
    names = {"q.weight": "q", "k.weight": "k", "v.weight": "v", "o.weight": "o", "g.weight": "g",
             "q_norm.weight": "q.norm", "k_norm.weight": "k.norm"}
    if m.v_mix:
        names["value_mix.weight"] = "vmix"
    return spec, names


def _rotated_attention(cfg: BugidraConfig, m: SoftmaxAttentionConfig):
    spec = PartSpec("normed_gqa_attention", dict(
        hidden_size=cfg.width, n_heads=m.heads, n_kv_heads=m.kv_heads, head_dim=m.dim, value_dim=m.vdim, scale=m.scale,
        position=_position(m.rot, m.dim, "half"), qk_norm="head", eps=cfg.eps, softcap=m.softcap))
    return spec, {"q.weight": "q", "k.weight": "k", "v.weight": "v", "o.weight": "o"}


def _retention(cfg: BugidraConfig, m: RetentionConfig):
    spec = PartSpec("retention", dict(hidden_size=cfg.width, n_heads=m.heads, head_dim=m.dim, value_dim=m.vdim, decay=m.decay,
                                      position=_position(m.rot, m.dim, "half"), eps=cfg.eps, gate="silu"))
    return spec, {"q.weight": "q", "k.weight": "k", "v.weight": "v", "g.weight": "g", "o.weight": "o"}


def _mixer(cfg: BugidraConfig, m, p: str, first_mix: bool):
    """The mixer's ``PartSpec`` and the file names of its tensors."""
    if isinstance(m, SoftmaxAttentionConfig):
        spec, names = _gated_attention(cfg, m, first_mix)
    elif isinstance(m, SideBySideConfig):
        left, left_names = _rotated_attention(cfg, m.left)
        right, right_names = _retention(cfg, m.right)
        spec = PartSpec("side_by_side", dict(hidden_size=cfg.width, left=left, right=right, eps=cfg.eps, factors=(0.5, 0.5)))
        names = {"left." + k: "left." + v for k, v in left_names.items()}
        names.update({"right." + k: "right." + v for k, v in right_names.items()})
        names.update({"left_out.weight": "left.out", "right_out.weight": "right.out"})
    elif isinstance(m, DeltaConfig):
        spec = PartSpec("gated_delta", dict(hidden_size=cfg.width, n_heads=m.heads, n_qk_heads=m.kv_heads, head_dim=m.dim,
                                            value_dim=m.vdim, conv_taps=m.conv, eps=cfg.eps))
        names = {"q.weight": "q", "k.weight": "k", "v.weight": "v", "q_conv.weight": "q.conv", "k_conv.weight": "k.conv",
                 "v_conv.weight": "v.conv", "b.weight": "b", "a.weight": "a", "A_log": "A_log", "dt_bias": "dt_bias",
                 "norm.weight": "norm", "g.weight": "g", "o.weight": "o"}
    else:
        raise TypeError(f"no mixer for {m!r}")
    return spec, {"mixer." + k: p + "mix." + v for k, v in names.items()}


def _norm_names(part: str, file_name: str) -> dict:
    return {part + ".weight": file_name, part + ".alpha": file_name + ".alpha", part + ".bias": file_name + ".b"}


def bugidra_spec(cfg: BugidraConfig) -> ModelSpec:
    norm = PartSpec("dynamic_tanh", dict(hidden_size=cfg.width))
    layers, ignored = [], []
    mixes = False
    for l, layer in enumerate(cfg.layers):
        p = f"l{l}."
        is_mix = isinstance(layer.mixer, SoftmaxAttentionConfig) and layer.mixer.v_mix
        mixer, names = _mixer(cfg, layer.mixer, p, first_mix=is_mix and not mixes)
        mixes = mixes or is_mix
        names.update(_norm_names("mixer_norm", p + "norm1"))
        ffn = None
        if layer.mlp is not None:
            ffn = PartSpec("gated_mlp", dict(hidden_size=cfg.width, intermediate_size=layer.mlp.ff, activation="gelu_tanh"))
            names.update({"ffn.gate.weight": p + "mlp.gate", "ffn.up.weight": p + "mlp.up", "ffn.down.weight": p + "mlp.down"})
            names.update(_norm_names("ffn_norm", p + "norm2"))
        else:
            ignored += [p + "norm2", p + "norm2.*"]
        layers.append(LayerSpec(PartSpec("prenorm", dict(mixer=mixer, feed_forward=ffn, norm=norm)), names))
    names = {"embedding.weight": "embed", "head.weight": "head"}
    names.update(_norm_names("final_norm", "final.norm"))
    return ModelSpec(
        architecture=cfg.architecture,
        hidden_size=cfg.width,
        vocab_size=cfg.vocab_size,
        max_position=cfg.max_position_embeddings,
        layers=layers,
        run_order=[RunEntry(l) for l in range(len(cfg.layers))],
        final_norm=norm,
        names=names,
        tied_head=False,
        eos_token_id=cfg.eos_token_id,
        eos_token_ids=(cfg.eos_token_id,) if cfg.eos_token_id is not None else (),
        embedding=PartSpec("scaled_token_embedding", dict(vocab_size=cfg.vocab_size, hidden_size=cfg.width, scale=cfg.embedding_scale)),
        ignored_tensors=tuple(ignored),
    )


register_architecture("Bugidra", BugidraConfig, bugidra_spec)
