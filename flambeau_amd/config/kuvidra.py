"""KuvidraConfig: a decoder whose config.json lists its layers one by one.

Every layer names its mixer (``latent_attention`` or ``mlstm``) with the mixer's sizes and its
feed-forward (``dense``, ``moe`` or none); ``loop`` says which stretch of layers runs several
times with the same weights.  Every size and constant that the file gives is read here, with its
type, and a missing or ill-typed key is named in the error; nothing is taken from a default that
the file could contradict.
"""
from __future__ import annotations

from dataclasses import dataclass

from .base import ConfigError, KeyReader


@dataclass(frozen=True)
class LatentAttentionConfig:
    heads: int
    dim: int            # query/key size per head
    vdim: int           # value size per head
    q_rank: int         # size of the queries' latent
    kv_rank: int        # size of the cached latent
    scale: float


@dataclass(frozen=True)
class MLstmConfig:
    heads: int
    dim: int
    vdim: int
    gate_cap: float


@dataclass(frozen=True)
class DenseMlpConfig:
    ff: int


@dataclass(frozen=True)
class MoeMlpConfig:
    experts: int
    top: int
    expert_ff: int
    shared_ff: int | None       # None: no shared expert


@dataclass(frozen=True)
class KuvidraLayer:
    type: str                   # "latent_attention" | "mlstm"
    mixer: object
    mlp: object                 # DenseMlpConfig | MoeMlpConfig | None


@dataclass(frozen=True)
class LoopConfig:
    start: int
    stop: int
    times: int


@dataclass(frozen=True)
class KuvidraConfig:
    vocab_size: int
    width: int
    eps: float
    layers: tuple
    loop: LoopConfig | None
    max_position_embeddings: int
    eos_token_id: int | None = None

    architecture = "Kuvidra"
    # the design names no longest sequence; this bounds block tables and default pools
    DEFAULT_MAX_POSITION = 1 << 17

    @classmethod
    def from_dict(cls, raw: dict, where: str = "config.json") -> "KuvidraConfig":
        r = KeyReader(raw, where)
        layers = []
        for lr in r.sections("layers"):
            kind = lr.string("type")
            m = lr.section("mixer")
            if kind == "latent_attention":
                mixer = LatentAttentionConfig(
                    heads=m.integer("heads", minimum=1), dim=m.integer("dim", minimum=1), vdim=m.integer("vdim", minimum=1),
                    q_rank=m.integer("q_rank", minimum=1), kv_rank=m.integer("kv_rank", minimum=1),
                    scale=m.number("scale", positive=True))
            elif kind == "mlstm":
                mixer = MLstmConfig(heads=m.integer("heads", minimum=1), dim=m.integer("dim", minimum=1),
                                    vdim=m.integer("vdim", minimum=1), gate_cap=m.number("gate_cap", positive=True))
            else:
                raise ConfigError(f"{lr.where}: unknown layer type '{kind}' (latent_attention, mlstm)")
            f = lr.section("mlp", default=None)
            if f is None:
                mlp = None
            else:
                fk = f.string("kind")
                if fk == "dense":
                    mlp = DenseMlpConfig(ff=f.integer("ff", minimum=1))
                elif fk == "moe":
                    router = f.section("router")
                    shared = f.section("shared", default=None)
                    mlp = MoeMlpConfig(experts=router.integer("experts", minimum=1), top=router.integer("top", minimum=1),
                                       expert_ff=f.section("expert").integer("ff", minimum=1),
                                       shared_ff=shared.integer("ff", minimum=1) if shared is not None else None)
                    if mlp.top > mlp.experts:
                        raise ConfigError(f"{f.where}: 'top' {mlp.top} exceeds 'experts' {mlp.experts}")
                else:
                    raise ConfigError(f"{f.where}: unknown feed-forward kind '{fk}' (dense, moe)")
            layers.append(KuvidraLayer(kind, mixer, mlp))
        if not layers:
            raise ConfigError(f"{where}: 'layers' is empty")
        lp = r.section("loop", default=None)
        loop = None
        if lp is not None:
            loop = LoopConfig(start=lp.integer("start", minimum=0), stop=lp.integer("stop", minimum=0),
                              times=lp.integer("times", minimum=1))
            if not loop.start < loop.stop <= len(layers):
                raise ConfigError(f"{lp.where}: layers {loop.start}..{loop.stop - 1} are not a stretch of the {len(layers)} layers")
        return cls(vocab_size=r.integer("vocab", minimum=1), width=r.integer("width", minimum=1),
                   eps=r.section("norm").number("eps", positive=True), layers=tuple(layers), loop=loop,
                   max_position_embeddings=r.integer("max_position_embeddings", default=cls.DEFAULT_MAX_POSITION, minimum=1),
                   eos_token_id=r.integer("eos_token_id", default=None, minimum=0))
