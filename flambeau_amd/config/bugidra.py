"""BugidraConfig: a pre-norm decoder whose config.json lists its layers one by one.

Every layer names its mixer: ``attention`` (softmax attention with normed, rotated, capped and gated
extras), ``parallel`` (softmax attention and a retention side by side) or ``delta`` (the gated delta
rule behind short convolutions), each with its sizes, and its feed-forward (``dense`` or none).  Every
size and constant that the file gives is read here, with its type, and a missing or ill-typed key is
named in the error.
"""
from __future__ import annotations

from dataclasses import dataclass

from .base import ConfigError, KeyReader


@dataclass(frozen=True)
class RotaryScaling:
    """The blend of a frequency ladder towards frequencies divided by ``factor``: dims whose wave turns
    fewer than ``slow`` times over ``original`` positions are divided, those that turn more than
    ``fast`` times are kept, the ones between are mixed linearly."""
    factor: float
    original: int
    fast: float
    slow: float


@dataclass(frozen=True)
class RotaryConfig:
    base: float
    dims: int
    scaling: RotaryScaling | None = None


@dataclass(frozen=True)
class SoftmaxAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: RotaryConfig | None
    softcap: float | None = None
    v_mix: bool = False


@dataclass(frozen=True)
class RetentionConfig:
    heads: int
    dim: int
    vdim: int
    decay: tuple
    rot: RotaryConfig | None


@dataclass(frozen=True)
class SideBySideConfig:
    left: SoftmaxAttentionConfig
    right: RetentionConfig


@dataclass(frozen=True)
class DeltaConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int


@dataclass(frozen=True)
class DenseMlpConfig:
    ff: int


@dataclass(frozen=True)
class BugidraLayer:
    type: str                   # "attention" | "parallel" | "delta"
    mixer: object
    mlp: object                 # DenseMlpConfig | None


def _rotary(m: KeyReader, dim: int):
    r = m.section("rot", default=None)
    if r is None:
        return None
    dims = r.integer("dims", minimum=2)
    if dims % 2 or dims > dim:
        raise ConfigError(f"{r.where}: 'dims' {dims} must be even and within the head's {dim} values")
    s = r.section("scaling", default=None)
    scaling = None
    if s is not None:
        scaling = RotaryScaling(factor=s.number("factor", positive=True), original=s.integer("original", minimum=1),
                                fast=s.number("fast", positive=True), slow=s.number("slow", positive=True))
    return RotaryConfig(base=r.number("base", positive=True), dims=dims, scaling=scaling)


def _softmax_attention(m: KeyReader) -> SoftmaxAttentionConfig:
    heads, kv_heads = m.integer("heads", minimum=1), m.integer("kv_heads", minimum=1)
    if heads % kv_heads:
        raise ConfigError(f"{m.where}: {heads} heads are not a multiple of {kv_heads} key/value heads")
    dim = m.integer("dim", minimum=1)
    return SoftmaxAttentionConfig(heads=heads, kv_heads=kv_heads, dim=dim, vdim=m.integer("vdim", minimum=1),
                                  scale=m.number("scale", positive=True), rot=_rotary(m, dim),
                                  softcap=m.number("softcap", default=None, positive=True),
                                  v_mix=m.boolean("v_mix", default=False))


def _retention(m: KeyReader) -> RetentionConfig:
    heads, dim = m.integer("heads", minimum=1), m.integer("dim", minimum=1)
    decay = m.raw.get("decay")
    if not isinstance(decay, list) or len(decay) != heads or not all(
            isinstance(d, (int, float)) and not isinstance(d, bool) for d in decay):
        raise ConfigError(f"{m.where}: 'decay' must be a list of {heads} numbers, one per head")
    return RetentionConfig(heads=heads, dim=dim, vdim=m.integer("vdim", minimum=1),
                           decay=tuple(float(d) for d in decay), rot=_rotary(m, dim))


@dataclass(frozen=True)
class BugidraConfig:
    vocab_size: int
    width: int
    eps: float
    embedding_scale: float
    layers: tuple
    max_position_embeddings: int
    eos_token_id: int | None = None

    architecture = "Bugidra"
    # the design names no longest sequence; this bounds block tables and default pools
    DEFAULT_MAX_POSITION = 1 << 17

    @classmethod
    def from_dict(cls, raw: dict, where: str = "config.json") -> "BugidraConfig":
        r = KeyReader(raw, where)
        layers = []
        for lr in r.sections("layers"):
            kind = lr.string("type")
            m = lr.section("mixer")
            if kind == "attention":
                mixer = _softmax_attention(m)
            elif kind == "parallel":
                mixer = SideBySideConfig(left=_softmax_attention(m.section("left")), right=_retention(m.section("right")))
            elif kind == "delta":
                heads, kv_heads = m.integer("heads", minimum=1), m.integer("kv_heads", minimum=1)
                if heads % kv_heads:
                    raise ConfigError(f"{m.where}: {heads} heads are not a multiple of {kv_heads} query/key heads")
                mixer = DeltaConfig(heads=heads, kv_heads=kv_heads, dim=m.integer("dim", minimum=1),
                                    vdim=m.integer("vdim", minimum=1), conv=m.integer("conv", minimum=1))
            else:
                raise ConfigError(f"{lr.where}: unknown layer type '{kind}' (attention, parallel, delta)")
            f = lr.section("mlp", default=None)
            mlp = None
            if f is not None:
                fk = f.string("kind")
                if fk != "dense":
                    raise ConfigError(f"{f.where}: unknown feed-forward kind '{fk}' (dense)")
                mlp = DenseMlpConfig(ff=f.integer("ff", minimum=1))
            layers.append(BugidraLayer(kind, mixer, mlp))
        if not layers:
            raise ConfigError(f"{where}: 'layers' is empty")
        emb = r.section("embedding", default=None)
        return cls(vocab_size=r.integer("vocab", minimum=1), width=r.integer("width", minimum=1),
                   eps=r.section("norm").number("eps", positive=True),
                   embedding_scale=emb.number("scale", default=1.0) if emb is not None else 1.0,
                   layers=tuple(layers),
                   max_position_embeddings=r.integer("max_position_embeddings", default=cls.DEFAULT_MAX_POSITION, minimum=1),
                   eos_token_id=r.integer("eos_token_id", default=None, minimum=0))
