"""FitevikConfig: a decoder whose config.json lists its layers one by one.

Every layer names its mixer, ``hgrn2`` (a linear recurrence whose forget gate is also its key) or
``attention`` (softmax attention inside a sliding window, with a distance bias, mixed heads and a sink; it may
read the keys and values of an earlier attention layer, ``kv_from``), with the mixer's sizes, and its
feed-forward: ``dense``, ``moe`` (routed experts) or none.  Every size and constant that the file gives is
read here, with its type, and a missing or ill-typed key is named in the error.
"""
from __future__ import annotations

from dataclasses import dataclass

from .base import ConfigError, KeyReader


@dataclass(frozen=True)
class Hgrn2Config:
    heads: int
    dim: int
    vdim: int


@dataclass(frozen=True)
class WindowAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int
    kv_from: int | None = None


@dataclass(frozen=True)
class DenseMlpConfig:
    ff: int


@dataclass(frozen=True)
class ExpertsMlpConfig:
    experts: int
    top: int
    ff: int


@dataclass(frozen=True)
class FitevikLayer:
    type: str                   # "hgrn2" | "attention"
    mixer: object
    mlp: object                 # DenseMlpConfig | ExpertsMlpConfig | None


def _attention(m: KeyReader, index: int, before: list) -> WindowAttentionConfig:
    heads, kv_heads = m.integer("heads", minimum=1), m.integer("kv_heads", minimum=1)
    if heads % kv_heads:
        raise ConfigError(f"{m.where}: {heads} heads are not a multiple of {kv_heads} key/value heads")
    mask = m.section("mask", default=None)                    # (a mixer without a mask sees every earlier token: window 0)
    cfg = WindowAttentionConfig(heads=heads, kv_heads=kv_heads, dim=m.integer("dim", minimum=1), vdim=m.integer("vdim", minimum=1),
                                scale=m.number("scale", positive=True), window=mask.integer("size", minimum=1) if mask is not None else 0,
                                kv_from=m.integer("kv_from", default=None, minimum=0))
    if cfg.kv_from is not None:
        src = before[cfg.kv_from].mixer if cfg.kv_from < index else None
        if not isinstance(src, WindowAttentionConfig) or src.kv_from is not None:
            raise ConfigError(f"{m.where}: 'kv_from' {cfg.kv_from} must name an earlier attention layer with keys and values of its own")
        if (src.heads, src.kv_heads, src.dim, src.vdim) != (cfg.heads, cfg.kv_heads, cfg.dim, cfg.vdim):
            raise ConfigError(f"{m.where}: layer {cfg.kv_from}, whose keys and values are read, has other head counts or sizes")
    return cfg


@dataclass(frozen=True)
class FitevikConfig:
    vocab_size: int
    width: int
    eps: float
    logit_scale: float
    max_position_embeddings: int
    layers: tuple
    eos_token_id: int | None = None

    architecture = "Fitevik"

    @classmethod
    def from_dict(cls, raw: dict, where: str = "config.json") -> "FitevikConfig":
        r = KeyReader(raw, where)
        layers: list = []
        for i, lr in enumerate(r.sections("layers")):
            kind = lr.string("type")
            m = lr.section("mixer")
            if kind == "hgrn2":
                mixer = Hgrn2Config(heads=m.integer("heads", minimum=1), dim=m.integer("dim", minimum=1), vdim=m.integer("vdim", minimum=1))
            elif kind == "attention":
                mixer = _attention(m, i, layers)
            else:
                raise ConfigError(f"{lr.where}: unknown layer type '{kind}' (hgrn2, attention)")
            f = lr.section("mlp", default=None)
            mlp = None
            if f is not None:
                fk = f.string("kind")
                if fk == "dense":
                    mlp = DenseMlpConfig(ff=f.integer("ff", minimum=1))
                elif fk == "moe":
                    router = f.section("router")
                    mlp = ExpertsMlpConfig(experts=router.integer("experts", minimum=1), top=router.integer("top", minimum=1),
                                           ff=f.section("expert").integer("ff", minimum=1))
                    if mlp.top > mlp.experts:
                        raise ConfigError(f"{f.where}: 'top' {mlp.top} of {mlp.experts} experts")
                else:
                    raise ConfigError(f"{f.where}: unknown feed-forward kind '{fk}' (dense, moe)")
            layers.append(FitevikLayer(kind, mixer, mlp))
        if not layers:
            raise ConfigError(f"{where}: 'layers' is empty")
        return cls(vocab_size=r.integer("vocab", minimum=1), width=r.integer("width", minimum=1),
                   eps=r.section("norm").number("eps", positive=True),
                   logit_scale=r.number("logit_scale", default=1.0),
                   max_position_embeddings=r.integer("max_positions", minimum=1),
                   layers=tuple(layers), eos_token_id=r.integer("eos_token_id", default=None, minimum=0))
