"""LenedraConfig: a decoder whose config.json lists its layers one by one.

Every layer names its mixer, ``attention`` (softmax attention whose keys are also its values, inside a sliding
window that keeps the first tokens) or ``parallel`` (chunked softmax attention with a sink beside a gated delta
rule), with the mixer's sizes and constants, and its feed-forward: ``dense``, ``moe`` (routed experts with groups,
identity experts and a shared expert) or none.  The residual stream may be kept in several copies (``streams``).
Every size and constant that the file gives is read here, with its type, and a missing or ill-typed key is named in
the error.  Two sizes are in no key of the file, the ranks of the delta rule's two projections of low rank: they are
read from the shapes of the tensors (``sizes_from_tensors``), unless the file gives them as ``decay_rank`` and
``gate_rank``, as a configuration without a weight file (random weights) must.
"""
from __future__ import annotations

from dataclasses import dataclass

from .base import ConfigError, KeyReader


@dataclass(frozen=True)
class KeptWindowAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int                 # 0: every earlier key
    keep_first: int


@dataclass(frozen=True)
class ChunkedAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    chunk: int                  # 0: every earlier key


@dataclass(frozen=True)
class DeltaRuleConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    decay_rank: int
    gate_rank: int


@dataclass(frozen=True)
class PairConfig:
    left: ChunkedAttentionConfig
    right: DeltaRuleConfig
    left_scale: float
    right_scale: float


@dataclass(frozen=True)
class DenseMlpConfig:
    ff: int


@dataclass(frozen=True)
class ExpertsMlpConfig:
    experts: int                # experts with matrices
    identity: int               # further outputs of the router that return their input
    top: int
    ff: int
    groups: int
    keep_groups: int
    scale: float
    shared_ff: int | None


@dataclass(frozen=True)
class LenedraLayer:
    type: str                   # "attention" | "parallel"
    mixer: object
    mlp: object                 # DenseMlpConfig | ExpertsMlpConfig | None


def _heads(m: KeyReader):
    heads, kv_heads = m.integer("heads", minimum=1), m.integer("kv_heads", minimum=1)
    if heads % kv_heads:
        raise ConfigError(f"{m.where}: {heads} heads are not a multiple of {kv_heads} key/value heads")
    return heads, kv_heads


def _attention(m: KeyReader) -> KeptWindowAttentionConfig:
    heads, kv_heads = _heads(m)
    mask = m.section("mask", default=None)                    # (a mixer without a mask sees every earlier token)
    dim = m.integer("dim", minimum=1)
    cfg = KeptWindowAttentionConfig(heads=heads, kv_heads=kv_heads, dim=dim, vdim=m.integer("vdim", default=dim, minimum=1),
                                    scale=m.number("scale", positive=True),
                                    window=mask.integer("size", minimum=1) if mask is not None else 0,
                                    keep_first=mask.integer("keep_first", default=0, minimum=0) if mask is not None else 0)
    if cfg.vdim != cfg.dim:
        raise ConfigError(f"{m.where}: the values are the keys, so 'vdim' {cfg.vdim} must equal 'dim' {cfg.dim}")
    return cfg


def _pair(m: KeyReader) -> PairConfig:
    l, r = m.section("left"), m.section("right")
    heads, kv_heads = _heads(l)
    mask = l.section("mask", default=None)
    left = ChunkedAttentionConfig(heads=heads, kv_heads=kv_heads, dim=l.integer("dim", minimum=1), vdim=l.integer("vdim", minimum=1),
                                  scale=l.number("scale", positive=True), chunk=mask.integer("size", minimum=1) if mask is not None else 0)
    heads, kv_heads = _heads(r)
    right = DeltaRuleConfig(heads=heads, kv_heads=kv_heads, dim=r.integer("dim", minimum=1), vdim=r.integer("vdim", minimum=1),
                            conv=r.integer("conv", minimum=1), decay_rank=r.integer("decay_rank", minimum=1),
                            gate_rank=r.integer("gate_rank", minimum=1))
    return PairConfig(left, right, left_scale=m.number("left_scale"), right_scale=m.number("right_scale"))


def _mlp(f: KeyReader):
    kind = f.string("kind")
    if kind == "dense":
        return DenseMlpConfig(ff=f.integer("ff", minimum=1))
    if kind != "moe":
        raise ConfigError(f"{f.where}: unknown feed-forward kind '{kind}' (dense, moe)")
    router = f.section("router")
    groups = router.section("groups", default=None)
    shared = f.section("shared", default=None)
    cfg = ExpertsMlpConfig(experts=router.integer("experts", minimum=1), identity=router.integer("identity", default=0, minimum=0),
                           top=router.integer("top", minimum=1), ff=f.section("expert").integer("ff", minimum=1),
                           groups=groups.integer("count", minimum=1) if groups is not None else 1,
                           keep_groups=groups.integer("keep", minimum=1) if groups is not None else 1,
                           scale=router.number("scale", default=1.0),
                           shared_ff=shared.integer("ff", minimum=1) if shared is not None else None)
    outputs = cfg.experts + cfg.identity
    if cfg.top > outputs:
        raise ConfigError(f"{f.where}: 'top' {cfg.top} of {outputs} experts")
    if outputs % cfg.groups or cfg.keep_groups > cfg.groups:
        raise ConfigError(f"{router.where}: {outputs} experts (identity experts included) in {cfg.groups} groups, of which {cfg.keep_groups} are kept")
    if cfg.keep_groups * (outputs // cfg.groups) < cfg.top:
        raise ConfigError(f"{router.where}: {cfg.keep_groups} groups of {outputs // cfg.groups} experts cannot give 'top' {cfg.top}")
    return cfg


@dataclass(frozen=True)
class LenedraConfig:
    vocab_size: int
    width: int
    eps: float
    embedding_scale: float
    logit_softcap: float | None
    streams: int | None             # None: one residual stream with plain sums
    max_position_embeddings: int
    layers: tuple
    eos_token_id: int | None = None

    architecture = "Lenedra"
    DEFAULT_MAX_POSITION = 1 << 20

    @staticmethod
    def sizes_from_tensors(raw: dict, shapes: dict) -> dict:
        """``raw`` with the sizes that only the tensors' shapes give filled in: the ranks of the delta rule's projections
        of low rank, from ``l<i>.mix.right.a1`` and ``.g1`` ([rank, width]).  Keys that the file has are left alone."""
        layers = raw.get("layers")
        if not isinstance(layers, list):
            return raw
        out = dict(raw, layers=[])
        for i, layer in enumerate(layers):
            right = layer.get("mixer", {}).get("right") if isinstance(layer, dict) and isinstance(layer.get("mixer"), dict) else None
            if isinstance(right, dict):
                right = dict(right)
                for key, tensor in (("decay_rank", f"l{i}.mix.right.a1"), ("gate_rank", f"l{i}.mix.right.g1")):
                    if key not in right and tensor in shapes and len(shapes[tensor]) == 2:
                        right[key] = int(shapes[tensor][0])
                layer = dict(layer, mixer=dict(layer["mixer"], right=right))
            out["layers"].append(layer)
        return out

    @classmethod
    def from_dict(cls, raw: dict, where: str = "config.json") -> "LenedraConfig":
        r = KeyReader(raw, where)
        layers: list = []
        for lr in r.sections("layers"):
            kind = lr.string("type")
            m = lr.section("mixer")
            if kind == "attention":
                mixer = _attention(m)
            elif kind == "parallel":
                mixer = _pair(m)
            else:
                raise ConfigError(f"{lr.where}: unknown layer type '{kind}' (attention, parallel)")
            f = lr.section("mlp", default=None)
            layers.append(LenedraLayer(kind, mixer, _mlp(f) if f is not None else None))
        if not layers:
            raise ConfigError(f"{where}: 'layers' is empty")
        emb = r.section("embedding", default=None)
        cap = r.number("logit_softcap", default=None)
        if cap is not None and not cap > 0.0:
            raise ConfigError(f"{where}: key 'logit_softcap' must be > 0, got {cap}")
        return cls(vocab_size=r.integer("vocab", minimum=1), width=r.integer("width", minimum=1),
                   eps=r.section("norm").number("eps", positive=True),
                   embedding_scale=emb.number("scale", default=1.0) if emb is not None else 1.0,
                   logit_softcap=cap, streams=r.integer("streams", default=None, minimum=1),
                   max_position_embeddings=r.integer("max_positions", default=cls.DEFAULT_MAX_POSITION, minimum=1),
                   layers=tuple(layers), eos_token_id=r.integer("eos_token_id", default=None, minimum=0))
