"""Lenedra as a description of parts.

A pre-norm decoder whose residual stream is kept in several copies (hyper-connections, ``hyper_prenorm`` blocks over a
``HyperStream``; without ``streams`` in config.json plain ``prenorm`` blocks), whose norms are root-mean-square norms
with the weight stored around zero, behind an embedding that is multiplied by a constant and in front of a head whose
logits pass a soft cap.  Mixers, layer by layer as config.json lists them:

* ``attention``: ``mixed_heads_attention`` with biased projections, no value projection (a key's raw projection is also its value), a norm per
  head with a gain shared by the heads, a distance bias with slopes 2^(-8 (h + 1) / heads), a sliding window beside
  which the first tokens stay visible, a biased output projection;
* ``parallel``: ``side_by_side`` (no norms, a factor each) of ``mixed_heads_attention`` with biased projections, a
  chunked mask and a sink, and ``gated_delta`` with a decay per head and key dim, decay and output gate through
  projections of low rank, and a sigmoid gate.

Feed-forwards: ``swiglu``, or ``routed_experts`` with the grouped softmax router, identity experts and an ungated
shared expert, or none.

Tensor names: ``embed``, ``final.norm``, ``head`` and per layer ``l<i>.``: ``norm1``, ``norm2``, ``mix.*``, ``mlp.*``,
``hc1.*``, ``hc2.*``; biases are the matrix's name with ``.b``.
"""
from __future__ import annotations

from ..config.lenedra import DenseMlpConfig, ExpertsMlpConfig, KeptWindowAttentionConfig, LenedraConfig, PairConfig
from ..parts import PartSpec
from ..registry import register_architecture
from .decoder import LayerSpec, ModelSpec, RunEntry

SLOPE_EXPONENT = 8.0          # slope of head h: 2^(-8 (h + 1) / heads)
UNIT_EPS = 1e-6               # inside the root that makes the delta rule's q and k unit vectors


def _mixer(cfg: LenedraConfig, l: int):
    m, p = cfg.layers[l].mixer, f"l{l}.mix."
    if isinstance(m, KeptWindowAttentionConfig):
        spec = PartSpec("mixed_heads_attention", dict(
            hidden_size=cfg.width, n_heads=m.heads, n_kv_heads=m.kv_heads, head_dim=m.dim, value_dim=m.dim, window=m.window,
            keep_first=m.keep_first if m.window else 0, scale=m.scale, qk_norm="head_gain", eps=cfg.eps,
            slope_exponent=SLOPE_EXPONENT, bias=True, out_bias=True, values="keys"))
        names = {"q.weight": "q", "q.bias": "q.b", "k.weight": "k", "k.bias": "k.b", "q_norm.weight": "q.norm",
                 "k_norm.weight": "k.norm", "o.weight": "o", "o.bias": "o.b"}
        return spec, {"mixer." + k: p + v for k, v in names.items()}
    if isinstance(m, PairConfig):
        a, d = m.left, m.right
        left = PartSpec("mixed_heads_attention", dict(
            hidden_size=cfg.width, n_heads=a.heads, n_kv_heads=a.kv_heads, head_dim=a.dim, value_dim=a.vdim, chunk=a.chunk,
            scale=a.scale, eps=cfg.eps, sink=True, bias=True))
        right = PartSpec("gated_delta", dict(
            hidden_size=cfg.width, n_heads=d.heads, n_qk_heads=d.kv_heads, head_dim=d.dim, value_dim=d.vdim, conv_taps=d.conv,
            eps=cfg.eps, unit_eps=UNIT_EPS, decay="key_dim", decay_rank=d.decay_rank, gate_rank=d.gate_rank, gate="sigmoid"))
        spec = PartSpec("side_by_side", dict(hidden_size=cfg.width, left=left, right=right, factors=(m.left_scale, m.right_scale),
                                             normed=False))
        names = {"left." + k: "left." + v for k, v in {
            "q.weight": "q", "q.bias": "q.b", "k.weight": "k", "k.bias": "k.b", "v.weight": "v", "v.bias": "v.b", "sink": "sink",
            "o.weight": "o"}.items()}
        names.update({"right." + k: "right." + v for k, v in {
            "q.weight": "q", "k.weight": "k", "v.weight": "v", "q_conv.weight": "q.conv", "k_conv.weight": "k.conv",
            "v_conv.weight": "v.conv", "b.weight": "b", "A_log": "A_log", "dt_bias": "dt_bias", "norm.weight": "norm",
            "a1.weight": "a1", "a2.weight": "a2", "g1.weight": "g1", "g2.weight": "g2", "o.weight": "o"}.items()})
        return spec, {"mixer." + k: p + v for k, v in names.items()}
    raise TypeError(f"no mixer for {m!r}")


def _feed_forward(cfg: LenedraConfig, f, p: str):
    if isinstance(f, DenseMlpConfig):
        spec = PartSpec("swiglu", dict(hidden_size=cfg.width, intermediate_size=f.ff))
        names = {"gate.weight": "gate", "up.weight": "up", "down.weight": "down"}
    elif isinstance(f, ExpertsMlpConfig):
        spec = PartSpec("routed_experts", dict(
            hidden_size=cfg.width, n_experts=f.experts, top=f.top, expert_size=f.ff, shared_size=f.shared_ff, shared_gate=False,
            scoring="softmax_grouped", weight_on="output", correction=True, n_groups=f.groups, keep_groups=f.keep_groups,
            n_identity=f.identity, weight_scale=f.scale))
        names = {"router.weight": "router", "correction": "correction"}
        for e in range(f.experts):
            names.update({f"e{e}.gate.weight": f"e{e}.gate", f"e{e}.up.weight": f"e{e}.up", f"e{e}.down.weight": f"e{e}.down"})
        if f.shared_ff is not None:
            names.update({"shared.gate.weight": "shared.gate", "shared.up.weight": "shared.up", "shared.down.weight": "shared.down"})
    else:
        raise TypeError(f"no feed-forward for {f!r}")
    return spec, {"ffn." + k: p + "mlp." + v for k, v in names.items()}


def lenedra_spec(cfg: LenedraConfig) -> ModelSpec:
    norm = PartSpec("rmsnorm", dict(hidden_size=cfg.width, eps=cfg.eps, unit_offset=True))
    layers, run_order, unread = [], [], []
    for l, layer in enumerate(cfg.layers):
        p = f"l{l}."
        mixer, names = _mixer(cfg, l)
        names["mixer_norm.weight"] = p + "norm1"
        ffn = None
        if layer.mlp is not None:
            ffn, ffn_names = _feed_forward(cfg, layer.mlp, p)
            names.update(ffn_names)
            names["ffn_norm.weight"] = p + "norm2"
        if cfg.streams is not None:
            for sub, file in (("hc_mixer", "hc1"), ("hc_ffn", "hc2")) if ffn is not None else (("hc_mixer", "hc1"),):
                names.update({f"{sub}.{k}": f"{p}{file}.{k}" for k in ("in", "out", "mix")})
            block = PartSpec("hyper_prenorm", dict(mixer=mixer, feed_forward=ffn, norm=norm, n_streams=cfg.streams))
        else:
            block = PartSpec("prenorm", dict(mixer=mixer, feed_forward=ffn, norm=norm))
        layers.append(LayerSpec(block, names))
        run_order.append(RunEntry(l))
        if ffn is None:                         # (a file may still hold the second sublayer's norm and numbers: nothing reads them)
            unread += [f"{p}norm2", f"{p}hc2.*"]
    return ModelSpec(
        architecture=cfg.architecture,
        hidden_size=cfg.width,
        vocab_size=cfg.vocab_size,
        max_position=cfg.max_position_embeddings,
        layers=layers,
        run_order=run_order,
        final_norm=norm,
        names={"embedding.weight": "embed", "final_norm.weight": "final.norm", "head.weight": "head"},
        tied_head=False,
        eos_token_id=cfg.eos_token_id,
        eos_token_ids=(cfg.eos_token_id,) if cfg.eos_token_id is not None else (),
        embedding=PartSpec("scaled_token_embedding", dict(vocab_size=cfg.vocab_size, hidden_size=cfg.width, scale=cfg.embedding_scale)),
        head=PartSpec("capped_linear_head", dict(vocab_size=cfg.vocab_size, hidden_size=cfg.width, softcap=cfg.logit_softcap)),
        residual_streams=cfg.streams,
        ignored_tensors=tuple(unread),
    )


register_architecture("Lenedra", LenedraConfig, lenedra_spec)
