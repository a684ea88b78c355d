"""Fitevik as a description of parts.

A decoder that norms what a sublayer RETURNS, x += LayerNorm(Mixer(x)), x += LayerNorm(FeedForward(x))
(``outnorm`` blocks; the sublayers read the stream itself), behind an embedding that adds a learned row per
position and is normed, and in front of a normed head whose logits are multiplied by a constant.  Mixers,
layer by layer as config.json lists them:

* ``hgrn2``: the ``hgrn2`` linear recurrence (forget gates per key dim above a learned lower bound);
* ``attention``: ``mixed_heads_attention``: a norm over the whole projection of q and of k, no rotation, a
  distance bias with slopes 2^(-8 (h + 1) / heads), the heads' scores mixed by a learned matrix, a sliding
  window, a sink in the softmax's denominator.  With ``kv_from`` the layer has no keys and values of its own:
  its run-order entry reads the cache of the layer named, which then keeps the widest window among its readers.

Feed-forwards: ``mlp`` with biases and the square of relu, or ``routed_experts`` (ungated experts with the
square of relu, a router with a bias, weights = softmax over the chosen logits), or none.

Tensor names: ``embed``, ``pos``, ``embed.norm``, ``final.norm`` (biases ``.b``), ``head`` and per layer
``l<i>.``: ``norm1``, ``norm2``, ``mix.*``, ``mlp.*``.
"""
from __future__ import annotations

from ..config.fitevik import DenseMlpConfig, ExpertsMlpConfig, FitevikConfig, Hgrn2Config, WindowAttentionConfig
from ..parts import PartSpec
from ..registry import register_architecture
from .decoder import LayerSpec, ModelSpec, RunEntry

SLOPE_EXPONENT = 8.0          # slope of head h: 2^(-8 (h + 1) / heads)


def _mixer(cfg: FitevikConfig, l: int, cache_windows: dict):
    m, p = cfg.layers[l].mixer, f"l{l}.mix."
    if isinstance(m, Hgrn2Config):
        spec = PartSpec("hgrn2", dict(hidden_size=cfg.width, n_heads=m.heads, head_dim=m.dim, value_dim=m.vdim, eps=cfg.eps))
        names = {"q.weight": "q", "f.weight": "f", "f.bias": "f.b", "lower": "lower", "v.weight": "v", "norm.weight": "norm", "o.weight": "o"}
    elif isinstance(m, WindowAttentionConfig):
        own = m.kv_from is None
        spec = PartSpec("mixed_heads_attention", dict(
            hidden_size=cfg.width, n_heads=m.heads, n_kv_heads=m.kv_heads, head_dim=m.dim, value_dim=m.vdim, window=m.window,
            scale=m.scale, qk_norm="projection", eps=cfg.eps, slope_exponent=SLOPE_EXPONENT, head_mix=True, sink=True, own_kv=own,
            cache_window=cache_windows[l if own else m.kv_from]))
        names = {"q.weight": "q", "q_norm.weight": "q.norm", "talk": "talk", "sink": "sink", "o.weight": "o"}
        if own:
            names.update({"k.weight": "k", "v.weight": "v", "k_norm.weight": "k.norm"})
    else:
        raise TypeError(f"no mixer for {m!r}")
    return spec, {"mixer." + k: p + v for k, v in names.items()}


def _feed_forward(cfg: FitevikConfig, f, p: str):
    if isinstance(f, DenseMlpConfig):
        spec = PartSpec("mlp", dict(hidden_size=cfg.width, intermediate_size=f.ff, activation="relu2", bias=True))
        names = {"up.weight": "up", "up.bias": "up.b", "down.weight": "down", "down.bias": "down.b"}
    elif isinstance(f, ExpertsMlpConfig):
        spec = PartSpec("routed_experts", dict(hidden_size=cfg.width, n_experts=f.experts, top=f.top, expert_size=f.ff,
                                               scoring="softmax_chosen", weight_on="output", gated=False, activation="relu2",
                                               router_bias=True))
        names = {"router.weight": "router", "router.bias": "router.b"}
        for e in range(f.experts):
            names.update({f"e{e}.up.weight": f"e{e}.up", f"e{e}.down.weight": f"e{e}.down"})
    else:
        raise TypeError(f"no feed-forward for {f!r}")
    return spec, {"ffn." + k: p + "mlp." + v for k, v in names.items()}


def fitevik_spec(cfg: FitevikConfig) -> ModelSpec:
    norm = PartSpec("layernorm", dict(hidden_size=cfg.width, eps=cfg.eps))
    # a cache keeps what the widest window among the layers that read it needs (0: everything, where one of them has no window)
    cache_windows: dict = {}
    for l, layer in enumerate(cfg.layers):
        if isinstance(layer.mixer, WindowAttentionConfig):
            owner = l if layer.mixer.kv_from is None else layer.mixer.kv_from
            kept, window = cache_windows.get(owner), layer.mixer.window
            cache_windows[owner] = window if kept is None else (0 if kept == 0 or window == 0 else max(kept, window))
    layers, run_order = [], []
    for l, layer in enumerate(cfg.layers):
        p = f"l{l}."
        mixer, names = _mixer(cfg, l, cache_windows)
        names.update({"mixer_norm.weight": p + "norm1", "mixer_norm.bias": p + "norm1.b"})
        ffn = None
        if layer.mlp is not None:
            ffn, ffn_names = _feed_forward(cfg, layer.mlp, p)
            names.update(ffn_names)
            names.update({"ffn_norm.weight": p + "norm2", "ffn_norm.bias": p + "norm2.b"})
        layers.append(LayerSpec(PartSpec("outnorm", dict(mixer=mixer, feed_forward=ffn, norm=norm)), names))
        run_order.append(RunEntry(l, cache_of=getattr(layer.mixer, "kv_from", None)))
    names = {"embedding.weight": "embed", "embedding.positions": "pos", "embedding.norm.weight": "embed.norm",
             "embedding.norm.bias": "embed.norm.b", "final_norm.weight": "final.norm", "final_norm.bias": "final.norm.b",
             "head.weight": "head"}
    return ModelSpec(
        architecture=cfg.architecture,
        hidden_size=cfg.width,
        vocab_size=cfg.vocab_size,
        max_position=cfg.max_position_embeddings,
        layers=layers,
        run_order=run_order,
        final_norm=norm,
        names=names,
        tied_head=False,
        eos_token_id=cfg.eos_token_id,
        eos_token_ids=(cfg.eos_token_id,) if cfg.eos_token_id is not None else (),
        embedding=PartSpec("positional_token_embedding", dict(vocab_size=cfg.vocab_size, hidden_size=cfg.width,
                                                              max_positions=cfg.max_position_embeddings, norm=norm)),
        head=PartSpec("scaled_linear_head", dict(vocab_size=cfg.vocab_size, hidden_size=cfg.width, scale=cfg.logit_scale)),
    )


register_architecture("Fitevik", FitevikConfig, fitevik_spec)
