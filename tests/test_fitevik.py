"""Fitevik without a GPU: its configuration, its description as parts, what its layers keep per request, its
tensor names, random weights as a folder, and the plain implementation's own invariants."""
import json
import math

import numpy as np
import pytest
import torch

import plain_fitevik as pf
from fitevik_configs import CONFIGS, read_model, write_model


def _spec(name):
    from flambeau_amd.registry import config_from_dict
    arch, cfg = config_from_dict(CONFIGS[name]["config"], "test")
    return arch, cfg, arch.build_spec(cfg)


def test_the_architecture_is_found_by_its_name():
    from flambeau_amd.registry import known_architectures
    assert {"Fitevik", "Bugidra", "Kuvidra", "MistralForCausalLM"} <= set(known_architectures())
    arch, cfg, spec = _spec("K")
    assert arch.name == "Fitevik" and cfg.width == 40 and cfg.vocab_size == 83 and not spec.tied_head
    assert spec.embedding.kind == "positional_token_embedding" and spec.embedding.params["max_positions"] == 600
    assert spec.head.kind == "scaled_linear_head" and spec.head.params["scale"] == 0.5
    assert _spec("L")[2].head.params["scale"] == 1.0                      # no logit scale in the file


def test_every_size_comes_from_the_file():
    _, cfg, _ = _spec("K")
    l0, l1, l2, l3, l4 = cfg.layers
    assert (l0.type, l0.mixer.heads, l0.mixer.dim, l0.mixer.vdim, l0.mlp.ff) == ("hgrn2", 3, 8, 12, 24)
    m = l1.mixer
    assert (l1.type, m.heads, m.kv_heads, m.dim, m.vdim, m.scale, m.window, m.kv_from) == ("attention", 6, 2, 16, 8, 0.25, 13, None)
    assert (l1.mlp.experts, l1.mlp.top, l1.mlp.ff) == (5, 2, 16)
    assert (l2.mixer.kv_from, l2.mixer.window, l2.mixer.scale) == (1, 29, 0.3)
    assert l3.mlp is None and (l4.mixer.window, l4.mlp.top) == (300, 3)
    assert cfg.eps == 1e-5 and cfg.logit_scale == 0.5 and cfg.max_position_embeddings == 600


@pytest.mark.parametrize("damage,text", [
    (lambda c: c.pop("width"), "width"),
    (lambda c: c.pop("vocab"), "vocab"),
    (lambda c: c.pop("max_positions"), "max_positions"),
    (lambda c: c["norm"].pop("eps"), "eps"),
    (lambda c: c["layers"][0]["mixer"].pop("vdim"), "vdim"),
    (lambda c: c["layers"][1]["mixer"].pop("kv_heads"), "kv_heads"),
    (lambda c: c["layers"][1]["mixer"].pop("scale"), "scale"),
    (lambda c: c["layers"][1]["mixer"]["mask"].pop("size"), "size"),
    (lambda c: c["layers"][1]["mixer"]["mask"].update(size=0), "size"),
    (lambda c: c["layers"][0].update(type="conv"), "conv"),
    (lambda c: c["layers"][0]["mlp"].update(kind="gated"), "gated"),
    (lambda c: c["layers"][1]["mixer"].update(heads=5), "multiple"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=6), "top"),
    (lambda c: c["layers"][1]["mlp"]["expert"].pop("ff"), "ff"),
    (lambda c: c["layers"][2]["mixer"].update(kv_from=0), "kv_from"),            # a recurrent layer has no keys
    (lambda c: c["layers"][2]["mixer"].update(kv_from=2), "kv_from"),            # itself
    (lambda c: c["layers"][2]["mixer"].update(kv_from=4), "kv_from"),            # a later layer
    (lambda c: c["layers"][2]["mixer"].update(dim=32), "sizes"),                 # other sizes than the layer it reads
    (lambda c: c.update(layers=[]), "layers"),
])
def test_a_bad_file_is_refused_with_the_key_s_name(damage, text):
    from flambeau_amd.config import ConfigError
    from flambeau_amd.registry import config_from_dict
    raw = json.loads(json.dumps(CONFIGS["K"]["config"]))
    damage(raw)
    with pytest.raises(ConfigError, match=text):
        config_from_dict(raw, "test")


def test_a_layer_cannot_read_a_layer_that_reads_another():
    from flambeau_amd.config import ConfigError
    from flambeau_amd.registry import config_from_dict
    raw = json.loads(json.dumps(CONFIGS["L"]["config"]))
    raw["layers"][4]["mixer"]["kv_from"] = 3
    with pytest.raises(ConfigError, match="kv_from"):
        config_from_dict(raw, "test")


def test_parts_caches_and_names():
    """Which part every layer becomes, what it keeps per request, and under which names its tensors lie."""
    from flambeau_amd.models.decoder import DecoderModel
    from flambeau_amd.parts import PagedKVSpec, StateSpec
    _, cfg, spec = _spec("K")
    model = DecoderModel(spec, rt=None)
    specs, shares = model.cache_entries()
    # the reader has no cache of its own: its entry is its source's, which keeps the wider of the two windows
    assert shares == [None, None, 1, None, None]
    assert specs[0] == StateSpec((3 * 8 * 12,), torch.float32) and specs[3] == StateSpec((1 * 20 * 6,), torch.float32)
    assert specs[1] == PagedKVSpec(2, 16, 29) and specs[4] == PagedKVSpec(4, 24, 300)
    assert [type(b).__name__ for b in model.blocks] == ["OutputNormBlock"] * 5
    assert model.blocks[3].ffn is None and "ffn_norm.weight" not in model.blocks[3].tensors()
    assert [b.mixer.own_kv for b in model.blocks if hasattr(b.mixer, "own_kv")] == [True, False, True]
    assert [b.mixer.window for b in model.blocks if hasattr(b.mixer, "own_kv")] == [13, 29, 300]
    names = set(model.manifest())
    for n in ("embed", "pos", "embed.norm", "embed.norm.b", "head", "final.norm", "final.norm.b", "l0.norm1", "l0.norm1.b", "l0.norm2.b",
              "l0.mix.q", "l0.mix.f", "l0.mix.f.b", "l0.mix.lower", "l0.mix.v", "l0.mix.norm", "l0.mix.o", "l0.mlp.up", "l0.mlp.up.b",
              "l0.mlp.down.b", "l1.mix.q", "l1.mix.k", "l1.mix.v", "l1.mix.q.norm", "l1.mix.k.norm", "l1.mix.talk", "l1.mix.sink",
              "l1.mlp.router", "l1.mlp.router.b", "l1.mlp.e0.up", "l1.mlp.e4.down", "l2.mix.q", "l2.mix.q.norm", "l2.mix.talk"):
        assert n in names, n
    for n in ("l2.mix.k", "l2.mix.v", "l2.mix.k.norm", "l3.norm2", "l3.mlp.up", "l1.mlp.e0.gate", "l1.mlp.e5.up", "l1.mlp.e0.up.b"):
        assert n not in names, n
    man = model.manifest()
    assert man["pos"][2].shape == (600, 40) and man["l1.mix.talk"][2].shape == (6, 6) and man["l1.mix.sink"][2].shape == (6,)
    assert man["l1.mix.q.norm"][2].shape == (6 * 16,) and man["l1.mix.k.norm"][2].shape == (2 * 16,) and man["l0.mix.norm"][2].shape == (12,)
    assert man["l0.mix.lower"][2].shape == (3 * 8,) and man["l1.mlp.router.b"][2].shape == (5,)
    # two readers of one source: the source keeps the widest window of the three
    l = DecoderModel(_spec("L")[2], rt=None)
    specs, shares = l.cache_entries()
    assert shares == [None, None, None, 2, 2] and specs[2] == PagedKVSpec(2, 32, 64) and specs[0] == PagedKVSpec(1, 16, 1)


def test_a_mixer_without_a_mask_sees_everything():
    """No ``mask``: window 0; a cache that such a layer reads keeps every key, whatever window its owner has."""
    from flambeau_amd.models.decoder import DecoderModel
    from flambeau_amd.parts import PagedKVSpec
    from flambeau_amd.registry import config_from_dict
    raw = json.loads(json.dumps(CONFIGS["K"]["config"]))
    del raw["layers"][2]["mixer"]["mask"]                      # the reader of layer 1, whose own window is 13
    del raw["layers"][4]["mixer"]["mask"]
    arch, cfg = config_from_dict(raw, "test")
    assert cfg.layers[2].mixer.window == 0 and cfg.layers[1].mixer.window == 13
    model = DecoderModel(arch.build_spec(cfg), rt=None)
    specs, _ = model.cache_entries()
    assert specs[1] == PagedKVSpec(2, 16, 0) and specs[4] == PagedKVSpec(4, 24, 0)
    assert [b.mixer.window for b in model.blocks if hasattr(b.mixer, "own_kv")] == [13, 0, 0]
    # the plain side reads the same file the same way
    assert pf.window_of(raw["layers"][2]["mixer"]) == 0 and pf.window_of(raw["layers"][1]["mixer"]) == 13


def test_random_weights_as_a_folder(tmp_path):
    from flambeau_amd.models.decoder import DecoderModel
    from flambeau_amd.weights.loader import SafetensorsDir, check_against_manifest
    for name in CONFIGS:
        d = write_model(name, tmp_path / name, "bfloat16")
        src = SafetensorsDir(d)
        assert check_against_manifest(DecoderModel(_spec(name)[2], rt=None).manifest(), src) == []
        src.close()
        cfg, t = read_model(d)
        logits = pf.forward(cfg, t, [1, 2, 3, 4, 5])
        assert logits.shape == (5, cfg["vocab"]) and np.isfinite(logits).all() and np.abs(logits).max() > 0.05
        lows = [v for n, v in t.items() if n.endswith(".lower")]
        assert all((v >= 0).all() and (v <= 1).all() for v in lows)


def test_the_plain_implementation_is_causal_and_its_parts_matter(tmp_path):
    d = write_model("K", tmp_path / "K", "float32")
    cfg, t = read_model(d)
    toks = list(np.random.default_rng(1).integers(0, 83, 60))
    a, layers = pf.forward(cfg, t, toks, keep_layers=True)
    b = pf.forward(cfg, t, toks[:25])
    assert np.allclose(a[:25], b, atol=1e-12)
    other = list(toks)
    other[0] = (other[0] + 1) % 83
    assert np.abs(pf.forward(cfg, t, other)[-1] - a[-1]).max() > 1e-7        # through the recurrences' memories
    assert len(layers) == 5 and all(np.abs(layers[i + 1] - layers[i]).max() > 1e-3 for i in range(4))
    # every constant of the file changes the result
    for path, value in (("layers.1.mixer.scale", 0.6), ("layers.1.mixer.mask.size", 12), ("layers.2.mixer.mask.size", 30),
                        ("layers.4.mixer.mask.size", 40), ("layers.1.mlp.router.top", 1), ("logit_scale", 0.25), ("norm.eps", 1e-2)):
        c = json.loads(json.dumps(cfg))
        at = c
        keys = path.split(".")
        for k in keys[:-1]:
            at = at[int(k)] if k.isdigit() else at[k]
        at[keys[-1]] = value
        assert np.abs(pf.forward(c, t, toks)[-1] - a[-1]).max() > 1e-6, path
    # and every tensor that is a constant's neighbour: positions, sink, the mixing matrix, the lower bounds, the biases
    for name in ("pos", "l1.mix.sink", "l2.mix.talk", "l0.mix.lower", "l0.mix.f.b", "l1.mlp.router.b", "l0.mlp.down.b", "l2.norm1.b",
                 "embed.norm.b", "final.norm.b"):
        u = dict(t)
        u[name] = t[name] * 0.5 + 0.01
        assert np.abs(pf.forward(cfg, u, toks)[-1] - a[-1]).max() > 1e-6, name
    # the reader reads its source's keys: other key weights in the source move the reader even where the source's own output is cut off
    u = dict(t)
    u["l1.mix.o"] = np.zeros_like(t["l1.mix.o"])
    base = pf.forward(cfg, u, toks)
    u["l1.mix.k"] = t["l1.mix.k"][::-1].copy()
    assert np.abs(pf.forward(cfg, u, toks)[-1] - base[-1]).max() > 1e-6


def test_the_recurrence_written_out_by_hand():
    """Three tokens of HGRN2 for one head of two key dims and two value dims, the sums written out."""
    rng = np.random.default_rng(0)
    W, D, Dv, eps = 5, 2, 2, 1e-5
    t = {"m.q": rng.normal(size=(D, W)), "m.f": rng.normal(size=(D, W)), "m.f.b": rng.normal(size=D), "m.lower": np.array([0.2, 0.7]),
         "m.v": rng.normal(size=(Dv, W)), "m.norm": np.array([1.5, 0.5]), "m.o": np.eye(W)[:, :Dv]}
    h = rng.normal(size=(3, W))
    got, S = pf.hgrn2(h, dict(heads=1, dim=D, vdim=Dv), t, "m.", eps)
    sg = lambda z: 1 / (1 + math.exp(-z))
    f = [[t["m.lower"][d] + (1 - t["m.lower"][d]) * sg(h[i] @ t["m.f"][d] + t["m.f.b"][d]) for d in range(D)] for i in range(3)]
    q = [[(z := h[i] @ t["m.q"][d]) * sg(z) for d in range(D)] for i in range(3)]
    v = [[h[i] @ t["m.v"][e] for e in range(Dv)] for i in range(3)]
    # S_2[d][e] = (1 - f_2) v_2 + f_2 (1 - f_1) v_1 + f_2 f_1 (1 - f_0) v_0
    S2 = [[(1 - f[2][d]) * v[2][e] + f[2][d] * (1 - f[1][d]) * v[1][e] + f[2][d] * f[1][d] * (1 - f[0][d]) * v[0][e] for e in range(Dv)]
          for d in range(D)]
    assert np.allclose(S[0], S2, atol=1e-12)
    o = np.array([sum(S2[d][e] * q[2][d] for d in range(D)) for e in range(Dv)])
    o = o / math.sqrt((o * o).mean() + eps) * t["m.norm"]
    assert np.allclose(got[2, :Dv], o, atol=1e-12) and np.allclose(got[2, Dv:], 0)
    # a forget gate never falls below its lower bound, and a bound of one keeps the memory empty for ever
    assert all(f[i][d] >= t["m.lower"][d] for i in range(3) for d in range(D))
    t["m.lower"] = np.ones(D)
    assert np.allclose(pf.hgrn2(h, dict(heads=1, dim=D, vdim=Dv), t, "m.", eps)[1], 0)


def test_the_attention_written_out_by_hand():
    """Two heads over one key/value head, a window of two keys: bias, mixing, mask and sink, term by term."""
    q = np.array([[[1.0, 0.0], [0.0, 2.0]], [[0.5, 0.5], [1.0, -1.0]], [[2.0, 1.0], [0.0, 1.0]]])       # [T, H, D]
    k = np.array([[[1.0, 1.0]], [[0.0, 1.0]], [[2.0, -1.0]]])                                              # [T, G, D]
    v = np.array([[[1.0, 0.0, 0.0]], [[0.0, 1.0, 0.0]], [[0.0, 0.0, 1.0]]])
    slopes = pf.head_slopes(2)
    assert np.allclose(slopes, [2.0 ** -4, 2.0 ** -8])
    talk, sink, scale = np.array([[1.0, 0.5], [-0.25, 2.0]]), np.array([0.3, -1.0]), 0.7
    out = pf.mixed_softmax_attention(q, k, v, 2, scale, slopes, talk, sink)
    i = 2                                                   # sees positions 1 and 2, not 0
    raw = {(g, j): scale * (q[i, g] @ k[j, 0]) - slopes[g] * (i - j) for g in range(2) for j in (1, 2)}
    for h in range(2):
        s = {j: talk[h, 0] * raw[(0, j)] + talk[h, 1] * raw[(1, j)] for j in (1, 2)}
        den = math.exp(s[1]) + math.exp(s[2]) + math.exp(sink[h])
        assert np.allclose(out[i, h], [0.0, math.exp(s[1]) / den, math.exp(s[2]) / den], atol=1e-12)
    # the first token sees itself and the sink only: its weights sum to less than one
    s0 = talk[0, 0] * scale * (q[0, 0] @ k[0, 0]) + talk[0, 1] * scale * (q[0, 1] @ k[0, 0])
    assert np.allclose(out[0, 0], [math.exp(s0) / (math.exp(s0) + math.exp(sink[0])), 0, 0], atol=1e-12)
    # positions continue where a prompt's first part ended
    later = pf.mixed_softmax_attention(q[2:], k, v, 2, scale, slopes, talk, sink, first=2)
    assert np.allclose(later[0], out[2], atol=1e-14)


def test_the_experts_written_out_by_hand():
    rng = np.random.default_rng(3)
    W, F, E = 4, 3, 4
    t = {"f.router": rng.normal(size=(E, W)), "f.router.b": np.array([0.0, 5.0, 0.0, -5.0])}
    for e in range(E):
        t[f"f.e{e}.up"], t[f"f.e{e}.down"] = rng.normal(size=(F, W)), rng.normal(size=(W, F))
    h = rng.normal(size=(1, W))
    z = h[0] @ t["f.router"].T + t["f.router.b"]
    a, b = np.argsort(-z)[:2]
    assert a == 1                                           # the bias decides
    wa = 1 / (1 + math.exp(z[b] - z[a]))                    # softmax over the two chosen logits alone
    one = lambda e: np.square(np.maximum(h[0] @ t[f"f.e{e}.up"].T, 0)) @ t[f"f.e{e}.down"].T
    got = pf.routed_experts(h, {"router": {"experts": E, "top": 2}}, t, "f.")
    assert np.allclose(got[0], wa * one(a) + (1 - wa) * one(b), atol=1e-12)
    assert np.allclose(pf.routed_experts(h, {"router": {"experts": E, "top": 1}}, t, "f.")[0], one(a), atol=1e-12)
