"""Lenedra without a GPU: its configuration, its description as parts, what its layers keep per request, its tensor
names, random weights as a folder, the cache manager's kept first tokens and chunks, and the plain implementation's
own invariants."""
import json

import numpy as np
import pytest
import torch

import plain_lenedra as pl
from lenedra_configs import CONFIGS, read_model, write_model


def _spec(name):
    from flambeau_amd.registry import config_from_dict
    arch, cfg = config_from_dict(CONFIGS[name]["config"], "test")
    return arch, cfg, arch.build_spec(cfg)


def test_the_architecture_is_found_by_its_name():
    from flambeau_amd.registry import known_architectures
    assert {"Lenedra", "Fitevik", "Bugidra", "Kuvidra", "MistralForCausalLM"} <= set(known_architectures())
    arch, cfg, spec = _spec("E")
    assert arch.name == "Lenedra" and cfg.width == 40 and cfg.vocab_size == 83 and not spec.tied_head
    assert spec.embedding.kind == "scaled_token_embedding" and spec.embedding.params["scale"] == 3.0
    assert spec.head.kind == "capped_linear_head" and spec.head.params["softcap"] == 9.0
    assert spec.residual_streams == 3 and all(l.block.kind == "hyper_prenorm" and l.block.params["n_streams"] == 3 for l in spec.layers)
    _, f, fs = _spec("F")                                                  # no soft cap, no factor; one copy is still hyper-connections
    assert fs.head.params["softcap"] is None and fs.embedding.params["scale"] == 1.0 and fs.residual_streams == 1
    _, g, gs = _spec("G")                                                  # no 'streams': the plain pre-norm layer
    assert gs.residual_streams is None and all(l.block.kind == "prenorm" for l in gs.layers)
    assert spec.final_norm.params["unit_offset"] is True


def test_every_size_comes_from_the_file():
    _, cfg, _ = _spec("E")
    l0, l1, l2, l3, l4 = cfg.layers
    m = l0.mixer
    assert (l0.type, m.heads, m.kv_heads, m.dim, m.scale, m.window, m.keep_first, l0.mlp.ff) == ("attention", 6, 2, 16, 0.25, 13, 11, 24)
    a, d = l1.mixer.left, l1.mixer.right
    assert (l1.type, a.heads, a.kv_heads, a.dim, a.vdim, a.scale, a.chunk) == ("parallel", 4, 2, 8, 12, 0.3, 10)
    assert (d.heads, d.kv_heads, d.dim, d.vdim, d.conv, d.decay_rank, d.gate_rank) == (4, 2, 8, 12, 3, 5, 7)
    assert (l1.mixer.left_scale, l1.mixer.right_scale) == (0.7, 1.2)
    f = l1.mlp
    assert (f.experts, f.identity, f.top, f.ff, f.groups, f.keep_groups, f.scale, f.shared_ff) == (6, 2, 2, 16, 4, 2, 1.5, 12)
    f = l2.mlp
    assert (f.experts, f.identity, f.top, f.groups, f.keep_groups, f.scale, f.shared_ff) == (3, 0, 3, 1, 1, 1.0, None)
    assert l3.mlp is None and l3.mixer.left.chunk == 290 and (l4.mixer.window, l4.mixer.keep_first) == (29, 40)
    assert cfg.eps == 1e-5 and cfg.embedding_scale == 3.0 and cfg.logit_softcap == 9.0 and cfg.streams == 3
    _, h, _ = _spec("H")
    assert (h.layers[1].mixer.window, h.layers[1].mixer.keep_first) == (0, 0)             # no mask


@pytest.mark.parametrize("damage,text", [
    (lambda c: c.pop("width"), "width"),
    (lambda c: c.pop("vocab"), "vocab"),
    (lambda c: c["norm"].pop("eps"), "eps"),
    (lambda c: c.update(streams=0), "streams"),
    (lambda c: c.update(logit_softcap=-1.0), "logit_softcap"),
    (lambda c: c["layers"][0]["mixer"].pop("dim"), "dim"),
    (lambda c: c["layers"][0]["mixer"].update(vdim=8), "vdim"),                      # the values are the keys
    (lambda c: c["layers"][0]["mixer"].pop("scale"), "scale"),
    (lambda c: c["layers"][0]["mixer"]["mask"].pop("size"), "size"),
    (lambda c: c["layers"][0]["mixer"]["mask"].update(size=0), "size"),
    (lambda c: c["layers"][0]["mixer"]["mask"].update(keep_first=-1), "keep_first"),
    (lambda c: c["layers"][0].update(type="conv"), "conv"),
    (lambda c: c["layers"][0]["mlp"].update(kind="gated"), "gated"),
    (lambda c: c["layers"][0]["mixer"].update(heads=5), "multiple"),
    (lambda c: c["layers"][1]["mixer"].pop("left_scale"), "left_scale"),
    (lambda c: c["layers"][1]["mixer"]["left"].pop("vdim"), "vdim"),
    (lambda c: c["layers"][1]["mixer"]["right"].pop("conv"), "conv"),
    (lambda c: c["layers"][1]["mixer"]["right"].pop("decay_rank"), "decay_rank"),    # (no weight file to read it from)
    (lambda c: c["layers"][1]["mixer"]["right"].update(heads=3), "multiple"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=9), "top"),
    (lambda c: c["layers"][1]["mlp"]["router"]["groups"].update(count=3), "groups"),  # 8 outputs in 3 groups
    (lambda c: c["layers"][1]["mlp"]["router"]["groups"].update(keep=5), "groups"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=5), "top"),                 # two groups of two hold four
    (lambda c: c["layers"][1]["mlp"]["expert"].pop("ff"), "ff"),
    (lambda c: c.update(layers=[]), "layers"),
])
def test_a_bad_file_is_refused_with_the_key_s_name(damage, text):
    from flambeau_amd.config import ConfigError
    from flambeau_amd.registry import config_from_dict
    raw = json.loads(json.dumps(CONFIGS["E"]["config"]))
    damage(raw)
    with pytest.raises(ConfigError, match=text):
        config_from_dict(raw, "test")


def test_the_ranks_of_the_low_rank_projections_come_from_the_tensors_shapes(tmp_path):
    """A file of the design names no rank: the folder's tensors say it; a key in the file wins over them."""
    from flambeau_amd.config.lenedra import LenedraConfig
    from flambeau_amd.registry import config_from_dir
    d = write_model("E", tmp_path / "m", drop_ranks=True)
    raw = json.loads((d / "config.json").read_text())
    assert "decay_rank" not in raw["layers"][1]["mixer"]["right"]
    _, cfg = config_from_dir(d)
    assert (cfg.layers[1].mixer.right.decay_rank, cfg.layers[1].mixer.right.gate_rank) == (5, 7)
    assert (cfg.layers[3].mixer.right.decay_rank, cfg.layers[3].mixer.right.gate_rank) == (3, 3)
    filled = LenedraConfig.sizes_from_tensors(CONFIGS["E"]["config"], {"l1.mix.right.a1": (99, 40), "l1.mix.right.g1": (98, 40)})
    assert filled["layers"][1]["mixer"]["right"]["decay_rank"] == 5


def test_parts_caches_and_tensor_names(tmp_path):
    from flambeau_amd.models.decoder import DecoderModel
    from flambeau_amd.parts import JoinedCacheSpec, PagedKVSpec, StateSpec
    _, cfg, spec = _spec("E")
    model = DecoderModel(spec, rt=None)
    kinds = [type(b.mixer).__name__ for b in model.blocks]
    assert kinds == ["MixedHeadsAttention", "SideBySide", "MixedHeadsAttention", "SideBySide", "MixedHeadsAttention"]
    specs, shares = model.cache_entries()
    assert shares == [None] * 5
    assert specs[0] == PagedKVSpec(2, 16, 13, 11, 0) and specs[2] == PagedKVSpec(3, 16, 300, 2, 0) and specs[4] == PagedKVSpec(4, 8, 29, 40, 0)
    assert isinstance(specs[1], JoinedCacheSpec) and specs[1].paged == PagedKVSpec(2, 16, 0, 0, 10)      # (heads stored max(8, 12) -> 16 wide)
    d = cfg.layers[1].mixer.right
    channels = 2 * d.kv_heads * d.dim + d.heads * d.vdim
    assert specs[1].states == (None, StateSpec((d.heads * d.dim * d.vdim + (d.conv - 1) * channels,), torch.float32))
    assert specs[3].paged.chunk == 290
    names = set(model.manifest())
    for n in ("embed", "head", "final.norm", "l0.norm1", "l0.norm2", "l0.mix.q", "l0.mix.q.b", "l0.mix.k.b", "l0.mix.q.norm", "l0.mix.k.norm",
              "l0.mix.o.b", "l0.hc1.in", "l0.hc1.out", "l0.hc1.mix", "l0.hc2.mix", "l1.mix.left.q.b", "l1.mix.left.v", "l1.mix.left.v.b",
              "l1.mix.left.sink", "l1.mix.left.o", "l1.mix.right.q.conv", "l1.mix.right.b", "l1.mix.right.A_log", "l1.mix.right.dt_bias",
              "l1.mix.right.a1", "l1.mix.right.a2", "l1.mix.right.g1", "l1.mix.right.g2", "l1.mix.right.norm", "l1.mix.right.o",
              "l1.mlp.router", "l1.mlp.correction", "l1.mlp.e5.down", "l1.mlp.shared.up", "l3.hc1.mix"):
        assert n in names, n
    for n in ("l0.mix.v", "l1.mix.left.o.b", "l1.mlp.e6.gate", "l2.mlp.shared.gate", "l3.norm2", "l3.hc2.in", "l1.mix.left.q.norm", "l1.mix.left_out"):
        assert n not in names, n
    shapes = {n: tuple(ts.shape) for n, (_, _, ts) in model.manifest().items()}
    assert shapes["l1.mlp.router"] == (8, 40) and shapes["l1.mlp.correction"] == (8,) and shapes["l0.mix.q.norm"] == (16,)
    assert shapes["l1.mix.right.a2"] == (32, 5) and shapes["l1.mix.right.dt_bias"] == (32,) and shapes["l1.mix.right.A_log"] == (4,)
    assert shapes["l0.hc1.mix"] == (3, 3) and shapes["l0.hc1.in"] == (3,)
    # the plain pre-norm model has no such numbers
    assert not any(".hc" in n for n in DecoderModel(_spec("G")[2], rt=None).manifest())
    dd = write_model("F", tmp_path / "F")
    conf, t = read_model(dd)
    assert set(t) == set(DecoderModel(_spec("F")[2], rt=None).manifest()) and t["l0.hc1.mix"].shape == (1, 1)


def test_pages_of_kept_first_tokens_stay_and_chunks_pass():
    """The manager gives a windowed group's pages back as the window passes them, all but those that hold a kept first
    token; a chunked group keeps the newest run of positions alone."""
    from flambeau_amd.cache.manager import CacheManager, GroupSpec
    ps = 4
    mgr = CacheManager([GroupSpec(window=6, keep_first=5), GroupSpec(window=6), GroupSpec(chunk=10), GroupSpec()], n_pages=40, page_size=ps,
                       max_slots=2, max_seq_len=200)
    assert mgr.admit("a") is not None
    at = 0
    for k in (3, 9, 1, 1, 14, 2, 1, 30, 1):
        mgr.ensure("a", at + k)
        mgr.advance("a", k)
        at += k
        mgr.check_invariants()
        for g, spec in enumerate(mgr.groups):
            held = {b for b, p in enumerate(mgr.table_row("a", g)) if p >= 0}
            # what the next query (at position ``at``) and every later one can still see
            if spec.window:
                lo = at - spec.window + 1
            elif spec.chunk:
                lo = at - at % spec.chunk
            else:
                lo = 0
            needed = {j // ps for j in range(max(lo, 0), at)} | {j // ps for j in range(min(spec.keep_first, at))}
            assert needed <= held, (g, at)
            assert held <= needed | {b for b in held if b * ps + ps > max(lo, 0)}, (g, at)     # nothing wholly below the edge is kept...
            if spec.keep_first and at > 20:
                assert {0, 1} <= held and 2 not in held                                          # ...but the kept tokens' pages
    mgr.release("a")
    assert mgr.free_pages() == [40] * 4


# ---------------------------------------------------------------- the plain implementation's own invariants
def test_the_plain_model_is_causal_and_every_constant_matters():
    cfg, t = read_model_of("E")
    toks = list(np.random.default_rng(0).integers(0, 83, size=60))
    base = pl.forward(cfg, t, toks)
    assert np.allclose(pl.forward(cfg, t, toks[:41])[:41], base[:41], rtol=0, atol=1e-9)
    changed = toks[:]
    changed[50] = (changed[50] + 1) % 83
    other = pl.forward(cfg, t, changed)
    assert np.allclose(other[:50], base[:50], rtol=0, atol=1e-9) and np.abs(other[50:] - base[50:]).max() > 1e-3

    def differs(edit):
        c = json.loads(json.dumps(cfg))
        edit(c)
        return np.abs(pl.forward(c, t, toks) - base).max() > 1e-6
    assert differs(lambda c: c["embedding"].update(scale=3.1))
    assert differs(lambda c: c.update(logit_softcap=8.0))
    assert differs(lambda c: c["norm"].update(eps=1e-2))
    assert differs(lambda c: c["layers"][0]["mixer"]["mask"].update(size=12))
    assert differs(lambda c: c["layers"][0]["mixer"]["mask"].update(keep_first=10))
    assert differs(lambda c: c["layers"][0]["mixer"].update(scale=0.26))
    assert differs(lambda c: c["layers"][1]["mixer"]["left"]["mask"].update(size=11))
    assert differs(lambda c: c["layers"][1]["mixer"].update(left_scale=0.71))
    assert differs(lambda c: c["layers"][1]["mixer"].update(right_scale=1.21))
    assert differs(lambda c: c["layers"][1]["mlp"]["router"].update(scale=1.6))
    assert differs(lambda c: c["layers"][1]["mlp"]["router"]["groups"].update(keep=1))
    assert differs(lambda c: c["layers"][1]["mlp"]["router"].update(top=3))
    import re
    for name in sorted(t):                                   # every tensor is read (an expert only if a token chooses it)
        if re.search(r"\.mlp\.e\d+\.", name) and not name.startswith("l2."):
            continue
        if name == "l2.mlp.correction":                      # (all three experts are chosen there: the choice has nothing to decide)
            continue
        bumped = dict(t)
        bumped[name] = t[name] + 0.05 + 0.3 * np.random.default_rng(1).normal(size=t[name].shape)     # (uneven: a shift of all router scores alike changes nothing)
        assert np.abs(pl.forward(cfg, bumped, toks) - base).max() > 1e-7, name


def read_model_of(name, tmp=[]):
    import pathlib
    import tempfile
    if not tmp:
        tmp.append(pathlib.Path(tempfile.mkdtemp()))
    d = tmp[0] / name
    if not d.exists():
        write_model(name, d)
    return read_model(d)


def test_masks_written_out():
    w = pl.window_mask(6, 2, keep_first=1).astype(int)
    assert w.tolist() == [[1, 0, 0, 0, 0, 0], [1, 1, 0, 0, 0, 0], [1, 1, 1, 0, 0, 0], [1, 0, 1, 1, 0, 0], [1, 0, 0, 1, 1, 0], [1, 0, 0, 0, 1, 1]]
    c = pl.chunk_mask(5, 2).astype(int)
    assert c.tolist() == [[1, 0, 0, 0, 0], [1, 1, 0, 0, 0], [0, 0, 1, 0, 0], [0, 0, 1, 1, 0], [0, 0, 0, 0, 1]]
    assert pl.distance_slopes(4).tolist() == [0.25, 0.0625, 0.015625, 0.00390625]


def test_a_sink_takes_weight_and_gives_nothing():
    """One head, two tokens, keys that score 0: the weights are 1 / (n + e^sink) each."""
    q, k = np.zeros((2, 1, 3)), np.ones((2, 1, 3))
    v = np.array([[[2.0, 0.0]], [[0.0, 4.0]]])
    o = pl.softmax_attention(q, k, v, pl.window_mask(2, 5), 1.0, sink=np.array([np.log(2.0)]))
    assert np.allclose(o[0, 0], [2.0 / 3.0, 0.0]) and np.allclose(o[1, 0], [2.0 / 4.0, 4.0 / 4.0])
    o = pl.softmax_attention(q, k, v, pl.window_mask(2, 5), 1.0, slopes=np.array([np.log(3.0)]))       # the bias: e^(-slope * distance)
    assert np.allclose(o[1, 0], [2.0 * (1 / 3) / (1 + 1 / 3), 4.0 / (1 + 1 / 3)])


def test_two_tokens_of_the_delta_rule_written_out():
    """One head, key and value of one and two dims, no convolution taps beyond the token's own."""
    W = 2
    t = {"p.q": np.array([[1.0, 0.0]]), "p.k": np.array([[0.0, 1.0]]), "p.v": np.eye(2), "p.q.conv": np.ones((1, 1)), "p.k.conv": np.ones((1, 1)),
         "p.v.conv": np.ones((2, 1)), "p.b": np.zeros((1, W)), "p.a1": np.zeros((1, W)), "p.a2": np.zeros((1, 1)), "p.dt_bias": np.array([0.0]),
         "p.A_log": np.array([0.0]), "p.g1": np.zeros((1, W)), "p.g2": np.zeros((2, 1)), "p.norm": np.ones(2), "p.o": np.eye(2)}
    h = np.array([[1.0, 2.0], [3.0, -1.0]])
    m = dict(heads=1, kv_heads=1, dim=1, vdim=2, conv=1)
    silu = lambda z: z / (1 + np.exp(-z))
    q = np.sign(silu(h[:, 0]))          # unit vectors of one dim (the 1e-6 under the root aside), times dim^-1/2 = 1
    k = np.sign(silu(h[:, 1]))
    v = silu(h)
    g = np.exp(-np.log(2.0))            # exp(-exp(0) softplus(0))
    S = 0.5 * k[0] * v[0]               # beta = sigmoid(0) = 1/2
    o0 = S * q[0]
    S = g * S
    S = S + k[1] * 0.5 * (v[1] - S * k[1])
    o1 = S * q[1]
    want = np.stack([o0, o1])
    want = want / np.sqrt((want ** 2).mean(axis=1, keepdims=True) + 1e-5) * 0.5          # the heads' norm, the gate sigmoid(0)
    got = pl.gated_delta_rule(h, m, t, "p.", 1e-5)
    assert np.allclose(got, want, atol=1e-5)


def test_the_router_written_out():
    """Four outputs in two groups, one kept: the correction lifts group 1 although group 0 holds the largest score, and
    inside group 1 a negative choice score still beats what lies outside (which counts as minus infinity, not 0)."""
    z = np.log(np.array([[0.4, 0.1, 0.3, 0.2]]))
    corr = np.array([0.0, 0.0, -0.25, -0.5])
    chosen, w = pl.route(z, corr + np.array([0, 0, 0.5, 0]), top=2, groups=2, keep=1, scale=2.0)       # choice: .4 .1 | .55 -.3
    assert chosen.tolist() == [[2, 3]] and np.allclose(w, [[2.0 * 0.3 / 0.5, 2.0 * 0.2 / 0.5]])
    chosen, w = pl.route(z, corr, top=2, groups=2, keep=1, scale=1.0)                                  # choice: .4 .1 | .05 -.3
    assert chosen.tolist() == [[0, 1]] and np.allclose(w, [[0.8, 0.2]])
    chosen, _ = pl.route(z, corr, top=2, groups=2, keep=2, scale=1.0)
    assert chosen.tolist() == [[0, 1]]
    chosen, _ = pl.route(z, np.zeros(4), top=3, groups=1, keep=1, scale=1.0)
    assert chosen.tolist() == [[0, 2, 3]]


def test_hyper_connections_written_out():
    """Two copies, a sublayer that returns its input: u = in . x, x_t <- sum_s mix[s, t] x_s + out[t] u."""
    xs = np.array([[[1.0, 2.0]], [[3.0, 5.0]]])                      # [copies, tokens, width]
    t = {"p.in": np.array([2.0, -1.0]), "p.out": np.array([10.0, 100.0]), "p.mix": np.array([[1.0, 2.0], [3.0, 4.0]])}
    got = pl.hyper_sublayer(xs, t, "p.", np.zeros(2), 0.0, lambda h: h * np.sqrt(((2 * xs[0] - xs[1]) ** 2).mean()))   # (undo the norm)
    u = 2 * xs[0] - xs[1]
    assert np.allclose(got[0], 1 * xs[0] + 3 * xs[1] + 10 * u) and np.allclose(got[1], 2 * xs[0] + 4 * xs[1] + 100 * u)
