"""Fitevik on the GPU against the plain implementation: every mechanism alone, the layers one by one, and
whole models in every cutting (whole prompts, single tokens, portions down to two tokens, mixed batches over
a small poisoned pool whose pages and slots are used again), in 32-bit and in bfloat16, at sizes of the
tests' own."""
import json

import numpy as np
import pytest
import torch

import plain_fitevik as pf
import replay_helpers as rh
from fitevik_configs import CONFIGS, read_model, write_model
from test_bugidra_gpu import CUTS, TOL, _x, bound_part, run_mixer, runner_for
from test_kuvidra_gpu import close, make_rt, make_step

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = ["float32", "bfloat16"]
TORCH = {"float32": torch.float32, "bfloat16": torch.bfloat16}


@pytest.fixture(scope="module")
def dirs(tmp_path_factory):
    base = tmp_path_factory.mktemp("fitevik")
    out = {}
    for name in CONFIGS:
        for store in DTYPES:
            out[(name, store)] = write_model(name, base / f"{name}-{store}", store)
    for store in DTYPES:          # (weights are stored in the dtype they are run in: the plain side reads the same numbers)
        out[("sharp", store)] = write_model("K", base / f"K-sharp-{store}", store, sharpen=8.0)
        out[("memory", store)] = write_model("K", base / f"K-memory-{store}", store, remember=True)
    return out


_refs = {}


def reference(d, reqs):
    out = {}
    cfg = t = None
    for rid, toks in reqs.items():
        key = (str(d), tuple(toks))
        if key not in _refs:
            if cfg is None:
                cfg, t = read_model(d)
            _refs[key] = pf.forward(cfg, t, toks)
        out[rid] = _refs[key]
    return out


def computed(r, rt):
    from flambeau_amd.parts import Product
    r = r.compute(rt) if isinstance(r, Product) else r
    return r.double().cpu().numpy()


# ---------------------------------------------------------------- each mechanism alone
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("W", [52, 40, 37, 42, 256, 1000])
def test_layer_norm_ahead_and_behind(dtype, W):
    """The norm as a part: of a row, of picked rows, with a delta added on the way, and as the norm of a
    sublayer's output added to the stream (which the kernel also leaves in the compute dtype)."""
    from flambeau_amd.parts import NORMS, PartSpec
    rt = make_rt(dtype)
    n, eps = 37, 3e-4
    norm, plain = bound_part(NORMS, PartSpec("layernorm", dict(hidden_size=W, eps=eps)), dtype, rt, seed=W, prefix="n.")
    x = torch.randn(n, W, generator=torch.Generator().manual_seed(2)) * 3 + 1.5        # a mean that is not zero
    d = torch.randn(n, W, generator=torch.Generator().manual_seed(3))
    out = torch.empty(n, W, dtype=TORCH[dtype], device=DEV)
    xs = x.to(DEV).contiguous()
    norm.forward(xs, out, delta=d.to(DEV), store_sum=True)
    want = pf.layer_norm((x + d).double().numpy(), plain, "n", eps)
    tol = 3e-6 if dtype == "float32" else 1e-2
    assert np.abs(out.double().cpu().numpy() - want).max() < tol * np.abs(want).max()
    assert torch.equal(xs.cpu(), x + d)                         # the sum went back into the stream
    rows = torch.tensor([5, 0, 36], dtype=torch.int32, device=DEV)
    picked = torch.empty(3, W, dtype=TORCH[dtype], device=DEV)
    norm.forward(xs, picked, rows=rows)
    assert torch.equal(picked, out[rows.long()])
    # behind a sublayer: stream += norm(delta)
    resid = x.to(DEV).contiguous()
    cast = torch.empty(n, W, dtype=TORCH[dtype], device=DEV) if dtype != "float32" else None
    norm.add_to(resid, (d * 40).to(DEV).contiguous(), cast=cast)       # (the norm takes the output's size away)
    want = x.double().numpy() + pf.layer_norm((d * 40).double().numpy(), plain, "n", eps)
    assert np.abs(resid.double().cpu().numpy() - want).max() < 3e-6 * np.abs(want).max()    # the stream is 32-bit in both dtypes
    if cast is not None:
        assert torch.equal(cast, resid.to(TORCH[dtype]))
    # a row of equal values has no deviation: eps alone stands under the root, the bias comes out
    flat = torch.full((2, W), 7.0, device=DEV)
    o = torch.empty(2, W, dtype=torch.float32, device=DEV)
    from flambeau_amd.kernels import ops
    ops.layernorm(flat, norm.weight, norm.bias, o, eps)
    assert torch.allclose(o, norm.bias.expand(2, W), atol=1e-6)


@pytest.mark.parametrize("W", [256, 4096, 1000])
def test_layer_norm_bits_do_not_depend_on_the_step_s_size(W):
    """A step of few rows keeps its rows in registers, a large one reads them three times: the same sums in the
    same order, so a row's bits are the same in both."""
    from flambeau_amd.kernels import ops
    g = torch.Generator().manual_seed(W)
    x = (torch.randn(300, W, generator=g) * 2 + 0.5).to(DEV)
    d = torch.randn(300, W, generator=g).to(DEV)
    w, b = (1 + 0.1 * torch.randn(W, generator=g)).to(DEV), torch.randn(W, generator=g).to(DEV)
    big = ops.layernorm(x, w, b, torch.empty(300, W, device=DEV), 1e-5, delta=d)
    few = ops.layernorm(x[:7].contiguous(), w, b, torch.empty(7, W, device=DEV), 1e-5, delta=d[:7].contiguous())
    assert torch.equal(big[:7], few)
    r_big, r_few = x.clone(), x[:7].clone()
    ops.layernorm_add(d, w, b, r_big, 1e-5)
    ops.layernorm_add(d[:7].contiguous(), w, b, r_few, 1e-5)
    assert torch.equal(r_big[:7], r_few)


@pytest.mark.parametrize("dtype", DTYPES)
def test_embedding_with_learned_positions_and_the_scaled_head(dtype):
    from flambeau_amd.parts import EMBEDDINGS, HEADS, PartSpec
    rt = make_rt(dtype)
    V, W, P, eps = 11, 44, 30, 1e-5
    norm = PartSpec("layernorm", dict(hidden_size=W, eps=eps))
    emb, plain = bound_part(EMBEDDINGS, PartSpec("positional_token_embedding", dict(vocab_size=V, hidden_size=W, max_positions=P, norm=norm)),
                            dtype, rt, seed=4, scale=1.0, prefix="")
    t = {"embed": plain["weight"], "pos": plain["positions"], "embed.norm": plain["norm"], "embed.norm.b": plain["norm.b"]}
    step = make_step([(7, 3), (0, 2), (28, 2)], 8, 12)
    toks = [3, 10, 0, 3, 3, 9, 1]
    step.tokens = torch.tensor(toks, dtype=torch.int32, device=DEV)
    got = emb.forward(step.tokens, torch.empty(7, W, dtype=torch.float32, device=DEV), step=step)
    want = pf.embed(toks, [7, 8, 9, 0, 1, 28, 29], t, eps)
    assert np.abs(got.double().cpu().numpy() - want).max() < 3e-6 * np.abs(want).max()
    assert np.abs(want[3] - want[4]).max() > 0.1                 # one token at two positions
    with pytest.raises(RuntimeError):
        emb.forward(step.tokens, torch.empty(7, W, dtype=torch.float32, device=DEV))
    for scale in (0.3, 1.0):
        head = HEADS.create(PartSpec("scaled_linear_head", dict(vocab_size=V, hidden_size=W, scale=scale)))
        w = (torch.randn(V, W, generator=torch.Generator().manual_seed(6)) * 0.3).to(TORCH[dtype])
        head.bind({"weight": w.to(DEV)}, rt)
        x = _x(5, W, dtype, 7)
        logits = head.forward(x.to(DEV), 5)
        want = x.double().numpy() @ w.double().numpy().T * scale
        assert np.abs(logits.double().cpu().numpy()[:5] - want).max() < (3e-6 if dtype == "float32" else 1e-2) * np.abs(want).max()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("W,F", [(40, 24), (36, 50), (64, 128)])
def test_feed_forward_with_biases_and_squared_relu(dtype, W, F):
    from flambeau_amd.parts import FEED_FORWARDS, PartSpec
    rt = make_rt(dtype)
    part, plain = bound_part(FEED_FORWARDS, PartSpec("mlp", dict(hidden_size=W, intermediate_size=F, activation="relu2", bias=True)),
                             dtype, rt, seed=F)
    x = _x(70, W, dtype, 5) * 2
    got = computed(part.forward(x.to(DEV), None), rt)
    want = pf.dense_mlp(x.double().numpy(), plain, "m.")
    assert np.abs(got - want).max() < TOL[dtype] * np.abs(want).max()
    assert np.abs(want - pf.dense_mlp(x.double().numpy(), dict(plain, **{"m.up.b": plain["m.up.b"] * 0}), "m.")).max() > 1e-2


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("W,F,E,top,n", [(40, 16, 5, 2, 70), (36, 20, 4, 1, 33), (64, 32, 8, 3, 150), (48, 8, 3, 3, 9), (32, 64, 16, 2, 1)])
def test_ungated_experts_weighted_by_the_chosen_logits(dtype, W, F, E, top, n):
    from flambeau_amd.parts import FEED_FORWARDS, PartSpec
    rt = make_rt(dtype)
    part, plain = bound_part(FEED_FORWARDS, PartSpec("routed_experts", dict(
        hidden_size=W, n_experts=E, top=top, expert_size=F, scoring="softmax_chosen", weight_on="output", gated=False,
        activation="relu2", router_bias=True)), dtype, rt, seed=E + top, scale=0.4)
    assert not any("gate" in k for k in part.tensors())
    x = _x(n, W, dtype, 5) * 2
    got = computed(part.forward(x.to(DEV), None), rt)
    h = x.double().numpy()
    want = pf.routed_experts(h, {"router": {"experts": E, "top": top}}, plain, "m.")
    z = np.sort(h @ plain["m.router"].T + plain["m.router.b"], axis=1)
    sure = (z[:, E - top] - z[:, E - top - 1] > 0.05) if top < E else np.ones(n, bool)      # no close call between the last chosen and the next
    assert sure.sum() >= 0.6 * n
    assert np.abs(got - want)[sure].max() < TOL[dtype] * np.abs(want).max()


HGRN_SHAPES = [(3, 8, 12), (1, 20, 6), (2, 64, 32), (4, 32, 32), (2, 16, 64), (5, 128, 40), (1, 1, 1)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,D,Dv", HGRN_SHAPES)
def test_hgrn2_alone(dtype, H, D, Dv):
    """The recurrence whose forget gate also decides what is written, in three cuttings; the state lives in a
    slot between steps, and in 32-bit no bit depends on the cutting."""
    from flambeau_amd.parts import MIXERS, PartSpec
    rt = make_rt(dtype)
    W, eps = 40, 2e-5
    fix = {"lower": lambda v: torch.sigmoid(v * 6)}           # bounds between nought and one, some next to either
    mixer, plain = bound_part(MIXERS, PartSpec("hgrn2", dict(hidden_size=W, n_heads=H, head_dim=D, value_dim=Dv, eps=eps)),
                              dtype, rt, seed=H * D + Dv, fix=fix)
    x = _x(90, W, dtype, 5)
    want, _ = pf.hgrn2(x.double().numpy(), dict(heads=H, dim=D, vdim=Dv), plain, "m.", eps)
    runs = [run_mixer(mixer, rt, x, cuts) for cuts in CUTS]
    for got, cuts in zip(runs, CUTS):
        assert np.abs(got - want).max() < TOL[dtype] * np.abs(want).max(), cuts
    if dtype == "float32":
        assert np.array_equal(runs[0], runs[1]) and np.array_equal(runs[0], runs[2])


def test_hgrn2_without_bound_and_bias():
    from flambeau_amd.parts import MIXERS, PartSpec
    rt = make_rt("float32")
    W, H, D, Dv, eps = 24, 2, 12, 10, 1e-5
    mixer, plain = bound_part(MIXERS, PartSpec("hgrn2", dict(hidden_size=W, n_heads=H, head_dim=D, value_dim=Dv, eps=eps,
                                                             lower_bound=False, gate_bias=False)), "float32", rt, seed=3)
    assert "lower" not in mixer.tensors() and "f.bias" not in mixer.tensors()
    plain.update({"m.lower": np.zeros(H * D), "m.f.b": np.zeros(H * D)})
    x = _x(50, W, "float32", 5)
    want, _ = pf.hgrn2(x.double().numpy(), dict(heads=H, dim=D, vdim=Dv), plain, "m.", eps)
    got = run_mixer(mixer, rt, x, [20, 1, 1, 28])
    assert np.abs(got - want).max() < 3e-5 * np.abs(want).max()


def mixed_spec(W, H, G, D, Dv, window, scale, eps, **kw):
    from flambeau_amd.parts import PartSpec
    return PartSpec("mixed_heads_attention", dict(dict(hidden_size=W, n_heads=H, n_kv_heads=G, head_dim=D, value_dim=Dv, window=window,
                                                       scale=scale, qk_norm="projection", eps=eps, slope_exponent=8.0, head_mix=True, sink=True), **kw))


def plain_mixed(h, plain, H, G, D, Dv, window, scale, eps, exponent=8.0, kv=None, first=0):
    """The mixer from the plain functions; ``kv``: another layer's keys and values."""
    n = h.shape[0]
    m = dict(heads=H, kv_heads=G, dim=D, vdim=Dv)
    k, v = kv if kv is not None else pf.keys_and_values(h, m, plain, "m.", eps)
    q = pf.rms_norm(h @ plain["m.q"].T, plain["m.q.norm"], eps).reshape(n, H, D)
    slopes = None if exponent is None else np.array([2.0 ** (-exponent * (g + 1) / H) for g in range(H)])
    out = pf.mixed_softmax_attention(q[first:], k, v, window, scale, slopes, plain.get("m.talk"), plain.get("m.sink"), first=first)
    return out.reshape(n - first, -1) @ plain["m.o"].T


ATT_SHAPES = [
    # H, G, D, Dv, window
    (6, 2, 16, 8, 13), (3, 1, 10, 6, 1), (4, 4, 12, 20, 300), (8, 1, 32, 32, 70), (2, 2, 32, 32, 64), (1, 1, 72, 40, 33), (5, 5, 8, 8, 2),
    (16, 4, 64, 64, 100), (4, 2, 24, 40, 0),
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,Dv,window", ATT_SHAPES)
def test_mixed_heads_attention_alone(dtype, H, G, D, Dv, window):
    """Norm over the whole projection, distance bias, mixed heads, window and sink against the plain functions, whole
    and in portions that cross the window's edge, page borders and the kernels' chunks; sinks large enough to matter."""
    from flambeau_amd.parts import MIXERS
    rt = make_rt(dtype, max_tokens=512)
    W, n, eps, scale = 40, 150 if window < 200 else 420, 2e-5, 0.5
    fix = {"sink": lambda v: v * 8}
    mixer, plain = bound_part(MIXERS, mixed_spec(W, H, G, D, Dv, window, scale, eps), dtype, rt, seed=H + D, fix=fix)
    assert mixer.cache_spec().window == window
    x = _x(n, W, dtype, 5)
    h = x.double().numpy()
    want = plain_mixed(h, plain, H, G, D, Dv, window, scale, eps)
    without = plain_mixed(h, {k: v for k, v in plain.items() if k != "m.sink"}, H, G, D, Dv, window, scale, eps)
    assert np.abs(want - without).max() > 0.05 * np.abs(want).max()
    cuttings = ([n], [60, 4, 1, 1, 70, 2, 12] + [1] * (n - 150), [1] * 30 + [n - 30]) if n == 150 else ([n], [330, 7, 1, 1] + [1] * 81)
    for cuts in cuttings:
        assert sum(cuts) == n
        got = run_mixer(mixer, rt, x, cuts, n_pages=70)
        assert np.abs(got - want).max() < TOL[dtype] * np.abs(want).max(), cuts[:8]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("exponent,head_mix,sink", [(None, False, False), (8.0, False, False), (None, True, False), (None, False, True), (3.0, True, True)])
def test_every_step_before_the_softmax_is_a_parameter(dtype, exponent, head_mix, sink):
    """Bias, mixing and sink one by one and together; none of them: plain softmax attention inside a window."""
    from flambeau_amd.parts import MIXERS
    rt = make_rt(dtype)
    W, n, eps, scale, H, G, D, Dv, window = 40, 100, 1e-5, 0.6, 4, 2, 16, 24, 21
    mixer, plain = bound_part(MIXERS, mixed_spec(W, H, G, D, Dv, window, scale, eps, slope_exponent=exponent, head_mix=head_mix, sink=sink),
                              dtype, rt, seed=11, fix={"sink": lambda v: v * 8})
    assert ("talk" in mixer.tensors()) == head_mix and ("sink" in mixer.tensors()) == sink
    x = _x(n, W, dtype, 6)
    want = plain_mixed(x.double().numpy(), plain, H, G, D, Dv, window, scale, eps, exponent=exponent)
    for cuts in ([n], [50, 3, 1, 1, 45], [1] * 25 + [75]):
        got = run_mixer(mixer, rt, x, cuts)
        assert np.abs(got - want).max() < TOL[dtype] * np.abs(want).max(), cuts


def pointing_weights(H, G, D):
    """Weights under which the query at position i points at ONE key: the model width holds two vectors of G * D
    values per token; the keys read the second, u_i, the queries the first, which the test sets to u_(i - back)."""
    W = 2 * G * D
    wq, wk = torch.zeros(H * D, W), torch.zeros(G * D, W)
    for h in range(H):
        g = h // (H // G)
        for d in range(D):
            wq[h * D + d, g * D + d] = 1.0
    for e in range(G * D):
        wk[e, G * D + e] = 1.0
    return W, wq, wk


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window,page", [(13, 8), (64, 16), (300, 16), (1, 8), (129, 32)])
def test_one_key_stands_out_at_every_distance(dtype, window, page):
    """Every query points at the one key ``back`` tokens behind it (its score is some twenty above the others', so it
    takes nearly all the weight if it is seen): the window's last key inside and the first outside, the query's own and
    its neighbour, far keys, and with them keys on either side of every page border; in a whole prompt, in portions and
    token by token.  A key that is lost or one too many turns the output round."""
    from flambeau_amd.parts import MIXERS
    rt = make_rt(dtype, max_tokens=512)
    H, G, D, Dv, eps, scale = 4, 2, 32, 16, 1e-6, 0.8
    W, wq, wk = pointing_weights(H, G, D)
    n = max(2 * window + 40, 120) if window < 200 else 420
    gen = torch.Generator().manual_seed(window)
    u = torch.randn(n, G * D, generator=gen)
    one = lambda v: torch.ones_like(v)
    for back in sorted({0, 1, window - 2, window - 1, window, window + 1, window // 2} - {-1}):
        if back < 0:
            continue
        a = torch.roll(u, back, 0)
        a[:back] = torch.randn(back, G * D, generator=gen)                    # (no such key yet)
        x = torch.cat([a, u], dim=1).to(TORCH[dtype])
        fix = {"q.weight": lambda v: wq, "k.weight": lambda v: wk, "q_norm.weight": one, "k_norm.weight": one,
               "talk": lambda v: torch.eye(H) + 0.1 * v, "sink": lambda v: v}
        # (slopes 2^-4 .. 2^-16: the bias leaves most heads their far keys)
        mixer, plain = bound_part(MIXERS, mixed_spec(W, H, G, D, Dv, window, scale, eps, slope_exponent=16.0), dtype, rt, seed=5, fix=fix)
        h = x.double().numpy()
        want = plain_mixed(h, plain, H, G, D, Dv, window, scale, eps, exponent=16.0)
        if back in (window - 1, window) and window > 1:        # the plain side itself turns round when the window moves by one key
            moved = plain_mixed(h, plain, H, G, D, Dv, window - 1 if back == window - 1 else window + 1, scale, eps, exponent=16.0)
            assert np.abs(moved[-1] - want[-1]).max() > 0.3 * np.abs(want).max(), back
        tail = min(n - 1, window + 20)
        for cuts in ([n], [n - tail] + [1] * tail, [7, 2, 9, 16, 1, 15, 33, 3] + [n - 86 - 30] + [1] * 30):
            assert sum(cuts) == n
            got = run_mixer(mixer, rt, x, cuts, page_size=page, n_pages=n // page + 6)
            err = np.abs(got - want).max(axis=1)
            worst = int(err.argmax())
            assert err[worst] < (1e-4 if dtype == "float32" else 0.1) * np.abs(want).max(), (back, cuts[:3], worst)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("w_source,w_reader", [(13, 29), (40, 40), (64, 17)])
def test_a_layer_that_reads_another_layer_s_keys(dtype, w_source, w_reader):
    """The reader has no key and value projections; its queries, window, mixing matrix and sinks are its own, the
    keys and values those the source wrote into the cache they share, which keeps the wider of the two windows."""
    from flambeau_amd.cache.storage import CacheStorage
    from flambeau_amd.parts import MIXERS
    rt = make_rt(dtype)
    W, n, eps, H, G, D, Dv, page = 40, 150, 1e-5, 6, 2, 16, 8, 8
    keep = max(w_source, w_reader)
    source, ps = bound_part(MIXERS, mixed_spec(W, H, G, D, Dv, w_source, 0.4, eps, cache_window=keep), dtype, rt, seed=1)
    reader, pr = bound_part(MIXERS, mixed_spec(W, H, G, D, Dv, w_reader, 0.7, eps, own_kv=False, cache_window=keep), dtype, rt, seed=2)
    assert not {"k.weight", "v.weight", "k_norm.weight"} & set(reader.tensors()) and source.cache_spec() == reader.cache_spec()
    xs, xr = _x(n, W, dtype, 3), _x(n, W, dtype, 4)            # the two layers read different streams
    kv = pf.keys_and_values(xs.double().numpy(), dict(kv_heads=G, dim=D, vdim=Dv), ps, "m.", eps)
    want_s = plain_mixed(xs.double().numpy(), ps, H, G, D, Dv, w_source, 0.4, eps)
    want_r = plain_mixed(xr.double().numpy(), pr, H, G, D, Dv, w_reader, 0.7, eps, kv=kv)
    for cuts in ([n], [60, 4, 1, 1, 70, 2, 12], [1] * 40 + [110]):
        store = CacheStorage([source.cache_spec(), reader.cache_spec()], [None, 0], rt.device, rt.dtype, n_pages=30, page_size=page, max_slots=2)
        for p in store.pools:
            p.fill_(float("nan"))
        assert store.entries[0].writes and not store.entries[1].writes and len(store.pools) == 1
        got_s, got_r, at = [], [], 0
        for k in cuts:
            step = make_step([(at, k)], page, 30, slots=[1], seed=2)
            got_s.append(computed(source.forward(xs[at:at + k].to(DEV).contiguous(), step, store.entries[0]), rt))
            got_r.append(computed(reader.forward(xr[at:at + k].to(DEV).contiguous(), step, store.entries[1]), rt))
            at += k
        assert np.abs(np.concatenate(got_s) - want_s).max() < TOL[dtype] * np.abs(want_s).max(), cuts
        assert np.abs(np.concatenate(got_r) - want_r).max() < TOL[dtype] * np.abs(want_r).max(), cuts
    with pytest.raises(RuntimeError):
        reader.forward(xr[:4].to(DEV).contiguous(), make_step([(0, 4)], page, 30), store.entries[0])


def test_single_tokens_behind_a_long_window_deal_their_keys_out():
    """Few rows over more than 256 keys: the tuned kernel set gives a token's keys to several blocks and joins them;
    the result is the one-block kernel's within rounding, and the plain implementation's."""
    from flambeau_amd.kernels import mixed_attention
    from flambeau_amd.parts import MIXERS
    rt = make_rt("bfloat16", max_tokens=1024)
    W, H, G, D, Dv, eps, n = 40, 4, 2, 32, 32, 1e-5, 900
    for window in (700, 0):
        mixer, plain = bound_part(MIXERS, mixed_spec(W, H, G, D, Dv, window, 0.5, eps), "bfloat16", rt, seed=7, fix={"sink": lambda v: v * 8})
        assert isinstance(mixer.kernels, mixed_attention.TunedMixedAttention)
        x = _x(n, W, "bfloat16", 5)
        want = plain_mixed(x.double().numpy(), plain, H, G, D, Dv, window, 0.5, eps, first=n - 20)
        seen = []
        orig = type(mixer.kernels).signature
        mixer.kernels.signature = lambda batch, w, k=mixer.kernels: seen.append(orig(k, batch, w)) or seen[-1]
        got = run_mixer(mixer, rt, x, [n - 20, 3] + [1] * 17, page_size=16, n_pages=64)
        del mixer.kernels.signature
        assert seen[0] == (0, 0) and max(seen)[1] >= 4       # the prompt: one block per tile; the single tokens: parts of 64 keys
        assert np.abs(got[n - 20:] - want).max() < 3e-2 * np.abs(want).max(), window


def test_the_matrix_core_kernel_at_the_size_of_a_real_layer():
    """32 heads over 8 key/value heads of 128, a window of 1,024: a prompt of 2,048 tokens whose keys are dealt out in
    parts of 512, a portion beside it, and single tokens whose keys are dealt out in parts of 64, on the matrix cores
    against the plain kernel (which the other tests hold against the plain implementation) with the same weights."""
    from flambeau_amd.engine import Runtime
    from flambeau_amd.kernels import mixed_attention
    from flambeau_amd.parts import MIXERS
    W, H, G, D, window, n = 128, 32, 8, 128, 1024, 2060
    x = _x(n, W, "bfloat16", 3)
    outs = []
    for tuned in (True, False):
        rt = Runtime(DEV, torch.bfloat16, 2304, tuned)
        mixer, _ = bound_part(MIXERS, mixed_spec(W, H, G, D, D, window, D ** -0.5 * 4, 1e-5), "bfloat16", rt, seed=9, fix={"sink": lambda v: v * 8})
        assert isinstance(mixer.kernels, mixed_attention.TunedMixedAttention) == tuned
        outs.append([run_mixer(mixer, rt, x, cuts, page_size=16, n_pages=140) for cuts in ([2048] + [1] * 12, [700, 40, 1308] + [2] * 6)])
    for got, want in zip(*outs):
        err = np.abs(got - want).max(axis=1)
        assert np.isfinite(got).all() and err.max() < 3e-2 * np.abs(want).max(), int(err.argmax())


# ---------------------------------------------------------------- layer by layer
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_the_stream_after_every_layer(dirs, name, dtype):
    from flambeau_amd.engine import StepEntry
    d = dirs[(name, dtype)]
    runner = runner_for(d, dtype, n_pages=16, page_size=CONFIGS[name]["page_size"], step_programs=False, decode_graphs=False)
    seen = []
    for b in runner.model.blocks:
        def wrapped(stream, step, cache, fwd=b.forward):
            fwd(stream, step, cache)
            seen.append(stream.flush().double().cpu().numpy())
        b.forward = wrapped
    toks = rh.make_requests(CONFIGS[name]["config"]["vocab"], [37], seed=1)["r0"]
    assert runner.begin("a")
    runner.step([StepEntry("a", toks, [0])])
    cfg, t = read_model(d)
    _, want = pf.forward(cfg, t, toks, keep_layers=True)
    assert len(seen) == len(want)
    for i, (g, w) in enumerate(zip(seen, want)):
        assert np.abs(g - w).max() < (2e-5 if dtype == "float32" else 1e-1) * np.abs(w).max(), f"layer {i}"


# ---------------------------------------------------------------- whole models in every cutting
LENGTHS = {"K": [40, 70, 97, 1, 33, 64, 2, 90, 340, 128, 21], "L": [97, 1, 150, 64, 31, 2, 120, 17, 65],
           "M": [150, 64, 3, 65, 1, 200, 31, 90], "N": [40, 100, 7, 64, 130, 2, 55], "P": [90, 33, 1, 140, 64, 2, 17, 120, 75, 200, 48, 100]}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_every_cutting(dirs, name, dtype):
    d = dirs[(name, dtype)]
    ps = CONFIGS[name]["page_size"]
    reqs = rh.make_requests(CONFIGS[name]["config"]["vocab"], LENGTHS[name], seed=5)
    ref = reference(d, reqs)
    for mode, steps in [("whole", rh.trace_whole(reqs)), ("tail", rh.trace_tail(reqs)), ("portions", rh.trace_portions(reqs)),
                        ("mixed", rh.trace_mixed(reqs, seed=13))]:
        peak = rh.peak_tokens(steps)
        runner = runner_for(d, dtype, n_pages=peak // ps, page_size=ps, max_tokens=max(peak, 256), slots=4)
        got = rh.run_in_process(runner, steps)
        pools = runner.manager.pools
        assert sum(p.n_acquired for p in pools) > sum(p.n_pages for p in pools), mode       # pages were used again
        assert not runner.manager.live and runner.manager.n_free_slots == 4
        close(got, ref, dtype, f"{name} {mode}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_single_tokens_replay_graphs_where_no_state_is_advanced(dirs, dtype):
    """A model of attention layers alone captures its decode steps (padded to a bucket: rows without pages
    ride along); one with a recurrent layer never does.  Both give the plain logits."""
    from flambeau_amd.engine import StepEntry
    d = dirs[("N", dtype)]
    reqs = rh.make_requests(90, [20, 33, 5], seed=12)
    ref = reference(d, reqs)
    runner = runner_for(d, dtype, n_pages=24, page_size=16, max_tokens=256)
    assert runner.decode_graphs
    assert not runner_for(dirs[("K", dtype)], dtype, n_pages=24, page_size=8).decode_graphs
    got = {}
    for rid, toks in reqs.items():
        assert runner.begin(rid)
        runner.step([StepEntry(rid, toks[:3], [])])
    for i in range(3, 33):
        live = [rid for rid, toks in reqs.items() if i < len(toks)]
        rows = runner.step([StepEntry(rid, [reqs[rid][i]], [0]) for rid in live]).cpu().double().numpy()
        for rid, row in zip(live, rows):
            got[(rid, i)] = row
    assert runner._graphs
    close(got, ref, dtype, "graphs")


def test_a_batch_equals_each_request_alone(dirs):
    """Unequal requests in one step against each alone: in 32-bit not a bit differs, whatever the
    neighbours, pages and slots are."""
    from flambeau_amd.engine import StepEntry
    d = dirs[("K", "float32")]
    reqs = rh.make_requests(83, [50, 3, 1, 77], seed=9)
    alone = {}
    for rid, toks in reqs.items():
        r = runner_for(d, "float32", n_pages=32, page_size=8)
        assert r.begin(rid)
        alone[rid] = r.step([StepEntry(rid, toks, list(range(len(toks))))]).cpu().numpy().copy()
    r = runner_for(d, "float32", n_pages=32, page_size=8)
    for rid in ("x", "y"):                  # two requests come and go first: other slots, other pages, states that are not zero
        assert r.begin(rid)
        r.step([StepEntry(rid, [1, 2, 3, 4, 5, 6, 7, 8, 9], [])])
    r.end("x"); r.end("y")
    for rid in reversed(list(reqs)):
        assert r.begin(rid)
    both = r.step([StepEntry(rid, toks, list(range(len(toks)))) for rid, toks in reqs.items()]).cpu().numpy()
    at = 0
    for rid, toks in reqs.items():
        assert np.array_equal(both[at:at + len(toks)], alone[rid]), rid
        at += len(toks)


@pytest.mark.parametrize("dtype", DTYPES)
def test_peaked_attention_over_far_keys_and_page_borders(dirs, dtype):
    """Score scales eight times as large: softmax puts nearly all weight on single keys, hundreds of tokens
    back or next to a page's or a window's edge alike, so one key lost or one too many shows in the logits."""
    d = dirs[("sharp", dtype)]
    reqs = rh.make_requests(83, [380, 131], seed=2)
    ref = reference(d, reqs)
    blunt = reference(dirs[("K", dtype)], reqs)
    assert np.abs(ref["r0"] - blunt["r0"]).max() > 0.05 * np.abs(ref["r0"]).max()
    for mode, steps in [("whole", rh.trace_whole(reqs)), ("tail", rh.trace_tail(reqs, tail=40)),
                        ("portions", rh.trace_portions(reqs, sizes=(7, 2, 8, 9, 16, 1, 15, 33, 3)))]:
        runner = runner_for(d, dtype, n_pages=64, page_size=8)
        close(rh.run_in_process(runner, steps), ref, dtype, f"sharp {mode}", bf16=8e-2)


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_memory_and_long_decoding(dirs, dtype):
    """Forget gates next to one: the first tokens stay in the memories for hundreds of steps (the plain logits
    at the end change when the first token does), through 340 single-token steps, during which the widest
    window (300 keys) passes over decoded tokens and the pages behind it are given back."""
    d = dirs[("memory", dtype)]
    toks = rh.make_requests(83, [400], seed=4)["r0"]
    reqs = {"r0": toks}
    ref = reference(d, reqs)
    other = reference(d, {"r0": [(toks[0] + 1) % 83] + toks[1:]})
    assert np.abs(ref["r0"][-1] - other["r0"][-1]).max() > 1e-3 * np.abs(ref["r0"]).max()
    runner = runner_for(d, dtype, n_pages=56, page_size=8)
    close(rh.run_in_process(runner, rh.trace_tail(reqs, tail=340)), ref, dtype, "memory")


@pytest.mark.parametrize("dtype", DTYPES)
def test_first_tokens(dirs, dtype):
    """Requests of one and two tokens, alone, side by side, and continued one token at a time: the first token
    sees itself and the sink, and writes into an empty memory."""
    d = dirs[("K", dtype)]
    reqs = rh.make_requests(83, [1, 2, 1, 3], seed=7)
    ref = reference(d, reqs)
    steps = [dict(entries=[dict(id=rid, tokens=toks[:1], want=[0]) for rid, toks in reqs.items()], end=["r0", "r2"]),
             dict(entries=[dict(id="r1", tokens=reqs["r1"][1:], want=[0]), dict(id="r3", tokens=reqs["r3"][1:2], want=[0])], end=["r1"]),
             dict(entries=[dict(id="r3", tokens=reqs["r3"][2:], want=[0])], end=["r3"])]
    close(rh.run_in_process(runner_for(d, dtype, n_pages=8, page_size=8), steps), ref, dtype, "first tokens")


def test_a_slot_that_is_used_again_starts_from_zero(dirs):
    """One state slot: every request inherits the slot of the one before, whose memories are not zero, and
    still gives the plain logits."""
    d = dirs[("L", "float32")]
    reqs = rh.make_requests(61, [30, 9, 1, 44], seed=8)
    ref = reference(d, reqs)
    runner = runner_for(d, "float32", n_pages=8, page_size=16, slots=1)
    close(rh.run_in_process(runner, rh.trace_portions(reqs, sizes=(5, 2, 11))), ref, "float32", "one slot")


# ---------------------------------------------------------------- through the entry points
@pytest.mark.parametrize("dtype", DTYPES)
def test_greedy_generation_through_the_engine(dirs, dtype):
    """``generate``: scheduler, portions, batching, device sampler.  Every token is the plain
    implementation's argmax (or within rounding of it)."""
    from flambeau_amd import generate
    d = dirs[("K", dtype)]
    cfg, t = read_model(d)
    prompts = [p for p in rh.make_requests(83, [7, 19, 1, 30, 12], seed=3).values()]
    outs = generate(str(d), prompts, max_new_tokens=10, dtype=dtype, page_size=8, inflight_slots=3, prefill_chunk_tokens=16)
    turned = 0
    for prompt, out in zip(prompts, outs):
        assert len(out) == 10
        toks = list(prompt)
        for tok in out:
            logits = pf.forward(cfg, t, toks)[-1]
            best = int(np.argmax(logits))
            if not (tok == best or logits[best] - logits[tok] < (1e-4 if dtype == "float32" else 3e-2) * np.abs(logits).max()):
                turned += 1
            toks.append(tok)
    assert turned <= (0 if dtype == "float32" else 2), turned


@pytest.mark.parametrize("dtype", DTYPES)
def test_trace_replay_as_a_program(dirs, tmp_path, dtype):
    d = dirs[("M", dtype)]
    reqs = rh.make_requests(150, [40, 70, 97, 33, 64, 12, 90, 55], seed=6)
    ref = reference(d, reqs)
    steps = rh.trace_mixed(reqs, seed=3)
    stats = {}
    got = rh.run_program(d, dtype, steps, tmp_path / "o", rh.peak_tokens(steps), 150, extra=("--poison-cache",), stats=stats)
    assert stats["handed_out"] > stats["pool"]
    close(got, ref, dtype, "trace_run")


def test_the_command_line_serves_it(tmp_path):
    """``random-weights`` -> ``inspect`` -> ``infer --json`` on a Fitevik configuration, greedy in 32-bit with so
    few slots and pages that requests wait and are pre-empted (a pre-empted request starts again from a
    zeroed state): exactly the plain implementation's tokens."""
    import subprocess
    import sys
    cfg = CONFIGS["K"]["config"]
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    d = tmp_path / "model"

    def cli(*args):
        r = subprocess.run([sys.executable, "-m", "flambeau_amd", *map(str, args)], capture_output=True, text=True, timeout=600, cwd=str(rh.ROOT))
        assert r.returncode == 0, f"{args}\n{r.stdout[-2000:]}\n{r.stderr[-4000:]}"
        return r
    cli("random-weights", "--config", tmp_path / "config.json", "--out", d, "--seed", 5, "--std", 0.16, "--gain-std", 0.1, "--dtype", "float32")
    seen = cli("inspect", d).stdout
    assert "architecture: Fitevik" in seen and "tensors fit the model" in seen and "l1.mix.talk" in seen
    prompts = list(rh.make_requests(83, [3, 30, 17], seed=6).values())
    flags = []
    for p in prompts:
        flags += ["--prompt", ",".join(map(str, p))]
    out = json.loads(cli("infer", "--model", d, *flags, "--max-tokens", 18, "--dtype", "float32", "--json", "--inflight-slots", 2,
                         "--paged-kv", 5, "--page-size", 16, "--prefill-chunk-tokens", 16, "--max-queue-depth", 4).stdout)
    conf, t = read_model(d)
    for p, o in zip(prompts, out["outputs"]):
        toks = list(p)
        for tok in o:
            logits = pf.forward(conf, t, toks)[-1]
            best = int(np.argmax(logits))
            assert tok == best or logits[best] - logits[tok] < 1e-4 * np.abs(logits).max()
            toks.append(tok)
        assert len(o) == 18
