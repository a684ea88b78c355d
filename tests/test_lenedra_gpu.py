"""Lenedra on the GPU against the plain implementation: every mechanism alone, the layers one by one, and whole
models in every cutting (whole prompts, single tokens, portions down to two tokens, mixed batches over a small
poisoned pool whose pages and slots are used again), in 32-bit and in bfloat16, at sizes of the tests' own."""
import json

import numpy as np
import pytest
import torch

import plain_lenedra as pl
import replay_helpers as rh
from lenedra_configs import CONFIGS, read_model, write_model
from test_bugidra_gpu import CUTS, TOL, _x, bound_part, run_mixer, runner_for
from test_kuvidra_gpu import close, make_rt

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = ["float32", "bfloat16"]
TORCH = {"float32": torch.float32, "bfloat16": torch.bfloat16}


@pytest.fixture(scope="module")
def dirs(tmp_path_factory):
    base = tmp_path_factory.mktemp("lenedra")
    out = {}
    for name in CONFIGS:
        for store in DTYPES:
            # (one configuration leaves the ranks of the projections of low rank to the tensors' shapes)
            out[(name, store)] = write_model(name, base / f"{name}-{store}", store, drop_ranks=name == "E")
    for store in DTYPES:          # (weights are stored in the dtype they are run in: the plain side reads the same numbers)
        out[("sharp", store)] = write_model("E", base / f"E-sharp-{store}", store, sharpen=8.0)
        out[("memory", store)] = write_model("E", base / f"E-memory-{store}", store, remember=True)
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
            _refs[key] = pl.forward(cfg, t, toks)
        out[rid] = _refs[key]
    return out


# ---------------------------------------------------------------- each mechanism alone
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("S,W", [(1, 40), (2, 37), (3, 256), (5, 52), (4, 1000), (16, 24)])
def test_hyper_connections_alone(dtype, S, W):
    """The kernels under the stream in S copies against the equations: the copies of the embedding, a sublayer's output
    written into all copies at once, the next sublayer's input with its norm fused or apart, the sum of the copies, and
    picked rows."""
    from flambeau_amd.kernels import ops
    g = torch.Generator().manual_seed(S * 1000 + W)
    n, eps = 19, 2e-5
    x0 = torch.randn(n, W, generator=g) * 2
    t = {"in": torch.randn(S, generator=g), "out": torch.randn(S, generator=g), "mix": torch.eye(S) + 0.3 * torch.randn(S, S, generator=g)}
    t2 = {"in": torch.randn(S, generator=g), "out": torch.randn(S, generator=g), "mix": torch.randn(S, S, generator=g)}
    gain = 1 + 0.2 * torch.randn(W, generator=g)
    y1, y2 = torch.randn(n, W, generator=g), torch.randn(n, W, generator=g)
    dev = lambda v: v.to(DEV).contiguous()
    xs = ops.hyper_spread(dev(x0), torch.empty(n, S * W, device=DEV), S)
    assert torch.equal(xs.view(n, S, W).cpu(), x0[:, None, :].expand(n, S, W))
    # the first sublayer's input: nothing waits to be written
    u = torch.empty(n, W, device=DEV)
    h = torch.empty(n, W, dtype=TORCH[dtype], device=DEV)
    ops.hyper_step(xs, S, in_w=dev(t["in"]), u_out=u, gain=dev(gain), eps=eps, normed=h)
    copies = np.repeat(x0.double().numpy()[None], S, axis=0)                       # [S, n, W] as the plain side keeps them
    want_u = np.tensordot(t["in"].double().numpy(), copies, axes=(0, 0))
    want_h = pl.rms_norm(want_u, gain.double().numpy(), eps)
    tol = 3e-6 if dtype == "float32" else 1e-2
    size = lambda w: np.abs(copies).max() * (1 + float(w.abs().sum()))           # (sums of S terms that cancel: rounding goes with the terms)
    assert np.abs(u.double().cpu().numpy() - want_u).max() < 3e-6 * size(t["in"])
    assert np.abs(h.double().cpu().numpy() - want_h).max() < tol * np.abs(want_h).max() * (1 + S / 4)
    # its output is written while the second sublayer's input is read (one kernel), then the second's alone, then the sum
    ops.hyper_step(xs, S, y=dev(y1), mix=dev(t["mix"]), out_w=dev(t["out"]), in_w=dev(t2["in"]), u_out=u, gain=dev(gain), eps=eps, normed=h)
    plain = {"p.in": t["in"].double().numpy(), "p.out": t["out"].double().numpy(), "p.mix": t["mix"].double().numpy()}
    copies = pl.hyper_sublayer(copies, plain, "p.", np.zeros(W), eps, lambda _: y1.double().numpy())
    assert np.abs(xs.view(n, S, W).double().cpu().numpy().transpose(1, 0, 2) - copies).max() < 3e-6 * S * np.abs(copies).max()
    want_u = np.tensordot(t2["in"].double().numpy(), copies, axes=(0, 0))
    assert np.abs(u.double().cpu().numpy() - want_u).max() < 3e-6 * size(t2["in"])
    assert np.abs(h.double().cpu().numpy() - pl.rms_norm(want_u, gain.double().numpy(), eps)).max() < tol * 4 * (1 + S / 4)
    bias = torch.randn(W, generator=g)                 # (a bias of the sublayer's last product rides in the same kernel)
    ops.hyper_step(xs, S, y=dev(y2), y_bias=dev(bias), mix=dev(t2["mix"]), out_w=dev(t2["out"]))
    plain = {"p.in": t2["in"].double().numpy(), "p.out": t2["out"].double().numpy(), "p.mix": t2["mix"].double().numpy()}
    copies = pl.hyper_sublayer(copies, plain, "p.", np.zeros(W), eps, lambda _: (y2 + bias).double().numpy())
    total = torch.empty(n, W, device=DEV)
    ops.hyper_step(xs, S, in_w=torch.ones(S, device=DEV), u_out=total)
    assert np.abs(total.double().cpu().numpy() - copies.sum(axis=0)).max() < 3e-6 * S * np.abs(copies).max()
    rows = torch.tensor([7, 0, 18], dtype=torch.int32, device=DEV)
    picked = torch.empty(3, W, device=DEV)
    ops.hyper_step(xs, S, in_w=torch.ones(S, device=DEV), u_out=picked, rows=rows)
    assert torch.equal(picked, total[rows.long()])


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_norm_with_its_weight_around_zero_the_scaled_embedding_and_the_capped_head(dtype):
    from flambeau_amd.parts import EMBEDDINGS, HEADS, NORMS, PartSpec
    rt = make_rt(dtype)
    V, W, eps, cap = 23, 44, 1e-5, 2.5
    norm, plain = bound_part(NORMS, PartSpec("rmsnorm", dict(hidden_size=W, eps=eps, unit_offset=True)), dtype, rt, seed=1, prefix="n.")
    x = torch.randn(9, W, generator=torch.Generator().manual_seed(2)) * 3
    out = torch.empty(9, W, dtype=TORCH[dtype], device=DEV)
    norm.forward(x.to(DEV).contiguous(), out)
    want = pl.rms_norm(x.double().numpy(), 1.0 + plain["n"], eps)          # (the stored weight lives around zero)
    assert np.abs(plain["n"]).mean() < 0.5 and np.abs(out.double().cpu().numpy() - want).max() < (3e-6 if dtype == "float32" else 1e-2) * np.abs(want).max()
    emb, pe = bound_part(EMBEDDINGS, PartSpec("scaled_token_embedding", dict(vocab_size=V, hidden_size=W, scale=7.0)), dtype, rt, seed=3, prefix="")
    head, ph = bound_part(HEADS, PartSpec("capped_linear_head", dict(vocab_size=V, hidden_size=W, softcap=cap)), dtype, rt, seed=4, prefix="head.", scale=1.0)
    toks = [5, 0, 22, 5]
    got = emb.forward(torch.tensor(toks, dtype=torch.int32, device=DEV), torch.empty(4, W, device=DEV))
    assert np.abs(got.double().cpu().numpy() - pl.embed(toks, {"embed": pe["weight"]}, 7.0)).max() < 1e-5
    h = _x(6, W, dtype, 5)
    logits = head.forward(h.to(DEV).contiguous(), 6).double().cpu().numpy()
    z = h.double().numpy() @ ph["head"].T
    assert np.abs(z).max() > 2 * cap                                             # the cap bites
    assert np.abs(logits - cap * np.tanh(z / cap)).max() < (1e-5 if dtype == "float32" else 2e-2) * cap
    none = HEADS.create(PartSpec("capped_linear_head", dict(vocab_size=V, hidden_size=W, softcap=None)))
    assert none.softcap is None


def kept_spec(W, H, G, D, window, keep, scale, eps, slope_exponent=8.0):
    from flambeau_amd.parts import PartSpec
    return PartSpec("mixed_heads_attention", dict(hidden_size=W, n_heads=H, n_kv_heads=G, head_dim=D, value_dim=D, window=window,
                                                  keep_first=keep if window else 0, scale=scale, qk_norm="head_gain", eps=eps,
                                                  slope_exponent=slope_exponent, bias=True, out_bias=True, values="keys"))


def mask_dict(window, keep):
    return None if not window else {"size": window, "keep_first": keep}


KEPT_SHAPES = [
    # H, G, D, window, kept first tokens
    (6, 2, 16, 13, 11), (3, 1, 10, 1, 0), (4, 4, 12, 300, 2), (6, 1, 32, 70, 1), (2, 2, 32, 64, 70), (1, 1, 72, 33, 40), (5, 5, 8, 2, 9),
    (16, 4, 64, 100, 33), (4, 2, 24, 0, 0),
    (2, 1, 136, 140, 5),          # heads wider than the matrix-core kernel takes: in bfloat16 the plain kernel, its keys dealt out to parts
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,window,keep", KEPT_SHAPES)
def test_attention_whose_keys_are_its_values_alone(dtype, H, G, D, window, keep):
    """Biased projections, values that are the keys before their norm, the heads' norm with a shared gain, the distance
    bias, the window beside the kept first tokens and the biased output projection against the plain function, whole
    and in portions that cross the window's edge, the kept tokens' edge, page borders and the kernels' chunks."""
    from flambeau_amd.parts import MIXERS
    rt = make_rt(dtype, max_tokens=512)
    W, n, eps, scale = 40, 150 if window < 200 else 420, 2e-5, 0.5 if D < 100 else 0.15
    mixer, plain = bound_part(MIXERS, kept_spec(W, H, G, D, window, keep, scale, eps), dtype, rt, seed=H + D)
    spec = mixer.cache_spec()
    assert (spec.window, spec.keep_first, spec.chunk) == (window, keep if window else 0, 0) and "v.weight" not in mixer.tensors()
    x = _x(n, W, dtype, 5)
    m = dict(heads=H, kv_heads=G, dim=D, scale=scale, mask=mask_dict(window, keep))
    want = pl.attention(x.double().numpy(), m, plain, "m.", eps)
    if window and keep and window + keep < n // 2:                 # the kept tokens matter: without them the late rows differ
        without = pl.attention(x.double().numpy(), dict(m, mask={"size": window}), plain, "m.", eps)
        assert np.abs(want[-1] - without[-1]).max() > 2e-4 * np.abs(want).max()
    cuttings = ([n], [60, 4, 1, 1, 70, 2, 12] + [1] * (n - 150), [1] * 30 + [n - 30]) if n == 150 else ([n], [330, 7, 1, 1] + [1] * 81)
    for cuts in cuttings:
        assert sum(cuts) == n
        got = run_mixer(mixer, rt, x, cuts, n_pages=70)
        assert np.abs(got - want).max() < TOL[dtype] * np.abs(want).max(), cuts[:8]


def chunked_spec(W, H, G, D, Dv, chunk, scale, eps):
    from flambeau_amd.parts import PartSpec
    return PartSpec("mixed_heads_attention", dict(hidden_size=W, n_heads=H, n_kv_heads=G, head_dim=D, value_dim=Dv, chunk=chunk,
                                                  scale=scale, eps=eps, sink=True, bias=True))


CHUNK_SHAPES = [(4, 2, 8, 12, 10), (3, 1, 10, 6, 1), (2, 1, 24, 8, 290), (4, 1, 48, 32, 64), (2, 2, 32, 32, 0), (5, 5, 16, 8, 33), (8, 2, 64, 64, 120),
                (2, 1, 136, 40, 145)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,Dv,chunk", CHUNK_SHAPES)
def test_chunked_attention_with_a_sink_alone(dtype, H, G, D, Dv, chunk):
    """A query sees the earlier keys of its own run of positions, counted from position 0 wherever a portion begins;
    sinks large enough to matter."""
    from flambeau_amd.parts import MIXERS
    rt = make_rt(dtype, max_tokens=512)
    W, n, eps, scale = 40, 150 if chunk < 200 else 420, 1e-5, 0.5 if D < 100 else 0.1          # (wide heads: sums of many products)
    mixer, plain = bound_part(MIXERS, chunked_spec(W, H, G, D, Dv, chunk, scale, eps), dtype, rt, seed=H + Dv, fix={"sink": lambda v: v * 8})
    spec = mixer.cache_spec()
    assert (spec.window, spec.keep_first, spec.chunk) == (0, 0, chunk)
    x = _x(n, W, dtype, 6)
    m = dict(heads=H, kv_heads=G, dim=D, vdim=Dv, scale=scale, mask={"size": chunk} if chunk else None)
    want = pl.chunked_sink_attention(x.double().numpy(), m, plain, "m.")
    flat = pl.chunked_sink_attention(x.double().numpy(), m, dict(plain, **{"m.sink": plain["m.sink"] - 50}), "m.")
    assert np.abs(want - flat).max() > 0.05 * np.abs(want).max()
    cuttings = ([n], [60, 4, 1, 1, 70, 2, 12] + [1] * (n - 150), [1] * 30 + [n - 30]) if n == 150 else ([n], [285, 7, 1, 1] + [1] * 126)
    for cuts in cuttings:
        assert sum(cuts) == n
        got = run_mixer(mixer, rt, x, cuts, n_pages=70)
        assert np.abs(got - want).max() < TOL[dtype] * np.abs(want).max(), cuts[:8]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window,keep,chunk", [(1500, 7, 0), (0, 0, 0), (0, 0, 700)])
def test_long_prompts_whose_keys_are_dealt_out_in_large_parts(dtype, window, keep, chunk):
    """Two thousand tokens: a whole prompt whose tiles do not fill the chip deals its keys out in parts of 512, portions
    and single tokens behind it in parts of 64; the kept first tokens ride with the first part.  Queries far behind the
    window's edge still see the kept tokens, which carry a large share of the weight here."""
    from flambeau_amd.parts import MIXERS
    rt = make_rt(dtype, max_tokens=2048)
    W, n, eps, scale, H, G, D = 40, 2000, 1e-5, 0.5, 4, 2, 32
    if chunk:
        mixer, plain = bound_part(MIXERS, chunked_spec(W, H, G, D, 16, chunk, scale, eps), dtype, rt, seed=3)
    else:
        mixer, plain = bound_part(MIXERS, kept_spec(W, H, G, D, window, keep, scale, eps, slope_exponent=20.0), dtype, rt, seed=3)
    x = _x(n, W, dtype, 4)
    x[:keep] *= 3                                              # (keys that stand out among two thousand)
    h = x.double().numpy()
    if chunk:
        want = pl.chunked_sink_attention(h, dict(heads=H, kv_heads=G, dim=D, vdim=16, scale=scale, mask={"size": chunk}), plain, "m.")
    else:
        orig = pl.distance_slopes
        pl.distance_slopes = lambda H: np.array([2.0 ** (-20.0 * (g + 1) / H) for g in range(H)])
        try:
            m = dict(heads=H, kv_heads=G, dim=D, scale=scale, mask=mask_dict(window, keep))
            want = pl.attention(h, m, plain, "m.", eps)
            if keep:
                without = pl.attention(h, dict(m, mask={"size": window}), plain, "m.", eps)
                assert np.abs(want[-1] - without[-1]).max() > 1e-3 * np.abs(want[-1]).max()
        finally:
            pl.distance_slopes = orig
    for cuts in ([n], [1700, 200, 60, 17] + [1] * 23, [900, 1000, 100]):
        assert sum(cuts) == n
        got = run_mixer(mixer, rt, x, cuts, page_size=16, n_pages=140)
        assert np.abs(got - want).max() < TOL[dtype] * np.abs(want).max(), cuts[:4]


def pointing_weights(H, G, D):
    """Weights under which a query points at ONE key: the model width holds two vectors of G * D values per token; the
    keys read the second, u_i, the queries the first, which the test sets to the u of the key it means."""
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
@pytest.mark.parametrize("window,keep,page", [(13, 3, 8), (64, 20, 16), (300, 1, 16), (1, 9, 8), (129, 40, 32)])
def test_one_key_stands_out_at_the_edges_of_the_window_and_of_the_kept_tokens(dtype, window, keep, page):
    """Every query points at ONE key (its score is some twenty above the others', so it takes nearly all the weight if it
    is seen): the key ``back`` tokens behind it, for the window's last key inside and the first outside, the query's own
    and its neighbour; or the key at a fixed place near the start, the last kept token and the first that is not; in a
    whole prompt, in portions and token by token, over pages of several sizes."""
    from flambeau_amd.parts import MIXERS
    rt = make_rt(dtype, max_tokens=512)
    H, G, D, eps, scale = 4, 2, 32, 1e-6, 0.8
    W, wq, wk = pointing_weights(H, G, D)
    n = max(2 * window + 40, 120) if window < 200 else 420
    gen = torch.Generator().manual_seed(window)
    u = torch.randn(n, G * D, generator=gen)
    one, zero = (lambda v: torch.ones_like(v)), (lambda v: torch.zeros_like(v))
    fix = {"q.weight": lambda v: wq, "k.weight": lambda v: wk, "q_norm.weight": one, "k_norm.weight": one, "q.bias": zero, "k.bias": zero}
    cases = [("back", b) for b in sorted({0, 1, window - 1, window, window + 1, window // 2}) if b >= 0]
    cases += [("at", j) for j in sorted({0, keep - 1, keep, keep + 1}) if j >= 0]
    for kind, k in cases:
        if kind == "back":
            a = torch.roll(u, k, 0)
            a[:k] = torch.randn(k, G * D, generator=gen)                    # (no such key yet)
        else:
            a = u[k].expand(n, G * D).clone()
        x = torch.cat([a, u], dim=1).to(TORCH[dtype])
        # (slopes 2^-4 .. 2^-16: the bias leaves most heads their far keys)
        mixer, plain = bound_part(MIXERS, kept_spec(W, H, G, D, window, keep, scale, eps, slope_exponent=16.0), dtype, rt, seed=5, fix=fix)
        h = x.double().numpy()

        def plain_side(window, keep):
            orig = pl.distance_slopes
            pl.distance_slopes = lambda H: np.array([2.0 ** (-16.0 * (g + 1) / H) for g in range(H)])
            try:
                return pl.attention(h, dict(heads=H, kv_heads=G, dim=D, scale=scale, mask={"size": window, "keep_first": keep}), plain, "m.", eps)
            finally:
                pl.distance_slopes = orig
        want = plain_side(window, keep)
        # the plain side itself turns round when the edge in question moves by one key
        if kind == "back" and k in (window - 1, window) and window > 1 and k >= keep:
            moved = plain_side(window - 1 if k == window - 1 else window + 1, keep)
            assert np.abs(moved[-1] - want[-1]).max() > 0.3 * np.abs(want).max(), (kind, k)
        if kind == "at" and k in (keep - 1, keep) and keep >= 1 and window + keep + 2 < n:
            moved = plain_side(window, keep - 1 if k == keep - 1 else keep + 1)
            assert np.abs(moved[-1] - want[-1]).max() > 0.3 * np.abs(want).max(), (kind, k)
        tail = min(n - 1, window + 20)
        for cuts in ([n], [n - tail] + [1] * tail, [7, 2, 9, 16, 1, 15, 33, 3] + [n - 86 - 30] + [1] * 30):
            assert sum(cuts) == n
            got = run_mixer(mixer, rt, x, cuts, page_size=page, n_pages=n // page + 6)
            err = np.abs(got - want).max(axis=1)
            worst = int(err.argmax())
            assert err[worst] < (1e-4 if dtype == "float32" else 0.1) * np.abs(want).max(), (kind, k, cuts[:3], worst)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("chunk,page", [(10, 8), (64, 16), (290, 16), (1, 8), (33, 32)])
def test_one_key_stands_out_at_the_edges_of_a_chunk(dtype, chunk, page):
    """Every query points at the key ``back`` tokens behind it: seen if both lie in the same run of positions, which
    for one ``back`` holds for some queries and not for others; the sink takes the weight of a query whose key is hidden."""
    from flambeau_amd.parts import MIXERS
    rt = make_rt(dtype, max_tokens=512)
    H, G, D, Dv, eps, scale = 4, 2, 32, 16, 1e-6, 0.8
    W, wq, wk = pointing_weights(H, G, D)
    n = max(3 * chunk + 17, 120) if chunk < 200 else 420
    gen = torch.Generator().manual_seed(chunk)
    u = torch.randn(n, G * D, generator=gen)
    zero = lambda v: torch.zeros_like(v)
    fix = {"q.weight": lambda v: wq, "k.weight": lambda v: wk, "q.bias": zero, "k.bias": zero, "sink": lambda v: v * 3}
    for back in sorted({0, 1, chunk - 1, chunk, chunk // 2, 3}):
        a = torch.roll(u, back, 0)
        a[:back] = torch.randn(back, G * D, generator=gen)
        x = torch.cat([a, u], dim=1).to(TORCH[dtype])
        mixer, plain = bound_part(MIXERS, chunked_spec(W, H, G, D, Dv, chunk, scale * 2, eps), dtype, rt, seed=5, fix=fix)
        m = dict(heads=H, kv_heads=G, dim=D, vdim=Dv, scale=scale * 2)
        want = pl.chunked_sink_attention(x.double().numpy(), dict(m, mask={"size": chunk}), plain, "m.")
        if 0 < back < chunk:                                    # chunks cut one position earlier hide other keys
            moved = pl.chunked_sink_attention(x.double().numpy(), dict(m, mask={"size": chunk + 1}), plain, "m.")
            assert np.abs(moved - want).max() > 0.3 * np.abs(want).max(), back
        tail = min(n - 1, chunk + 20)
        for cuts in ([n], [n - tail] + [1] * tail, [7, 2, 9, 16, 1, 15, 33, 3] + [n - 86 - 30] + [1] * 30):
            assert sum(cuts) == n
            got = run_mixer(mixer, rt, x, cuts, page_size=page, n_pages=n // page + 6)
            err = np.abs(got - want).max(axis=1)
            worst = int(err.argmax())
            assert err[worst] < (1e-4 if dtype == "float32" else 0.1) * np.abs(want).max(), (back, cuts[:3], worst)


def delta_spec(W, H, G, D, Dv, taps, ra, rg, eps):
    from flambeau_amd.parts import PartSpec
    return PartSpec("gated_delta", dict(hidden_size=W, n_heads=H, n_qk_heads=G, head_dim=D, value_dim=Dv, conv_taps=taps, eps=eps,
                                        decay="key_dim", decay_rank=ra, gate_rank=rg, gate="sigmoid"))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,Dv,taps,ra,rg", [(4, 2, 12, 20, 4, 5, 7), (3, 3, 6, 10, 1, 1, 2), (2, 1, 20, 36, 2, 9, 3), (4, 4, 64, 32, 3, 24, 24),
                                               (1, 1, 130, 17, 5, 6, 40), (4, 4, 32, 64, 4, 24, 24)])
def test_delta_rule_with_a_decay_per_key_dim_alone(dtype, H, G, D, Dv, taps, ra, rg):
    """Convolutions, unit vectors, a decay per head and key dim and an output gate through projections of low rank, the
    recurrence and the heads' norm against the plain function; in 32-bit no bit depends on the cutting."""
    from flambeau_amd.parts import MIXERS
    rt = make_rt(dtype)
    W, n, eps = 40, 90, 1e-5
    fix = {"A_log": lambda v: v * 3 - 1.0, "dt_bias": lambda v: v * 3, "a2.weight": lambda v: v * 4}
    mixer, plain = bound_part(MIXERS, delta_spec(W, H, G, D, Dv, taps, ra, rg, eps), dtype, rt, seed=D, fix=fix)
    x = _x(n, W, dtype, 8)
    m = dict(heads=H, kv_heads=G, dim=D, vdim=Dv, conv=taps)
    want = pl.gated_delta_rule(x.double().numpy(), m, plain, "m.", eps)
    # the decays differ between the key dims of a head: with their mean in every dim the output is another
    flat = dict(plain)
    flat["m.a2"] = np.repeat(plain["m.a2"].reshape(H, D, ra).mean(axis=1, keepdims=True), D, axis=1).reshape(H * D, ra)
    assert np.abs(pl.gated_delta_rule(x.double().numpy(), m, flat, "m.", eps) - want).max() > 1e-2 * np.abs(want).max()
    results = [run_mixer(mixer, rt, x, cuts) for cuts in CUTS]
    for got in results:
        assert np.abs(got - want).max() < (5e-5 if dtype == "float32" else 5e-2) * np.abs(want).max()
    if dtype == "float32":
        assert np.array_equal(results[0], results[1]) and np.array_equal(results[0], results[2])


@pytest.mark.parametrize("dtype", DTYPES)
def test_two_mixers_side_by_side_with_a_factor_each(dtype):
    from flambeau_amd.parts import MIXERS, PartSpec
    rt = make_rt(dtype)
    W, n, eps = 40, 90, 1e-4
    left = dict(heads=6, kv_heads=3, dim=16, vdim=8, scale=0.5, mask={"size": 21})
    right = dict(heads=3, kv_heads=1, dim=8, vdim=12, conv=3)
    spec = PartSpec("side_by_side", dict(hidden_size=W, left=chunked_spec(W, 6, 3, 16, 8, 21, 0.5, eps), right=delta_spec(W, 3, 1, 8, 12, 3, 4, 6, eps),
                                         factors=(0.3, 1.7), normed=False))
    mixer, plain = bound_part(MIXERS, spec, dtype, rt, seed=3)
    assert "left_out.weight" not in mixer.tensors()
    x = _x(n, W, dtype, 9)
    want = pl.parallel(x.double().numpy(), dict(left=left, right=right, left_scale=0.3, right_scale=1.7), plain, "m.", eps)
    for cuts in CUTS:
        got = run_mixer(mixer, rt, x, cuts)
        assert np.abs(got - want).max() < (3e-5 if dtype == "float32" else 4e-2) * np.abs(want).max(), cuts


ROUTERS = [
    # experts, identity, top, groups, kept groups, scale
    (6, 2, 2, 4, 2, 1.5), (12, 2, 3, 2, 1, 2.5), (5, 1, 1, 3, 1, 1.0), (8, 4, 3, 3, 2, 2.0), (3, 0, 3, 1, 1, 1.0), (6, 2, 2, 2, 2, 0.7),
    (70, 10, 4, 8, 3, 1.0), (4, 0, 1, 4, 1, 3.0),
]


@pytest.mark.parametrize("E,ident,top,groups,keep,scale", ROUTERS)
def test_the_router_alone(E, ident, top, groups, keep, scale):
    """The picks and weights of the grouped router against the plain function: corrections large enough to turn the
    choice round (and negative, so that a choice score of 0 would beat what a kept group holds), groups, identity
    experts; every (token, expert) pair has its place in exactly one tile of its expert."""
    from flambeau_amd.kernels import ops
    n, N = 97, E + ident
    g = torch.Generator().manual_seed(E * 10 + top)
    z = torch.randn(n, N, generator=g) * 2
    corr = torch.randn(N, generator=g) * 0.3 - 0.8
    P = n * top
    i32 = lambda k, *s: torch.empty(k, *s, dtype=torch.int32, device=DEV)
    place, src_row, tiles = i32(P), i32(P), i32(ops.moe_max_tiles(P, N), 4)
    src_scale, pair_w = torch.empty(P, device=DEV), torch.empty(P, device=DEV)
    ops.moe_route_grouped(z.to(DEV), 0, N, ident, top, corr.to(DEV), groups, keep, scale, place, src_row, src_scale, pair_w, tiles)
    chosen, w = pl.route(z.double().numpy(), corr.double().numpy(), top, groups, keep, scale)
    plain_choice = pl.route(z.double().numpy(), np.zeros(N), top, groups, keep, scale)[0]
    assert top == N or (np.sort(plain_choice, axis=1) != np.sort(chosen, axis=1)).any()            # the correction matters
    if groups > keep and top > keep:                     # (the best `keep` outputs always lie in the best `keep` groups)
        free = pl.route(z.double().numpy(), corr.double().numpy(), top, 1, 1, scale)[0]
        assert (np.sort(free, axis=1) != np.sort(chosen, axis=1)).any()                # and so do the groups
    expert_of = np.full(P, -7)
    for e, p0, m, flag in tiles.cpu().numpy():
        if m > 0:
            assert (expert_of[p0:p0 + m] == -7).all() and (flag == 1) == (e < 0)
            expert_of[p0:p0 + m] = e if flag == 0 else -1                               # (-1: an identity expert's tile)
    assert (expert_of != -7).all()
    place, src_row, src_scale = place.cpu().numpy(), src_row.cpu().numpy(), src_scale.cpu().numpy()
    for t in range(n):
        mine = sorted((int(expert_of[place[t * top + k]]), float(src_scale[place[t * top + k]])) for k in range(top))
        ref = sorted((int(e) if e < E else -1, float(x)) for e, x in zip(chosen[t], w[t]))
        assert [a for a, _ in mine] == [a for a, _ in ref], t
        assert max(abs(a - b) for (_, a), (_, b) in zip(mine, ref)) < 5e-6 * scale, t
        assert all(src_row[place[t * top + k]] == t for k in range(top))


def experts_spec(W, f):
    from flambeau_amd.parts import PartSpec
    r = f["router"]
    g = r.get("groups") or {"count": 1, "keep": 1}
    return PartSpec("routed_experts", dict(hidden_size=W, n_experts=r["experts"], top=r["top"], expert_size=f["expert"]["ff"],
                                           shared_size=(f.get("shared") or {}).get("ff"), shared_gate=False, scoring="softmax_grouped",
                                           weight_on="output", correction=True, n_groups=g["count"], keep_groups=g["keep"],
                                           n_identity=r.get("identity", 0), weight_scale=r.get("scale", 1.0)))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n,W,f", [
    (37, 40, dict(kind="moe", router=dict(experts=6, identity=2, top=2, groups=dict(count=4, keep=2), scale=1.5), expert=dict(ff=16), shared=dict(ff=12))),
    (150, 64, dict(kind="moe", router=dict(experts=8, identity=4, top=3, groups=dict(count=3, keep=2), scale=2.0), expert=dict(ff=32), shared=dict(ff=32))),
    (5, 36, dict(kind="moe", router=dict(experts=4, top=1), expert=dict(ff=20))),
    (64, 48, dict(kind="moe", router=dict(experts=3, identity=1, top=4), expert=dict(ff=24), shared=dict(ff=8))),
])
def test_experts_with_identity_experts_and_a_shared_expert_alone(dtype, n, W, f):
    from flambeau_amd.parts import FEED_FORWARDS
    rt = make_rt(dtype)
    part, plain = bound_part(FEED_FORWARDS, experts_spec(W, f), dtype, rt, seed=n, prefix="f.", fix={"correction": lambda v: v * 0.3})
    x = _x(n, W, dtype, 3)
    h = x.double().numpy()
    want = pl.experts_ff(h, f, plain, "f.")
    got = part.forward(x.to(DEV).contiguous(), None).double().cpu().numpy()
    # rows whose last chosen and first left-out choice scores are a rounding apart may turn either way: leave them out
    r = f["router"]
    z = h @ plain["f.router"].T
    e = np.exp(z - z.max(axis=1, keepdims=True))
    c = np.sort(e / e.sum(axis=1, keepdims=True) + plain["f.correction"], axis=1)[:, ::-1]
    sure = np.ones(n, dtype=bool) if r["top"] >= z.shape[1] else (c[:, r["top"] - 1] - c[:, r["top"]]) > (1e-5 if dtype == "float32" else 1e-2)
    assert sure.sum() > 0.4 * n
    assert np.abs(got - want)[sure].max() < (3e-5 if dtype == "float32" else 4e-2) * np.abs(want).max()
    if r.get("identity"):                                  # identity experts carry weight: without them the output differs
        chosen, _ = pl.route(z, plain["f.correction"], r["top"], (r.get("groups") or {"count": 1})["count"], (r.get("groups") or {"keep": 1})["keep"], 1.0)
        assert (chosen >= r["experts"]).any()


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
    want = []
    pl.forward(cfg, t, toks, layer_outputs=want)
    assert len(seen) == len(want)
    for i, (g, w) in enumerate(zip(seen, want)):
        err = np.abs(g - w).max(axis=1) / np.abs(w).max()
        if dtype == "float32":
            assert err.max() < 2e-5, f"layer {i}"
        else:               # (a token whose choice of experts is a close call may turn the other way in bfloat16, and is then far off)
            assert np.median(err) < 5e-2 and (err > 1e-1).mean() <= 0.2, f"layer {i}"


# ---------------------------------------------------------------- whole models in every cutting
LENGTHS = {"E": [40, 70, 97, 1, 33, 64, 2, 90, 340, 128, 21], "F": [97, 1, 150, 64, 31, 2, 120, 17, 65],
           "G": [150, 64, 3, 65, 1, 200, 31, 90], "H": [40, 100, 7, 64, 130, 2, 55]}


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
    """A model of attention layers alone captures its decode steps (padded to a bucket: rows without pages ride along);
    one with a recurrent layer never does.  Both give the plain logits."""
    from flambeau_amd.engine import StepEntry
    d = dirs[("H", dtype)]
    reqs = rh.make_requests(90, [20, 33, 5], seed=12)
    ref = reference(d, reqs)
    runner = runner_for(d, dtype, n_pages=24, page_size=16, max_tokens=256)
    assert runner.decode_graphs
    assert not runner_for(dirs[("E", dtype)], dtype, n_pages=24, page_size=8).decode_graphs
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
    """Unequal requests in one step against each alone: in 32-bit not a bit differs, whatever the neighbours, pages
    and slots are."""
    from flambeau_amd.engine import StepEntry
    d = dirs[("E", "float32")]
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
    """Score scales eight times as large: softmax puts nearly all weight on single keys, hundreds of tokens back, among
    the kept first tokens or next to a page's, a window's or a chunk's edge alike, so one key lost or one too many shows
    in the logits."""
    d = dirs[("sharp", dtype)]
    reqs = rh.make_requests(83, [380, 131], seed=2)
    ref = reference(d, reqs)
    blunt = reference(dirs[("E", dtype)], reqs)
    assert np.abs(ref["r0"] - blunt["r0"]).max() > 0.05 * np.abs(ref["r0"]).max()
    for mode, steps in [("whole", rh.trace_whole(reqs)), ("tail", rh.trace_tail(reqs, tail=40)),
                        ("portions", rh.trace_portions(reqs, sizes=(7, 2, 8, 9, 16, 1, 15, 33, 3)))]:
        runner = runner_for(d, dtype, n_pages=64, page_size=8)
        close(rh.run_in_process(runner, steps), ref, dtype, f"sharp {mode}", bf16=8e-2)


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_memory_and_long_decoding(dirs, dtype):
    """Decays next to one: the first tokens stay in the memories for hundreds of steps (the plain logits at the end
    change when the first token does), through 340 single-token steps, during which the widest window (300 keys) and
    the chunks of 10 and of 290 positions pass over decoded tokens and the pages behind them are given back, all but
    those of the kept first tokens."""
    d = dirs[("memory", dtype)]
    toks = rh.make_requests(83, [397], seed=4)["r0"]
    reqs = {"r0": toks}
    ref = reference(d, reqs)
    other = reference(d, {"r0": [(toks[0] + 1) % 83] + toks[1:]})
    assert np.abs(ref["r0"][-1] - other["r0"][-1]).max() > 1e-3 * np.abs(ref["r0"]).max()
    runner = runner_for(d, dtype, n_pages=56, page_size=8)
    steps = rh.trace_tail(reqs, tail=340)
    from flambeau_amd.engine import StepEntry
    got = rh.run_in_process(runner, [dict(s, end=[]) for s in steps])              # (the request stays live: what does it still hold?)
    held = {g: [b for b, p in enumerate(runner.manager.table_row("r0", g)) if p >= 0] for g in range(len(runner.manager.groups))}
    for g, spec in enumerate(runner.manager.groups):
        if spec.window and spec.keep_first:                 # the kept tokens' pages are still there, the rest of the start is not
            kept_blocks = -(-spec.keep_first // 8)
            assert held[g][:kept_blocks] == list(range(kept_blocks)) and held[g][kept_blocks] >= (397 - spec.window) // 8, (g, held[g][:8])
        elif spec.chunk:
            assert held[g][0] == (397 - 397 % spec.chunk) // 8, (g, held[g][:4])
    runner.end("r0")
    close(got, ref, dtype, "memory")


@pytest.mark.parametrize("dtype", DTYPES)
def test_first_tokens(dirs, dtype):
    """Requests of one and two tokens, alone, side by side, and continued one token at a time: the first token sees itself
    and the sink, writes into an empty memory, and its convolutions see zeros before it."""
    d = dirs[("E", dtype)]
    reqs = rh.make_requests(83, [1, 2, 1, 3], seed=7)
    ref = reference(d, reqs)
    steps = [dict(entries=[dict(id=rid, tokens=toks[:1], want=[0]) for rid, toks in reqs.items()], end=["r0", "r2"]),
             dict(entries=[dict(id="r1", tokens=reqs["r1"][1:], want=[0]), dict(id="r3", tokens=reqs["r3"][1:2], want=[0])], end=["r1"]),
             dict(entries=[dict(id="r3", tokens=reqs["r3"][2:], want=[0])], end=["r3"])]
    close(rh.run_in_process(runner_for(d, dtype, n_pages=8, page_size=8), steps), ref, dtype, "first tokens")


def test_a_slot_that_is_used_again_starts_from_zero(dirs):
    """One state slot: every request inherits the slot of the one before, whose memories and kept inputs are not zero,
    and still gives the plain logits."""
    d = dirs[("F", "float32")]
    reqs = rh.make_requests(61, [30, 9, 1, 44], seed=8)
    ref = reference(d, reqs)
    runner = runner_for(d, "float32", n_pages=8, page_size=16, slots=1)
    close(rh.run_in_process(runner, rh.trace_portions(reqs, sizes=(5, 2, 11))), ref, "float32", "one slot")


# ---------------------------------------------------------------- through the entry points
@pytest.mark.parametrize("dtype", DTYPES)
def test_greedy_generation_through_the_engine(dirs, dtype):
    """``generate``: scheduler, portions, batching, device sampler.  Every token is the plain implementation's argmax
    (or within rounding of it)."""
    from flambeau_amd import generate
    d = dirs[("E", dtype)]
    cfg, t = read_model(d)
    prompts = [p for p in rh.make_requests(83, [7, 19, 1, 30, 12], seed=3).values()]
    outs = generate(str(d), prompts, max_new_tokens=10, dtype=dtype, page_size=8, inflight_slots=3, prefill_chunk_tokens=16)
    turned = 0
    for prompt, out in zip(prompts, outs):
        assert len(out) == 10
        toks = list(prompt)
        for tok in out:
            logits = pl.forward(cfg, t, toks)[-1]
            best = int(np.argmax(logits))
            if not (tok == best or logits[best] - logits[tok] < (1e-4 if dtype == "float32" else 3e-2) * np.abs(logits).max()):
                turned += 1
            toks.append(tok)
    assert turned <= (0 if dtype == "float32" else 2), turned


@pytest.mark.parametrize("dtype", DTYPES)
def test_trace_replay_as_a_program(dirs, tmp_path, dtype):
    d = dirs[("G", dtype)]
    reqs = rh.make_requests(150, [40, 70, 97, 33, 64, 12, 90, 55], seed=6)
    ref = reference(d, reqs)
    steps = rh.trace_mixed(reqs, seed=3)
    stats = {}
    got = rh.run_program(d, dtype, steps, tmp_path / "o", rh.peak_tokens(steps), 150, extra=("--poison-cache",), stats=stats)
    assert stats["handed_out"] > stats["pool"]
    close(got, ref, dtype, "trace_run")


def test_the_command_line_serves_it(tmp_path):
    """``random-weights`` -> ``inspect`` -> ``infer --json`` on a Lenedra configuration, greedy in 32-bit with so few
    slots and pages that requests wait and are pre-empted (a pre-empted request starts again from a zeroed state): exactly
    the plain implementation's tokens."""
    import subprocess
    import sys
    cfg = CONFIGS["E"]["config"]
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    d = tmp_path / "model"

    def cli(*args):
        r = subprocess.run([sys.executable, "-m", "flambeau_amd", *map(str, args)], capture_output=True, text=True, timeout=600, cwd=str(rh.ROOT))
        assert r.returncode == 0, f"{args}\n{r.stdout[-2000:]}\n{r.stderr[-4000:]}"
        return r
    cli("random-weights", "--config", tmp_path / "config.json", "--out", d, "--seed", 5, "--std", 0.16, "--gain-std", 0.1, "--dtype", "float32")
    seen = cli("inspect", d).stdout
    assert "architecture: Lenedra" in seen and "tensors fit the model" in seen and "l1.hc2.mix" in seen and "l1.mix.right.a2" in seen
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
            logits = pl.forward(conf, t, toks)[-1]
            best = int(np.argmax(logits))
            assert tok == best or logits[best] - logits[tok] < 1e-4 * np.abs(logits).max()
            toks.append(tok)
        assert len(o) == 18
