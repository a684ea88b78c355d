"""Small Lenedra configurations for the tests, and their random weights.

They differ from one another in every size and option, layer by layer: the order of the two kinds of layers, the
number of copies of the residual stream (several, one, none: plain sums), one to six query heads per key/value
head, key and value sizes that differ and are no multiples of 8, windows of one key, of a few, across pages and
beyond 256 keys, more kept first tokens than a page or a window holds, one or none, mixers without a mask, chunks of
one position, of a few and beyond 256, convolutions of one to five taps, ranks of the projections of low rank that
differ, routers with and without groups, with all groups kept, with one, two or no identity experts, with one, some
and all experts per token, with and without a shared expert, layers without a feed-forward, a soft cap and an
embedding factor that are absent, widths and vocabularies that are no multiples of 8."""
import json

import torch

from flambeau_amd.weights import SafetensorsFile, write_random_model, write_safetensors


def att(heads, kv_heads, dim, scale, window, keep_first=None):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, scale=scale)
    if window is not None:                  # (None: no mask, every earlier key is seen)
        m["mask"] = {"size": window}
        if keep_first is not None:
            m["mask"]["keep_first"] = keep_first
    return {"type": "attention", "mixer": m}


def pair(left, right, left_scale, right_scale):
    """left: (heads, kv_heads, dim, vdim, scale, chunk or None); right: (heads, kv_heads, dim, vdim, conv, decay_rank, gate_rank)."""
    H, G, D, Dv, scale, chunk = left
    l = dict(heads=H, kv_heads=G, dim=D, vdim=Dv, scale=scale)
    if chunk is not None:
        l["mask"] = {"size": chunk}
    H, G, D, Dv, conv, ra, rg = right
    r = dict(heads=H, kv_heads=G, dim=D, vdim=Dv, conv=conv, decay_rank=ra, gate_rank=rg)
    return {"type": "parallel", "mixer": dict(left=l, right=r, left_scale=left_scale, right_scale=right_scale)}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, identity=None, groups=None, scale=None, shared=None):
    router = {"experts": experts, "top": top}
    if identity is not None:
        router["identity"] = identity
    if groups is not None:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    if scale is not None:
        router["scale"] = scale
    f = {"kind": "moe", "router": router, "expert": {"ff": ff}}
    if shared is not None:
        f["shared"] = {"ff": shared}
    return f


def model(vocab, width, eps, layers, streams=None, embedding_scale=None, softcap=None):
    cfg = {"architecture": "Lenedra", "vocab": vocab, "width": width, "norm": {"eps": eps},
           "layers": [dict(l, mlp=m) for l, m in layers]}
    if streams is not None:
        cfg["streams"] = streams
    if embedding_scale is not None:
        cfg["embedding"] = {"scale": embedding_scale}
    if softcap is not None:
        cfg["logit_softcap"] = softcap
    return cfg


CONFIGS = {
    # three copies of the stream; both kinds of layers; three query heads per key/value head; kept first tokens that fill
    # more than a page of 8; a window beyond 256 keys; two of four groups kept; all experts per token in the last layer
    "E": dict(config=model(83, 40, 1e-5, [
        (att(6, 2, 16, 0.25, 13, 11), dense(24)),
        (pair((4, 2, 8, 12, 0.3, 10), (4, 2, 8, 12, 3, 5, 7), 0.7, 1.2), moe(6, 2, 16, identity=2, groups=(4, 2), scale=1.5, shared=12)),
        (att(3, 3, 10, 0.3, 300, 2), moe(3, 3, 8)),
        (pair((2, 1, 24, 8, 0.2, 290), (3, 1, 20, 6, 1, 3, 3), 1.0, 0.5), None),
        (att(4, 4, 8, 0.35, 29, 40), moe(5, 1, 12, identity=1, groups=(3, 1), shared=20)),
    ], streams=3, embedding_scale=3.0, softcap=9.0), seed=3, std=0.16, page_size=8),
    # one copy of the stream (its numbers still act); starts with a pair; a window of one key; chunks of one position;
    # sizes that are no multiples of 8; no identity experts, no groups, no soft cap, no embedding factor
    "F": dict(config=model(61, 36, 3e-4, [
        (pair((3, 1, 10, 6, 0.35, 1), (2, 2, 12, 10, 5, 4, 9), 0.5, 0.9), moe(4, 1, 20, shared=8)),
        (att(3, 1, 10, 0.35, 1, 0), dense(20)),
        (att(2, 2, 32, 0.2, 64), None),
        (pair((2, 2, 32, 32, 0.15, None), (4, 4, 16, 8, 2, 6, 2), 1.3, 0.4), moe(6, 2, 12, identity=2, groups=(2, 2), scale=0.7)),
    ], streams=1), seed=11, std=0.2, page_size=16),
    # no copies at all: the plain pre-norm layer with its fused norms; sizes in steps of 16 and 32, which in bfloat16 run
    # on the matrix cores; six query heads per key/value head; one kept token
    "G": dict(config=model(150, 64, 1e-5, [
        (att(6, 1, 32, 0.18, 70, 1), moe(8, 3, 32, identity=4, groups=(3, 2), scale=2.0, shared=32)),
        (pair((4, 2, 32, 32, 0.2, 48), (4, 2, 32, 64, 4, 8, 16), 0.6, 1.1), dense(96)),
        (att(4, 2, 64, 0.12, 33, 20), None),
    ], embedding_scale=5.0, softcap=20.0), seed=21, std=0.12, page_size=16),
    # attention layers only: no mixer advances a state, so steps of single tokens replay captured graphs; two copies; a
    # mixer without a mask
    "H": dict(config=model(90, 48, 1e-6, [
        (att(4, 2, 16, 0.3, 20, 5), dense(40)),
        (att(4, 2, 16, 0.4, None), moe(4, 2, 24, identity=2, groups=(2, 1), scale=2.5)),
        (att(3, 3, 8, 0.5, 9, 3), dense(24)),
    ], streams=2, embedding_scale=2.0, softcap=6.0), seed=41, std=0.15, page_size=16),
}

STORE = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def sharpened(config, factor):
    """The configuration with every softmax mixer's score scale multiplied: softmax becomes peaked and single keys
    carry the output."""
    cfg = json.loads(json.dumps(config))
    for layer in cfg["layers"]:
        m = layer["mixer"]
        (m if layer["type"] == "attention" else m["left"])["scale"] *= factor
    return cfg


def write_model(name, out_dir, store="float32", sharpen=1.0, remember=False, edit=None, drop_ranks=False):
    """The folder of a configuration.  ``sharpen``: see ``sharpened``; ``remember`` makes the recurrent memories long
    (decays next to one, weak writes); ``edit(tensors)`` changes tensors before they are written; ``drop_ranks`` leaves
    the ranks of the projections of low rank out of config.json, as a file of the design has it."""
    c = CONFIGS[name]
    config = sharpened(c["config"], sharpen) if sharpen != 1.0 else json.loads(json.dumps(c["config"]))
    d = write_random_model(config, out_dir, seed=c["seed"], std=c["std"], gain_std=0.1, store_dtype=STORE[store])
    if drop_ranks:
        for layer in config["layers"]:
            if layer["type"] == "parallel":
                del layer["mixer"]["right"]["decay_rank"], layer["mixer"]["right"]["gate_rank"]
    (d / "config.json").write_text(json.dumps(config, indent=1))
    if remember or edit:
        f = SafetensorsFile(d / "model.safetensors")
        tensors = {n: f.read(n) for n in f.names()}
        f.close()
        if remember:
            for n in tensors:
                if n.endswith(".A_log"):
                    tensors[n] = torch.full_like(tensors[n], -6.0)
        if edit:
            edit(tensors)
        write_safetensors(d / "model.safetensors", tensors)
    return d


def read_model(model_dir):
    """``(config dictionary, {name: float64 array})`` as the plain implementation takes them."""
    cfg = json.loads((model_dir / "config.json").read_text())
    f = SafetensorsFile(model_dir / "model.safetensors")
    tensors = {n: f.read(n).to(torch.float64).numpy() for n in f.names()}
    f.close()
    return cfg, tensors
