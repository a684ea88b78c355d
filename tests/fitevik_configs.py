"""Small Fitevik configurations for the tests, and their random weights.

They differ from one another in every size and option, layer by layer: the order of the two kinds of layers,
one to eight query heads per key/value head, key and value sizes that differ either way and are no multiples
of 8, windows of one key, of a few, across several pages and beyond 256 keys, layers that read the keys and
values of an earlier layer through a narrower, an equal and a wider window, one, some and all experts per
token, layers without a feed-forward, a logit scale that is no power of two or absent, widths and vocabularies
that are no multiples of 8, mixers without a mask."""
import json

import torch

from flambeau_amd.weights import SafetensorsFile, write_random_model, write_safetensors


def hgrn(heads, dim, vdim):
    return {"type": "hgrn2", "mixer": dict(heads=heads, dim=dim, vdim=vdim)}


def att(heads, kv_heads, dim, vdim, scale, window, kv_from=None):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale)
    if window is not None:                  # (None: no mask, every earlier key is seen)
        m["mask"] = {"size": window}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff):
    return {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}


def model(vocab, width, eps, logit_scale, max_positions, layers):
    cfg = {"architecture": "Fitevik", "vocab": vocab, "width": width, "norm": {"eps": eps}, "max_positions": max_positions,
           "layers": [dict(l, mlp=m) for l, m in layers]}
    if logit_scale is not None:
        cfg["logit_scale"] = logit_scale
    return cfg


CONFIGS = {
    # both kinds of layers; three query heads per key/value head; a reader with a wider window than its source; a window
    # beyond 256 keys (single tokens then deal their keys out to several blocks); all experts per token in the last layer
    "K": dict(config=model(83, 40, 1e-5, 0.5, 600, [
        (hgrn(3, 8, 12), dense(24)),
        (att(6, 2, 16, 8, 0.25, 13), moe(5, 2, 16)),
        (att(6, 2, 16, 8, 0.3, 29, kv_from=1), dense(48)),
        (hgrn(1, 20, 6), None),
        (att(4, 4, 12, 20, 0.3, 300), moe(3, 3, 8)),
    ]), seed=3, std=0.16, page_size=8),
    # starts with attention; a window of one key; one expert per token; sizes that are no multiples of 8; two readers
    # of one source (narrower and equal windows); no logit scale in the file
    "L": dict(config=model(61, 36, 3e-4, None, 400, [
        (att(3, 1, 10, 6, 0.35, 1), moe(4, 1, 20)),
        (hgrn(2, 64, 32), dense(20)),
        (att(2, 2, 32, 32, 0.2, 64), None),
        (att(2, 2, 32, 32, 0.15, 17, kv_from=2), dense(28)),
        (att(2, 2, 32, 32, 0.25, 64, kv_from=2), moe(2, 2, 12)),
    ]), seed=11, std=0.2, page_size=16),
    # sizes in steps of 16 and 32, which in bfloat16 run on the matrix cores; eight query heads per key/value head
    "M": dict(config=model(150, 64, 1e-5, 0.3, 512, [
        (hgrn(4, 32, 32), moe(8, 3, 32)),
        (att(8, 1, 32, 32, 0.18, 70), dense(96)),
        (hgrn(2, 16, 64), dense(64)),
        (att(4, 2, 64, 32, 0.12, 33), None),
    ]), seed=21, std=0.12, page_size=16),
    # attention layers only: no mixer advances a state, so steps of single tokens replay captured graphs
    "N": dict(config=model(90, 48, 1e-6, 2.0, 256, [
        (att(4, 2, 16, 16, 0.3, 20), dense(40)),
        (att(4, 2, 16, 16, 0.4, 50, kv_from=0), moe(4, 2, 24)),
        (att(3, 3, 8, 12, 0.5, 9), dense(24)),
    ]), seed=41, std=0.15, page_size=16),
    # mixers without a mask: a reader that sees every key of a source whose own window is narrow, and a layer of its own
    "P": dict(config=model(70, 32, 1e-5, 1.5, 300, [
        (att(4, 2, 16, 16, 0.3, 11), dense(24)),
        (hgrn(2, 8, 8), None),
        (att(4, 2, 16, 16, 0.35, None, kv_from=0), moe(3, 2, 8)),
        (att(2, 1, 8, 24, 0.4, None), dense(16)),
    ]), seed=51, std=0.18, page_size=16),
}

STORE = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def sharpened(config, factor):
    """The configuration with every attention layer's score scale multiplied (queries and keys are normed, so
    scaling a projection would change nothing): softmax becomes peaked and single keys carry the output."""
    cfg = json.loads(json.dumps(config))
    for layer in cfg["layers"]:
        if layer["type"] == "attention":
            layer["mixer"]["scale"] *= factor
    return cfg


def write_model(name, out_dir, store="float32", sharpen=1.0, remember=False, edit=None):
    """The folder of a configuration.  ``sharpen``: see ``sharpened``; ``remember`` makes the recurrent memories
    long (lower bounds of the forget gates next to one); ``edit(tensors)`` changes tensors before they are written."""
    c = CONFIGS[name]
    config = sharpened(c["config"], sharpen) if sharpen != 1.0 else json.loads(json.dumps(c["config"]))
    d = write_random_model(config, out_dir, seed=c["seed"], std=c["std"], gain_std=0.1, store_dtype=STORE[store])
    (d / "config.json").write_text(json.dumps(config, indent=1))       # exactly the keys the design has
    if remember or edit:
        f = SafetensorsFile(d / "model.safetensors")
        tensors = {n: f.read(n) for n in f.names()}
        f.close()
        if remember:
            for n in tensors:
                if n.endswith(".lower"):
                    tensors[n] = torch.full_like(tensors[n], 0.996)
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
