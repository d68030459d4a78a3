"""Small Biberax configurations and weights for the tests.  The configurations differ from each
other in every size and option: numbers of heads (also as many key/value heads as query heads, one
key/value head, a group of sixteen and more heads), key and value sizes (equal and unequal, also no
multiples of 16 or of 8), rotated dimensions (part of the head, all of it, none), frequency scaling (with
all three ranges in use, and none), chunks (shorter than a page, no multiple of a page or a tile,
longer than any sequence, none), bias tables of several sizes with a farthest distance inside and
beyond the sequences, experts (one chosen, several, all), layers without a feed-forward or without a
shared expert, and the order of the layers."""

from __future__ import annotations

import json

import torch


def rotary(heads, kv_heads, dim, vdim, chunk, rot, scale, base=10000.0, scaling=None):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if chunk:
        mixer["mask"] = {"size": chunk}
    if rot:
        mixer["rot"] = {"dims": rot, "base": base}
        if scaling:
            mixer["rot"]["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return {"type": "attention", "mixer": mixer}


def biased(heads, kv_heads, dim, farthest, rows, scale):
    return {"type": "attention_2", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim,
                                             "scale": scale, "bias_max": farthest, "bias_rows": rows}}


def dense(layer, ff):
    return dict(layer, mlp={"kind": "dense", "ff": ff})


def routed(layer, ff, limit, experts, top, shared=None):
    mlp = {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top}}
    if shared:
        mlp["shared"] = {"ff": shared[0], "limit": shared[1]}
    return dict(layer, mlp=mlp)


def bare(layer):
    return dict(layer, mlp=None)


def config(width, vocab, layers, eps=1e-5):
    return {"architecture": "Biberax", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}


CASES = {
    # both mixers and both feed-forwards; a chunk of 24 on pages of 8; a bias table of 12 rows that ends inside the
    # sequences; scaled frequencies whose three ranges are all in use
    "A": dict(page_size=8, raw=config(64, 128, [
        dense(rotary(4, 2, 32, 16, chunk=24, rot=16, scale=0.25, base=100.0, scaling=(8.0, 1.0, 4.0, 64)), 96),
        routed(biased(4, 2, 24, farthest=60, rows=12, scale=0.2), 32, 2.0, experts=6, top=2, shared=(40, 1.0)),
        routed(rotary(4, 2, 32, 16, chunk=24, rot=16, scale=0.25, base=100.0, scaling=(8.0, 1.0, 4.0, 64)), 32, 2.0,
               experts=6, top=2, shared=(40, 1.0)),
    ])),
    # other sizes everywhere: the biased mixer first, six heads over three and over one, sizes that are no multiple
    # of 16, a chunk that is no multiple of a page or of a key tile, rotation of the whole head without scaling, a
    # farthest distance beyond the sequences, one expert a token and no shared expert, a layer without feed-forward
    "B": dict(page_size=16, raw=config(96, 200, [
        routed(biased(6, 3, 40, farthest=5000, rows=20, scale=0.15), 24, 0.7, experts=5, top=1),
        bare(rotary(6, 1, 40, 40, chunk=37, rot=40, scale=0.1, base=500.0)),
        dense(rotary(3, 3, 24, 24, chunk=1000, rot=8, scale=0.3), 160),
        routed(biased(6, 3, 40, farthest=90, rows=6, scale=0.15), 48, 1.5, experts=3, top=3, shared=(24, 3.0)),
    ], eps=1e-6)),
    # as many key/value heads as query heads, no chunks and no rotation (plain causal attention with a one in the
    # denominator), a chunk shorter than a page, a group of sixteen heads on one key/value head
    "C": dict(page_size=16, raw=config(32, 64, [
        dense(rotary(2, 2, 16, 16, chunk=None, rot=0, scale=0.5), 48),
        routed(rotary(2, 2, 16, 16, chunk=5, rot=16, scale=0.5, scaling=(2.0, 1.0, 2.0, 16)), 16, 1.0, experts=4, top=2,
               shared=(16, 0.5)),
        bare(biased(16, 1, 16, farthest=16, rows=8, scale=0.25)),
    ])),
    # key sizes that are no multiple of eight (padded in the cache), value sizes that are no multiple of four, three
    # query heads on one key/value head, a chunk of eleven, two rows in a bias table
    "D": dict(page_size=8, raw=config(48, 80, [
        routed(rotary(3, 1, 20, 6, chunk=11, rot=10, scale=0.2, base=50.0), 12, 1.0, experts=9, top=4, shared=(20, 2.0)),
        dense(biased(4, 2, 12, farthest=7, rows=2, scale=0.3), 56),
    ])),
}

SINGLE = {
    "rotary": dict(page_size=8, raw=config(64, 96, [
        bare(rotary(4, 2, 32, 16, chunk=20, rot=16, scale=0.2, scaling=(4.0, 1.0, 4.0, 32)))])),
    "biased": dict(page_size=8, raw=config(64, 96, [bare(biased(4, 2, 24, farthest=50, rows=10, scale=0.2))])),
    "dense": dict(page_size=8, raw=config(64, 96, [dense(rotary(2, 1, 16, 16, chunk=None, rot=0, scale=0.25), 72)])),
    "routed": dict(page_size=8, raw=config(64, 96, [
        routed(rotary(2, 1, 16, 16, chunk=None, rot=0, scale=0.25), 40, 1.2, experts=7, top=3, shared=(24, 0.8))])),
}


def make_tensors(raw: dict, seed: int, sharpen: float = 1.0, spread: float = 1.0) -> dict:
    """Random bfloat16 weights for ``raw`` through the package's seeded random-weights mode, then:
    query weights and biases of the mixers times ``sharpen`` (peaked attention shows a wrong key), all
    matrices times ``spread``; bias tables, sinks and router biases are drawn wide enough to matter."""
    from lockstep_amd.config import config_from_dict
    from lockstep_amd.weights import random_tensors

    cfg = config_from_dict(raw)
    tensors = random_tensors(cfg, seed, std=0.08 * spread, norm_std=0.2, dtype=torch.bfloat16)
    g = torch.Generator().manual_seed(seed + 1000)
    for i, layer in enumerate(raw["layers"]):
        if sharpen != 1.0:
            for name in (f"l{i}.mix.q", f"l{i}.mix.q.b"):
                if name in tensors:
                    tensors[name] = (tensors[name].float() * sharpen).to(torch.bfloat16)
        for name, width in ((f"l{i}.mix.rel", 1.0), (f"l{i}.mix.sink", 1.5), (f"l{i}.mlp.router.b", 0.3)):
            if name in tensors:
                tensors[name] = (torch.randn(tensors[name].shape, generator=g) * width).to(torch.bfloat16)
        if f"l{i}.mlp.router" in tensors:       # routers that decide clearly: no close calls between experts
            tensors[f"l{i}.mlp.router"] = (tensors[f"l{i}.mlp.router"].float() * 6.0).to(torch.bfloat16)
    return tensors


def write_model(folder, raw: dict, tensors: dict):
    from lockstep_amd.weights import save_file

    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(raw))
    save_file(tensors, folder / "model.safetensors")
    return folder
