"""Small Bikovik configurations and weights for the tests.  The configurations differ from each
other in every size and option: numbers of heads (also one that no power of two divides, and as
many key/value heads as query heads), key and value sizes (also equal ones, and ones that are no
multiple of 16), rotated dimensions (part of the head, all of it), windows (shorter and longer
than the sequences), kept first tokens (none, some), value mixing (none, a source alone, a source
and two mixers), layers without a feed-forward, the order of the layers, and the constants."""

from __future__ import annotations

import json

import torch


def attention(heads, kv_heads, dim, vdim, window, keep_first, rot, scale, v_mix, base=10000.0):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
             "mask": {"size": window, "keep_first": keep_first}, "rot": {"dims": rot, "base": base}}
    if v_mix:
        mixer["v_mix"] = True
    return {"type": "attention", "mixer": mixer}


def hgrn2(heads, dim, vdim):
    return {"type": "hgrn2", "mixer": {"heads": heads, "dim": dim, "vdim": vdim}}


def retention(heads, dim, vdim, rot, decay, base=10000.0):
    return {"type": "retention", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay,
                                           "rot": {"dims": rot, "base": base}}}


def with_mlp(layer, ff, limit):
    return dict(layer, mlp=None if ff is None else {"kind": "dense", "ff": ff, "limit": limit})


def config(width, vocab, layers, scale=4.0, softcap=20.0, eps=1e-5):
    return {"architecture": "Bikovik", "vocab": vocab, "width": width, "embedding": {"scale": scale},
            "norm": {"eps": eps}, "logit_softcap": softcap, "layers": layers}


CASES = {
    # every mixer, a window shorter than the sequences that keeps three first tokens, a source and a mixer of values
    "A": dict(page_size=8, raw=config(64, 128, [
        with_mlp(hgrn2(2, 16, 32), 96, 2.0),
        with_mlp(attention(4, 2, 32, 16, window=24, keep_first=3, rot=8, scale=0.25, v_mix=True), 96, 2.0),
        with_mlp(retention(2, 32, 16, rot=32, decay=[0.9, 0.99]), 96, 2.0),
        with_mlp(attention(4, 2, 32, 16, window=24, keep_first=3, rot=8, scale=0.25, v_mix=True), 96, 2.0),
    ])),
    # other sizes everywhere: six and three heads, sizes that are no multiples of 16, rotation over the whole head,
    # no kept tokens, a window longer than any sequence with kept tokens that then never matter, a layer without
    # feed-forward, one head, attention first
    "B": dict(page_size=16, raw=config(96, 200, [
        with_mlp(attention(6, 3, 48, 24, window=40, keep_first=0, rot=48, scale=0.1, v_mix=False, base=500.0), 160, 0.7),
        with_mlp(retention(3, 24, 40, rot=12, decay=[0.8, 0.95, 0.999]), None, None),
        with_mlp(hgrn2(1, 40, 24), 160, 0.7),
        with_mlp(attention(3, 1, 24, 40, window=1000, keep_first=5, rot=8, scale=0.3, v_mix=True), 64, 1.5),
    ], scale=1.0, softcap=8.0, eps=1e-6)),
    # as many key/value heads as query heads, keys as large as values, a source of values and two mixers, a window
    # of one page, kept tokens beyond the first page
    "C": dict(page_size=8, raw=config(32, 64, [
        with_mlp(attention(2, 2, 16, 16, window=8, keep_first=10, rot=16, scale=0.5, v_mix=True), 48, 1.0),
        with_mlp(attention(2, 2, 16, 16, window=8, keep_first=10, rot=16, scale=0.5, v_mix=True), None, None),
        with_mlp(attention(2, 2, 16, 16, window=8, keep_first=10, rot=16, scale=0.5, v_mix=True), 48, 1.0),
    ], scale=2.0, softcap=5.0)),
}

SINGLE = {
    "attention": dict(page_size=8, raw=config(64, 96, [
        with_mlp(attention(4, 2, 32, 16, window=20, keep_first=2, rot=16, scale=0.2, v_mix=False), None, None)])),
    "hgrn2": dict(page_size=8, raw=config(64, 96, [with_mlp(hgrn2(2, 24, 40), None, None)])),
    "retention": dict(page_size=8, raw=config(64, 96, [
        with_mlp(retention(2, 24, 40, rot=8, decay=[0.7, 0.97]), None, None)])),
}


def make_tensors(raw: dict, seed: int, sharpen: float = 1.0, spread: float = 1.0) -> dict:
    """Random bfloat16 weights for ``raw`` through the package's seeded random-weights mode, then:
    query weights and biases of the attention layers times ``sharpen`` (peaked attention shows a
    wrong key), all matrices times ``spread``."""
    from lockstep_amd.config import config_from_dict
    from lockstep_amd.weights import random_tensors

    cfg = config_from_dict(raw)
    tensors = random_tensors(cfg, seed, std=0.08 * spread, norm_std=0.2, dtype=torch.bfloat16)
    for i, layer in enumerate(raw["layers"]):
        if layer["type"] == "attention" and sharpen != 1.0:
            for name in (f"l{i}.mix.q", f"l{i}.mix.q.b"):
                tensors[name] = (tensors[name].float() * sharpen).to(torch.bfloat16)
    return tensors


def write_model(folder, raw: dict, tensors: dict):
    from lockstep_amd.weights import save_file

    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(raw))
    save_file(tensors, folder / "model.safetensors")
    return folder
