"""Bikovik: a decoder whose layers each name their own mixer -- talking-heads attention over a
sliding window that keeps the first tokens, HGRN2 or retention -- between Dynamic Tanh norms, with
a clamped gated feed-forward (or none), a scaled embedding and soft-capped logits.

``config.json`` is nested: ``architecture`` (the name), ``vocab``, ``width``, ``embedding.scale``,
``norm.eps``, ``logit_softcap`` and ``layers``, a list whose entries give ``type`` (``attention``,
``hgrn2``, ``retention``), the mixer's sizes and constants under ``mixer`` and the feed-forward
under ``mlp`` (``kind``, ``ff``, ``limit``; null for a layer without one).  Layer ``i``'s tensors
start with ``l<i>.``: ``norm1``, ``norm2`` (each with ``.b`` and ``.alpha``), ``mix.*``, ``mlp.*``;
beside them ``embed``, ``final.norm`` and ``head``.  ``model_spec`` states all of this as parts.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any

from .base import ConfigError, LayerSpec, ModelConfig, ModelSpec, PartSpec, ScheduleEntry
from .registry import register_architecture

#: the slope of the sigmoid in the gated feed-forward, fixed by the design
GATE_SLOPE = 1.702


def _need(mapping, key: str, where: str):
    if not isinstance(mapping, dict) or key not in mapping:
        raise ConfigError(f"config.json: {where} lacks the key {key!r}")
    return mapping[key]


def _positive_int(value, what: str) -> int:
    if not isinstance(value, int) or isinstance(value, bool) or value <= 0:
        raise ConfigError(f"{what} must be a positive integer, got {value!r}")
    return value


@register_architecture
@dataclass(frozen=True)
class BikovikConfig(ModelConfig):
    architecture: str
    vocab: int
    width: int
    embedding: Any
    norm: Any
    logit_softcap: float
    layers: Any

    architecture_names = ("Bikovik", "bikovik")

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_dict(cls, raw) -> "BikovikConfig":
        # what the file does not mention does not exist: no soft cap, an embedding as stored
        raw = dict(raw)
        raw.setdefault("logit_softcap", None)
        raw.setdefault("embedding", {"scale": 1.0})
        return super().from_dict(raw)

    def to_dict(self) -> dict:
        return {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                "embedding": dict(self.embedding), "norm": dict(self.norm), "logit_softcap": self.logit_softcap,
                "layers": [dict(layer) for layer in self.layers]}

    def init_scheme(self):
        return {"std": 0.05, "norm_std": 0.1}

    def validate(self) -> None:
        _positive_int(self.vocab, "vocab")
        _positive_int(self.width, "width")
        if not float(_need(self.norm, "eps", "norm")) > 0:
            raise ConfigError("norm.eps must be positive")
        if not isinstance(self.embedding, dict):
            raise ConfigError("embedding must be a mapping")
        if not isinstance(self.layers, (list, tuple)) or not self.layers:
            raise ConfigError("layers must be a non-empty list")
        for i, layer in enumerate(self.layers):
            kind = _need(layer, "type", f"layers[{i}]")
            if kind not in ("attention", "hgrn2", "retention"):
                raise ConfigError(f"layers[{i}].type {kind!r} is not one of attention, hgrn2, retention")
            _need(layer, "mixer", f"layers[{i}]")
            mlp = layer.get("mlp")
            if mlp is not None and _need(mlp, "kind", f"layers[{i}].mlp") != "dense":
                raise ConfigError(f"layers[{i}].mlp.kind {mlp['kind']!r} is not built; known: dense")

    # -- the mixers as parts ------------------------------------------------------------
    def _rotation(self, m, where: str) -> PartSpec:
        if m.get("rot") is None or not m["rot"].get("dims"):
            return PartSpec("no_position", {})
        rot = m["rot"]
        dims = _positive_int(_need(rot, "dims", where + ".rot"), where + ".rot.dims")
        if dims % 2 or dims > int(m["dim"]):
            raise ConfigError(f"{where}.rot.dims {dims} must be even and at most dim {m['dim']}")
        return PartSpec("rope_half", {"rotary_dim": dims, "theta": float(_need(rot, "base", where + ".rot"))})

    def _mixer(self, i: int, layer, first_mixing) -> PartSpec:
        kind, m, where = layer["type"], layer["mixer"], f"layers[{i}].mixer"
        sizes = {"hidden_size": self.width,
                 "num_heads": _positive_int(_need(m, "heads", where), where + ".heads"),
                 "head_dim": _positive_int(_need(m, "dim", where), where + ".dim"),
                 "value_dim": _positive_int(_need(m, "vdim", where), where + ".vdim")}
        if kind == "attention":
            mask = _need(m, "mask", where)
            v_mix = None
            if m.get("v_mix"):
                v_mix = "source" if i == first_mixing else "mix"
            return PartSpec("talking_attention", dict(
                sizes, num_kv_heads=_positive_int(_need(m, "kv_heads", where), where + ".kv_heads"),
                position=self._rotation(m, where), window=_positive_int(_need(mask, "size", where + ".mask"), "mask.size"),
                keep_first=int(mask.get("keep_first") or 0), scale=float(_need(m, "scale", where)), bias=True,
                v_mix=v_mix))
        eps = float(self.norm["eps"])
        if kind == "hgrn2":
            return PartSpec("hgrn2", dict(sizes, eps=eps))
        decay = [float(v) for v in _need(m, "decay", where)]
        return PartSpec("retention", dict(sizes, eps=eps, decay=tuple(decay), position=self._rotation(m, where)))

    def model_spec(self) -> ModelSpec:
        width = self.width
        norm = PartSpec("dynamic_tanh", {"size": width})
        arrangement = PartSpec("prenorm_residual", {"mixer_prefix": "mix", "feed_forward_prefix": "mlp",
                                                    "mixer_norm_name": "norm1", "feed_forward_norm_name": "norm2"})
        mixing = [i for i, layer in enumerate(self.layers) if layer["type"] == "attention" and layer["mixer"].get("v_mix")]
        first_mixing = mixing[0] if mixing else None
        layers = []
        for i, layer in enumerate(self.layers):
            mlp = layer.get("mlp")
            feed_forward = None
            if mlp is not None:
                feed_forward = PartSpec("clamped_gated_mlp", {
                    "hidden_size": width, "intermediate_size": _positive_int(_need(mlp, "ff", f"layers[{i}].mlp"), "mlp.ff"),
                    "limit": float(_need(mlp, "limit", f"layers[{i}].mlp")), "alpha": GATE_SLOPE})
            layers.append(LayerSpec(
                prefix=f"l{i}", arrangement=arrangement, mixer=self._mixer(i, layer, first_mixing),
                feed_forward=feed_forward, mixer_norm=norm,
                feed_forward_norm=norm if mlp is not None else PartSpec("dynamic_tanh", {"size": width, "optional": True})))
        shapes = {(layers[i].mixer["num_kv_heads"], layers[i].mixer["value_dim"]) for i in mixing}
        if len(shapes) > 1:
            raise ConfigError(f"layers that mix values must agree on kv_heads and vdim, got {sorted(shapes)}")
        return ModelSpec(
            hidden_size=width, vocab_size=self.vocab,
            embedding=PartSpec("token_embedding", {"name": "embed", "vocab_size": self.vocab, "hidden_size": width,
                                                   "scale": float(self.embedding.get("scale", 1.0))}),
            layers=tuple(layers),
            schedule=tuple(ScheduleEntry(layer=i, cache=i) for i in range(len(layers))),
            final_norm=PartSpec("dynamic_tanh", {"size": width, "name": "final.norm"}),
            head=PartSpec("linear_head", {"name": "head", "tied_to": None, "vocab_size": self.vocab,
                                          "hidden_size": width, "softcap": float(self.logit_softcap) if self.logit_softcap else None}),
            max_positions=None)
