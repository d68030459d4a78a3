"""Biberax: a decoder whose layers each name one of two attention mixers and one of two
feed-forwards, between root-mean-square norms.

* ``attention``: grouped heads, rotation of the leading dimensions of a head in neighbouring pairs
  with frequencies stretched by wavelength, keys of the query's own chunk only, a softmax with a one
  in its denominator, a sigmoid gate on the heads' outputs.
* ``attention_2``: biased projections, values that are the keys as projected, a norm over the whole
  query and key projections, a learned bias by (bucketed) distance, all earlier keys, a learned sink a
  head, the same gate, a biased output projection.
* feed-forward ``dense`` (a gated unit with the tanh form of GELU) or ``moe`` (routed small experts with
  clamped gated units, and a shared expert).

``config.json`` is nested: ``architecture`` (the name), ``vocab``, ``width``, ``norm.eps`` and
``layers``, a list whose entries give ``type``, the mixer's sizes and constants under ``mixer`` and the
feed-forward under ``mlp`` (null for a layer without one).  Layer ``i``'s tensors start with ``l<i>.``:
``norm1``, ``norm2``, ``mix.*``, ``mlp.*``; beside them ``embed``, ``final.norm`` and ``head``.
``model_spec`` states all of this as parts.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any

from .base import ConfigError, LayerSpec, ModelConfig, ModelSpec, PartSpec, ScheduleEntry
from .registry import register_architecture

#: the slope of the sigmoid in the experts' gated unit, fixed by the design
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
class BiberaxConfig(ModelConfig):
    architecture: str
    vocab: int
    width: int
    norm: Any
    layers: Any

    architecture_names = ("Biberax", "biberax")

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    def to_dict(self) -> dict:
        return {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                "norm": dict(self.norm), "layers": [dict(layer) for layer in self.layers]}

    def init_scheme(self):
        return {"std": 0.05, "norm_std": 0.1}

    def validate(self) -> None:
        _positive_int(self.vocab, "vocab")
        _positive_int(self.width, "width")
        if not float(_need(self.norm, "eps", "norm")) > 0:
            raise ConfigError("norm.eps must be positive")
        if not isinstance(self.layers, (list, tuple)) or not self.layers:
            raise ConfigError("layers must be a non-empty list")
        for i, layer in enumerate(self.layers):
            kind = _need(layer, "type", f"layers[{i}]")
            if kind not in ("attention", "attention_2"):
                raise ConfigError(f"layers[{i}].type {kind!r} is not one of attention, attention_2")
            _need(layer, "mixer", f"layers[{i}]")
            mlp = layer.get("mlp")
            if mlp is not None and _need(mlp, "kind", f"layers[{i}].mlp") not in ("dense", "moe"):
                raise ConfigError(f"layers[{i}].mlp.kind {mlp['kind']!r} is not one of dense, moe")
        self.model_spec()        # every key the layers need, now rather than at the first step

    # -- the mixers as parts ------------------------------------------------------------
    def _rotation(self, m, where: str) -> PartSpec:
        rot = m.get("rot")
        if rot is None or not rot.get("dims"):
            return PartSpec("no_position", {})
        dims = _positive_int(_need(rot, "dims", where + ".rot"), where + ".rot.dims")
        if dims % 2 or dims > int(m["dim"]):
            raise ConfigError(f"{where}.rot.dims {dims} must be even and at most dim {m['dim']}")
        scaling = rot.get("scaling")
        if scaling is not None:
            scaling = {key: float(_need(scaling, key, where + ".rot.scaling")) for key in ("factor", "low", "high", "original")}
        return PartSpec("rope_scaled", {"rotary_dim": dims, "theta": float(_need(rot, "base", where + ".rot")),
                                        "pairing": "neighbours", "scaling": scaling})

    def _mixer(self, i: int, layer) -> PartSpec:
        kind, m, where = layer["type"], layer["mixer"], f"layers[{i}].mixer"
        sizes = {"hidden_size": self.width,
                 "num_heads": _positive_int(_need(m, "heads", where), where + ".heads"),
                 "num_kv_heads": _positive_int(_need(m, "kv_heads", where), where + ".kv_heads"),
                 "head_dim": _positive_int(_need(m, "dim", where), where + ".dim"),
                 "value_dim": _positive_int(_need(m, "vdim", where), where + ".vdim"),
                 "scale": float(_need(m, "scale", where)), "gate": True}
        if sizes["num_heads"] % sizes["num_kv_heads"]:
            raise ConfigError(f"{where}: {sizes['num_heads']} heads are not a multiple of {sizes['num_kv_heads']} kv_heads")
        if kind == "attention":
            mask = m.get("mask")
            chunk = _positive_int(_need(mask, "size", where + ".mask"), where + ".mask.size") if mask else None
            return PartSpec("sink_attention", dict(sizes, position=self._rotation(m, where), chunk=chunk, sink="zero"))
        if sizes["value_dim"] != sizes["head_dim"]:
            raise ConfigError(f"{where}: the values are the keys, so vdim {sizes['value_dim']} must equal dim {sizes['head_dim']}")
        farthest = float(_need(m, "bias_max", where))
        if not farthest > 1:
            raise ConfigError(f"{where}.bias_max must exceed 1")
        bias = {"farthest": farthest}
        if m.get("bias_rows"):               # (sizes the table of random weights; a checkpoint's table says it itself)
            bias["rows"] = _positive_int(m["bias_rows"], where + ".bias_rows")
        return PartSpec("sink_attention", dict(
            sizes, position=PartSpec("no_position", {}), sink="learned", bias=True, out_bias=True,
            qk_norm=float(self.norm["eps"]), shared_kv=True, distance_bias=bias))

    def _feed_forward(self, i: int, mlp) -> PartSpec:
        where = f"layers[{i}].mlp"
        if mlp["kind"] == "dense":
            return PartSpec("gated_mlp", {
                "hidden_size": self.width, "intermediate_size": _positive_int(_need(mlp, "ff", where), where + ".ff"),
                "activation": "gelu_tanh", "gate_name": "gate", "up_name": "up", "down_name": "down"})
        router, expert = _need(mlp, "router", where), _need(mlp, "expert", where)
        experts = _positive_int(_need(router, "experts", where + ".router"), where + ".router.experts")
        top = _positive_int(_need(router, "top", where + ".router"), where + ".router.top")
        if top > experts:
            raise ConfigError(f"{where}.router.top {top} exceeds its {experts} experts")
        shared = mlp.get("shared")
        shared_spec = None
        if shared is not None:
            shared_spec = PartSpec("clamped_gated_mlp", {
                "hidden_size": self.width,
                "intermediate_size": _positive_int(_need(shared, "ff", where + ".shared"), where + ".shared.ff"),
                "limit": float(_need(shared, "limit", where + ".shared")), "alpha": GATE_SLOPE})
        return PartSpec("routed_experts", {
            "hidden_size": self.width,
            "intermediate_size": _positive_int(_need(expert, "ff", where + ".expert"), where + ".expert.ff"),
            "experts": experts, "top": top, "limit": float(_need(expert, "limit", where + ".expert")),
            "alpha": GATE_SLOPE, "shared": shared_spec})

    def model_spec(self) -> ModelSpec:
        width, eps = self.width, float(self.norm["eps"])
        arrangement = PartSpec("prenorm_residual", {"mixer_prefix": "mix", "feed_forward_prefix": "mlp",
                                                    "mixer_norm_name": "norm1", "feed_forward_norm_name": "norm2"})
        layers = []
        for i, layer in enumerate(self.layers):
            mlp = layer.get("mlp")
            layers.append(LayerSpec(
                prefix=f"l{i}", arrangement=arrangement, mixer=self._mixer(i, layer),
                feed_forward=None if mlp is None else self._feed_forward(i, mlp),
                mixer_norm=PartSpec("rmsnorm", {"size": width, "eps": eps, "name": f"l{i}.norm1"}),
                feed_forward_norm=PartSpec("rmsnorm", {"size": width, "eps": eps, "name": f"l{i}.norm2",
                                                       "optional": mlp is None})))
        return ModelSpec(
            hidden_size=width, vocab_size=self.vocab,
            embedding=PartSpec("token_embedding", {"name": "embed", "vocab_size": self.vocab, "hidden_size": width}),
            layers=tuple(layers),
            schedule=tuple(ScheduleEntry(layer=i, cache=i) for i in range(len(layers))),
            final_norm=PartSpec("rmsnorm", {"size": width, "eps": eps, "name": "final.norm"}),
            head=PartSpec("linear_head", {"name": "head", "tied_to": None, "vocab_size": self.vocab, "hidden_size": width}),
            max_positions=None)
