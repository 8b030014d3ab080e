"""The Musutar decoder: its config.json and the parts it is made of.

config.json names everything that can differ between models of the design:

    architecture "Musutar", vocab, width, streams (the residual's copies), norm.eps, canon.taps (the convolution in
    front of every mixer), and `layers`, one entry a layer: `type` ("attention" | "lightning"), `mixer` (its sizes)
    and `mlp` ({"kind": "dense", "ff": n} or null).

    attention mixer: heads, kv_heads, dim, vdim, conv (taps of the convolution behind q/k/v), rot {base, dims,
    scaling {factor, original, fast, slow}}, scale, mask {size}, kv_from (a layer whose keys and values are used).
    lightning mixer: heads, dim, vdim, decay (one per head).

Tensors: `embed`, `head`, `final.norm`; layer i under `l<i>.`: `norm1`, `norm2`, `mix.*`, `mlp.up`, `mlp.down`,
`hc<q>.in|out|mix`, `canon1`, `rg<q>`, `rg<q>.b`. Linear weights are [out, in]. Nothing here fixes a size.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional

from .model_config import ConfigError, LayerCall, LayerSpec, ModelSpec, PartSpec

# the design sets no limit on positions; the engine needs one for its block tables
DEFAULT_MAX_POSITIONS = 131072


def _need(data: Mapping[str, Any], key: str, kind, where: str):
    if not isinstance(data, Mapping) or key not in data or data[key] is None:
        raise ConfigError(f"config.json: {where} lacks '{key}'")
    try:
        return kind(data[key])
    except (TypeError, ValueError) as exc:
        raise ConfigError(f"config.json: {where} '{key}' = {data[key]!r} is not {kind.__name__}") from exc


@dataclass(frozen=True)
class MusutarConfig:
    data: Mapping[str, Any]
    max_positions: int = DEFAULT_MAX_POSITIONS

    architecture = "Musutar"

    @property
    def vocab_size(self) -> int:
        return int(self.data["vocab"])

    @property
    def hidden_size(self) -> int:
        return int(self.data["width"])

    @property
    def num_layers(self) -> int:
        return len(self.data["layers"])

    @classmethod
    def from_dict(cls, data: Mapping[str, Any]) -> "MusutarConfig":
        vocab, width = _need(data, "vocab", int, "the model"), _need(data, "width", int, "the model")
        if vocab < 1 or width < 1:
            raise ConfigError("vocab and width must be >= 1")
        _need(data.get("norm") or {}, "eps", float, "norm")
        streams = data.get("streams")
        if streams is not None and not 1 <= int(streams) <= 8:
            raise ConfigError("streams must be 1 to 8")
        canon = data.get("canon")
        if canon and not 1 <= _need(canon, "taps", int, "canon") <= 16:
            raise ConfigError("canon.taps must be 1 to 16")
        layers = data.get("layers")
        if not isinstance(layers, (list, tuple)) or not layers:
            raise ConfigError("config.json lacks 'layers'")
        for i, layer in enumerate(layers):
            where = f"layer {i}"
            kind = _need(layer, "type", str, where)
            mixer = layer.get("mixer")
            heads, dim = _need(mixer, "heads", int, where), _need(mixer, "dim", int, where)
            _need(mixer, "vdim", int, where)
            if heads < 1 or dim < 1 or int(mixer["vdim"]) < 1:
                raise ConfigError(f"{where}: heads, dim and vdim must be >= 1")
            if kind == "attention":
                kv_heads = _need(mixer, "kv_heads", int, where)
                if kv_heads < 1 or heads % kv_heads:
                    raise ConfigError(f"{where}: heads must be a positive multiple of kv_heads")
                _need(mixer, "scale", float, where)
                rot = mixer.get("rot")
                if rot:
                    dims = _need(rot, "dims", int, where + " rot")
                    _need(rot, "base", float, where + " rot")
                    if dims < 2 or dims % 2 or dims > dim:
                        raise ConfigError(f"{where}: rot.dims must be even and at most dim")
                    if rot.get("scaling"):
                        for key in ("factor", "original", "fast", "slow"):
                            _need(rot["scaling"], key, float, where + " rot.scaling")
                if mixer.get("mask") and _need(mixer["mask"], "size", int, where + " mask") < 1:
                    raise ConfigError(f"{where}: mask.size must be >= 1")
                if mixer.get("conv") is not None and not 1 <= int(mixer["conv"]) <= 16:
                    raise ConfigError(f"{where}: conv must be 1 to 16 taps")
                source = mixer.get("kv_from")
                if source is not None:
                    source = int(source)
                    if not 0 <= source < i or layers[source].get("type") != "attention" or \
                            layers[source]["mixer"].get("kv_from") is not None:
                        raise ConfigError(f"{where}: kv_from must name an earlier attention layer with keys of its own")
                    theirs = layers[source]["mixer"]
                    if any(int(theirs[k]) != int(mixer[k]) for k in ("kv_heads", "dim", "vdim")):
                        raise ConfigError(f"{where}: kv_from names a layer with other head sizes")
            elif kind == "lightning":
                decay = mixer.get("decay")
                if not isinstance(decay, (list, tuple)) or len(decay) != heads:
                    raise ConfigError(f"{where}: decay must hold one value for each of the {heads} heads")
            else:
                raise ConfigError(f"{where}: unknown layer type {kind!r}")
            mlp = layer.get("mlp")
            if mlp is not None:
                if _need(mlp, "kind", str, where + " mlp") != "dense":
                    raise ConfigError(f"{where}: unknown mlp kind {mlp['kind']!r}")
                if _need(mlp, "ff", int, where + " mlp") < 1:
                    raise ConfigError(f"{where}: mlp.ff must be >= 1")
        return cls(data=dict(data), max_positions=int(data.get("max_positions") or DEFAULT_MAX_POSITIONS))

    def to_dict(self) -> dict:
        return dict(self.data)

    def _kept_windows(self) -> dict:
        """For every attention layer with keys of its own: how far back its cache must reach, the widest window
        among itself and the layers that borrow from it (None: everything)."""
        layers = self.data["layers"]
        window = lambda m: (m.get("mask") or {}).get("size")
        kept = {i: window(l["mixer"]) for i, l in enumerate(layers)
                if l["type"] == "attention" and l["mixer"].get("kv_from") is None}
        for layer in layers:
            source = layer["mixer"].get("kv_from") if layer["type"] == "attention" else None
            if source is not None:
                mine = window(layer["mixer"])
                if kept[int(source)] is not None:
                    kept[int(source)] = None if mine is None else max(int(kept[int(source)]), int(mine))
        return kept

    def model_spec(self) -> ModelSpec:
        data = self.data
        width, eps = self.hidden_size, float(data["norm"]["eps"])
        taps = int(data["canon"]["taps"]) if data.get("canon") else 0
        kept = self._kept_windows()
        layers = []
        for i, layer in enumerate(data["layers"]):
            base = f"l{i}."
            m = layer["mixer"]
            if layer["type"] == "attention":
                rot = m.get("rot")
                window = (m.get("mask") or {}).get("size")
                mixer = PartSpec("conv_gated_attention", base + "mix.", {
                    "hidden_size": width, "num_heads": int(m["heads"]), "num_kv_heads": int(m["kv_heads"]),
                    "head_dim": int(m["dim"]), "value_dim": int(m["vdim"]), "conv_taps": int(m.get("conv") or 0),
                    "window": None if window is None else int(window),
                    "keep": kept.get(i, None if window is None else int(window)),
                    "scale": float(m["scale"]), "output_gate": True,
                    "kv_from": None if m.get("kv_from") is None else int(m["kv_from"]),
                    "position": PartSpec("rope_scaled", "", {"dims": int(rot["dims"]), "base": float(rot["base"]),
                                                             "scaling": rot.get("scaling")}) if rot else None,
                })
            else:
                mixer = PartSpec("decay_linear_attention", base + "mix.", {
                    "hidden_size": width, "num_heads": int(m["heads"]), "head_dim": int(m["dim"]),
                    "value_dim": int(m["vdim"]), "decay": tuple(float(d) for d in m["decay"]), "eps": eps,
                })
            parts = {"mixer": mixer,
                     "mixer_norm": PartSpec("layernorm", base, {"size": width, "eps": eps, "weight_name": "norm1"})}
            if layer.get("mlp") is not None:
                parts["feed_forward"] = PartSpec("dense_mlp", base + "mlp.", {
                    "hidden_size": width, "intermediate_size": int(layer["mlp"]["ff"]), "activation": "relu2",
                    "up_name": "up", "down_name": "down"})
                parts["feed_forward_norm"] = PartSpec("layernorm", base, {"size": width, "eps": eps, "weight_name": "norm2"})
            block = PartSpec("hyper_connections", base, {
                "hidden_size": width, "streams": None if data.get("streams") is None else int(data["streams"]),
                "gated": True, "input_taps": taps})
            layers.append(LayerSpec(block, parts))
        return ModelSpec(
            architecture=self.architecture,
            vocab_size=self.vocab_size,
            hidden_size=width,
            max_positions=self.max_positions,
            embedding=PartSpec("token_embedding", "", {"vocab_size": self.vocab_size, "hidden_size": width,
                                                       "weight_name": "embed"}),
            layers=tuple(layers),
            order=tuple(LayerCall(l) for l in range(len(layers))),
            final_norm=PartSpec("layernorm", "final.", {"size": width, "eps": eps, "weight_name": "norm"}),
            head=PartSpec("lm_head", "", {"vocab_size": self.vocab_size, "hidden_size": width, "tied_to": None,
                                          "weight_name": "head"}),
        )
