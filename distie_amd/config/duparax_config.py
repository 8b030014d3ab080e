"""The Duparax decoder: its config.json and the parts it is made of.

config.json names everything that can differ between models of the design:

    architecture "Duparax", vocab, width, norm.eps, logit_scale, and `layers`, one entry a layer: `type`
    ("parallel" | "rglru"), `mixer` (its sizes) and `mlp` (or null).

    parallel mixer: `left` {heads, kv_heads, dim, vdim, scale, q_temp {coef, every}} (softmax attention with biases,
    no rotation) and `right` {heads, dim, vdim, tau} (gated linear attention), side by side.
    rglru mixer: width, blocks, conv (taps).
    mlp: {"kind": "dense", "ff"} or {"kind": "moe", "router" {experts, top}, "expert" {ff}, "shared" {ff}}.

Tensors: `embed`, `head`, `final.norm`; layer i under `l<i>.`: `norm1`, `norm1b`, `norm2`, `norm2b`, `mix.*`,
`mlp.*`. Linear weights are [out, in]. One size is not in config.json: the rank of the projection that the gated
linear attention's decay goes through. With a model folder at hand it is the first dimension of the tensor
`l<i>.mix.right.a1` (`with_tensor_shapes`); a configuration without a folder (random weights) names it as
`right.rank`. Nothing here fixes a size.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping

from .model_config import ConfigError, LayerCall, LayerSpec, ModelSpec, PartSpec
from .musutar_config import DEFAULT_MAX_POSITIONS, _need


@dataclass(frozen=True)
class DuparaxConfig:
    data: Mapping[str, Any]
    max_positions: int = DEFAULT_MAX_POSITIONS

    architecture = "Duparax"

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
    def from_dict(cls, data: Mapping[str, Any]) -> "DuparaxConfig":
        vocab, width = _need(data, "vocab", int, "the model"), _need(data, "width", int, "the model")
        if vocab < 1 or width < 1:
            raise ConfigError("vocab and width must be >= 1")
        _need(data.get("norm") or {}, "eps", float, "norm")
        if data.get("logit_scale") is not None:
            _need(data, "logit_scale", float, "the model")
        layers = data.get("layers")
        if not isinstance(layers, (list, tuple)) or not layers:
            raise ConfigError("config.json lacks 'layers'")
        for i, layer in enumerate(layers):
            where = f"layer {i}"
            kind = _need(layer, "type", str, where)
            mixer = layer.get("mixer")
            if not isinstance(mixer, Mapping):
                raise ConfigError(f"config.json: {where} lacks 'mixer'")
            if kind == "parallel":
                left, right = mixer.get("left"), mixer.get("right")
                heads, kv_heads = _need(left, "heads", int, where + " left"), _need(left, "kv_heads", int, where + " left")
                if heads < 1 or kv_heads < 1 or heads % kv_heads:
                    raise ConfigError(f"{where}: left.heads must be a positive multiple of left.kv_heads")
                if _need(left, "dim", int, where + " left") < 1 or _need(left, "vdim", int, where + " left") < 1:
                    raise ConfigError(f"{where}: left.dim and left.vdim must be >= 1")
                if not _need(left, "scale", float, where + " left") > 0:
                    raise ConfigError(f"{where}: left.scale must be positive")
                temp = left.get("q_temp")
                if temp:
                    _need(temp, "coef", float, where + " left.q_temp")
                    if _need(temp, "every", int, where + " left.q_temp") < 1:
                        raise ConfigError(f"{where}: left.q_temp.every must be >= 1")
                for key in ("heads", "dim", "vdim"):
                    if _need(right, key, int, where + " right") < 1:
                        raise ConfigError(f"{where}: right.{key} must be >= 1")
                if not _need(right, "tau", float, where + " right") > 0:
                    raise ConfigError(f"{where}: right.tau must be positive")
            elif kind == "rglru":
                channels, blocks = _need(mixer, "width", int, where), _need(mixer, "blocks", int, where)
                if channels < 1 or blocks < 1 or channels % blocks:
                    raise ConfigError(f"{where}: width must be a positive multiple of blocks")
                if not 1 <= _need(mixer, "conv", int, where) <= 16:
                    raise ConfigError(f"{where}: conv must be 1 to 16 taps")
            else:
                raise ConfigError(f"{where}: unknown layer type {kind!r}")
            mlp = layer.get("mlp")
            if mlp is None:
                continue
            mlp_kind = _need(mlp, "kind", str, where + " mlp")
            if mlp_kind == "dense":
                if _need(mlp, "ff", int, where + " mlp") < 1:
                    raise ConfigError(f"{where}: mlp.ff must be >= 1")
            elif mlp_kind == "moe":
                router = mlp.get("router")
                experts, top = _need(router, "experts", int, where + " router"), _need(router, "top", int, where + " router")
                if not 1 <= top <= experts:
                    raise ConfigError(f"{where}: router.top must be between 1 and router.experts")
                if _need(mlp.get("expert"), "ff", int, where + " expert") < 1:
                    raise ConfigError(f"{where}: expert.ff must be >= 1")
                if mlp.get("shared") and _need(mlp["shared"], "ff", int, where + " shared") < 1:
                    raise ConfigError(f"{where}: shared.ff must be >= 1")
            else:
                raise ConfigError(f"{where}: unknown mlp kind {mlp_kind!r}")
        return cls(data=dict(data), max_positions=int(data.get("max_positions") or DEFAULT_MAX_POSITIONS))

    def to_dict(self) -> dict:
        return dict(self.data)

    def with_tensor_shapes(self, shapes: Mapping[str, tuple]) -> "DuparaxConfig":
        """The sizes that only the tensors tell: each gated linear attention's decay rank."""
        data = dict(self.data)
        layers = []
        for i, layer in enumerate(data["layers"]):
            name = f"l{i}.mix.right.a1"
            if layer.get("type") == "parallel" and name in shapes and len(shapes[name]) == 2:
                right = dict(layer["mixer"]["right"], rank=int(shapes[name][0]))
                layer = dict(layer, mixer=dict(layer["mixer"], right=right))
            layers.append(layer)
        data["layers"] = layers
        return type(self)(data=data, max_positions=self.max_positions)

    @staticmethod
    def _rank(right: Mapping[str, Any], layer: int) -> int:
        if right.get("rank") is None:
            raise ConfigError(f"layer {layer}: the decay's rank comes from the tensors of a model folder, or from "
                              f"'rank' in the layer's right mixer")
        return int(right["rank"])

    def model_spec(self) -> ModelSpec:
        data = self.data
        width, eps = self.hidden_size, float(data["norm"]["eps"])
        norm = lambda base, name: PartSpec("rmsnorm", base, {"size": width, "eps": eps, "weight_name": name})
        layers = []
        for i, layer in enumerate(data["layers"]):
            base = f"l{i}."
            m = layer["mixer"]
            if layer["type"] == "parallel":
                left, right = m["left"], m["right"]
                mixer = PartSpec("parallel_mixers", base + "mix.", {"hidden_size": width, "eps": eps, "scale": 0.5, "mixers": {
                    "left": PartSpec("conv_gated_attention", base + "mix.left.", {
                        "hidden_size": width, "num_heads": int(left["heads"]), "num_kv_heads": int(left["kv_heads"]),
                        "head_dim": int(left["dim"]), "value_dim": int(left["vdim"]), "conv_taps": 0, "window": None,
                        "scale": float(left["scale"]), "output_gate": False, "bias": True, "position": None,
                        "q_temp": dict(left["q_temp"]) if left.get("q_temp") else None}),
                    "right": PartSpec("gated_linear_attention", base + "mix.right.", {
                        "hidden_size": width, "num_heads": int(right["heads"]), "head_dim": int(right["dim"]),
                        "value_dim": int(right["vdim"]), "tau": float(right["tau"]), "eps": eps,
                        "decay_rank": self._rank(right, i)}),
                }})
            else:
                mixer = PartSpec("rglru", base + "mix.", {
                    "hidden_size": width, "width": int(m["width"]), "blocks": int(m["blocks"]),
                    "conv_taps": int(m["conv"]), "rate": 8.0})
            parts = {"mixer": mixer, "mixer_norm": norm(base, "norm1"), "mixer_post_norm": norm(base, "norm1b")}
            mlp = layer.get("mlp")
            if mlp is not None:
                if mlp["kind"] == "dense":
                    parts["feed_forward"] = PartSpec("swiglu", base + "mlp.", {
                        "hidden_size": width, "intermediate_size": int(mlp["ff"]),
                        "gate_name": "gate", "up_name": "up", "down_name": "down"})
                else:
                    parts["feed_forward"] = PartSpec("routed_experts", base + "mlp.", {
                        "hidden_size": width, "num_experts": int(mlp["router"]["experts"]),
                        "top": int(mlp["router"]["top"]), "expert_size": int(mlp["expert"]["ff"]),
                        "shared_size": int(mlp["shared"]["ff"]) if mlp.get("shared") else 0})
                parts["feed_forward_norm"] = norm(base, "norm2")
                parts["feed_forward_post_norm"] = norm(base, "norm2b")
            layers.append(LayerSpec(PartSpec("sandwich_residual", base, {}), parts))
        return ModelSpec(
            architecture=self.architecture,
            vocab_size=self.vocab_size,
            hidden_size=width,
            max_positions=self.max_positions,
            embedding=PartSpec("token_embedding", "", {"vocab_size": self.vocab_size, "hidden_size": width,
                                                       "weight_name": "embed"}),
            layers=tuple(layers),
            order=tuple(LayerCall(l) for l in range(len(layers))),
            final_norm=PartSpec("rmsnorm", "final.", {"size": width, "eps": eps, "weight_name": "norm"}),
            head=PartSpec("lm_head", "", {"vocab_size": self.vocab_size, "hidden_size": width, "tied_to": None,
                                          "weight_name": "head", "scale": float(data.get("logit_scale") or 1.0)}),
        )
