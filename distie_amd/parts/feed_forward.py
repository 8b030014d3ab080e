"""Feed-forwards. Gated: down(silu(gate x) * up x), no biases
(worker/src/inference/qwen2/model.py:228-236). Gate and up are one matrix product:
their weights are stacked at load."""

from __future__ import annotations

import torch

from .base import FeedForward, ParamSpec, register_part


class SwiGLU(FeedForward):
    def __init__(self, spec) -> None:
        super().__init__(spec)
        self.hidden_size = int(spec.params["hidden_size"])
        self.intermediate_size = int(spec.params["intermediate_size"])
        self.gate_up_weight = self.down_weight = None

    def param_specs(self):
        return {
            "gate_proj.weight": ParamSpec((self.intermediate_size, self.hidden_size)),
            "up_proj.weight": ParamSpec((self.intermediate_size, self.hidden_size)),
            "down_proj.weight": ParamSpec((self.hidden_size, self.intermediate_size)),
        }

    def load(self, tensors) -> None:
        gate, up = tensors["gate_proj.weight"], tensors["up_proj.weight"]
        dtype = torch.float32 if torch.float32 in (gate.dtype, up.dtype) else gate.dtype
        self.gate_up_weight = torch.cat([gate.to(dtype), up.to(dtype)], dim=0).contiguous()
        self.down_weight = tensors["down_proj.weight"].contiguous()

    def prepare(self, ops) -> None:
        ops.prepare_linear(self.gate_up_weight, gated=True, role="gate_up")
        ops.prepare_linear(self.down_weight, role="down")

    def forward(self, ops, x, ctx):
        return ops.linear(ops.linear_silu_mul(x, self.gate_up_weight), self.down_weight)


class DenseMLP(FeedForward):
    """down(act(up x)), no gate and no biases; `activation` names the function ("relu2": the square of
    max(z, 0)). Tensors `up` [ff, C] and `down` [C, ff] under the names the spec gives."""

    def __init__(self, spec) -> None:
        super().__init__(spec)
        self.hidden_size = int(spec.params["hidden_size"])
        self.intermediate_size = int(spec.params["intermediate_size"])
        self.activation = str(spec.params.get("activation", "relu2"))
        self.up_name = spec.params.get("up_name", "up_proj.weight")
        self.down_name = spec.params.get("down_name", "down_proj.weight")
        self.up_weight = self.down_weight = None

    def param_specs(self):
        return {self.up_name: ParamSpec((self.intermediate_size, self.hidden_size)),
                self.down_name: ParamSpec((self.hidden_size, self.intermediate_size))}

    def load(self, tensors) -> None:
        self.up_weight = tensors[self.up_name].contiguous()
        self.down_weight = tensors[self.down_name].contiguous()

    def prepare(self, ops) -> None:
        ops.prepare_linear(self.up_weight, role="up")
        ops.prepare_linear(self.down_weight, role="down")

    def forward(self, ops, x, ctx):
        return ops.linear(ops.linear_act(x, self.up_weight, self.activation), self.down_weight)


register_part("feed_forward", "swiglu", SwiGLU)
register_part("feed_forward", "dense_mlp", DenseMLP)
