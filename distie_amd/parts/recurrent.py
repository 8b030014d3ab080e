"""A recurrent block with a real-gated linear recurrent unit (the "RG-LRU" of Griffin: De et al., "Griffin: Mixing
Gated Linear Recurrences with Local Attention for Efficient Language Models").

Two branches of `width` channels read the mixer's input h:

    y = gelu_tanh(W_y h + b_y)
    u = conv(W_x h + b_x)          a causal convolution over time for each channel (`conv` [width, taps], bias
                                   `conv.b`; the last column is the current token's; zeros before the start)

u is cut into `blocks` equal parts, and in part b, with square matrices `ra[b]`, `ri[b]` ([out, in]) and biases:

    r = sigmoid(ra[b] u_b + ra.b[b]),   i = sigmoid(ri[b] u_b + ri.b[b])
    a = exp(-rate * r * softplus(lam)),          S_t = a S_(t-1) + sqrt(1 - a^2) * i * u

from S = 0, the first token included; the result is W_o (S * y). `rate` is 8 in the design this was written for.
The state S is float32 [width] for each request, and the convolution's last taps - 1 inputs are state as well. The
gates, a, the square root and the recurrence are float32 in either precision. Both branches are one matrix product:
their weights are stacked at load (y first).
"""

from __future__ import annotations

import torch

from ..config.model_config import PartSpec
from .base import FixedState, Mixer, ParamSpec, TensorDecl, register_part


class GatedLinearRecurrentUnit(Mixer):
    def __init__(self, spec: PartSpec) -> None:
        super().__init__(spec)
        p = spec.params
        self.hidden_size = int(p["hidden_size"])
        self.width = int(p["width"])
        self.blocks = int(p["blocks"])
        self.taps = int(p["conv_taps"])
        self.rate = float(p.get("rate", 8.0))
        if self.blocks < 1 or self.width % self.blocks:
            raise ValueError("the recurrent unit's width must be a multiple of its blocks")
        if self.taps < 1:
            raise ValueError("the convolution has at least one tap")
        self.in_weight = self.in_bias = self.conv_weight = self.conv_bias = None
        self.recur_weight = self.recur_bias = self.input_weight = self.input_bias = self.lam = self.out_weight = None

    def cache_requirement(self):
        tensors = [TensorDecl("state", (self.width,), torch.float32)]
        if self.taps > 1:
            tensors.append(TensorDecl("conv", (self.taps - 1, self.width), torch.float32))
        return FixedState(tuple(tensors))

    def param_specs(self):
        R, C, n = self.width, self.hidden_size, self.width // self.blocks
        return {"y": ParamSpec((R, C)), "y.b": ParamSpec((R,)), "x": ParamSpec((R, C)), "x.b": ParamSpec((R,)),
                "conv": ParamSpec((R, self.taps)), "conv.b": ParamSpec((R,)),
                "ra": ParamSpec((self.blocks, n, n)), "ra.b": ParamSpec((self.blocks, n)),
                "ri": ParamSpec((self.blocks, n, n)), "ri.b": ParamSpec((self.blocks, n)),
                "lam": ParamSpec((R,)), "o": ParamSpec((C, R))}

    def load(self, tensors) -> None:
        y, x = tensors["y"], tensors["x"]
        dtype = torch.float32 if torch.float32 in (y.dtype, x.dtype) else y.dtype
        self.in_weight = torch.cat([y.to(dtype), x.to(dtype)], dim=0).contiguous()
        self.in_bias = torch.cat([tensors["y.b"].float(), tensors["x.b"].float()]).contiguous()
        self.conv_weight = tensors["conv"].contiguous()
        self.conv_bias = tensors["conv.b"].float().contiguous()
        self.recur_weight, self.input_weight = tensors["ra"].contiguous(), tensors["ri"].contiguous()
        self.recur_bias, self.input_bias = tensors["ra.b"].float().contiguous(), tensors["ri.b"].float().contiguous()
        self.lam = tensors["lam"].float().contiguous()
        self.out_weight = tensors["o"].contiguous()

    def prepare(self, ops) -> None:
        ops.prepare_linear(self.in_weight, role="qkv")
        ops.prepare_linear(self.out_weight, role="attn_out")

    def forward(self, ops, x, ctx, cache, writes_cache: bool):
        R = self.width
        product = ops.dense(ops.linear(x, self.in_weight, self.in_bias))
        history = cache["conv"] if self.taps > 1 else None
        u = ops.causal_conv(product[:, R:2 * R], self.conv_weight, history, ctx.meta, bias=self.conv_bias)
        a, gated = ops.lru_gates(u, self.recur_weight, self.recur_bias, self.input_weight, self.input_bias, self.lam,
                                 self.rate)
        mixed = ops.lru_scan(a, gated, cache["state"], ctx.meta, product[:, :R], "gelu_tanh", ctx.act_dtype)
        return ops.linear(mixed, self.out_weight)


register_part("mixer", "rglru", GatedLinearRecurrentUnit)
