"""Linear attention with a fixed decay per head ("lightning attention"), as a state that is carried from token to token.

q = silu(W_q h), k = silu(W_k h) (heads x dim), v = silu(W_v h) (heads x value_dim), laid out head by head. Per head

    S_t = decay_h * S_(t-1) + k_t v_t^T,        o_t = S_t^T q_t

with no other scale. The concatenated heads go through an RMS norm over all of them together (weight `norm`),
times sigmoid(W_g h), then the output projection. The state starts at zero, is float32 [heads, dim, value_dim] for
each request, and everything behind the activations (products, decay, sums, the norm) is float32 in either
precision. The four projections are one matrix product: their weights are stacked at load.
"""

from __future__ import annotations

import torch

from ..config.model_config import PartSpec
from .base import FixedState, Mixer, ParamSpec, register_part


class DecayLinearAttention(Mixer):
    def __init__(self, spec: PartSpec) -> None:
        super().__init__(spec)
        p = spec.params
        self.hidden_size = int(p["hidden_size"])
        self.num_heads = int(p["num_heads"])
        self.head_dim = int(p["head_dim"])
        self.value_dim = int(p.get("value_dim") or self.head_dim)
        self.eps = float(p["eps"])
        self.decay_values = tuple(float(d) for d in p["decay"])
        if len(self.decay_values) != self.num_heads:
            raise ValueError(f"{len(self.decay_values)} decays for {self.num_heads} heads")
        self.in_weight = self.out_weight = self.norm_weight = self.decay = None

    def cache_requirement(self):
        return FixedState.of((self.num_heads, self.head_dim, self.value_dim))

    def param_specs(self):
        qk, v = self.num_heads * self.head_dim, self.num_heads * self.value_dim
        return {"q": ParamSpec((qk, self.hidden_size)), "k": ParamSpec((qk, self.hidden_size)),
                "v": ParamSpec((v, self.hidden_size)), "g": ParamSpec((v, self.hidden_size)),
                "o": ParamSpec((self.hidden_size, v)), "norm": ParamSpec((v,), "ones")}

    def load(self, tensors) -> None:
        stacked = [tensors[name] for name in "qkvg"]
        dtype = torch.float32 if any(t.dtype == torch.float32 for t in stacked) else stacked[0].dtype
        self.in_weight = torch.cat([t.to(dtype) for t in stacked], dim=0).contiguous()
        self.out_weight = tensors["o"].contiguous()
        self.norm_weight = tensors["norm"].contiguous()
        self.decay = torch.tensor(self.decay_values, dtype=torch.float64).to(torch.float32).to(self.out_weight.device)

    def prepare(self, ops) -> None:
        ops.prepare_linear(self.in_weight, role="qkv")
        ops.prepare_linear(self.out_weight, role="attn_out")

    def forward(self, ops, x, ctx, cache, writes_cache: bool):
        product = ops.dense(ops.linear(x, self.in_weight))
        mixed = ops.decay_scan(product, cache["state"], self.decay, ctx.meta, self.num_heads, self.head_dim, self.value_dim)
        first = self.num_heads * (2 * self.head_dim + self.value_dim)
        gates = product[:, first:first + self.num_heads * self.value_dim]
        normed = ops.rmsnorm_gate(mixed, self.norm_weight, self.eps, gates, ctx.act_dtype)
        return ops.linear(normed, self.out_weight)


class GatedLinearAttention(Mixer):
    """Linear attention whose state forgets channel by channel, by a gate computed from the token.

    q = W_q h * dim^(-1/2), k = W_k h (heads x dim), v = W_v h (heads x value_dim), no activation. A decay for
    every key channel, alpha = sigmoid(z)^(1 / tau) with z = W_a2 (W_a1 h) + b_a2 (a projection through `decay_rank`
    dimensions), laid out like k. Per head

        S_t = diag(alpha_t) S_(t-1) + k_t v_t^T,        o_t = S_t^T q_t.

    Every head's o goes through an RMS norm over its value_dim columns (weight `norm` [value_dim], the same for all
    heads), the heads side by side are multiplied by silu(W_g h) and projected by W_o. The state starts at zero and
    is float32 [heads, dim, value_dim] for each request; the decay (sigmoid, logarithm, power), the products k v^T
    and S^T q and the norm are float32 in either precision; z is not rounded on its way into the recurrence. q, k, v,
    the gate and W_a1 are one matrix product (their weights are stacked at load); z is made from its last columns,
    inside the scan for steps of few rows."""

    def __init__(self, spec: PartSpec) -> None:
        super().__init__(spec)
        p = spec.params
        self.hidden_size = int(p["hidden_size"])
        self.num_heads = int(p["num_heads"])
        self.head_dim = int(p["head_dim"])
        self.value_dim = int(p.get("value_dim") or self.head_dim)
        self.decay_rank = int(p["decay_rank"])
        self.tau = float(p["tau"])
        self.eps = float(p["eps"])
        if not self.tau > 0:
            raise ValueError("tau must be positive")
        self.q_scale = float(p.get("q_scale", self.head_dim ** -0.5))
        self.in_weight = self.up_weight = self.up_bias = self.out_weight = self.norm_weight = None

    def cache_requirement(self):
        return FixedState.of((self.num_heads, self.head_dim, self.value_dim))

    def param_specs(self):
        qk, v = self.num_heads * self.head_dim, self.num_heads * self.value_dim
        return {"q": ParamSpec((qk, self.hidden_size)), "k": ParamSpec((qk, self.hidden_size)),
                "v": ParamSpec((v, self.hidden_size)), "g": ParamSpec((v, self.hidden_size)),
                "o": ParamSpec((self.hidden_size, v)), "norm": ParamSpec((self.value_dim,), "ones"),
                "a1": ParamSpec((self.decay_rank, self.hidden_size)), "a2": ParamSpec((qk, self.decay_rank)),
                "a2.b": ParamSpec((qk,))}

    def load(self, tensors) -> None:
        stacked = [tensors[name] for name in "qkvg"]
        dtype = torch.float32 if any(t.dtype == torch.float32 for t in stacked) else stacked[0].dtype
        stacked.append(tensors["a1"])
        dtype = torch.float32 if any(t.dtype == torch.float32 for t in stacked) else stacked[0].dtype
        self.in_weight = torch.cat([t.to(dtype) for t in stacked], dim=0).contiguous()
        self.up_weight = tensors["a2"].contiguous()
        self.up_bias = tensors["a2.b"].float().contiguous()
        self.out_weight = tensors["o"].contiguous()
        self.norm_weight = tensors["norm"].contiguous()

    def prepare(self, ops) -> None:
        ops.prepare_linear(self.in_weight, role="qkv")
        ops.prepare_linear(self.out_weight, role="attn_out")

    def forward(self, ops, x, ctx, cache, writes_cache: bool):
        product = ops.dense(ops.linear(x, self.in_weight))
        first = self.num_heads * (2 * self.head_dim + self.value_dim)
        behind = first + self.num_heads * self.value_dim
        low = product[:, behind:behind + self.decay_rank]
        mixed = ops.gated_decay_scan(product, None, cache["state"], ctx.meta, self.num_heads, self.head_dim,
                                     self.value_dim, self.q_scale, self.tau, (low, self.up_weight, self.up_bias))
        gates = product[:, first:behind]
        normed = ops.rmsnorm_gate(mixed, self.norm_weight, self.eps, gates, ctx.act_dtype, group=self.value_dim,
                                  gate="silu")
        return ops.linear(normed, self.out_weight)


register_part("mixer", "decay_linear_attention", DecayLinearAttention)
register_part("mixer", "gated_linear_attention", GatedLinearAttention)
