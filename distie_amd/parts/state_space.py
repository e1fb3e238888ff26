"""A selective state-space mixer in its scalar-decay form (Mamba-2: Dao and Gu, "Transformers are SSMs: Generalized
Models and Efficient Algorithms Through Structured State Space Duality").

H heads of `value_dim` channels (inner = H * value_dim), a state of `state_size` rows a head, G groups of B and C
(head h reads group h // (H / G)). One projection of the mixer's input gives, side by side,

    z (inner) | x (inner) | B (G * state_size) | C (G * state_size) | dt (H).

x, B and C together go through a causal convolution over time for each channel (`conv` [channels, taps], bias `conv.b`;
the last column is the current token's; zeros before the start) and silu. With d = softplus(dt + dt_bias) and
a = exp(-exp(A_log) * d), per head

    S_t = a S_(t-1) + d * B_t x_t^T     (S is state_size x value_dim),        y_t = S_t^T C_t + D x_t.

The heads side by side are multiplied by silu(z), then RMS-normed in `norm_groups` equal parts (each by its own root
mean square) times `norm`, then projected by `o`: the gate stands in front of the norm. The state starts at zero and is
float32 [H, state_size, value_dim] for each request; the convolution's last taps - 1 inputs are state as well. Softplus,
both exponentials, the state, its products and sums, the gate and the norm are float32 in either precision.
"""

from __future__ import annotations

import torch

from ..config.model_config import PartSpec
from .base import FixedState, Mixer, ParamSpec, TensorDecl, register_part


class StateSpaceDuality(Mixer):
    def __init__(self, spec: PartSpec) -> None:
        super().__init__(spec)
        p = spec.params
        self.hidden_size = int(p["hidden_size"])
        self.num_heads = int(p["num_heads"])
        self.value_dim = int(p["value_dim"])
        self.state_size = int(p["state_size"])
        self.groups = int(p.get("groups") or 1)
        self.taps = int(p["conv_taps"])
        self.norm_groups = int(p.get("norm_groups") or 1)
        self.eps = float(p["eps"])
        self.inner = self.num_heads * self.value_dim
        if self.num_heads % self.groups or self.inner % self.norm_groups:
            raise ValueError("state-space mixer: heads must be a multiple of groups, heads * value_dim of norm_groups")
        if self.taps < 1:
            raise ValueError("the convolution has at least one tap")
        self.conv_channels = self.inner + 2 * self.groups * self.state_size
        self.in_width = 2 * self.inner + 2 * self.groups * self.state_size + self.num_heads
        self.in_weight = self.conv_weight = self.conv_bias = self.dt_bias = self.a_log = self.skip = None
        self.norm_weight = self.out_weight = None

    def cache_requirement(self):
        tensors = [TensorDecl("state", (self.num_heads, self.state_size, self.value_dim), torch.float32)]
        if self.taps > 1:
            tensors.append(TensorDecl("conv", (self.taps - 1, self.conv_channels), torch.float32))
        return FixedState(tuple(tensors))

    def param_specs(self):
        H, C = self.num_heads, self.hidden_size
        return {"in": ParamSpec((self.in_width, C)), "conv": ParamSpec((self.conv_channels, self.taps)),
                "conv.b": ParamSpec((self.conv_channels,)), "dt_bias": ParamSpec((H,)), "A_log": ParamSpec((H,)),
                "D": ParamSpec((H,)), "norm": ParamSpec((self.inner,), "ones"), "o": ParamSpec((C, self.inner))}

    def load(self, tensors) -> None:
        self.in_weight = tensors["in"].contiguous()
        self.conv_weight = tensors["conv"].contiguous()
        self.conv_bias = tensors["conv.b"].float().contiguous()
        self.dt_bias = tensors["dt_bias"].float().contiguous()
        self.a_log = tensors["A_log"].float().contiguous()
        self.skip = tensors["D"].float().contiguous()
        self.norm_weight = tensors["norm"].contiguous()
        self.out_weight = tensors["o"].contiguous()

    def prepare(self, ops) -> None:
        self.capturable = bool(ops.ssm_scan_captures(self.state_size))
        ops.prepare_linear(self.in_weight, role="qkv")
        ops.prepare_linear(self.out_weight, role="attn_out")

    def forward(self, ops, x, ctx, cache, writes_cache: bool):
        inner, channels = self.inner, self.conv_channels
        product = ops.dense(ops.linear(x, self.in_weight))
        history = cache["conv"] if self.taps > 1 else None
        xbc = ops.causal_conv(product[:, inner:inner + channels], self.conv_weight, history, ctx.meta,
                              bias=self.conv_bias, act="silu")
        y = ops.ssm_scan(xbc, product[:, inner + channels:inner + channels + self.num_heads], self.dt_bias, self.a_log,
                         self.skip, cache["state"], ctx.meta, self.num_heads, self.value_dim, self.state_size, self.groups)
        normed = ops.rmsnorm_gate(y, self.norm_weight, self.eps, product[:, :inner], ctx.act_dtype,
                                  group=inner // self.norm_groups, gate="silu", gate_first=True)
        return ops.linear(normed, self.out_weight)


register_part("mixer", "state_space_duality", StateSpaceDuality)
