"""Feed-forwards. Gated: down(silu(gate x) * up x), no biases
(worker/src/inference/qwen2/model.py:228-236). Gate and up are one matrix product:
their weights are stacked at load."""

from __future__ import annotations

import torch

from .base import FeedForward, ParamSpec, register_part


class SwiGLU(FeedForward):
    """down(act(gate x) * up x), act = silu unless `activation` names another ("gelu_tanh"); the tensors' names
    behind the prefix come from the spec (`gate_name`, `up_name`, `down_name`)."""

    def __init__(self, spec) -> None:
        super().__init__(spec)
        self.hidden_size = int(spec.params["hidden_size"])
        self.intermediate_size = int(spec.params["intermediate_size"])
        self.gate_name = spec.params.get("gate_name", "gate_proj.weight")
        self.up_name = spec.params.get("up_name", "up_proj.weight")
        self.down_name = spec.params.get("down_name", "down_proj.weight")
        self.activation = str(spec.params.get("activation", "silu"))
        if self.activation not in ("silu", "gelu_tanh", "relu", "relu2"):
            raise ValueError(f"no gated activation named {self.activation!r}")
        self.gate_up_weight = self.down_weight = None

    def param_specs(self):
        return {
            self.gate_name: ParamSpec((self.intermediate_size, self.hidden_size)),
            self.up_name: ParamSpec((self.intermediate_size, self.hidden_size)),
            self.down_name: ParamSpec((self.hidden_size, self.intermediate_size)),
        }

    def load(self, tensors) -> None:
        gate, up = tensors[self.gate_name], tensors[self.up_name]
        dtype = torch.float32 if torch.float32 in (gate.dtype, up.dtype) else gate.dtype
        self.gate_up_weight = torch.cat([gate.to(dtype), up.to(dtype)], dim=0).contiguous()
        self.down_weight = tensors[self.down_name].contiguous()

    def prepare(self, ops) -> None:
        ops.prepare_linear(self.gate_up_weight, gated=True, role="gate_up")
        ops.prepare_linear(self.down_weight, role="down")

    def forward(self, ops, x, ctx):
        if self.activation == "silu":
            return ops.linear(ops.linear_silu_mul(x, self.gate_up_weight), self.down_weight)
        return ops.linear(ops.linear_glu(x, self.gate_up_weight, self.activation), self.down_weight)


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


class RoutedExperts(FeedForward):
    """A mixture of gated feed-forwards. A router (`router` [E, C], bias `router.b`) gives every token a logit for
    each of the E experts, in float32; the token uses the `top` experts with the largest logits, weighted by the
    softmax over those logits alone. Expert e is down_e(silu(gate_e x) * up_e x) with tensors `e<e>.gate`, `e<e>.up`
    [F, C] and `e<e>.down` [C, F], no biases. `shared_size` > 0: one more expert of that size (`shared.*`) that every
    token uses with weight one.

    Variants, each a parameter: `router_bias` False: no `router.b`. `scoring` "sigmoid": an expert's weight is
    sigmoid(z) of its own logit, not renormalised over the chosen (the `top` largest scores are the `top` largest
    logits). `weight_on` "input": the weight multiplies what the expert reads, expert(w x), instead of what it
    returns. `activation` "clamped_glu": with g = min(gate x, limit) and u = clamp(up x, -limit, limit) the hidden
    values are g * sigmoid(slope * g) * (u + up_shift). Since gate and up are linear, gate (w x) = w (gate x): the
    weight is applied to the stacked product's columns, in float32, in front of the clamps.

    All experts' gate and up weights are stacked into one matrix (the shared expert's behind them), all down weights
    side by side into another: one product gives every expert's hidden values for every token, those of the experts a
    token did not choose are multiplied by zero and the chosen ones by their weight, and the second product adds
    the experts up. What a token's unchosen experts compute is wasted (E / top times the products of a grouped
    kernel); no host-side decision depends on the routing, so the step can be recorded into a graph."""

    def __init__(self, spec) -> None:
        super().__init__(spec)
        p = spec.params
        self.hidden_size = int(p["hidden_size"])
        self.num_experts = int(p["num_experts"])
        self.top = int(p["top"])
        self.expert_size = int(p["expert_size"])
        self.shared_size = int(p.get("shared_size") or 0)
        if not 1 <= self.top <= self.num_experts:
            raise ValueError("a token uses between one and all of the experts")
        self.has_router_bias = bool(p.get("router_bias", True))
        self.scoring = str(p.get("scoring", "softmax"))
        self.weight_on = str(p.get("weight_on", "output"))
        self.activation = str(p.get("activation", "silu_glu"))
        if self.scoring not in ("softmax", "sigmoid") or self.weight_on not in ("input", "output") or \
                self.activation not in ("silu_glu", "clamped_glu"):
            raise ValueError("routed experts: scoring is softmax or sigmoid, weight_on input or output, activation "
                             "silu_glu or clamped_glu")
        self.plain = self.activation == "silu_glu" and self.weight_on == "output"
        if not self.plain and self.shared_size:
            raise ValueError("routed experts: a shared expert goes with the plain gated activation only")
        self.limit = float(p.get("limit") or 0.0)
        self.slope = float(p.get("slope", 1.0))
        self.up_shift = float(p.get("up_shift", 0.0))
        if self.activation == "clamped_glu" and not self.limit > 0:
            raise ValueError("routed experts: the clamped activation needs a positive limit")
        self.router_weight = self.router_bias = self.gate_up_weight = self.down_weight = None

    def _experts(self):
        return [(f"e{e}.", self.expert_size) for e in range(self.num_experts)] + \
            ([("shared.", self.shared_size)] if self.shared_size else [])

    def param_specs(self):
        specs = {"router": ParamSpec((self.num_experts, self.hidden_size))}
        if self.has_router_bias:
            specs["router.b"] = ParamSpec((self.num_experts,))
        for prefix, size in self._experts():
            specs[prefix + "gate"] = ParamSpec((size, self.hidden_size))
            specs[prefix + "up"] = ParamSpec((size, self.hidden_size))
            specs[prefix + "down"] = ParamSpec((self.hidden_size, size))
        return specs

    def load(self, tensors) -> None:
        self.router_weight = tensors["router"].contiguous()
        self.router_bias = tensors["router.b"].float().contiguous() if self.has_router_bias else None
        names = [prefix for prefix, _ in self._experts()]
        stacked = [tensors[n + "gate"] for n in names] + [tensors[n + "up"] for n in names]
        dtype = torch.float32 if any(t.dtype == torch.float32 for t in stacked) else stacked[0].dtype
        self.gate_up_weight = torch.cat([t.to(dtype) for t in stacked], dim=0).contiguous()
        down = [tensors[n + "down"] for n in names]
        dtype = torch.float32 if any(t.dtype == torch.float32 for t in down) else down[0].dtype
        self.down_weight = torch.cat([t.to(dtype) for t in down], dim=1).contiguous()

    def prepare(self, ops) -> None:
        ops.prepare_linear(self.gate_up_weight, gated=self.plain, role="gate_up")
        ops.prepare_linear(self.down_weight, role="down")

    def forward(self, ops, x, ctx):
        x = ops.dense(x)
        if not self.plain:
            hidden = ops.route_experts_glu(x, self.router_weight, self.router_bias, self.top, self.scoring,
                                           ops.linear(x, self.gate_up_weight), self.num_experts, self.expert_size,
                                           self.limit if self.activation == "clamped_glu" else None, self.slope,
                                           self.up_shift, self.weight_on == "input")
            return ops.linear(hidden, self.down_weight)
        experts, gates = ops.route_topk(x, self.router_weight, self.router_bias, self.top, self.scoring)
        hidden = ops.dense(ops.linear_silu_mul(x, self.gate_up_weight))
        hidden = ops.route_scale(hidden, experts, gates, self.num_experts, self.expert_size)
        return ops.linear(hidden, self.down_weight)


register_part("feed_forward", "swiglu", SwiGLU)
register_part("feed_forward", "routed_experts", RoutedExperts)
register_part("feed_forward", "dense_mlp", DenseMLP)
