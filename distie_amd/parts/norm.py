"""Norms. RMS norm: y = weight * x * rsqrt(mean(x^2) + eps), statistics in float32
(worker/src/inference/qwen2/model.py:77-90). The reference multiplies by the weight
after rounding back to the model dtype; here the product is rounded once."""

from __future__ import annotations

import torch

from .base import Norm, ParamSpec, register_part


class RMSNorm(Norm):
    """`offset`: what is added to the stored weight (1 for designs whose files hold the weight minus one:
    y = x / rms(x) * (1 + w)); the sum is made once at load, in float32, and is the weight from then on."""

    fused_kind = "rms"          # what `Ops.hyper_step` calls this norm when it computes it while reading the streams

    def __init__(self, spec) -> None:
        super().__init__(spec)
        self.size = int(spec.params["size"])
        self.eps = float(spec.params["eps"])
        self.weight_name = spec.params.get("weight_name", "weight")      # the tensor's name behind the prefix
        self.offset = float(spec.params.get("offset") or 0.0)
        self.weight = None

    def param_specs(self):
        return {self.weight_name: ParamSpec((self.size,), "zeros" if self.offset else "ones")}

    def load(self, tensors) -> None:
        self.weight = tensors[self.weight_name].contiguous()
        if self.offset:
            self.weight = (self.weight.float() + self.offset).contiguous()

    def apply(self, ops, x, out_dtype):
        return ops.rmsnorm(x, self.weight, self.eps, out_dtype)

    def add_apply(self, ops, residual, delta, out_dtype):
        return ops.add_rmsnorm(residual, delta, self.weight, self.eps, out_dtype)


class LayerNorm(Norm):
    """Centred norm with a weight and no bias: y = (x - mean) / sqrt(var + eps) * weight, where var is the mean of
    the squared deviations; statistics in float32."""

    fused_kind = "layer"

    def __init__(self, spec) -> None:
        super().__init__(spec)
        self.size = int(spec.params["size"])
        self.eps = float(spec.params["eps"])
        self.weight = None
        self._one = None

    def param_specs(self):
        return {self.spec.params.get("weight_name", "weight"): ParamSpec((self.size,), "ones")}

    def load(self, tensors) -> None:
        self.weight = tensors[self.spec.params.get("weight_name", "weight")].contiguous()
        self._one = torch.ones(1, dtype=torch.float32, device=self.weight.device)

    def apply(self, ops, x, out_dtype):
        return ops.layernorm(x, self.weight, self.eps, out_dtype)

    def add_apply(self, ops, residual, delta, out_dtype):
        rows, width = residual.shape
        return ops.hyper_step(residual.view(rows, 1, width), delta=delta, mix=self._one.view(1, 1), write=self._one,
                              read=self._one, norm_weight=self.weight, norm="layer", eps=self.eps, out_dtype=out_dtype)[1]


register_part("norm", "rmsnorm", RMSNorm)
register_part("norm", "layernorm", LayerNorm)
