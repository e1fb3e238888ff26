"""Grouped-query attention over the paged cache with what some designs put around it:

* a short causal convolution over time on every channel of q, k and v, directly behind the projections and
  before the rotation (`conv_taps`; filters `<q|k|v>.conv` [channels, taps], no bias); the last taps - 1
  projected rows of a request are part of its state;
* a rotation of only the first dimensions of a head, with scaled frequencies (whatever the `position` part gives:
  its frequencies and the factor on cosine and sine);
* keys of size `head_dim` and values of another size `value_dim`;
* an output gate: the concatenated heads times sigmoid(W_g h), h being the mixer's input, before the output projection
  (`output_gate` True: a gate for every value column, `g` [heads * value_dim, C]; "head": one number for each head,
  `g` [heads, C]);
* biases on q, k and v (`bias`: tensors `<q|k|v>.b`, added in the projection);
* a query temperature by position (`q_temp` = {coef, every}): q at position p is multiplied by
  1 + coef * ln(floor((p + 1) / every) + 1), in float32, so that later queries weigh their keys more sharply;
* a norm on every head of q and k (`qk_norm` = {eps, offset}): RMS norm over the head's `head_dim` values with the
  weights `q.norm` and `k.norm` [head_dim] (each shared by all heads; `offset` is added to the stored weight),
  behind the convolution and before the rotation, in float32;
* a sink in the softmax (`sink`): a learned number per query head (`sink` [heads]) whose exponential is one more term
  of the denominator; it has no key and no value, is not scaled, and counts once whatever the window;
* keys and values borrowed from an earlier layer (`kv_from`): such a layer has no k or v tensors; it reads the other
  layer's cache (keys as they lie there, convolved and rotated; values convolved) with queries, window and everything
  else of its own. The lending layer must keep its pages for as long as a borrower looks back (`keep`).

score = q . k * scale over the keys j with 0 <= i - j < window (all j <= i without a window), ordinary softmax.
The projections (and the gate's) are one matrix product: their weights are stacked at load. The kernels
work on one head size: max(head_dim, value_dim) rounded up to what the matrix-core kernels take, with zeros in the
places beyond (they add nothing to a score and come out as zeros that are dropped).
"""

from __future__ import annotations

import bisect

import torch

from ..config.model_config import PartSpec
from ..kernels.interface import ScoreExtras
from .attention import PagedKV, context_classes
from .base import Borrowed, CacheNeeds, FixedState, Mixer, ParamSpec, TensorDecl, build_part, register_part


def padded_head_dim(dim: int, value_dim: int) -> int:
    """The head size the attention kernels run at: a multiple of 32 up to 128 (every kernel takes those, in
    either precision), a multiple of 16 beyond."""
    widest = max(dim, value_dim)
    step = 32 if widest <= 128 else 16
    return -(-widest // step) * step


class ConvGatedAttention(Mixer):
    FIRST_CONTEXT = 1024

    def __init__(self, spec: PartSpec) -> None:
        super().__init__(spec)
        p = spec.params
        self.hidden_size = int(p["hidden_size"])
        self.num_heads = int(p["num_heads"])
        self.num_kv_heads = int(p["num_kv_heads"])
        self.head_dim = int(p["head_dim"])
        self.value_dim = int(p.get("value_dim") or self.head_dim)
        self.conv_taps = int(p.get("conv_taps") or 0)
        self.window = p.get("window")
        self.keep = p.get("keep", self.window)          # how far back the cache must reach (None: everything)
        self.scale = float(p.get("scale", self.head_dim ** -0.5))
        gate = p.get("output_gate", True)
        self.output_gate = bool(gate)
        self.gate_per_head = gate == "head"
        self.kv_from = p.get("kv_from")
        self.bias = bool(p.get("bias", False))
        temp = p.get("q_temp")
        self.q_temp = (float(temp["coef"]), int(temp["every"])) if temp else None
        if self.q_temp is not None and self.q_temp[1] < 1:
            raise ValueError("q_temp.every must be >= 1")
        if self.num_heads % self.num_kv_heads:
            raise ValueError("num_heads must be a multiple of num_kv_heads")
        norm = p.get("qk_norm")
        self.qk_norm = (float(norm["eps"]), float(norm.get("offset") or 0.0)) if norm else None
        self.sink = bool(p.get("sink", False))
        self.q_norm_weight = self.k_norm_weight = self.extras = None
        self.position = build_part("position", p.get("position") or PartSpec("none"))
        self.padded_dim = padded_head_dim(self.head_dim, self.value_dim)
        self.has_kv = self.kv_from is None
        q, k, v = self.num_heads * self.head_dim, self.num_kv_heads * self.head_dim, self.num_kv_heads * self.value_dim
        self.conv_channels = q + (k + v if self.has_kv else 0)
        self.out_width = self.num_heads * self.value_dim
        self.gate_width = self.num_heads if self.gate_per_head else self.out_width
        self.in_weight = self.in_bias = self.conv_weight = self.out_weight = None

    def _projections(self):
        q, k, v = self.num_heads * self.head_dim, self.num_kv_heads * self.head_dim, self.num_kv_heads * self.value_dim
        return [("q", q)] + ([("k", k), ("v", v)] if self.has_kv else [])

    def cache_requirement(self):
        paged = PagedKV(self.num_kv_heads, self.padded_dim, self.keep) if self.has_kv else Borrowed(int(self.kv_from))
        state = None
        if self.conv_taps > 1:
            state = FixedState((TensorDecl("conv", (self.conv_taps - 1, self.conv_channels), torch.float32),))
        return CacheNeeds(paged, state)

    def param_specs(self):
        specs = {}
        for name, rows in self._projections():
            specs[name] = ParamSpec((rows, self.hidden_size))
        if self.bias:
            for name, rows in self._projections():
                specs[name + ".b"] = ParamSpec((rows,))
        if self.conv_taps:
            for name, rows in self._projections():
                specs[name + ".conv"] = ParamSpec((rows, self.conv_taps))
        if self.qk_norm is not None:
            init = "zeros" if self.qk_norm[1] else "ones"
            specs["q.norm"] = ParamSpec((self.head_dim,), init)
            if self.has_kv:
                specs["k.norm"] = ParamSpec((self.head_dim,), init)
        if self.sink:
            specs["sink"] = ParamSpec((self.num_heads,))
        if self.output_gate:
            specs["g"] = ParamSpec((self.gate_width, self.hidden_size))
        specs["o"] = ParamSpec((self.hidden_size, self.out_width))
        return specs

    def load(self, tensors) -> None:
        stacked = [tensors[name] for name, _ in self._projections()] + ([tensors["g"]] if self.output_gate else [])
        dtype = torch.float32 if any(t.dtype == torch.float32 for t in stacked) else stacked[0].dtype
        self.in_weight = torch.cat([t.to(dtype) for t in stacked], dim=0).contiguous()
        if self.bias:
            biases = [tensors[name + ".b"].float() for name, _ in self._projections()]
            if self.output_gate:
                biases.append(torch.zeros(self.gate_width, dtype=torch.float32, device=biases[0].device))
            self.in_bias = torch.cat(biases).contiguous()
        if self.conv_taps:
            self.conv_weight = torch.cat([tensors[name + ".conv"] for name, _ in self._projections()], dim=0).contiguous()
        self.out_weight = tensors["o"].contiguous()
        if self.qk_norm is not None:
            self.q_norm_weight = (tensors["q.norm"].float() + self.qk_norm[1]).contiguous()
            if self.has_kv:
                self.k_norm_weight = (tensors["k.norm"].float() + self.qk_norm[1]).contiguous()
        if self.sink:
            self.extras = ScoreExtras(sinks=tensors["sink"].float().contiguous())
        self.position.to_device(self.out_weight.device)

    def prepare(self, ops) -> None:
        ops.prepare_linear(self.in_weight, role="qkv")
        ops.prepare_linear(self.out_weight, role="attn_out")

    def capture_context(self, longest: int, limit: int):
        classes = context_classes(limit, self.FIRST_CONTEXT)
        return classes[min(bisect.bisect_left(classes, longest), len(classes) - 1)]

    def forward(self, ops, x, ctx, cache, writes_cache: bool):
        product = ops.linear(x, self.in_weight, self.in_bias)
        if self.output_gate or self.conv_taps:
            product = ops.dense(product)            # the gate's columns are read here; a filter reads earlier rows
        k_cache, v_cache = cache["k"], cache["v"]
        state = cache["conv"] if self.conv_taps > 1 else None
        q = ops.conv_rope_kv_write(product, self.conv_weight, state, ctx.meta, cache.group, k_cache, v_cache,
                                   self.position.rotary(), self.position.rotary_magnitude(), self.num_heads,
                                   self.num_kv_heads, self.head_dim, self.value_dim, self.padded_dim, self.has_kv,
                                   writes_cache and self.has_kv, self.q_temp,
                                   None if self.qk_norm is None else (self.q_norm_weight, self.k_norm_weight, self.qk_norm[0]))
        mixed = ops.paged_attention(q, ctx.meta, cache.group, k_cache, v_cache, self.num_heads, self.num_kv_heads,
                                    self.padded_dim, self.scale, self.window, self.extras)
        if self.output_gate:
            gates = product[:, self.conv_channels:self.conv_channels + self.gate_width]
            if self.gate_per_head:
                mixed = ops.sigmoid_gate(mixed, self.num_heads, self.padded_dim, self.value_dim, gates, per_head=True)
            else:
                mixed = ops.sigmoid_gate(mixed, self.num_heads, self.padded_dim, self.value_dim, gates)
        elif self.padded_dim != self.value_dim:
            mixed = ops.sigmoid_gate(mixed, self.num_heads, self.padded_dim, self.value_dim, None)
        return ops.linear(mixed, self.out_weight)


register_part("mixer", "conv_gated_attention", ConvGatedAttention)
