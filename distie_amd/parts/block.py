"""Arrangements. Pre-norm residual: h += mixer(norm(h)); h += feed_forward(norm(h))
(worker/src/inference/qwen2/model.py:279-290). Each sub-layer's output is left pending
on the stream; the next norm adds it while it reads the stream."""

from __future__ import annotations

import torch

from .base import Block, CacheNeeds, FixedState, ParamSpec, ResidualStream, StepContext, TensorDecl, register_part


class PreNormResidual(Block):
    CHILDREN = {"mixer_norm": "norm", "mixer": "mixer", "feed_forward_norm": "norm", "feed_forward": "feed_forward"}

    def forward(self, ops, stream: ResidualStream, ctx: StepContext, cache, writes_cache: bool) -> None:
        normed = self.mixer_norm.of_stream(ops, stream, ctx.act_dtype)
        stream.pending = self.mixer.forward(ops, normed, ctx, cache["mixer"], writes_cache)
        normed = self.feed_forward_norm.of_stream(ops, stream, ctx.act_dtype)
        stream.pending = self.feed_forward.forward(ops, normed, ctx)


class HyperConnections(Block):
    """Pre-norm sub-layers on several residual streams ("hyper-connections"), with two optional extras around
    each sub-layer.

    There are S copies x_1 .. x_S of the residual, all equal to the embedding output at the start. Sub-layer q
    (1: the mixer, 2: the feed-forward, which a layer may lack) owns a read vector `hc<q>.in` [S], a write vector
    `hc<q>.out` [S] and a matrix `hc<q>.mix` [S, S] indexed [from, to]:

        u = sum_s in[s] x_s;   h = norm(u);   y = sublayer(h);   x_j <- sum_s mix[s, j] x_s + out[j] * y

    for all j at once from the old streams. After the last layer the residual is the sum of the streams. The
    streams are float32; a sub-layer's y stays pending and is written by the same kernel that reads the
    streams for the next sub-layer (`Ops.hyper_step`). `streams` None: one stream, read, written and kept
    with weight 1 (the plain pre-norm residual), and no such tensors.

    `gated` : y is multiplied element by element by sigmoid(W h + b) (`rg<q>`, `rg<q>.b`), h being the normed
    input of the sub-layer.
    `input_taps` > 0: the mixer reads h + conv(h) instead of h, a causal convolution over time with a filter of
    that many taps for each channel (`canon1` [C, taps]); the last taps - 1 rows of h are part of a request's
    state. The gate above reads h before this convolution."""

    CHILDREN = {"mixer_norm": "norm", "mixer": "mixer", "feed_forward_norm": "norm", "feed_forward": "feed_forward"}
    OPTIONAL = ("feed_forward_norm", "feed_forward")

    def __init__(self, spec, parts) -> None:
        super().__init__(spec, parts)
        p = spec.params
        self.width = int(p["hidden_size"])
        self.streams = p.get("streams")
        self.count = int(self.streams) if self.streams is not None else 1
        self.gated = bool(p.get("gated", False))
        self.input_taps = int(p.get("input_taps") or 0)
        if self.count < 1 or self.input_taps < 0:
            raise ValueError("streams must be >= 1 and input_taps >= 0")
        if (self.feed_forward is None) != (self.feed_forward_norm is None):
            raise ValueError("a feed-forward and its norm come together")
        self.subs = (1, 2) if self.feed_forward is not None else (1,)
        self.read, self.write, self.mix, self.gate_weight, self.gate_bias = {}, {}, {}, {}, {}
        self.input_filter = None
        self._ones = None

    def param_specs(self):
        specs = {}
        S, C = self.count, self.width
        for q in self.subs:
            if self.streams is not None:
                specs.update({f"hc{q}.in": ParamSpec((S,), "ones"), f"hc{q}.out": ParamSpec((S,), "ones"),
                              f"hc{q}.mix": ParamSpec((S, S), "eye")})
        if self.input_taps:
            specs["canon1"] = ParamSpec((C, self.input_taps))
        for q in self.subs:
            if self.gated:
                specs.update({f"rg{q}": ParamSpec((C, C)), f"rg{q}.b": ParamSpec((C,))})
        return specs

    def load(self, tensors) -> None:
        device = next(iter(tensors.values())).device if tensors else None
        for q in self.subs:
            if self.streams is not None:
                self.read[q] = tensors[f"hc{q}.in"].float().contiguous()
                self.write[q] = tensors[f"hc{q}.out"].float().contiguous()
                self.mix[q] = tensors[f"hc{q}.mix"].float().contiguous()
                device = self.read[q].device
            if self.gated:
                self.gate_weight[q] = tensors[f"rg{q}"].contiguous()
                self.gate_bias[q] = tensors[f"rg{q}.b"].float().contiguous()
        if self.input_taps:
            self.input_filter = tensors["canon1"].contiguous()
        self._device = device

    def _constants(self, device):
        if self._ones is None or self._ones.device != device:
            self._ones = torch.ones(self.count, dtype=torch.float32, device=device)
            if self.streams is None:
                for q in self.subs:
                    self.read[q] = self.write[q] = self._ones
                    self.mix[q] = self._ones.view(1, 1)
        return self._ones

    def prepare(self, ops) -> None:
        for q in self.subs:
            if self.gated:
                ops.prepare_linear(self.gate_weight[q], role="residual_gate")

    def cache_requirements(self):
        needs = super().cache_requirements()
        if self.input_taps > 1:
            needs["input_conv"] = FixedState((TensorDecl("history", (self.input_taps - 1, self.width), torch.float32),))
        return needs

    def _enter(self, ops, stream: ResidualStream, q: int, norm, act_dtype):
        """Write what is pending on the streams, read them for sub-layer q -> the sub-layer's normed input."""
        kind = getattr(norm, "fused_kind", None)
        common = dict(read=self.read[q], norm_weight=norm.weight if kind else None, norm=kind or "none",
                      eps=norm.eps if kind else 0.0, out_dtype=act_dtype if kind else torch.float32)
        lanes = stream.lanes
        if lanes is None:
            if stream.pending is not None:
                raise ValueError("streams start from a residual with nothing pending on it")
            x, h = ops.hyper_step(None, init=stream.hidden, **common)
            stream.lanes = {"x": x, "pending": None}
            stream.settle = self._settle
        elif lanes["pending"] is None:
            _, h = ops.hyper_step(lanes["x"], **common)
        else:
            delta, gate, mix, write = lanes["pending"]
            lanes["pending"] = None
            _, h = ops.hyper_step(lanes["x"], delta=delta, gate=gate, mix=mix, write=write, **common)
        return h if kind else norm.apply(ops, h, act_dtype)

    def _settle(self, ops, stream: ResidualStream) -> None:
        lanes, stream.lanes = stream.lanes, None
        ones = self._constants(lanes["x"].device)
        if lanes["pending"] is None:
            _, total = ops.hyper_step(lanes["x"], read=ones)
        else:
            delta, gate, mix, write = lanes["pending"]
            _, total = ops.hyper_step(lanes["x"], delta=delta, gate=gate, mix=mix, write=write, read=ones)
        stream.hidden, stream.pending = total, None

    def forward(self, ops, stream: ResidualStream, ctx: StepContext, cache, writes_cache: bool) -> None:
        self._constants(stream.hidden.device)
        h = self._enter(ops, stream, 1, self.mixer_norm, ctx.act_dtype)
        gate = ops.linear(h, self.gate_weight[1], self.gate_bias[1]) if self.gated else None
        if self.input_taps:
            history = cache["input_conv"]["history"] if self.input_taps > 1 else None
            h = ops.causal_conv(h, self.input_filter, history, ctx.meta, residual=True)
        y = self.mixer.forward(ops, h, ctx, cache["mixer"], writes_cache)
        stream.lanes["pending"] = (y, gate, self.mix[1], self.write[1])
        if self.feed_forward is None:
            return
        h = self._enter(ops, stream, 2, self.feed_forward_norm, ctx.act_dtype)
        gate = ops.linear(h, self.gate_weight[2], self.gate_bias[2]) if self.gated else None
        y = self.feed_forward.forward(ops, h, ctx)
        stream.lanes["pending"] = (y, gate, self.mix[2], self.write[2])


class SandwichResidual(Block):
    """A norm in front of each sub-layer and another behind it, the second inside the residual branch:

        x <- x + mixer_post_norm(mixer(mixer_norm(x)));   x <- x + feed_forward_post_norm(feed_forward(feed_forward_norm(x)))

    All four are RMS norms. A layer may have no feed-forward. A sub-layer's result stays pending with the norm that
    belongs behind it; the norm in front of the next sub-layer (or the model's last norm) adds it while it reads the
    residual (`Ops.add_normed_rmsnorm`: one kernel between two sub-layers)."""

    CHILDREN = {"mixer_norm": "norm", "mixer": "mixer", "mixer_post_norm": "norm",
                "feed_forward_norm": "norm", "feed_forward": "feed_forward", "feed_forward_post_norm": "norm"}
    OPTIONAL = ("feed_forward_norm", "feed_forward", "feed_forward_post_norm")

    def __init__(self, spec, parts) -> None:
        super().__init__(spec, parts)
        present = [self.feed_forward is None, self.feed_forward_norm is None, self.feed_forward_post_norm is None]
        if any(present) and not all(present):
            raise ValueError("a feed-forward and its two norms come together")
        for norm in (self.mixer_norm, self.mixer_post_norm, self.feed_forward_norm, self.feed_forward_post_norm):
            if norm is not None and getattr(norm, "fused_kind", None) != "rms":
                raise ValueError("the sandwich arrangement takes RMS norms")

    @staticmethod
    def _settle(ops, stream: ResidualStream) -> None:
        lanes, stream.lanes = stream.lanes, None
        if lanes and lanes.get("pending") is not None:
            delta, post = lanes["pending"]
            ops.add_normed(stream.hidden, delta, post.weight, post.eps)

    def _enter(self, ops, stream: ResidualStream, norm, act_dtype):
        """Add what is pending, through the norm behind its sub-layer, and norm the residual for the next one."""
        if stream.pending is not None:
            raise ValueError("the sandwich arrangement starts from a residual with nothing pending on it")
        pending = stream.lanes.get("pending") if stream.lanes else None
        if pending is None:
            return norm.apply(ops, stream.hidden, act_dtype)
        delta, post = pending
        stream.lanes["pending"] = None
        return ops.add_normed_rmsnorm(stream.hidden, delta, post.weight, post.eps, norm.weight, norm.eps, act_dtype)

    def forward(self, ops, stream: ResidualStream, ctx: StepContext, cache, writes_cache: bool) -> None:
        h = self._enter(ops, stream, self.mixer_norm, ctx.act_dtype)
        y = self.mixer.forward(ops, h, ctx, cache["mixer"], writes_cache)
        stream.lanes = {"pending": (y, self.mixer_post_norm)}
        stream.settle = self._settle
        if self.feed_forward is None:
            return
        h = self._enter(ops, stream, self.feed_forward_norm, ctx.act_dtype)
        y = self.feed_forward.forward(ops, h, ctx)
        stream.lanes["pending"] = (y, self.feed_forward_post_norm)


class BranchNormResidual(Block):
    """A norm on each sub-layer's result only, inside the residual branch; the sub-layers read the residual itself:

        x <- x + mixer_post_norm(mixer(x));   x <- x + feed_forward_post_norm(feed_forward(x))

    Both are RMS norms. A layer may have no feed-forward. The residual is float32; a sub-layer reads it rounded to
    the activations' precision (itself in a float32 engine). A sub-layer's result stays pending with its norm, and
    the read for the next sub-layer adds it (`Ops.add_normed_read`: one kernel between two sub-layers); the model's
    last norm finds the plain sum through `ResidualStream.close`."""

    CHILDREN = {"mixer": "mixer", "mixer_post_norm": "norm", "feed_forward": "feed_forward",
                "feed_forward_post_norm": "norm"}
    OPTIONAL = ("feed_forward", "feed_forward_post_norm")

    def __init__(self, spec, parts) -> None:
        super().__init__(spec, parts)
        if (self.feed_forward is None) != (self.feed_forward_post_norm is None):
            raise ValueError("a feed-forward and its norm come together")
        for norm in (self.mixer_post_norm, self.feed_forward_post_norm):
            if norm is not None and getattr(norm, "fused_kind", None) != "rms":
                raise ValueError("the branch-norm arrangement takes RMS norms")

    _settle = staticmethod(SandwichResidual._settle)

    @staticmethod
    def _read(ops, stream: ResidualStream, act_dtype):
        """Add what is pending, through its norm, and hand out the residual in the activations' precision."""
        if stream.pending is not None:
            raise ValueError("the branch-norm arrangement starts from a residual with nothing pending on it")
        pending = stream.lanes.get("pending") if stream.lanes else None
        if pending is None:
            return ops.read_residual(stream.hidden, act_dtype)
        delta, post = pending
        stream.lanes["pending"] = None
        return ops.add_normed_read(stream.hidden, delta, post.weight, post.eps, act_dtype)

    def forward(self, ops, stream: ResidualStream, ctx: StepContext, cache, writes_cache: bool) -> None:
        h = self._read(ops, stream, ctx.act_dtype)
        y = self.mixer.forward(ops, h, ctx, cache["mixer"], writes_cache)
        stream.lanes = {"pending": (y, self.mixer_post_norm)}
        stream.settle = self._settle
        if self.feed_forward is None:
            return
        h = self._read(ops, stream, ctx.act_dtype)
        y = self.feed_forward.forward(ops, h, ctx)
        stream.lanes["pending"] = (y, self.feed_forward_post_norm)


register_part("block", "prenorm_residual", PreNormResidual)
register_part("block", "branch_norm_residual", BranchNormResidual)
register_part("block", "sandwich_residual", SandwichResidual)
register_part("block", "hyper_connections", HyperConnections)
