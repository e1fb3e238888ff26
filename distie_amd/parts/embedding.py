"""The two ends of the model: the token embedding, h0[t] = E[ids[t]], and the head,
logits = h W^T without a bias (worker/src/inference/qwen2/model.py:297-303, 375-380). A head that is
tied to the embedding declares no tensor of its own and asks for the embedding's by name, so both use
one buffer (model.py:302-303); a file may still hold a copy under the head's name, which is ignored."""

from __future__ import annotations

from .base import Embedding, Head, ParamSpec, build_part, register_part


class TokenEmbedding(Embedding):
    """`norm` (a norm's PartSpec, with its own prefix): the looked-up rows go through it before they become the
    residual stream, which stays float32. `scale`: what the looked-up rows are multiplied by, in float32."""

    def __init__(self, spec) -> None:
        super().__init__(spec)
        self.vocab_size = int(spec.params["vocab_size"])
        self.hidden_size = int(spec.params["hidden_size"])
        self.weight_name = spec.params.get("weight_name", "weight")      # the tensor's name behind the prefix
        self.norm = build_part("norm", spec.params["norm"]) if spec.params.get("norm") is not None else None
        self.scale = float(spec.params.get("scale", 1.0))
        self.weight = None

    def parts(self):
        if self.norm is not None:
            yield from self.norm.parts()
        yield self

    def param_specs(self):
        return {self.weight_name: ParamSpec((self.vocab_size, self.hidden_size))}

    def load(self, tensors) -> None:
        self.weight = tensors[self.weight_name].contiguous()

    def forward(self, ops, ids, meta):
        hidden = ops.embed(ids, self.weight) if self.scale == 1.0 else ops.embed(ids, self.weight, self.scale)
        return hidden if self.norm is None else ops.dense(self.norm.apply(ops, hidden, hidden.dtype))


class LinearHead(Head):
    def __init__(self, spec) -> None:
        super().__init__(spec)
        self.vocab_size = int(spec.params["vocab_size"])
        self.hidden_size = int(spec.params["hidden_size"])
        self.tied_to = spec.params.get("tied_to")        # full name of the tensor to share, or None
        self.weight_name = spec.params.get("weight_name", "weight")
        self.scale = float(spec.params.get("scale", 1.0))       # what the logits are multiplied by
        cap = spec.params.get("cap")                             # logits <- cap * tanh(logits / cap), float32
        self.cap = None if cap is None else float(cap)
        if self.cap is not None and not self.cap > 0:
            raise ValueError("the cap of the logits must be positive")
        self.weight = None

    def param_specs(self):
        return {} if self.tied_to else {self.weight_name: ParamSpec((self.vocab_size, self.hidden_size))}

    def shared_specs(self):
        return {self.weight_name: self.tied_to} if self.tied_to else {}

    def optional_names(self):
        return [self.weight_name] if self.tied_to else []

    def load(self, tensors) -> None:
        self.weight = tensors[self.weight_name] if self.tied_to else tensors[self.weight_name].contiguous()

    def prepare(self, ops) -> None:
        ops.prepare_linear(self.weight, role="head")

    def forward(self, ops, normed):
        if self.scale == 1.0:
            logits = ops.linear_f32out(normed, self.weight)
        else:
            logits = ops.linear_f32out(normed, self.weight, None, self.scale)
        return logits if self.cap is None else ops.softcap(logits, self.cap)


register_part("embedding", "token_embedding", TokenEmbedding)
register_part("head", "lm_head", LinearHead)
