"""Attention whose keys and values are expanded from one small latent vector a token ("multi-head latent attention",
as in DeepSeek-V2), computed on the latent itself.

h is the mixer's input, H the number of heads; a head has `head_dim` query/key dimensions that are not rotated and
`rot_dim` that are, and values of `value_dim`.

    c_q = rms(W_dq h) * dq.norm                  the queries' latent, q_rank wide
    q   = W_uq c_q                               head by head (head_dim unrotated, rot_dim rotated)
    (c', r) = W_dkv h                            kv_rank + rot_dim rows
    c   = rms(c') * dkv.norm                     the latent that is cached; r, rotated, is one key part for all heads
    k_h = (W_uk,h c, rot(r)),   v_h = W_uv,h c
    score = (q_h[:head_dim] . W_uk,h c + rot(q_h[head_dim:]) . rot(r)) * scale

with an optional sink in the softmax's denominator (`sink` [H]) and W_o on the concatenated heads. The rotation pairs
neighbouring dimensions (`rotate` "neighbours": 2i with 2i + 1) or halves ("halves": i with i + rot_dim / 2).

Only c and the rotated r are kept, and attention runs on them directly: q_h . (W_uk,h c) = (W_uk,h^T q_h) . c, so with
the query of head h taken to the latent's space every head reads the same cached vector (c, rot(r)) as its key and c as
its value, which is attention with one key/value head of size kv_rank + rot_dim, and W_uv,h is applied to the weighted
sum of the c's afterwards. The kernels are the ones every attention layer uses (one key/value head, H query heads on
it); their head size is kv_rank + rot_dim rounded up to what they take, so that sum is bounded by their largest head
(beyond the matrix-core kernels' 256 the wave-per-token kernel serves, slowly).
The two down-projections are one matrix product (their weights are stacked at load), both norms, the rotation of r and
the cache write one kernel.
"""

from __future__ import annotations

import bisect

import torch

from ..config.model_config import PartSpec
from ..kernels.interface import ScoreExtras
from .attention import PagedKV, context_classes
from .base import Mixer, ParamSpec, build_part, register_part
from .conv_attention import padded_head_dim

LARGEST_HEAD = 1024         # what the attention kernels take (the matrix-core ones up to 256, the wave-per-token one beyond)


class LatentAttention(Mixer):
    FIRST_CONTEXT = 1024

    def __init__(self, spec: PartSpec) -> None:
        super().__init__(spec)
        p = spec.params
        self.hidden_size = int(p["hidden_size"])
        self.num_heads = int(p["num_heads"])
        self.head_dim = int(p["head_dim"])
        self.rot_dim = int(p["rot_dim"])
        self.value_dim = int(p["value_dim"])
        self.kv_rank = int(p["kv_rank"])
        self.q_rank = int(p["q_rank"])
        self.eps = float(p["eps"])
        self.scale = float(p.get("scale", (self.head_dim + self.rot_dim) ** -0.5))
        self.sink = bool(p.get("sink", False))
        rotate = str(p.get("rotate", "neighbours"))
        if rotate not in ("neighbours", "halves"):
            raise ValueError("latent attention rotates neighbours or halves")
        self.neighbours = rotate == "neighbours"
        if min(self.num_heads, self.head_dim, self.rot_dim, self.value_dim, self.kv_rank, self.q_rank) < 1 or self.rot_dim % 2:
            raise ValueError("latent attention: sizes must be >= 1 and rot_dim even")
        self.position = build_part("position", p.get("position") or PartSpec("none"))
        self.padded_dim = padded_head_dim(self.kv_rank + self.rot_dim, self.kv_rank)
        if self.padded_dim > LARGEST_HEAD:
            raise ValueError(f"latent attention: kv_rank + rot_dim = {self.kv_rank + self.rot_dim} is beyond the attention "
                             f"kernels' largest head ({LARGEST_HEAD})")
        self.down_weight = self.q_norm = self.kv_norm = self.q_up = self.key_up = self.value_up = self.out_weight = None
        self.extras = None

    def cache_requirement(self):
        return PagedKV(1, self.padded_dim, None)

    def param_specs(self):
        H, C = self.num_heads, self.hidden_size
        specs = {"dq": ParamSpec((self.q_rank, C)), "dq.norm": ParamSpec((self.q_rank,), "ones"),
                 "uq": ParamSpec((H * (self.head_dim + self.rot_dim), self.q_rank)),
                 "dkv": ParamSpec((self.kv_rank + self.rot_dim, C)), "dkv.norm": ParamSpec((self.kv_rank,), "ones"),
                 "uk": ParamSpec((H * self.head_dim, self.kv_rank)), "uv": ParamSpec((H * self.value_dim, self.kv_rank))}
        if self.sink:
            specs["sink"] = ParamSpec((H,))
        specs["o"] = ParamSpec((C, H * self.value_dim))
        return specs

    def load(self, tensors) -> None:
        H = self.num_heads
        stacked = [tensors["dq"], tensors["dkv"]]
        dtype = torch.float32 if any(t.dtype == torch.float32 for t in stacked) else stacked[0].dtype
        self.down_weight = torch.cat([t.to(dtype) for t in stacked], dim=0).contiguous()
        self.q_norm = tensors["dq.norm"].float().contiguous()
        self.kv_norm = tensors["dkv.norm"].float().contiguous()
        self.q_up = tensors["uq"].contiguous()
        # head h's key expansion transposed, [kv_rank, head_dim]: what takes a query to the latent's space
        self.key_up = tensors["uk"].view(H, self.head_dim, self.kv_rank).transpose(1, 2).contiguous()
        self.value_up = tensors["uv"].view(H, self.value_dim, self.kv_rank).contiguous()
        self.out_weight = tensors["o"].contiguous()
        if self.sink:
            self.extras = ScoreExtras(sinks=tensors["sink"].float().contiguous())
        self.position.to_device(self.out_weight.device)
        if self.position.rotary() is None or 2 * self.position.rotary().shape[0] != self.rot_dim:
            raise ValueError("latent attention: the rotation turns all rot_dim dimensions of the rotated part")

    def prepare(self, ops) -> None:
        ops.prepare_linear(self.down_weight, role="qkv")
        ops.prepare_linear(self.q_up, role="qkv")
        ops.prepare_linear(self.out_weight, role="attn_out")

    def capture_context(self, longest: int, limit: int):
        classes = context_classes(limit, self.FIRST_CONTEXT)
        return classes[min(bisect.bisect_left(classes, longest), len(classes) - 1)]

    def forward(self, ops, x, ctx, cache, writes_cache: bool):
        k_cache, v_cache = cache["k"], cache["v"]
        inv_freq, magnitude = self.position.rotary(), self.position.rotary_magnitude()
        down = ops.linear_f32out(x, self.down_weight, partial=True)
        latent = ops.latent_norm_rope_write(down, self.q_rank, self.q_norm, self.kv_rank, self.kv_norm, self.eps,
                                            self.rot_dim, inv_freq, magnitude, self.neighbours, ctx.meta, cache.group,
                                            k_cache, v_cache, writes_cache, ctx.act_dtype)
        q = ops.latent_queries(ops.linear(latent, self.q_up), self.key_up, self.num_heads, self.head_dim, self.rot_dim, self.padded_dim, inv_freq,
                               magnitude, self.neighbours, ctx.meta)
        mixed = ops.paged_attention(q, ctx.meta, cache.group, k_cache, v_cache, self.num_heads, 1, self.padded_dim,
                                    self.scale, None, self.extras)
        values = ops.heads_linear(mixed, self.value_up, self.padded_dim, self.value_dim)
        return ops.linear(values, self.out_weight)


register_part("mixer", "latent_attention", LatentAttention)
