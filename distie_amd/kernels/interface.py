"""The kernel surface: every device operation the parts and the engine use.

The product implementation is `HipOps` (hand-written HIP for gfx950, loaded from
shared libraries built out of `distie_amd/csrc`); there is no other implementation in
this package and no fallback: constructing `HipOps` without a GPU or without the
libraries raises. Parts never touch torch math directly; they call these methods, so
what runs on the device is exactly this list.

Conventions: T = tokens of the step (all requests, flattened), B = requests of the
step, `act` = the engine's activation dtype (bfloat16 or float32). The residual stream
is always float32. Weights may be bfloat16 or float32 whatever `act` is.
"""

from __future__ import annotations

import abc
from dataclasses import dataclass, field
from typing import List, Optional

import numpy as np
import torch


@dataclass
class GroupMeta:
    """Addressing of one cache group for one step."""

    block_table: torch.Tensor          # int32 [rows, W]; -1 where a page was given back. Row of request b:
    #                                    BatchMeta.table_rows[b] (the request's state slot: the tables live on the
    #                                    device from step to step), or b itself where table_rows is None
    slots: torch.Tensor                # int32 [T]; block * block_size + offset of each new token


@dataclass
class BatchMeta:
    """Device tensors that describe one flattened step (the reference's BatchMeta,
    worker/src/inference/qwen2/paged_attn.py:310-357, plus what windows, state slots and
    wanted rows need)."""

    num_tokens: int
    num_requests: int
    positions: torch.Tensor            # int32 [T] absolute position of each token
    token_request: torch.Tensor        # int32 [T] index of the request each token belongs to
    cu_q: torch.Tensor                 # int32 [B+1] prefix sums of the new-token counts
    kv_len: torch.Tensor               # int32 [B] tokens cached after this step (past + new)
    state_slots: torch.Tensor          # int32 [B] per-request state slot
    max_q: int                         # host copies, for launch geometry
    max_kv: int
    block_size: int
    groups: List[GroupMeta] = field(default_factory=list)
    # host mirrors (numpy) for parts that run per request on the host side
    host_cu_q: Optional[object] = None
    host_past: Optional[object] = None
    all_decode: bool = False           # every request brings exactly one token
    table_rows: Optional[torch.Tensor] = None    # int32 [B]: each request's row of the groups' block tables
    # In a captured step no launch may depend on how the step's tokens are spread over its requests (that is
    # known on the device only): `max_q` and `max_kv` are then bounds, and so is this, the most requests that
    # bring exactly one token (None: an implementation may count them from `host_cu_q`).
    singles_bound: Optional[int] = None
    scratch: dict = field(default_factory=dict)   # what an implementation computes once per step (cos/sin tables)


@dataclass(frozen=True)
class ScoreExtras:
    """What a variant of attention does to a score beyond scale, causal mask and window; everything None
    for plain attention. An implementation's kernel that does not take a field that is set refuses the call
    (it never ignores it), so a new variant is a kernel added behind this argument, not a changed signature.

    score(i, j) = q_i . k_j * scale; with `score_cap` c: c * tanh(score / c); with `head_slopes` s:
    + s[h] * (j - i), a bias by the distance to the key with a slope of the head's own (a position
    encoding that needs no rotation). With `sinks` z: the softmax's denominator holds exp(z[h]) beside the
    visible keys' terms, weight(i, j) = exp(score(i, j)) / (exp(z[h]) + sum_j' exp(score(i, j'))); the sink is
    not scaled, has no value and counts once for every query, whatever its window."""

    head_slopes: Optional[torch.Tensor] = None      # float32 [H] on the device
    score_cap: Optional[float] = None               # > 0
    sinks: Optional[torch.Tensor] = None            # float32 [H] on the device

    def __post_init__(self):
        if self.score_cap is not None and not self.score_cap > 0:
            raise ValueError("score_cap must be positive")

    @property
    def plain(self) -> bool:
        return self.head_slopes is None and self.score_cap is None and self.sinks is None

    @property
    def bends_scores(self) -> bool:
        """Something changes the scores themselves (a sink does not: it only joins the denominator)."""
        return self.head_slopes is not None or self.score_cap is not None


class Ops(abc.ABC):
    device: torch.device
    # True while the engine warms or records a captured step: launches then cost the host nothing when the
    # step is replayed, so an implementation may choose kernels by their time on the device alone
    captured: bool = False

    def upload(self, values: np.ndarray) -> torch.Tensor:
        """A small host array (row indexes, sampling parameters) as a device tensor of the same dtype and
        shape. An implementation makes this a copy that does not wait for the work queued before it."""
        return torch.from_numpy(np.ascontiguousarray(values)).to(self.device)

    def scatter_int32(self, table: torch.Tensor, index: torch.Tensor, value: torch.Tensor) -> None:
        """table.view(-1)[index] = value for int32 tensors on the device (distinct indexes): the block tables'
        changed entries of a step."""
        table.view(-1)[index.long()] = value

    @abc.abstractmethod
    def embed(self, ids: torch.Tensor, table: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
        """ids int32 [T], table [V, C] -> float32 [T, C], the rows times `scale` (in float32)."""

    @abc.abstractmethod
    def rmsnorm(self, x: torch.Tensor, weight: torch.Tensor, eps: float, out_dtype) -> torch.Tensor:
        """float32 [T, C] -> out_dtype [T, C]; statistics in float32.

        As with `linear`, an implementation may return the result in a form of its own that only its own
        operations read (the HIP kernels leave the norm of few rows to the product that reads it: the value
        is then not computed yet, and stays valid only until `x` is next written in place, which the
        implementation finds out and refuses). A part hands the result on to `linear`, `linear_silu_mul`,
        `linear_rope_kv_write`, `linear_f32out` or `gather_rows`; a part that computes on the values itself
        (indexing, `.float()`, any torch operation) calls `ops.dense(result)` first. The same holds for
        `add_rmsnorm`."""

    @abc.abstractmethod
    def add_rmsnorm(self, residual: torch.Tensor, delta: torch.Tensor, weight: torch.Tensor,
                    eps: float, out_dtype) -> torch.Tensor:
        """residual (float32, updated in place) += delta; returns rmsnorm(residual)."""

    @abc.abstractmethod
    def linear(self, x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
        """x [T, K] (act) times weight [N, K] transposed, plus bias [N] -> act [T, N].

        An implementation may return the product in a form of its own that only its
        `add_rmsnorm`, `silu_mul`, `rope_kv_write`, `linear`, `paged_attention` and `gather_rows`
        read (the HIP kernels return partial sums over slices of K for small batches, or, for few
        rows, a product not yet computed that adds itself to the residual stream if `add_rmsnorm`
        is what comes next); parts hand the result on to those operations, or as the `delta` of a
        `ResidualStream`, and do nothing else with it. A part that computes on the values itself
        calls `ops.dense(result)` first."""

    def dense(self, x):
        """The plain tensor of a result that `linear`, `rmsnorm` or `add_rmsnorm` returned in a form of
        its own; any other tensor as it is. For parts that compute on the values themselves."""
        return x

    def prepare_linear(self, weight: torch.Tensor, gated: bool = False, rotary=None, role: Optional[str] = None) -> None:
        """Called once for every weight of a `linear` after it is loaded (`gated`: the weight of a
        `linear_silu_mul`; `rotary = (num_heads, num_kv_heads, head_dim)`: the stacked q/k/v weight
        of a `linear_rope_kv_write`; `role`: what the part calls this product, so that a setting
        can name it). An implementation may build what its products need beside
        the tensor (the HIP kernels keep a second copy in the matrix cores' order for small
        batches)."""

    def linear_rope_kv_write(self, x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
                             meta: BatchMeta, group: int, k_cache: torch.Tensor, v_cache: torch.Tensor,
                             inv_freq: Optional[torch.Tensor], num_heads: int, num_kv_heads: int,
                             head_dim: int, write: bool) -> torch.Tensor:
        """rope_kv_write(linear(x, weight, bias), ...) for the stacked q/k/v weight; an
        implementation may fuse the two."""
        return self.rope_kv_write(self.linear(x, weight, bias), meta, group, k_cache, v_cache, inv_freq,
                                  num_heads, num_kv_heads, head_dim, write)

    def linear_silu_mul(self, x: torch.Tensor, gate_up_weight: torch.Tensor) -> torch.Tensor:
        """silu_mul(linear(x, gate_up_weight)) with gate_up_weight [2I, K] -> act [T, I]; an
        implementation may fuse the two."""
        return self.silu_mul(self.linear(x, gate_up_weight))

    @abc.abstractmethod
    def linear_f32out(self, x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
                      scale: float = 1.0, partial: bool = False) -> torch.Tensor:
        """As `linear`, result in float32 and not rounded (the logits; what enters a recurrence), times `scale`.
        `partial`: as with `linear`, the result may come in a form of the implementation's own, for the operations
        that say they take it (`latent_norm_rope_write`) and for `dense`."""

    @abc.abstractmethod
    def rope_kv_write(self, qkv: torch.Tensor, meta: BatchMeta, group: int, k_cache: torch.Tensor,
                      v_cache: torch.Tensor, inv_freq: Optional[torch.Tensor], num_heads: int,
                      num_kv_heads: int, head_dim: int, write: bool) -> torch.Tensor:
        """Rotate q and k of qkv [T, (H+2KH)*D] by each token's position (angles and
        trigonometry in float32; no rotation if inv_freq is None) and, if `write`, store the
        rotated k and v at the token's slot of k_cache [NB, KH, P, D] / v_cache [NB, KH, D, P]. Returns the
        rotated qkv (the argument itself if it was rotated in place)."""

    @abc.abstractmethod
    def paged_attention(self, qkv: torch.Tensor, meta: BatchMeta, group: int, k_cache: torch.Tensor,
                        v_cache: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int,
                        scale: float, window: Optional[int], extras: Optional[ScoreExtras] = None) -> torch.Tensor:
        """softmax(q k^T * scale) v over the cached keys 0..position of each token (the last
        `window` of them on a windowed layer), read through the block table -> act [T, H*D].
        `extras`: what a variant adds to the scores (`ScoreExtras`); None for plain attention."""

    # ---- several residual streams, short convolutions over time, decayed states, gates. An implementation that
    # ---- serves only models without them may leave these out: the bodies here refuse.
    def hyper_step(self, streams: Optional[torch.Tensor], *, init: Optional[torch.Tensor] = None, delta=None,
                   gate: Optional[torch.Tensor] = None, mix: Optional[torch.Tensor] = None,
                   write: Optional[torch.Tensor] = None, read: Optional[torch.Tensor] = None,
                   norm_weight: Optional[torch.Tensor] = None, norm: str = "none", eps: float = 0.0, out_dtype=None):
        """One step on S residual streams, float32 [T, S, C], updated in place -> (streams, h or None).

        `init` (float32 [T, C]): the streams do not exist yet and all start as `init` (`streams` is None).
        `delta` (act [T, C], with `mix` float32 [S, S] indexed [from, to] and `write` float32 [S]): all streams
        at once from the old ones, x_j <- sum_s mix[s, j] x_s + write[j] * delta * sigmoid(gate) (`gate` act
        [T, C] or a view with a row stride; None: no gate). `delta` and `gate` may be what `linear` returned, in
        whatever form. `read` (float32 [S]): h = norm(sum_s read[s] x_s)
        * norm_weight in `out_dtype`, from the updated streams; `norm` is "none" (h is the sum, float32 unless
        `out_dtype` says otherwise), "layer" ((u - mean) / sqrt(var + eps), var the mean of the squared deviations)
        or "rms" (u / sqrt(mean(u^2) + eps)). Statistics and sums in float32."""
        raise NotImplementedError(f"{type(self).__name__} has no residual streams")

    def layernorm(self, x: torch.Tensor, weight: torch.Tensor, eps: float, out_dtype) -> torch.Tensor:
        """float32 [T, C] -> (x - mean) / sqrt(var + eps) * weight, no bias, statistics in float32."""
        ones = torch.ones(1, dtype=torch.float32, device=x.device)
        return self.hyper_step(x.view(x.shape[0], 1, x.shape[1]), read=ones, norm_weight=weight, norm="layer",
                               eps=eps, out_dtype=out_dtype)[1]

    def causal_conv(self, x: torch.Tensor, weight: torch.Tensor, state: Optional[torch.Tensor], meta: BatchMeta,
                    residual: bool = False, bias: Optional[torch.Tensor] = None, act: Optional[str] = None) -> torch.Tensor:
        """x act [T, N] (or a view of columns with a row stride), weight [N, taps], bias float32 [N] or None
        -> y_t = bias + (x_t if residual) + sum_j weight[:, j] * x_(t - taps + 1 + j)
        within each request; what lies before the step's rows comes from `state` (float32 [slots + 1, taps - 1, N],
        the request's last taps - 1 inputs, oldest first, rows by `meta.state_slots`), which is moved on to the
        end of the step's rows. Sums in float32, in the order of j. `act`: one of `activation`'s names, applied to the
        float32 sum before it is rounded (None: none)."""
        raise NotImplementedError(f"{type(self).__name__} has no convolution over time")

    def conv_rope_kv_write(self, product: torch.Tensor, conv_weight: Optional[torch.Tensor],
                           state: Optional[torch.Tensor], meta: BatchMeta, group: int,
                           k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
                           inv_freq: Optional[torch.Tensor], magnitude: float, num_heads: int, num_kv_heads: int,
                           dim: int, value_dim: int, padded_dim: int, has_kv: bool, write: bool,
                           q_temp=None, qk_norm=None) -> torch.Tensor:
        """Behind attention's stacked projection. The first columns of `product` (act [T, W]) are q (num_heads x
        dim) and, if `has_kv`, k (num_kv_heads x dim) and v (num_kv_heads x value_dim); further columns are left
        alone. Each of these channels goes through `causal_conv` (no residual; `conv_weight` [channels, taps],
        None: no convolution; the state is moved on), the first 2 * len(inv_freq) dimensions of every q and k head
        are rotated by the token's position (pair (i, i + len(inv_freq)); cosine and sine both times
        `magnitude`), and, if `write`, k and v go to the token's slot of k_cache [pages, KH, P, padded_dim] /
        v_cache [pages, KH, padded_dim, P]. Returns q as act [T, num_heads * padded_dim], zeros beyond `dim`:
        what `paged_attention` reads with a head size of `padded_dim`.
        `q_temp` = (coef, every): a query temperature by position, q of the token at position p is multiplied by
        1 + coef * ln(floor((p + 1) / every) + 1), computed in float32 (None: none).
        `qk_norm` = (q_weight float32 [dim], k_weight float32 [dim] or None without keys, eps): behind the convolution
        and in front of the rotation every q and k head becomes x / sqrt(mean(x^2) + eps) * weight over its `dim`
        values, in float32 (None: none)."""
        raise NotImplementedError(f"{type(self).__name__} has no convolution over time")

    def sigmoid_gate(self, x: torch.Tensor, num_heads: int, head_stride: int, width: int,
                     gates: torch.Tensor, per_head: bool = False) -> torch.Tensor:
        """x act [T, num_heads * head_stride], of which the first `width` of every head count; gates act
        [T, num_heads * width] (or a view with a row stride) -> x * sigmoid(gates), act [T, num_heads * width]. `gates` None: the kept columns as they are.
        `per_head`: gates act [T, num_heads] (or such a view), one number for all of a head's columns."""
        raise NotImplementedError(f"{type(self).__name__} has no gates")

    def decay_scan(self, product: torch.Tensor, state: torch.Tensor, decay: torch.Tensor, meta: BatchMeta,
                   num_heads: int, dim: int, value_dim: int) -> torch.Tensor:
        """Linear attention with a decay per head, as a recurrence over each request's rows: with q = silu(.),
        k = silu(.) (num_heads x dim each) and v = silu(.) (num_heads x value_dim) taken from the first columns of
        `product` (act [T, W]), S <- decay[h] * S + k v^T and o = S^T q. `state` float32 [slots + 1, num_heads,
        dim, value_dim] (rows by `meta.state_slots`) is read and left as the step's last row leaves it.
        -> float32 [T, num_heads * value_dim]. Everything behind the activations in float32."""
        raise NotImplementedError(f"{type(self).__name__} has no decayed state")

    def rmsnorm_gate(self, x: torch.Tensor, weight: torch.Tensor, eps: float, gates: Optional[torch.Tensor],
                     out_dtype, group: Optional[int] = None, gate: str = "sigmoid", gate_first: bool = False) -> torch.Tensor:
        """float32 [T, N] -> x / sqrt(mean(x^2) + eps) * weight * sigmoid(gates) in `out_dtype` (gates act [T, N]
        or a view with a row stride; None: no gate). `group`: the mean is taken over every run of `group` columns
        by itself (a head), and `weight` [group] is the same for all of them; None: over all N, weight [N].
        `gate`: "sigmoid" or "silu" (times gates * sigmoid(gates)). With `group`, a weight of [N] is each column's own.
        `gate_first`: the gate multiplies x in front of the norm, (x * gate) / sqrt(mean((x * gate)^2) + eps) * weight,
        instead of its result."""
        raise NotImplementedError(f"{type(self).__name__} has no gated norm")

    # ---- a state with one decay per head and token (state-space duality), attention over a shared latent
    def ssm_scan(self, xbc: torch.Tensor, dt: torch.Tensor, dt_bias: torch.Tensor, a_log: torch.Tensor,
                 skip: torch.Tensor, state: torch.Tensor, meta: BatchMeta, num_heads: int, value_dim: int,
                 state_size: int, groups: int) -> torch.Tensor:
        """The selective state-space recurrence in its scalar-decay form, over each request's rows in order. `xbc` act
        [T, H * P + 2 * G * N] (or a view of columns): x (H heads of P = value_dim), then B and C (G groups of N =
        state_size each; head h reads group h // (H / G)). `dt` act [T, H] (or a view), `dt_bias`, `a_log`, `skip`
        float32 [H]. With d = softplus(dt + dt_bias) and a = exp(-exp(a_log) * d), per head

            S <- a * S + d * B x^T   (S is N x P),        y = S^T C + skip * x.

        `state` float32 [slots + 1, H, N, P] (rows by `meta.state_slots`) is read and left as the step's last row
        leaves it. -> float32 [T, H * P]. Softplus, exponentials, the state, its products and sums in float32."""
        raise NotImplementedError(f"{type(self).__name__} has no state-space recurrence")

    def ssm_scan_captures(self, state_size: int) -> bool:
        """Whether `ssm_scan` at this state size can run inside a captured step (its launches then must not hang on the
        step's row counts, which an implementation's kernel for large states may need)."""
        return True

    def latent_norm_rope_write(self, down: torch.Tensor, q_rank: int, q_weight: Optional[torch.Tensor], kv_rank: int,
                               kv_weight: torch.Tensor, eps: float, rot_dim: int, inv_freq: Optional[torch.Tensor],
                               magnitude: float, neighbours: bool, meta: BatchMeta, group: int, k_cache: torch.Tensor,
                               v_cache: torch.Tensor, write: bool, out_dtype) -> Optional[torch.Tensor]:
        """Behind latent attention's stacked down-projection. `down` float32 [T, q_rank + kv_rank + rot_dim] (or what
        `linear_f32out(..., partial=True)` returned): the
        queries' latent, the keys' and values' latent, and one rotated key part for all heads. Both latents go through
        an RMS norm of their own (x / sqrt(mean(x^2) + eps) * weight, float32). The normed queries' latent is returned
        in `out_dtype` [T, q_rank] (None if q_rank is 0). If `write`, the token's slot of the cache gets the normed
        latent c and the rotated key part as one key of one head, k_cache [pages, 1, P, DP] = (c, rotated part, zeros),
        and c again as its value, v_cache [pages, 1, DP, P]. The key part's 2 * len(inv_freq) dimensions are turned by
        the token's position, cosine and sine both times `magnitude`; `neighbours`: dimension 2i pairs with 2i + 1,
        else i with i + len(inv_freq)."""
        raise NotImplementedError(f"{type(self).__name__} has no latent attention")

    def heads_linear(self, x: torch.Tensor, weight: torch.Tensor, in_stride: int, out_stride: int,
                     out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """A product of its own for every head: x act [T, H * in_stride], head h's input its first K columns there;
        weight [H, N, K] -> act [T, H * out_stride], head h's N results the first of its out_stride columns. The
        other columns are zero, or what `out` (act [T, H * out_stride]) held. Sums in float32."""
        raise NotImplementedError(f"{type(self).__name__} has no products by head")

    def rope_heads(self, x: torch.Tensor, in_stride: int, in_offset: int, out: torch.Tensor, out_stride: int,
                   out_offset: int, num_heads: int, inv_freq: torch.Tensor, magnitude: float, neighbours: bool,
                   meta: BatchMeta) -> torch.Tensor:
        """The 2 * len(inv_freq) columns at `in_offset` of every head of x (act [T, H * in_stride]), turned by the
        token's position as in `latent_norm_rope_write`, written to the columns at `out_offset` of every head of `out`
        (act [T, H * out_stride]) -> out."""
        raise NotImplementedError(f"{type(self).__name__} has no rotation of head columns")

    def latent_queries(self, q: torch.Tensor, key_up: torch.Tensor, num_heads: int, dim: int, rot_dim: int,
                       padded_dim: int, inv_freq: Optional[torch.Tensor], magnitude: float, neighbours: bool,
                       meta: BatchMeta) -> torch.Tensor:
        """Latent attention's queries as the cache's one key head reads them. q act [T, H * (dim + rot_dim)] (or what
        `linear` returned), every
        head (dim unrotated, rot_dim rotated); key_up [H, kv_rank, dim], head h's key expansion transposed. Since
        q_h . (U_h c) = (U_h^T q_h) . c, head h's query against the cached (c, rotated key part) is
        (key_up[h] q_h[:dim], turned q_h[dim:], zeros) -> act [T, H * padded_dim]. An implementation may fuse the two."""
        q = self.dense(q)
        out = self.heads_linear(q, key_up, dim + rot_dim, padded_dim)
        if inv_freq is None:
            raise NotImplementedError("latent attention's rotated part needs a rotation")
        return self.rope_heads(q, dim + rot_dim, dim, out, padded_dim, key_up.shape[1], num_heads, inv_freq, magnitude,
                               neighbours, meta)

    # ---- sums of normed sub-layer outputs, states with a decay of their own for every channel and token, routed
    # ---- feed-forwards. As above: an implementation that serves no model with them may leave them out.
    def normed_sum(self, terms, weights, eps: float, scale: float):
        """scale * sum_i rmsnorm(terms[i]) * weights[i] -> float32 [T, C] (mixers side by side on one input, each
        result normed over the model width before they are added). `terms`: act [T, C] each, or what `linear`
        returned; `weights` float32 [C] each. An implementation may hand out a value that only `add_normed`,
        `add_normed_rmsnorm` and `dense` read."""
        raise NotImplementedError(f"{type(self).__name__} has no sum of normed terms")

    def add_normed(self, residual: torch.Tensor, delta, weight: torch.Tensor, eps: float) -> None:
        """residual (float32 [T, C], in place) += rmsnorm(delta) * weight: a sub-layer's result with a norm behind
        it. `delta`: act [T, C], what `linear` returned, or what `normed_sum` returned."""
        raise NotImplementedError(f"{type(self).__name__} has no norm behind a sub-layer")

    def read_residual(self, residual: torch.Tensor, out_dtype) -> torch.Tensor:
        """The residual (float32 [T, C]) as a sub-layer without a norm in front reads it: rounded to `out_dtype`,
        or the tensor itself where that is float32."""
        return residual if out_dtype == residual.dtype else residual.to(out_dtype)

    def add_normed_read(self, residual: torch.Tensor, delta, post_weight: torch.Tensor, post_eps: float,
                        out_dtype) -> torch.Tensor:
        """`add_normed`, then `read_residual`; an implementation may fuse the two."""
        self.add_normed(residual, delta, post_weight, post_eps)
        return self.read_residual(residual, out_dtype)

    def add_normed_rmsnorm(self, residual: torch.Tensor, delta, post_weight: torch.Tensor, post_eps: float,
                           weight: torch.Tensor, eps: float, out_dtype) -> torch.Tensor:
        """`add_normed`, then rmsnorm(residual) * weight in `out_dtype`; an implementation may fuse the two."""
        self.add_normed(residual, delta, post_weight, post_eps)
        return self.rmsnorm(residual, weight, eps, out_dtype)

    def gated_decay_scan(self, product: torch.Tensor, decay_logits: Optional[torch.Tensor], state: torch.Tensor,
                         meta: BatchMeta, num_heads: int, dim: int, value_dim: int, q_scale: float, tau: float,
                         decay_low=None) -> torch.Tensor:
        """Linear attention whose state decays by a factor of its own for every key channel and token: with q
        (num_heads x dim, times `q_scale`), k (num_heads x dim) and v (num_heads x value_dim) from the first columns
        of `product` (act [T, W]) and alpha = sigmoid(decay_logits)^(1 / tau) (decay_logits float32 [T, num_heads *
        dim]), per head S <- diag(alpha) S + k v^T (alpha scales the rows of S, one a key channel) and o = S^T q.
        `state` float32 [slots + 1, num_heads, dim, value_dim] (rows by `meta.state_slots`) is read and left as
        the step's last row leaves it. -> float32 [T, num_heads * value_dim]; decay, state and sums in float32.
        `decay_logits` None: they are still to be made from `decay_low` = (low act [T, rank] or a view of columns, up
        [num_heads * dim, rank], bias float32 [num_heads * dim]) as up . low + bias, float32 and not rounded; an
        implementation may make them inside the scan (`decay_logits_of` makes them as a product of their own)."""
        raise NotImplementedError(f"{type(self).__name__} has no gated decayed state")

    def decay_logits_of(self, decay_low) -> torch.Tensor:
        """The decay's logits as a product of their own: float32 [T, num_heads * dim]."""
        low, up, bias = decay_low
        return self.linear_f32out(low.contiguous(), up, bias)

    def lru_gates(self, u: torch.Tensor, recur_weight: torch.Tensor, recur_bias: torch.Tensor,
                  input_weight: torch.Tensor, input_bias: torch.Tensor, lam: torch.Tensor, rate: float):
        """The coefficients of a real-gated linear recurrent unit. u act [T, R] in B equal parts; the gates'
        weights are block-diagonal, [B, R/B, R/B] with each block [out, in], biases float32 [B, R/B]:
        r = sigmoid(W_r u + b_r), i = sigmoid(W_i u + b_i), a = exp(-rate * r * softplus(lam)) (lam float32 [R]),
        x = sqrt(1 - a^2) * i * u -> (a, x), float32 [T, R] each; sums and everything behind them in float32."""
        raise NotImplementedError(f"{type(self).__name__} has no gated linear recurrent unit")

    def lru_scan(self, a: torch.Tensor, x: torch.Tensor, state: torch.Tensor, meta: BatchMeta,
                 mul: Optional[torch.Tensor], mul_act: Optional[str], out_dtype) -> torch.Tensor:
        """h_t = a_t * h_(t-1) + x_t for every channel, over each request's rows in order (a, x float32 [T, R]);
        `state` float32 [slots + 1, R] (rows by `meta.state_slots`) holds h in front of the step and is left as the
        last row leaves it. -> h * act(mul) in `out_dtype` (`mul` act [T, R] or a view with a row stride, `mul_act`
        one of `activation`'s names or None for mul itself; `mul` None: h)."""
        raise NotImplementedError(f"{type(self).__name__} has no gated linear recurrent unit")

    def route_topk(self, x, weight: torch.Tensor, bias: Optional[torch.Tensor], top: int, scoring: str = "softmax"):
        """The router of a mixture of experts: z = weight x + bias in float32 (x act [T, C], weight [E, C], bias
        float32 [E] or None); for every row the `top` largest z (the lower index among equals) and, as weights,
        softmax over those alone (`scoring` "softmax") or sigmoid(z) of each, not renormalised ("sigmoid")
        -> (experts int32 [T, top], their weights float32 [T, top]), largest first."""
        raise NotImplementedError(f"{type(self).__name__} has no router")

    def route_glu(self, gate_up, experts: torch.Tensor, gates: torch.Tensor, num_experts: int, width: int,
                  limit: Optional[float], slope: float, up_shift: float, on_input: bool) -> torch.Tensor:
        """The hidden values of routed gated experts from the stacked product. `gate_up` act [T, 2 * num_experts *
        width] (or what `linear` returned): every expert's gate columns, expert after expert, then every expert's up
        columns. For expert e of a row with weight w (zero result if the row did not choose e):
        g, u = gate and up columns, times w if `on_input`; with `limit`: g <- min(g, limit), u <- clamp(u, -limit,
        limit); hidden = g * sigmoid(slope * g) * (u + up_shift), times w unless `on_input`
        -> act [T, num_experts * width], in float32 behind the product's rounding."""
        raise NotImplementedError(f"{type(self).__name__} has no routed feed-forward")

    def route_experts_glu(self, x, router_weight: torch.Tensor, router_bias: Optional[torch.Tensor], top: int,
                          scoring: str, gate_up, num_experts: int, width: int, limit: Optional[float], slope: float,
                          up_shift: float, on_input: bool) -> torch.Tensor:
        """`route_topk` of x, then `route_glu` of `gate_up` with what it chose; an implementation may fuse the two."""
        experts, gates = self.route_topk(x, router_weight, router_bias, top, scoring)
        return self.route_glu(gate_up, experts, gates, num_experts, width, limit, slope, up_shift, on_input)

    def softcap(self, x: torch.Tensor, cap: float) -> torch.Tensor:
        """float32 [R, N] (in place) -> cap * tanh(x / cap)."""
        raise NotImplementedError(f"{type(self).__name__} has no cap on values")

    def route_scale(self, hidden: torch.Tensor, experts: torch.Tensor, gates: torch.Tensor, num_experts: int,
                    width: int) -> torch.Tensor:
        """hidden act [T, num_experts * width + more] (in place): the columns of expert e, [e * width, (e + 1) *
        width), times the row's weight for e, or zero if the row did not choose e; columns beyond the experts' (a
        part that every row uses) stay. -> hidden."""
        raise NotImplementedError(f"{type(self).__name__} has no routed feed-forward")

    def activation(self, x, kind: str) -> torch.Tensor:
        """Element by element on act [T, N]: "relu2" (the square of max(x, 0)), "silu", "gelu_tanh", "relu"."""
        raise NotImplementedError(f"{type(self).__name__} has no activation {kind!r}")

    def linear_act(self, x, weight: torch.Tensor, kind: str) -> torch.Tensor:
        """activation(linear(x, weight), kind); an implementation may fuse the two."""
        return self.activation(self.linear(x, weight), kind)

    def glu_mul(self, gate_up, kind: str) -> torch.Tensor:
        """[T, 2I] (or what `linear` returned) -> act(first half) * second half, [T, I]; `kind` one of `activation`'s
        names. "silu" is `silu_mul`."""
        if kind == "silu":
            return self.silu_mul(gate_up)
        raise NotImplementedError(f"{type(self).__name__} has no gated activation {kind!r}")

    def linear_glu(self, x: torch.Tensor, gate_up_weight: torch.Tensor, kind: str) -> torch.Tensor:
        """glu_mul(linear(x, gate_up_weight), kind); an implementation may fuse the two."""
        if kind == "silu":
            return self.linear_silu_mul(x, gate_up_weight)
        return self.glu_mul(self.linear(x, gate_up_weight), kind)

    @abc.abstractmethod
    def silu_mul(self, gate_up: torch.Tensor) -> torch.Tensor:
        """[T, 2I] -> silu(first half) * second half, [T, I]."""

    @abc.abstractmethod
    def gather_rows(self, x: torch.Tensor, rows: torch.Tensor) -> torch.Tensor:
        """x [T, C], rows int32 [R] -> x[rows]."""

    @abc.abstractmethod
    def argmax(self, logits: torch.Tensor) -> torch.Tensor:
        """float32 [R, V] -> int32 [R], lowest index among equals."""

    @abc.abstractmethod
    def sample(self, logits: torch.Tensor, temperature: torch.Tensor, seeds: torch.Tensor,
               counters: torch.Tensor) -> torch.Tensor:
        """Rows with temperature <= 0: argmax. Others: one draw from softmax(logits / t)
        with the uniform number hash(seed, counter) -> int32 [R]."""
