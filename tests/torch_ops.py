"""A test double of the kernel surface in plain torch, for tests of the engine's logic
(batching, cache, scheduler) on a machine without a GPU. It is not part of the product:
the package never selects it, and it computes each operation in the most direct way
(float32 math, loops over requests), reading the cache through the block table as the
kernels must."""

from __future__ import annotations

import math

import torch

from distie_amd.kernels.interface import Ops


class TorchOps(Ops):
    def __init__(self, device="cpu") -> None:
        self.device = torch.device(device)

    def embed(self, ids, table, scale=1.0):
        rows = table[ids.long()].float()
        return rows if scale == 1.0 else rows * scale

    def rmsnorm(self, x, weight, eps, out_dtype):
        x = x.float()
        y = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * weight.float()
        return y.to(out_dtype)

    def add_rmsnorm(self, residual, delta, weight, eps, out_dtype):
        residual += delta.float()
        return self.rmsnorm(residual, weight, eps, out_dtype)

    def linear(self, x, weight, bias=None):
        y = x.float() @ weight.float().T
        if bias is not None:
            y = y + bias.float()
        return y.to(x.dtype)

    def linear_f32out(self, x, weight, bias=None, scale=1.0, partial=False):
        y = x.float() @ weight.float().T
        if bias is not None:
            y = y + bias.float()
        return y * scale if scale != 1.0 else y

    def rope_kv_write(self, qkv, meta, group, k_cache, v_cache, inv_freq, num_heads, num_kv_heads,
                      head_dim, write):
        T = qkv.shape[0]
        view = qkv.view(T, num_heads + 2 * num_kv_heads, head_dim)
        if inv_freq is not None:
            ang = meta.positions.float()[:, None] * inv_freq.float()[None, :]
            rot = 2 * inv_freq.shape[0]
            cos, sin = ang.cos()[:, None, :], ang.sin()[:, None, :]
            qk = view[:, :num_heads + num_kv_heads, :rot].float()
            a, b = qk[..., :rot // 2], qk[..., rot // 2:]
            view[:, :num_heads + num_kv_heads, :rot] = torch.cat(
                [a * cos - b * sin, b * cos + a * sin], -1).to(qkv.dtype)
        if write:
            P = k_cache.shape[2]
            slots = meta.groups[group].slots.long()
            k = view[:, num_heads:num_heads + num_kv_heads]
            v = view[:, num_heads + num_kv_heads:]
            k_cache[slots // P, :, slots % P] = k.to(k_cache.dtype)
            v_cache[slots // P, :, :, slots % P] = v.to(v_cache.dtype)
        return qkv

    def paged_attention(self, qkv, meta, group, k_cache, v_cache, num_heads, num_kv_heads, head_dim,
                        scale, window, extras=None):
        T = qkv.shape[0]
        P = k_cache.shape[2]
        q_all = qkv[:, :num_heads * head_dim].reshape(T, num_heads, head_dim).float()      # (q may come without k and v)
        out = torch.zeros(T, num_heads, head_dim, dtype=torch.float32, device=qkv.device)
        table = meta.groups[group].block_table.long()
        if meta.table_rows is not None:
            table = table[meta.table_rows.long()]
        cu = meta.cu_q.tolist()
        rep = num_heads // num_kv_heads
        for b in range(meta.num_requests):
            for t in range(cu[b], cu[b + 1]):
                pos = int(meta.positions[t])
                first = 0 if window is None else max(0, pos - window + 1)
                keys = torch.arange(first, pos + 1, device=qkv.device)
                pages = table[b, keys // P]
                assert (pages >= 0).all(), "attention would read a page that was given back"
                k = k_cache[pages, :, keys % P].float()          # [n, KH, D]
                v = v_cache[pages, :, :, keys % P].float()
                k = k.repeat_interleave(rep, dim=1)
                v = v.repeat_interleave(rep, dim=1)
                s = torch.einsum("hd,nhd->hn", q_all[t], k) * scale
                if extras is not None and extras.score_cap is not None:
                    s = extras.score_cap * torch.tanh(s / extras.score_cap)
                if extras is not None and extras.head_slopes is not None:
                    s = s + extras.head_slopes.float()[:, None] * (keys - pos).float()[None, :]
                if extras is not None and extras.sinks is not None:
                    w = torch.softmax(torch.cat([s, extras.sinks.float()[:, None]], -1), -1)[:, :-1]
                else:
                    w = torch.softmax(s, -1)
                out[t] = torch.einsum("hn,nhd->hd", w, v)
        return out.view(T, num_heads * head_dim).to(qkv.dtype)

    # ---- residual streams, convolutions over time, decayed states, gates
    def hyper_step(self, streams, *, init=None, delta=None, gate=None, mix=None, write=None, read=None,
                   norm_weight=None, norm="none", eps=0.0, out_dtype=None):
        if init is not None:
            count = (read if read is not None else write).shape[0]
            streams = init.float()[:, None, :].repeat(1, count, 1)
        if delta is not None:
            d = delta.float()
            if gate is not None:
                d = d * torch.sigmoid(gate.float())
            streams.copy_(torch.einsum("sj,tsc->tjc", mix.float(), streams) + write.float()[None, :, None] * d[:, None, :])
        h = None
        if read is not None:
            u = torch.einsum("s,tsc->tc", read.float(), streams)
            if norm == "layer":
                mean = u.mean(-1, keepdim=True)
                u = (u - mean) / torch.sqrt(((u - mean) ** 2).mean(-1, keepdim=True) + eps) * norm_weight.float()
            elif norm == "rms":
                u = u / torch.sqrt((u ** 2).mean(-1, keepdim=True) + eps) * norm_weight.float()
            h = u.to(out_dtype or torch.float32)
        return streams, h

    def _history(self, x, state, meta, taps):
        """Per request: (rows of the step, its state row, the inputs with the state in front)."""
        cu = meta.cu_q.tolist()
        slots = meta.state_slots.tolist()
        for b in range(meta.num_requests):
            rows = slice(cu[b], cu[b + 1])
            past = state[slots[b]] if taps > 1 else x.new_zeros((0, x.shape[1]), dtype=torch.float32)
            yield rows, slots[b], torch.cat([past, x[rows].float()], 0)

    def _conv(self, x, weight, state, meta, residual):
        taps = weight.shape[1]
        out = torch.zeros(x.shape, dtype=torch.float32, device=x.device)
        for rows, slot, full in self._history(x, state, meta, taps):
            n = rows.stop - rows.start
            for j in range(taps):
                out[rows] += weight[:, j].float() * full[j:j + n]
            if taps > 1:
                state[slot] = full[-(taps - 1):]
        if residual:
            out += x.float()
        return out

    def causal_conv(self, x, weight, state, meta, residual=False, bias=None, act=None):
        y = self._conv(x, weight, state, meta, residual)
        y = y if bias is None else y + bias.float()
        return (y if act is None else self.activation(y, act)).to(x.dtype)

    def conv_rope_kv_write(self, product, conv_weight, state, meta, group, k_cache, v_cache, inv_freq, magnitude,
                           num_heads, num_kv_heads, dim, value_dim, padded_dim, has_kv, write, q_temp=None, qk_norm=None):
        T = product.shape[0]
        channels = num_heads * dim + (num_kv_heads * (dim + value_dim) if has_kv else 0)
        u = product[:, :channels]
        u = self._conv(u, conv_weight, state, meta, False) if conv_weight is not None else u.float()
        u = u.to(product.dtype).float()                   # the convolution's result in the activations' precision

        def turned(x):
            if inv_freq is None:
                return x
            pairs = inv_freq.shape[0]
            ang = meta.positions.float()[:, None] * inv_freq.float()[None, :]
            cos, sin = (ang.cos() * magnitude)[:, None, :], (ang.sin() * magnitude)[:, None, :]
            a, b = x[..., :pairs], x[..., pairs:2 * pairs]
            return torch.cat([a * cos - b * sin, b * cos + a * sin, x[..., 2 * pairs:]], -1)

        def normed(x, weight):
            if qk_norm is None:
                return x
            return x / torch.sqrt((x * x).mean(-1, keepdim=True) + qk_norm[2]) * weight.float()

        q = torch.zeros(T, num_heads, padded_dim, dtype=torch.float32, device=product.device)
        q[..., :dim] = turned(normed(u[:, :num_heads * dim].reshape(T, num_heads, dim), qk_norm and qk_norm[0]))
        if q_temp is not None:
            coef, every = q_temp
            steps = torch.div(meta.positions.long() + 1, int(every), rounding_mode="floor")
            q = q * (1.0 + float(coef) * torch.log(steps.float() + 1.0))[:, None, None]
        if has_kv and write:
            k = turned(normed(u[:, num_heads * dim:(num_heads + num_kv_heads) * dim].reshape(T, num_kv_heads, dim),
                              qk_norm and qk_norm[1]))
            v = u[:, (num_heads + num_kv_heads) * dim:].reshape(T, num_kv_heads, value_dim)
            P = k_cache.shape[2]
            slots = meta.groups[group].slots.long()
            k_cache[slots // P, :, slots % P, :dim] = k.to(k_cache.dtype)
            v_cache[slots // P, :, :value_dim, slots % P] = v.to(v_cache.dtype)
        return q.view(T, num_heads * padded_dim).to(product.dtype)

    def sigmoid_gate(self, x, num_heads, head_stride, width, gates, per_head=False):
        T = x.shape[0]
        kept = x.view(T, num_heads, head_stride)[..., :width].float()
        if gates is not None:
            g = torch.sigmoid(gates.float())
            kept = kept * (g[:, :, None] if per_head else g.view(T, num_heads, width))
        return kept.reshape(T, num_heads * width).to(x.dtype)

    def decay_scan(self, product, state, decay, meta, num_heads, dim, value_dim):
        T = product.shape[0]
        act = lambda z: z * torch.sigmoid(z)
        q = act(product[:, :num_heads * dim].float()).view(T, num_heads, dim)
        k = act(product[:, num_heads * dim:2 * num_heads * dim].float()).view(T, num_heads, dim)
        v = act(product[:, 2 * num_heads * dim:num_heads * (2 * dim + value_dim)].float()).view(T, num_heads, value_dim)
        out = torch.zeros(T, num_heads, value_dim, dtype=torch.float32, device=product.device)
        cu = meta.cu_q.tolist()
        slots = meta.state_slots.tolist()
        for b in range(meta.num_requests):
            s = state[slots[b]]
            for t in range(cu[b], cu[b + 1]):
                s = decay.float()[:, None, None] * s + k[t][:, :, None] * v[t][:, None, :]
                out[t] = torch.einsum("hde,hd->he", s, q[t])
            state[slots[b]] = s
        return out.view(T, num_heads * value_dim)

    def rmsnorm_gate(self, x, weight, eps, gates, out_dtype, group=None, gate="sigmoid", gate_first=False):
        T, N = x.shape
        factor = None
        if gates is not None:
            g = gates.float()
            factor = torch.sigmoid(g) if gate == "sigmoid" else g * torch.sigmoid(g)
        if gate_first and factor is not None:
            x = x * factor
        v = x.view(T, N // group, group) if group else x
        w = weight.float()
        if group and w.shape[0] == N:
            w = w.view(N // group, group)
        y = (v / torch.sqrt((v ** 2).mean(-1, keepdim=True) + eps) * w).reshape(T, N)
        if factor is not None and not gate_first:
            y = y * factor
        return y.to(out_dtype)

    # ---- a state with one decay a head and token, attention over a shared latent
    def ssm_scan(self, xbc, dt, dt_bias, a_log, skip, state, meta, num_heads, value_dim, state_size, groups):
        T = xbc.shape[0]
        H, P, N, G = num_heads, value_dim, state_size, groups
        x = xbc[:, :H * P].float().view(T, H, P)
        B = xbc[:, H * P:H * P + G * N].float().view(T, G, N).repeat_interleave(H // G, dim=1)
        C = xbc[:, H * P + G * N:H * P + 2 * G * N].float().view(T, G, N).repeat_interleave(H // G, dim=1)
        d = torch.nn.functional.softplus(dt.float() + dt_bias.float(), threshold=80.0)
        a = torch.exp(-torch.exp(a_log.float()) * d)
        out = torch.zeros(T, H, P, dtype=torch.float32, device=xbc.device)
        cu, slots = meta.cu_q.tolist(), meta.state_slots.tolist()
        for b in range(meta.num_requests):
            s = state[slots[b]]
            for t in range(cu[b], cu[b + 1]):
                s = a[t][:, None, None] * s + d[t][:, None, None] * B[t][:, :, None] * x[t][:, None, :]
                out[t] = torch.einsum("hnp,hn->hp", s, C[t]) + skip.float()[:, None] * x[t]
            state[slots[b]] = s
        return out.view(T, H * P)

    @staticmethod
    def _turn(x, positions, inv_freq, magnitude, neighbours):
        """x [..., 2 * pairs] with rows by token -> turned by each token's position."""
        pairs = inv_freq.shape[0]
        ang = positions.float()[:, None] * inv_freq.float()[None, :]
        shape = [x.shape[0]] + [1] * (x.dim() - 2) + [pairs]
        cos, sin = (ang.cos() * magnitude).view(shape), (ang.sin() * magnitude).view(shape)
        if neighbours:
            a, b = x[..., 0::2], x[..., 1::2]
            return torch.stack([a * cos - b * sin, b * cos + a * sin], -1).flatten(-2)
        a, b = x[..., :pairs], x[..., pairs:]
        return torch.cat([a * cos - b * sin, b * cos + a * sin], -1)

    def latent_norm_rope_write(self, down, q_rank, q_weight, kv_rank, kv_weight, eps, rot_dim, inv_freq, magnitude,
                               neighbours, meta, group, k_cache, v_cache, write, out_dtype):
        down = down.float()
        latent = self._rms(down[:, :q_rank], q_weight, eps).to(out_dtype) if q_rank else None
        if write:
            c = self._rms(down[:, q_rank:q_rank + kv_rank], kv_weight, eps)
            r = down[:, q_rank + kv_rank:q_rank + kv_rank + rot_dim]
            if inv_freq is not None:
                r = self._turn(r, meta.positions, inv_freq, magnitude, neighbours)
            P = k_cache.shape[2]
            slots = meta.groups[group].slots.long()
            k_cache[slots // P, 0, slots % P, :kv_rank] = c.to(k_cache.dtype)
            k_cache[slots // P, 0, slots % P, kv_rank:kv_rank + rot_dim] = r.to(k_cache.dtype)
            v_cache[slots // P, 0, :kv_rank, slots % P] = c.to(v_cache.dtype)
        return latent

    def heads_linear(self, x, weight, in_stride, out_stride, out=None):
        T = x.shape[0]
        H, N, K = weight.shape
        if out is None:
            out = torch.zeros(T, H * out_stride, dtype=x.dtype, device=x.device)
        y = torch.einsum("thk,hnk->thn", x.view(T, H, in_stride)[..., :K].float(), weight.float())
        out.view(T, H, out_stride)[..., :N] = y.to(x.dtype)
        return out

    def rope_heads(self, x, in_stride, in_offset, out, out_stride, out_offset, num_heads, inv_freq, magnitude,
                   neighbours, meta):
        T = x.shape[0]
        n = 2 * inv_freq.shape[0]
        part = x.view(T, num_heads, in_stride)[..., in_offset:in_offset + n].float()
        out.view(T, num_heads, out_stride)[..., out_offset:out_offset + n] = \
            self._turn(part, meta.positions, inv_freq, magnitude, neighbours).to(out.dtype)
        return out

    def glu_mul(self, gate_up, kind):
        inter = gate_up.shape[1] // 2
        g, u = gate_up[:, :inter].float(), gate_up[:, inter:].float()
        return (self.activation(g, kind) * u).to(gate_up.dtype)

    # ---- sums of normed terms, states with their own decays, routers
    @staticmethod
    def _rms(x, weight, eps):
        x = x.float()
        return x / torch.sqrt((x ** 2).mean(-1, keepdim=True) + eps) * weight.float()

    def normed_sum(self, terms, weights, eps, scale):
        return scale * sum(self._rms(t, w, eps) for t, w in zip(terms, weights))

    def add_normed(self, residual, delta, weight, eps):
        residual += self._rms(delta, weight, eps)

    def gated_decay_scan(self, product, decay_logits, state, meta, num_heads, dim, value_dim, q_scale, tau, decay_low=None):
        T = product.shape[0]
        if decay_logits is None:
            decay_logits = self.decay_logits_of(decay_low)
        H, D, E = num_heads, dim, value_dim
        q = product[:, :H * D].float().view(T, H, D) * q_scale
        k = product[:, H * D:2 * H * D].float().view(T, H, D)
        v = product[:, 2 * H * D:H * (2 * D + E)].float().view(T, H, E)
        alpha = torch.exp(torch.nn.functional.logsigmoid(decay_logits.float()) / tau).view(T, H, D)
        out = torch.zeros(T, H, E, dtype=torch.float32, device=product.device)
        cu, slots = meta.cu_q.tolist(), meta.state_slots.tolist()
        for b in range(meta.num_requests):
            s = state[slots[b]]
            for t in range(cu[b], cu[b + 1]):
                s = alpha[t][:, :, None] * s + k[t][:, :, None] * v[t][:, None, :]
                out[t] = torch.einsum("hde,hd->he", s, q[t])
            state[slots[b]] = s
        return out.view(T, H * E)

    def lru_gates(self, u, recur_weight, recur_bias, input_weight, input_bias, lam, rate):
        T, R = u.shape
        B = recur_weight.shape[0]
        parts = u.float().view(T, B, R // B)
        gate = lambda w, b: torch.sigmoid(torch.einsum("tbi,boi->tbo", parts, w.float()) + b.float()).reshape(T, R)
        r, i = gate(recur_weight, recur_bias), gate(input_weight, input_bias)
        a = torch.exp(-rate * r * torch.nn.functional.softplus(lam.float()))
        return a, torch.sqrt(1.0 - a * a) * i * u.float()

    def lru_scan(self, a, x, state, meta, mul, mul_act, out_dtype):
        out = torch.zeros_like(x)
        cu, slots = meta.cu_q.tolist(), meta.state_slots.tolist()
        for b in range(meta.num_requests):
            h = state[slots[b]]
            for t in range(cu[b], cu[b + 1]):
                h = a[t] * h + x[t]
                out[t] = h
            state[slots[b]] = h
        if mul is not None:
            out = out * (mul.float() if mul_act is None else self.activation(mul.float(), mul_act))
        return out.to(out_dtype)

    def route_topk(self, x, weight, bias, top, scoring="softmax"):
        z = x.float() @ weight.float().T
        if bias is not None:
            z = z + bias.float()
        order = torch.sort(z, dim=-1, descending=True, stable=True).indices[:, :top]
        chosen = torch.gather(z, 1, order)
        return order.to(torch.int32), torch.sigmoid(chosen) if scoring == "sigmoid" else torch.softmax(chosen, -1)

    def route_glu(self, gate_up, experts, gates, num_experts, width, limit, slope, up_shift, on_input):
        T = gate_up.shape[0]
        factor = torch.zeros(T, num_experts, dtype=torch.float32, device=gate_up.device)
        factor.scatter_(1, experts.long(), gates.float())
        chosen = torch.zeros(T, num_experts, dtype=torch.bool, device=gate_up.device)
        chosen.scatter_(1, experts.long(), True)
        g = gate_up[:, :num_experts * width].float().view(T, num_experts, width)
        u = gate_up[:, num_experts * width:].float().view(T, num_experts, width)
        if on_input:
            g, u = g * factor[:, :, None], u * factor[:, :, None]
        if limit is not None:
            g, u = g.clamp(max=limit), u.clamp(-limit, limit)
        hidden = g * torch.sigmoid(slope * g) * (u + up_shift)
        if not on_input:
            hidden = hidden * factor[:, :, None]
        hidden = torch.where(chosen[:, :, None], hidden, torch.zeros_like(hidden))
        return hidden.view(T, -1).to(gate_up.dtype)

    def softcap(self, x, cap):
        x.copy_(cap * torch.tanh(x / cap))
        return x

    def route_scale(self, hidden, experts, gates, num_experts, width):
        T = hidden.shape[0]
        factor = torch.zeros(T, num_experts, dtype=torch.float32, device=hidden.device)
        factor.scatter_(1, experts.long(), gates.float())
        routed = hidden[:, :num_experts * width].float().view(T, num_experts, width) * factor[:, :, None]
        hidden[:, :num_experts * width] = routed.view(T, -1).to(hidden.dtype)
        return hidden

    def activation(self, x, kind):
        z = x.float()
        if kind == "relu2":
            r = torch.relu(z) ** 2
        elif kind == "silu":
            r = z * torch.sigmoid(z)
        elif kind == "gelu_tanh":
            r = 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))
        elif kind == "relu":
            r = torch.relu(z)
        else:
            raise ValueError(kind)
        return r.to(x.dtype)

    def silu_mul(self, gate_up):
        inter = gate_up.shape[1] // 2
        g, u = gate_up[:, :inter].float(), gate_up[:, inter:].float()
        return (g * torch.sigmoid(g) * u).to(gate_up.dtype)

    def gather_rows(self, x, rows):
        return x[rows.long()].clone()

    def argmax(self, logits):
        return logits.argmax(-1).to(torch.int32)

    def sample(self, logits, temperature, seeds, counters):
        return plain_sample(logits, temperature, seeds, counters)


def plain_sample(logits, temperature, seeds, counters):
    """argmax where t <= 0; else the first index whose cumulative softmax weight (float64)
    exceeds u * total, u from the request's (seed, counter)."""
    from engine_util import plain_uniform as uniform_of

    out = []
    for row, t, seed, counter in zip(logits.double().cpu(), temperature.tolist(), seeds.tolist(), counters.tolist()):
        if t <= 0:
            out.append(int(row.argmax()))
            continue
        w = torch.exp((row - row.max()) / t)
        target = uniform_of(seed & ((1 << 64) - 1), counter & ((1 << 64) - 1)) * w.sum()
        hit = (torch.cumsum(w, 0) > target).nonzero()
        out.append(int(hit[0]) if len(hit) else int((w > 0).nonzero()[-1]))
    return torch.tensor(out, dtype=torch.int32, device=logits.device)
