"""The Dufelix decoder in the plainest way: float64, whole sequences, one function for each mechanism, loops where a
loop says it best. It shares no code with the package; the tests compare the engine with it.

Notation: T tokens, C the model width, rms(v) = v / sqrt(mean(v^2) + eps). Weights come as a dict by checkpoint name,
linear weights [out, in]."""

from __future__ import annotations

import math

import torch


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm(x, weight, eps):
    return rms(x, eps) * weight


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def frequencies(rot):
    """-> (float64 [dims / 2], the factor on cosine and sine). Stretched frequencies: the dimension at which a
    frequency makes `turns` turns over `original` positions is where(turns); between where(fast) and where(slow) the
    frequency goes linearly from its own value to its value over `factor`."""
    dims, base = int(rot["dims"]), float(rot["base"])
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=torch.float64)
    s = rot.get("scaling")
    if not s:
        return f, 1.0
    where = lambda turns: dims * math.log(float(s["original"]) / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(where(float(s["fast"]))), 0)
    hi = min(math.ceil(where(float(s["slow"]))), dims - 1)
    ramp = torch.tensor([min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0) for i in range(half)], dtype=torch.float64)
    return f / float(s["factor"]) * ramp + f * (1.0 - ramp), 0.1 * math.log(float(s["factor"])) + 1.0


def turn(x, positions, rot, neighbours):
    """x [T, heads, d]: the first rot.dims dimensions of every head turned by the position; pairs are (i, i + dims/2),
    or neighbours (2i, 2i + 1)."""
    if not rot:
        return x
    dims = int(rot["dims"])
    f, magnitude = frequencies(rot)
    angle = positions.double()[:, None] * f[None, :]
    cos, sin = (torch.cos(angle) * magnitude)[:, None, :], (torch.sin(angle) * magnitude)[:, None, :]
    out = x.clone()
    if neighbours:
        a, b = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = a * cos - b * sin
        out[..., 1:dims:2] = b * cos + a * sin
    else:
        a, b = x[..., :dims // 2], x[..., dims // 2:dims]
        out[..., :dims // 2] = a * cos - b * sin
        out[..., dims // 2:dims] = b * cos + a * sin
    return out


def causal_softmax(scores, sink=None):
    """scores [T, T] (query, key) -> weights with keys behind the query masked; `sink`: one more term exp(sink) in
    every row's denominator, with no key."""
    T = scores.shape[0]
    visible = torch.tril(torch.ones(T, T, dtype=torch.bool))
    scores = scores.masked_fill(~visible, -math.inf)
    top = scores.max(-1, keepdim=True).values
    if sink is not None:
        top = torch.maximum(top, sink.reshape(1, 1))
    e = torch.exp(scores - top)
    total = e.sum(-1, keepdim=True)
    if sink is not None:
        total = total + torch.exp(sink - top)
    return e / total


def attention(h, w, p, m, positions):
    """Grouped-query attention with a partial rotation by halves and one gate a head."""
    T = h.shape[0]
    H, G, D, E = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = turn((h @ w[p + "q"].T).view(T, H, D), positions, m.get("rot"), False)
    k = turn((h @ w[p + "k"].T).view(T, G, D), positions, m.get("rot"), False)
    v = (h @ w[p + "v"].T).view(T, G, E)
    gate = torch.sigmoid(h @ w[p + "g"].T)
    heads = []
    for i in range(H):
        j = i // (H // G)
        weights = causal_softmax(q[:, i] @ k[:, j].T * float(m["scale"]))
        heads.append(weights @ v[:, j] * gate[:, i:i + 1])
    return torch.cat(heads, -1) @ w[p + "o"].T


def latent_attention(h, w, p, m, positions, eps):
    """Queries, keys and values through latents; one rotated key part for all heads; a sink in the softmax."""
    T = h.shape[0]
    H, D, R, E, rank = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"])
    q = (norm(h @ w[p + "dq"].T, w[p + "dq.norm"], eps) @ w[p + "uq"].T).view(T, H, D + R)
    q_plain, q_turned = q[..., :D], turn(q[..., D:], positions, m["rot"], True)
    down = h @ w[p + "dkv"].T
    latent = norm(down[:, :rank], w[p + "dkv.norm"], eps)
    k_turned = turn(down[:, rank:].view(T, 1, R), positions, m["rot"], True)[:, 0]
    k_plain = (latent @ w[p + "uk"].T).view(T, H, D)
    v = (latent @ w[p + "uv"].T).view(T, H, E)
    heads = []
    for i in range(H):
        scores = (q_plain[:, i] @ k_plain[:, i].T + q_turned[:, i] @ k_turned.T) * float(m["scale"])
        heads.append(causal_softmax(scores, w[p + "sink"][i]) @ v[:, i])
    return torch.cat(heads, -1) @ w[p + "o"].T


def short_convolution(x, filters, bias):
    """x [T, N], filters [N, taps] (the last column is the current token's), zeros before the start."""
    T, taps = x.shape[0], filters.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, x.shape[1], dtype=x.dtype), x])
    return sum(padded[j:j + T] * filters[:, j] for j in range(taps)) + bias


def state_space_scan(x, B, C, dt, a_log, skip):
    """x [T, H, P], B and C [T, H, N] (already spread over the heads), dt [T, H] (behind softplus) -> y [T, H, P]."""
    T, H, P = x.shape
    state = torch.zeros(H, B.shape[-1], P, dtype=torch.float64)
    y = torch.zeros(T, H, P, dtype=torch.float64)
    rate = -torch.exp(a_log)
    for t in range(T):
        state = torch.exp(rate * dt[t])[:, None, None] * state + dt[t][:, None, None] * B[t][:, :, None] * x[t][:, None, :]
        y[t] = torch.einsum("hnp,hn->hp", state, C[t]) + skip[:, None] * x[t]
    return y


def mamba2(h, w, p, m, eps):
    T = h.shape[0]
    H, P, N, G = int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m["groups"])
    inner = H * P
    z, xbc, dt = torch.split(h @ w[p + "in"].T, [inner, inner + 2 * G * N, H], dim=-1)
    xbc = silu(short_convolution(xbc, w[p + "conv"], w[p + "conv.b"]))
    x = xbc[:, :inner].view(T, H, P)
    B = xbc[:, inner:inner + G * N].view(T, G, N).repeat_interleave(H // G, dim=1)
    C = xbc[:, inner + G * N:].view(T, G, N).repeat_interleave(H // G, dim=1)
    y = state_space_scan(x, B, C, softplus(dt + w[p + "dt_bias"]), w[p + "A_log"], w[p + "D"])
    gated = y.reshape(T, inner) * silu(z)
    parts = int(m["norm_groups"])
    normed = rms(gated.view(T, parts, inner // parts), eps).reshape(T, inner) * w[p + "norm"]
    return normed @ w[p + "o"].T


def feed_forward(h, w, p):
    return (gelu_tanh(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def mixer(kind, h, w, p, m, positions, eps):
    if kind == "attention":
        return attention(h, w, p, m, positions)
    if kind == "latent_attention":
        return latent_attention(h, w, p, m, positions, eps)
    return mamba2(h, w, p, m, eps)


def forward(cfg, weights, ids):
    """-> (float64 logits [T, vocab], the residual behind every layer)."""
    w = {name: t.double() for name, t in weights.items()}
    eps = float(cfg["norm"]["eps"])
    ids = torch.as_tensor(ids, dtype=torch.long)
    positions = torch.arange(len(ids))
    x = w["embed"][ids] * float((cfg.get("embedding") or {}).get("scale", 1.0))
    after = []
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{layer['weights_of'] if layer.get('weights_of') is not None else i}."
        h = norm(x, w[p + "norm1"], eps)
        x = x + norm(mixer(layer["type"], h, w, p + "mix.", layer["mixer"], positions, eps), w[p + "norm1b"], eps)
        if layer.get("mlp"):
            h = norm(x, w[p + "norm2"], eps)
            x = x + norm(feed_forward(h, w, p + "mlp."), w[p + "norm2b"], eps)
        after.append(x.clone())
    return norm(x, w["final.norm"], eps) @ w["head"].T, after
