"""The Sekazen decoder written out plainly, in float64, one function per mechanism, from the design's equations. It
shares no code with the package: the tests compare the engine with this.

Notation: T tokens, C the model width; rms(v) = v / sqrt(mean(v^2) + eps) over the last dimension.

    x0 = rms(embed[token]) (1 + w_e)
    a layer:  x <- x + rms(mixer(x)) (1 + w_1);   x <- x + rms(ff(x)) (1 + w_2)       (a layer may have no ff)
    logits = cap tanh((rms(x) (1 + w_f)) embed^T / cap)

Mixer: H query heads on G key/value heads; q, k get an RMS norm over every head (weight as stored, shared by the
heads), then the first `dims` dimensions of every head are turned by the position's angles; score = q . k * scale
over the keys j with 0 <= i - j < window; the softmax's denominator holds exp(sink_h) as one more term. A layer with
`kv_from` takes another layer's turned keys and its values.
Feed-forward: scores s = sigmoid(W_r h); the `top` largest choose the experts; expert e gets s_e h as its input;
g = min(W_g u, limit), v = clamp(W_u u, -limit, limit), out = W_d (g sigmoid(1.702 g) (v + 1)); the outputs are added.
"""

from __future__ import annotations

import math

import torch


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_one_plus(x, weight, eps):
    """The norms of the model width: the stored weight is the distance from one."""
    return rms(x, eps) * (1.0 + weight)


def frequencies(rot):
    """f_i for i < dims / 2, with the bands of the scaling: short wavelengths stay, long ones are divided by the
    factor, those between are blended."""
    dims = int(rot["dims"])
    scaling = rot.get("scaling")
    out = []
    for i in range(dims // 2):
        f = float(rot["base"]) ** (-2.0 * i / dims)
        if scaling:
            wavelength = 2.0 * math.pi / f
            short, long_ = scaling["original"] / scaling["high"], scaling["original"] / scaling["low"]
            if wavelength > long_:
                f = f / scaling["factor"]
            elif wavelength >= short:
                s = (scaling["original"] / wavelength - scaling["low"]) / (scaling["high"] - scaling["low"])
                f = (1.0 - s) * f / scaling["factor"] + s * f
        out.append(f)
    return torch.tensor(out, dtype=torch.float64)


def turn(x, positions, rot):
    """x [T, heads, dim]: dimension i pairs with i + dims / 2; (u, v) -> (u cos a - v sin a, v cos a + u sin a)."""
    if not rot:
        return x
    dims = int(rot["dims"])
    half = dims // 2
    angle = positions.double()[:, None] * frequencies(rot)[None, :]
    c, s = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


def softmax_with_sink(scores, visible, sink):
    """scores [T, T] of one head, visible [T, T] bool, sink a number: weights over the visible keys whose
    denominator also holds exp(sink)."""
    scores = scores.masked_fill(~visible, -math.inf)
    top = torch.maximum(scores.max(-1, keepdim=True).values, torch.as_tensor(sink, dtype=scores.dtype))
    e = torch.exp(scores - top)
    return e / (e.sum(-1, keepdim=True) + torch.exp(sink - top))


def visible_keys(T, window):
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    ok = j <= i
    if window is not None:
        ok = ok & (i - j < int(window))
    return ok


def queries(h, w, p, m, eps, positions):
    T = h.shape[0]
    q = (h @ w[p + "q"].T).view(T, m["heads"], m["dim"])
    return turn(rms(q, eps) * w[p + "q.norm"], positions, m.get("rot"))


def keys_values(h, w, p, m, eps, positions):
    T = h.shape[0]
    k = (h @ w[p + "k"].T).view(T, m["kv_heads"], m["dim"])
    v = (h @ w[p + "v"].T).view(T, m["kv_heads"], m["vdim"])
    return turn(rms(k, eps) * w[p + "k.norm"], positions, m.get("rot")), v


def attention(q, k, v, m, sinks):
    T, H = q.shape[0], m["heads"]
    per = H // m["kv_heads"]
    window = (m.get("mask") or {}).get("size")
    ok = visible_keys(T, window)
    out = []
    for head in range(H):
        scores = (q[:, head] @ k[:, head // per].T) * float(m["scale"])
        out.append(softmax_with_sink(scores, ok, sinks[head]) @ v[:, head // per])
    return torch.stack(out, dim=1).reshape(T, H * m["vdim"])


def expert(u, w, p, limit):
    g = torch.clamp(u @ w[p + "gate"].T, max=limit)
    v = torch.clamp(u @ w[p + "up"].T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (v + 1.0)) @ w[p + "down"].T


def router_scores(h, w, p):
    return torch.sigmoid(h @ w[p + "router"].T)


def mixture(h, w, p, mlp):
    scores = router_scores(h, w, p)
    top = int(mlp["router"]["top"])
    order = torch.sort(scores, dim=-1, descending=True, stable=True).indices[:, :top]
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e in order[t].tolist():
            out[t] += expert(scores[t, e] * h[t], w, f"{p}e{e}.", float(mlp["expert"]["limit"]))
    return out


def forward(cfg, weights, ids):
    """-> (float64 logits [T, vocab], the residual behind every layer [layers, T, C])."""
    w = {n: t.double() for n, t in weights.items()}
    eps = float(cfg["norm"]["eps"])
    ids = torch.as_tensor(ids, dtype=torch.long)
    positions = torch.arange(len(ids))
    x = norm_one_plus(w["embed"][ids], w["embed.norm"], eps)
    kept, after = {}, []
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        q = queries(x, w, p + "mix.", m, eps, positions)
        if m.get("kv_from") is None:
            kept[i] = keys_values(x, w, p + "mix.", m, eps, positions)
        k, v = kept[i if m.get("kv_from") is None else int(m["kv_from"])]
        y = attention(q, k, v, m, w[p + "mix.sink"]) @ w[p + "mix.o"].T
        x = x + norm_one_plus(y, w[p + "norm1"], eps)
        if layer.get("mlp"):
            x = x + norm_one_plus(mixture(x, w, p + "mlp.", layer["mlp"]), w[p + "norm2"], eps)
        after.append(x.clone())
    logits = norm_one_plus(x, w["final.norm"], eps) @ w["embed"].T
    cap = cfg.get("logit_softcap")
    if cap:
        logits = float(cap) * torch.tanh(logits / float(cap))
    return logits, torch.stack(after)
