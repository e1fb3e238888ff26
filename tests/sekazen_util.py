"""Small Sekazen models for the tests: configurations, random weights by tensor name, model folders. The names and
shapes of the tensors are written out here from the design, not taken from the package."""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch

import plain_sekazen as plain
from distie_amd.weights.safetensors_io import write_safetensors


def moe(experts=6, top=2, ff=24, limit=1.25):
    return {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff, "limit": limit}}


def scaling(factor=4.0, low=1.0, high=4.0, original=64):
    return {"factor": factor, "low": low, "high": high, "original": original}


def layer(heads=4, kv_heads=2, dim=16, vdim=24, scale=0.3, window=9, dims=8, base=100.0, scaled=True, kv_from=None,
          mlp="moe"):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if window:
        mixer["mask"] = {"size": window}
    if dims:
        mixer["rot"] = {"base": base, "dims": dims}
        if scaled:
            mixer["rot"]["scaling"] = scaling() if scaled is True else scaled
    if kv_from is not None:
        mixer["kv_from"] = kv_from
    return {"type": "attention", "mixer": mixer, "mlp": moe() if mlp == "moe" else mlp}


def make_config(layers, vocab=61, width=48, eps=1e-5, cap=6.0):
    cfg = {"architecture": "Sekazen", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if cap is not None:
        cfg["logit_softcap"] = cap
    return cfg


def tensor_shapes(cfg):
    """Checkpoint name -> shape, from the design."""
    C = cfg["width"]
    out = {"embed": (cfg["vocab"], C), "embed.norm": (C,), "final.norm": (C,)}
    for i, lay in enumerate(cfg["layers"]):
        p, m = f"l{i}.", lay["mixer"]
        H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        out.update({p + "norm1": (C,), p + "mix.q": (H * D, C), p + "mix.q.norm": (D,), p + "mix.sink": (H,),
                    p + "mix.o": (C, H * E)})
        if m.get("kv_from") is None:
            out.update({p + "mix.k": (G * D, C), p + "mix.v": (G * E, C), p + "mix.k.norm": (D,)})
        mlp = lay.get("mlp")
        if mlp:
            F = mlp["expert"]["ff"]
            out.update({p + "norm2": (C,), p + "mlp.router": (mlp["router"]["experts"], C)})
            for e in range(mlp["router"]["experts"]):
                out.update({p + f"mlp.e{e}.gate": (F, C), p + f"mlp.e{e}.up": (F, C), p + f"mlp.e{e}.down": (C, F)})
    return out


def random_weights(cfg, seed=0, dtype=torch.float32):
    """Values that keep every mechanism alive: projections ~ N(0, 1/in), the model-wide norms' weights near zero (they
    count from one), the heads' norms near one, sinks of the size of a score, router logits far apart, experts'
    hidden values that reach the clamps now and then. Rounded to `dtype` (the oracle computes with what the file
    holds)."""
    g = torch.Generator().manual_seed(seed)
    rnd = lambda *shape: torch.randn(*shape, generator=g)
    w = {}
    for name, shape in tensor_shapes(cfg).items():
        last = name.split(".")[-1]
        if name.endswith("q.norm") or name.endswith("k.norm"):
            t = 1.0 + 0.2 * rnd(*shape)
        elif last in ("norm", "norm1", "norm2"):
            t = 0.2 * rnd(*shape)
        elif last == "sink":
            t = 1.5 * rnd(*shape)
        elif last == "router":
            t = 3.0 * rnd(*shape) / math.sqrt(shape[-1])
        elif name == "embed":
            t = rnd(*shape)
        elif last in ("gate", "up"):
            t = 1.5 * rnd(*shape) / math.sqrt(shape[-1])
        else:
            t = rnd(*shape) / math.sqrt(shape[-1])
        w[name] = t.to(dtype)
    return w


def write_model(folder, cfg, weights) -> Path:
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(cfg))
    names = list(weights)
    write_safetensors(folder / "model.safetensors", [(n, weights[n].dtype, tuple(weights[n].shape)) for n in names],
                      ((n, weights[n].contiguous()) for n in names), {"format": "pt"})
    return folder


def oracle(cfg, weights, ids):
    """float64 logits of the plain implementation as float32 [T, vocab]."""
    return plain.forward(cfg, weights, ids)[0].float()


def router_gaps(cfg, weights, ids):
    """For every position: the smallest gap between the last chosen and the first unchosen router logit over the
    routed layers, relative to the largest logit of its row (1.0 where every expert is chosen). A token with a
    large gap chooses the same experts in bfloat16."""
    w = {n: t.double() for n, t in weights.items()}
    eps = float(cfg["norm"]["eps"])
    T = len(ids)
    positions = torch.arange(T)
    gaps = torch.ones(T, dtype=torch.float64)
    x = plain.norm_one_plus(w["embed"][torch.tensor(ids)], w["embed.norm"], eps)
    kept = {}
    for i, lay in enumerate(cfg["layers"]):
        p, m = f"l{i}.", lay["mixer"]
        q = plain.queries(x, w, p + "mix.", m, eps, positions)
        if m.get("kv_from") is None:
            kept[i] = plain.keys_values(x, w, p + "mix.", m, eps, positions)
        k, v = kept[i if m.get("kv_from") is None else int(m["kv_from"])]
        x = x + plain.norm_one_plus(plain.attention(q, k, v, m, w[p + "mix.sink"]) @ w[p + "mix.o"].T, w[p + "norm1"], eps)
        mlp = lay.get("mlp")
        if not mlp:
            continue
        top = mlp["router"]["top"]
        if top < mlp["router"]["experts"]:
            z = x @ w[p + "mlp.router"].T
            s = torch.sort(z, dim=-1, descending=True).values
            gaps = torch.minimum(gaps, (s[:, top - 1] - s[:, top]) / z.abs().max(-1).values)
        x = x + plain.norm_one_plus(plain.mixture(x, w, p + "mlp.", mlp), w[p + "norm2"], eps)
    return gaps


def random_ids(cfg, n, seed):
    return torch.randint(0, cfg["vocab"], (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def clear_ids(cfg, weights, n, seed, margin=0.12):
    """`n` random token ids none of which chooses its experts by a close call (`router_gaps`): the first token that
    does is drawn again (what stands before it stays as it is, being causal), until none is left."""
    g = torch.Generator().manual_seed(seed)
    ids = torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()
    for _ in range(40 * n):
        close = (router_gaps(cfg, weights, ids) < margin).nonzero()
        if not len(close):
            return ids
        ids[int(close[0])] = int(torch.randint(0, cfg["vocab"], (1,), generator=g))
    raise AssertionError("no sequence without a close call found")


def logit_error(got, want):
    """Per row: root mean square of the difference (its mean taken off), over that of the wanted logits."""
    d = got.double() - want.double()
    d = d - d.mean(-1, keepdim=True)
    ref = want.double() - want.double().mean(-1, keepdim=True)
    return (d.pow(2).mean(-1).sqrt() / ref.pow(2).mean().sqrt()).float()


TOL = {torch.float32: 5e-5, torch.bfloat16: 6e-2}
