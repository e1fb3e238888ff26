"""Small Dufelix models for the tests: configurations, random weights by tensor name, model folders. The names and
shapes of the tensors are written out here from the design, not taken from the package."""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch

import plain_dufelix as plain
from distie_amd.weights.safetensors_io import write_safetensors


def scaling(factor=4.0, original=32, fast=8.0, slow=1.0):
    return {"factor": factor, "original": original, "fast": fast, "slow": slow}


def rot(dims, base=100.0, scaled=True):
    out = {"base": base, "dims": dims}
    if scaled:
        out["scaling"] = scaling() if scaled is True else scaled
    return out


def dense(ff=40):
    return {"kind": "dense", "ff": ff}


def attention(heads=4, kv_heads=2, dim=16, vdim=24, scale=0.3, dims=8, base=100.0, scaled=True, mlp="dense", weights_of=None):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if dims:
        mixer["rot"] = rot(dims, base, scaled)
    return _layer("attention", mixer, mlp, weights_of)


def latent(heads=3, dim=12, rot_dim=8, vdim=20, kv_rank=24, q_rank=28, scale=0.25, base=100.0, scaled=True, mlp="dense",
           weights_of=None):
    mixer = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
             "scale": scale, "rot": rot(rot_dim, base, scaled)}
    return _layer("latent_attention", mixer, mlp, weights_of)


def mamba(heads=4, vdim=12, state=8, groups=2, conv=3, norm_groups=2, mlp="dense", weights_of=None):
    mixer = {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv, "norm_groups": norm_groups}
    return _layer("mamba2", mixer, mlp, weights_of)


def _layer(kind, mixer, mlp, weights_of):
    out = {"type": kind, "mixer": mixer, "mlp": dense() if mlp == "dense" else mlp}
    if weights_of is not None:
        out["weights_of"] = weights_of
    return out


def make_config(layers, vocab=61, width=48, eps=1e-5, embed_scale=3.0):
    return {"architecture": "Dufelix", "vocab": vocab, "width": width, "norm": {"eps": eps},
            "embedding": {"scale": embed_scale}, "layers": layers}


def tensor_shapes(cfg):
    """Checkpoint name -> shape, from the design. A layer that uses another layer's tensors has none."""
    C = cfg["width"]
    out = {"embed": (cfg["vocab"], C), "final.norm": (C,), "head": (cfg["vocab"], C)}
    for i, lay in enumerate(cfg["layers"]):
        if lay.get("weights_of") is not None:
            continue
        p, m = f"l{i}.", lay["mixer"]
        out.update({p + "norm1": (C,), p + "norm1b": (C,)})
        if lay["type"] == "attention":
            H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            out.update({p + "mix.q": (H * D, C), p + "mix.k": (G * D, C), p + "mix.v": (G * E, C), p + "mix.g": (H, C),
                        p + "mix.o": (C, H * E)})
        elif lay["type"] == "latent_attention":
            H, D, R, E, kv, qr = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
            out.update({p + "mix.dq": (qr, C), p + "mix.dq.norm": (qr,), p + "mix.uq": (H * (D + R), qr),
                        p + "mix.dkv": (kv + R, C), p + "mix.dkv.norm": (kv,), p + "mix.uk": (H * D, kv),
                        p + "mix.uv": (H * E, kv), p + "mix.sink": (H,), p + "mix.o": (C, H * E)})
        else:
            H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
            inner, channels = H * P, H * P + 2 * G * N
            out.update({p + "mix.in": (2 * inner + 2 * G * N + H, C), p + "mix.conv": (channels, m["conv"]),
                        p + "mix.conv.b": (channels,), p + "mix.dt_bias": (H,), p + "mix.A_log": (H,), p + "mix.D": (H,),
                        p + "mix.norm": (inner,), p + "mix.o": (C, inner)})
        if lay.get("mlp"):
            F = lay["mlp"]["ff"]
            out.update({p + "norm2": (C,), p + "norm2b": (C,), p + "mlp.gate": (F, C), p + "mlp.up": (F, C),
                        p + "mlp.down": (C, F)})
    return out


def random_weights(cfg, seed=0, dtype=torch.float32):
    """Values that keep every mechanism alive: projections ~ N(0, 1/in), norm weights around one, sinks of the size of
    a score, step sizes and decays spread so that some heads forget within a few tokens and others keep hundreds,
    convolution filters and skip weights of order one. Rounded to `dtype` (the oracle computes with what the file
    holds)."""
    g = torch.Generator().manual_seed(seed)
    rnd = lambda *shape: torch.randn(*shape, generator=g)
    w = {}
    for name, shape in tensor_shapes(cfg).items():
        last = name.split(".")[-1]
        if last in ("norm", "norm1", "norm2", "norm1b", "norm2b"):
            t = 1.0 + 0.2 * rnd(*shape)
        elif last == "sink":
            t = 1.5 * rnd(*shape)
        elif last == "dt_bias":
            t = torch.linspace(-3.0, 1.0, shape[0]) + 0.2 * rnd(*shape)
        elif last == "A_log":
            t = torch.linspace(-3.0, 1.0, shape[0]).flip(0) + 0.2 * rnd(*shape)
        elif last == "D":
            t = 1.0 + 0.3 * rnd(*shape)
        elif last == "conv":
            t = 0.6 * rnd(*shape)
        elif last == "b":
            t = 0.2 * rnd(*shape)
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


def random_ids(cfg, n, seed):
    return torch.randint(0, cfg["vocab"], (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def logit_error(got, want):
    """Per row: root mean square of the difference (its mean taken off), over that of the wanted logits."""
    d = got.double() - want.double()
    d = d - d.mean(-1, keepdim=True)
    ref = want.double() - want.double().mean(-1, keepdim=True)
    return (d.pow(2).mean(-1).sqrt() / ref.pow(2).mean().sqrt()).float()


TOL = {torch.float32: 5e-5, torch.bfloat16: 6e-2}
