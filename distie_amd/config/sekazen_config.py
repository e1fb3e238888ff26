"""The Sekazen decoder: its config.json and the parts it is made of.

config.json names everything that can differ between models of the design:

    architecture "Sekazen", vocab, width, norm.eps, logit_softcap, and `layers`, one entry a layer: `type`
    ("attention"), `mixer` (its sizes) and `mlp` (or null).

    attention mixer: heads, kv_heads, dim, vdim, rot {base, dims, scaling {factor, low, high, original}}, scale,
    mask {size} (the window), kv_from (a layer whose keys and values are used).
    mlp: {"kind": "moe", "router" {experts, top}, "expert" {ff, limit}}.

Tensors: `embed`, `embed.norm`, `final.norm`; layer i under `l<i>.`: `norm1`, `norm2`, `mix.q`, `mix.k`, `mix.v`,
`mix.o`, `mix.q.norm`, `mix.k.norm`, `mix.sink`, `mlp.router`, `mlp.e<e>.gate|up|down`. Linear weights are
[out, in]. The head is the embedding table. Nothing here fixes a size.

What the design fixes, and where it stands: the files hold the norms' weights minus one (`offset` 1 on every norm of
the model width, 0 on the per-head norms of queries and keys); the experts' activation g * sigmoid(1.702 g) * (u + 1)
(`slope`, `up_shift`); the router's sigmoid scores, not renormalised, on the experts' input.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping

from .model_config import ConfigError, LayerCall, LayerSpec, ModelSpec, PartSpec
from .musutar_config import DEFAULT_MAX_POSITIONS, _need

EXPERT_SLOPE = 1.702          # g * sigmoid(1.702 g): the sigmoid form of gelu
EXPERT_UP_SHIFT = 1.0         # ... times (u + 1)


@dataclass(frozen=True)
class SekazenConfig:
    data: Mapping[str, Any]
    max_positions: int = DEFAULT_MAX_POSITIONS

    architecture = "Sekazen"

    @property
    def vocab_size(self) -> int:
        return int(self.data["vocab"])

    @property
    def hidden_size(self) -> int:
        return int(self.data["width"])

    @property
    def num_layers(self) -> int:
        return len(self.data["layers"])

    @classmethod
    def from_dict(cls, data: Mapping[str, Any]) -> "SekazenConfig":
        vocab, width = _need(data, "vocab", int, "the model"), _need(data, "width", int, "the model")
        if vocab < 1 or width < 1:
            raise ConfigError("vocab and width must be >= 1")
        _need(data.get("norm") or {}, "eps", float, "norm")
        if data.get("logit_softcap") is not None and not _need(data, "logit_softcap", float, "the model") > 0:
            raise ConfigError("logit_softcap must be positive")
        layers = data.get("layers")
        if not isinstance(layers, (list, tuple)) or not layers:
            raise ConfigError("config.json lacks 'layers'")
        for i, layer in enumerate(layers):
            where = f"layer {i}"
            kind = _need(layer, "type", str, where)
            if kind != "attention":
                raise ConfigError(f"{where}: unknown layer type {kind!r}")
            mixer = layer.get("mixer")
            heads, kv_heads = _need(mixer, "heads", int, where), _need(mixer, "kv_heads", int, where)
            dim, vdim = _need(mixer, "dim", int, where), _need(mixer, "vdim", int, where)
            if heads < 1 or kv_heads < 1 or heads % kv_heads:
                raise ConfigError(f"{where}: heads must be a positive multiple of kv_heads")
            if dim < 1 or vdim < 1:
                raise ConfigError(f"{where}: dim and vdim must be >= 1")
            if not _need(mixer, "scale", float, where) > 0:
                raise ConfigError(f"{where}: scale must be positive")
            rot = mixer.get("rot")
            if rot:
                dims = _need(rot, "dims", int, where + " rot")
                if not _need(rot, "base", float, where + " rot") > 0:
                    raise ConfigError(f"{where}: rot.base must be positive")
                if dims < 2 or dims % 2 or dims > dim:
                    raise ConfigError(f"{where}: rot.dims must be even and at most dim")
                if rot.get("scaling"):
                    for key in ("factor", "low", "high", "original"):
                        _need(rot["scaling"], key, float, where + " rot.scaling")
                    if float(rot["scaling"]["high"]) == float(rot["scaling"]["low"]):
                        raise ConfigError(f"{where}: rot.scaling.high and low must differ")
            if mixer.get("mask") and _need(mixer["mask"], "size", int, where + " mask") < 1:
                raise ConfigError(f"{where}: mask.size must be >= 1")
            source = mixer.get("kv_from")
            if source is not None:
                source = int(source)
                if not 0 <= source < i or layers[source]["mixer"].get("kv_from") is not None:
                    raise ConfigError(f"{where}: kv_from must name an earlier layer with keys of its own")
                theirs = layers[source]["mixer"]
                if any(int(theirs[k]) != int(mixer[k]) for k in ("kv_heads", "dim", "vdim")):
                    raise ConfigError(f"{where}: kv_from names a layer with other head sizes")
            mlp = layer.get("mlp")
            if mlp is None:
                continue
            if _need(mlp, "kind", str, where + " mlp") != "moe":
                raise ConfigError(f"{where}: unknown mlp kind {mlp['kind']!r}")
            router = mlp.get("router")
            experts, top = _need(router, "experts", int, where + " router"), _need(router, "top", int, where + " router")
            if not 1 <= top <= experts:
                raise ConfigError(f"{where}: router.top must be between 1 and router.experts")
            if _need(mlp.get("expert"), "ff", int, where + " expert") < 1:
                raise ConfigError(f"{where}: expert.ff must be >= 1")
            if not _need(mlp["expert"], "limit", float, where + " expert") > 0:
                raise ConfigError(f"{where}: expert.limit must be positive")
        return cls(data=dict(data), max_positions=int(data.get("max_positions") or DEFAULT_MAX_POSITIONS))

    def to_dict(self) -> dict:
        return dict(self.data)

    def _kept_windows(self) -> dict:
        """For every layer with keys of its own: how far back its cache must reach, the widest window among itself
        and the layers that borrow from it (None: everything)."""
        layers = self.data["layers"]
        window = lambda m: (m.get("mask") or {}).get("size")
        kept = {i: window(l["mixer"]) for i, l in enumerate(layers) if l["mixer"].get("kv_from") is None}
        for layer in layers:
            source = layer["mixer"].get("kv_from")
            if source is not None and kept[int(source)] is not None:
                mine = window(layer["mixer"])
                kept[int(source)] = None if mine is None else max(int(kept[int(source)]), int(mine))
        return kept

    def model_spec(self) -> ModelSpec:
        data = self.data
        width, eps = self.hidden_size, float(data["norm"]["eps"])
        norm = lambda base, name: PartSpec("rmsnorm", base, {"size": width, "eps": eps, "weight_name": name, "offset": 1.0})
        kept = self._kept_windows()
        layers = []
        for i, layer in enumerate(data["layers"]):
            base = f"l{i}."
            m = layer["mixer"]
            rot = m.get("rot")
            window = (m.get("mask") or {}).get("size")
            mixer = PartSpec("conv_gated_attention", base + "mix.", {
                "hidden_size": width, "num_heads": int(m["heads"]), "num_kv_heads": int(m["kv_heads"]),
                "head_dim": int(m["dim"]), "value_dim": int(m["vdim"]), "conv_taps": 0,
                "window": None if window is None else int(window),
                "keep": kept.get(i, None if window is None else int(window)),
                "scale": float(m["scale"]), "output_gate": False, "bias": False, "sink": True,
                "qk_norm": {"eps": eps, "offset": 0.0},
                "kv_from": None if m.get("kv_from") is None else int(m["kv_from"]),
                "position": PartSpec("rope_banded", "", {"dims": int(rot["dims"]), "base": float(rot["base"]),
                                                         "scaling": rot.get("scaling")}) if rot else None,
            })
            parts = {"mixer": mixer, "mixer_post_norm": norm(base, "norm1")}
            mlp = layer.get("mlp")
            if mlp is not None:
                parts["feed_forward"] = PartSpec("routed_experts", base + "mlp.", {
                    "hidden_size": width, "num_experts": int(mlp["router"]["experts"]), "top": int(mlp["router"]["top"]),
                    "expert_size": int(mlp["expert"]["ff"]), "router_bias": False, "scoring": "sigmoid",
                    "weight_on": "input", "activation": "clamped_glu", "limit": float(mlp["expert"]["limit"]),
                    "slope": EXPERT_SLOPE, "up_shift": EXPERT_UP_SHIFT})
                parts["feed_forward_post_norm"] = norm(base, "norm2")
            layers.append(LayerSpec(PartSpec("branch_norm_residual", base, {}), parts))
        cap = data.get("logit_softcap")
        return ModelSpec(
            architecture=self.architecture,
            vocab_size=self.vocab_size,
            hidden_size=width,
            max_positions=self.max_positions,
            embedding=PartSpec("token_embedding", "", {"vocab_size": self.vocab_size, "hidden_size": width,
                                                       "weight_name": "embed", "norm": norm("embed.", "norm")}),
            layers=tuple(layers),
            order=tuple(LayerCall(l) for l in range(len(layers))),
            final_norm=norm("final.", "norm"),
            head=PartSpec("lm_head", "", {"vocab_size": self.vocab_size, "hidden_size": width, "tied_to": "embed",
                                          "weight_name": "head", "cap": None if cap is None else float(cap)}),
        )
