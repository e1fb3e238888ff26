"""The Dufelix decoder: its config.json and the parts it is made of.

config.json names everything that can differ between models of the design:

    architecture "Dufelix", vocab, width, norm.eps, embedding.scale, and `layers`, one entry a layer: `type`
    ("attention" | "latent_attention" | "mamba2"), `mixer` (its sizes), `mlp` ({"kind": "dense", "ff": n} or null) and,
    optionally, `weights_of`: another layer whose tensors (mixer, feed-forward, norms) this layer uses, with a cache
    or state of its own (its type and sizes are that layer's; an entry may repeat them).

    attention mixer: heads, kv_heads (heads if left out), dim, vdim (dim if left out), rot {base, dims, scaling {factor,
    original, fast, slow}} (no rotation if left out, plain frequencies without `scaling`), scale.
    latent_attention mixer: heads, dim, rot_dim, vdim, kv_rank, q_rank, rot (as above, dims = rot_dim), scale.
    mamba2 mixer: heads, vdim, state, groups, conv (taps), norm_groups (groups and norm_groups are one if left out).

Tensors: `embed`, `head`, `final.norm`; layer i under `l<i>.`: `norm1`, `norm1b`, `norm2`, `norm2b`, `mix.*`,
`mlp.gate|up|down`. Linear weights are [out, in]. Nothing here fixes a size. The one size a file may leave to a tensor's
shape is the rank of the queries' latent (`q_rank`, the rows of `l<i>.mix.dq`).

What the design fixes, and where it stands: a norm in front of and behind every sub-layer (`sandwich_residual`), the
tanh form of gelu in the gated feed-forward, rotation by halves in attention and by neighbours in latent attention, a
gate per head in attention, the sink in latent attention's softmax, the gate in front of the norm in the state-space
mixer.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping

from .model_config import ConfigError, LayerCall, LayerSpec, ModelSpec, PartSpec
from .musutar_config import DEFAULT_MAX_POSITIONS, _need

LAYER_TYPES = ("attention", "latent_attention", "mamba2")


def _check_rot(rot, limit: int, where: str) -> None:
    dims = _need(rot, "dims", int, where + " rot")
    if not _need(rot, "base", float, where + " rot") > 0:
        raise ConfigError(f"{where}: rot.base must be positive")
    if dims < 2 or dims % 2 or dims > limit:
        raise ConfigError(f"{where}: rot.dims must be even and at most the size it turns")
    if rot.get("scaling"):
        for key in ("factor", "original", "fast", "slow"):
            if not _need(rot["scaling"], key, float, where + " rot.scaling") > 0:
                raise ConfigError(f"{where}: rot.scaling.{key} must be positive")


@dataclass(frozen=True)
class DufelixConfig:
    data: Mapping[str, Any]
    max_positions: int = DEFAULT_MAX_POSITIONS

    architecture = "Dufelix"

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
    def from_dict(cls, data: Mapping[str, Any]) -> "DufelixConfig":
        vocab, width = _need(data, "vocab", int, "the model"), _need(data, "width", int, "the model")
        if vocab < 1 or width < 1:
            raise ConfigError("vocab and width must be >= 1")
        _need(data.get("norm") or {}, "eps", float, "norm")
        if data.get("embedding") is not None:
            _need(data["embedding"], "scale", float, "embedding")
        layers = data.get("layers")
        if not isinstance(layers, (list, tuple)) or not layers:
            raise ConfigError("config.json lacks 'layers'")
        for i, layer in enumerate(layers):
            where = f"layer {i}"
            kind = _need(layer, "type", str, where)
            if kind not in LAYER_TYPES:
                raise ConfigError(f"{where}: unknown layer type {kind!r}")
            source = layer.get("weights_of")
            if source is not None:
                owner = cls._owner(layers, i)
                theirs = layers[owner]
                if theirs.get("type") != kind:
                    raise ConfigError(f"{where}: a layer that uses layer {owner}'s tensors has its type")
                for key in ("mixer", "mlp"):
                    if key in layer and cls._sizes(layer[key]) != cls._sizes(theirs.get(key)):
                        raise ConfigError(f"{where}: a layer that uses layer {owner}'s tensors has its sizes")
                continue                                         # (its sizes are the owner's, checked there)
            m = layer.get("mixer")
            if kind == "attention":
                heads = _need(m, "heads", int, where)
                kv_heads = heads if m.get("kv_heads") is None else _need(m, "kv_heads", int, where)
                if heads < 1 or kv_heads < 1 or heads % kv_heads:
                    raise ConfigError(f"{where}: heads must be a positive multiple of kv_heads")
                if _need(m, "dim", int, where) < 1 or (m.get("vdim") is not None and _need(m, "vdim", int, where) < 1):
                    raise ConfigError(f"{where}: dim and vdim must be >= 1")
                if not _need(m, "scale", float, where) > 0:
                    raise ConfigError(f"{where}: scale must be positive")
                if m.get("rot"):
                    _check_rot(m["rot"], int(m["dim"]), where)
            elif kind == "latent_attention":
                for key in ("heads", "dim", "rot_dim", "vdim", "kv_rank"):
                    if _need(m, key, int, where) < 1:
                        raise ConfigError(f"{where}: {key} must be >= 1")
                if m.get("q_rank") is not None and int(m["q_rank"]) < 1:
                    raise ConfigError(f"{where}: q_rank must be >= 1")
                if not _need(m, "scale", float, where) > 0:
                    raise ConfigError(f"{where}: scale must be positive")
                if int(m["rot_dim"]) % 2:
                    raise ConfigError(f"{where}: rot_dim must be even")
                _check_rot(_need(m, "rot", dict, where), int(m["rot_dim"]), where)
                if int(m["rot"]["dims"]) != int(m["rot_dim"]):
                    raise ConfigError(f"{where}: rot.dims must equal rot_dim")
            else:
                for key in ("heads", "vdim", "state", "conv"):
                    if _need(m, key, int, where) < 1:
                        raise ConfigError(f"{where}: {key} must be >= 1")
                for key in ("groups", "norm_groups"):                      # one where a file leaves them out
                    if m.get(key) is not None and _need(m, key, int, where) < 1:
                        raise ConfigError(f"{where}: {key} must be >= 1")
                if int(m["heads"]) % int(m.get("groups") or 1):
                    raise ConfigError(f"{where}: heads must be a multiple of groups")
                if (int(m["heads"]) * int(m["vdim"])) % int(m.get("norm_groups") or 1):
                    raise ConfigError(f"{where}: heads * vdim must be a multiple of norm_groups")
            mlp = layer.get("mlp")
            if mlp is not None:
                if _need(mlp, "kind", str, where + " mlp") != "dense":
                    raise ConfigError(f"{where}: unknown mlp kind {mlp['kind']!r}")
                if _need(mlp, "ff", int, where + " mlp") < 1:
                    raise ConfigError(f"{where}: mlp.ff must be >= 1")
        return cls(data=dict(data), max_positions=int(data.get("max_positions") or DEFAULT_MAX_POSITIONS))

    @staticmethod
    def _owner(layers, i: int) -> int:
        """The layer whose tensors layer i uses: itself, or where its chain of `weights_of` ends."""
        seen = {i}
        while layers[i].get("weights_of") is not None:
            j = layers[i]["weights_of"]
            if isinstance(j, bool) or not isinstance(j, int) or not 0 <= j < len(layers) or j in seen:
                raise ConfigError(f"layer {i}: weights_of must name another layer of the model")
            seen.add(j)
            i = j
        return i

    @staticmethod
    def _sizes(value):
        """A mixer's or feed-forward's entry as numbers compare, whatever way a file wrote them (1 and 1.0 are one size)."""
        if isinstance(value, Mapping):
            return {k: DufelixConfig._sizes(v) for k, v in value.items()}
        if isinstance(value, (int, float)) and not isinstance(value, bool):
            return float(value)
        return value

    def to_dict(self) -> dict:
        return dict(self.data)

    def with_tensor_shapes(self, shapes: Mapping[str, tuple]) -> "DufelixConfig":
        """The one size that a file may leave to the tensors: the rank of the queries' latent."""
        data = dict(self.data)
        layers = []
        for i, layer in enumerate(data["layers"]):
            name = f"l{self._owner(data['layers'], i)}.mix.dq"
            if layer.get("type") == "latent_attention" and isinstance(layer.get("mixer"), Mapping) and \
                    layer["mixer"].get("q_rank") is None and name in shapes and len(shapes[name]) == 2:
                layer = dict(layer, mixer=dict(layer["mixer"], q_rank=int(shapes[name][0])))
            layers.append(layer)
        data["layers"] = layers
        return type(self)(data=data, max_positions=self.max_positions)

    def _mixer(self, kind: str, m: Mapping[str, Any], base: str, layer: int) -> PartSpec:
        width, eps = self.hidden_size, float(self.data["norm"]["eps"])
        rot = m.get("rot")
        position = PartSpec("rope_scaled", "", {"dims": int(rot["dims"]), "base": float(rot["base"]),
                                                "scaling": rot.get("scaling")}) if rot else None
        if kind == "attention":
            return PartSpec("conv_gated_attention", base, {
                "hidden_size": width, "num_heads": int(m["heads"]), "num_kv_heads": int(m.get("kv_heads") or m["heads"]),
                "head_dim": int(m["dim"]), "value_dim": int(m.get("vdim") or m["dim"]), "conv_taps": 0, "window": None,
                "scale": float(m["scale"]), "output_gate": "head", "bias": False, "position": position})
        if kind == "latent_attention":
            if m.get("q_rank") is None:
                raise ConfigError(f"layer {layer}: the rank of the queries' latent comes from the tensors of a model "
                                  f"folder, or from 'q_rank' in the layer's mixer")
            return PartSpec("latent_attention", base, {
                "hidden_size": width, "num_heads": int(m["heads"]), "head_dim": int(m["dim"]),
                "rot_dim": int(m["rot_dim"]), "value_dim": int(m["vdim"]), "kv_rank": int(m["kv_rank"]),
                "q_rank": int(m["q_rank"]), "scale": float(m["scale"]), "eps": eps, "sink": True,
                "rotate": "neighbours", "position": position})
        return PartSpec("state_space_duality", base, {
            "hidden_size": width, "num_heads": int(m["heads"]), "value_dim": int(m["vdim"]),
            "state_size": int(m["state"]), "groups": int(m.get("groups") or 1), "conv_taps": int(m["conv"]),
            "norm_groups": int(m.get("norm_groups") or 1), "eps": eps})

    def model_spec(self) -> ModelSpec:
        data = self.data
        width, eps = self.hidden_size, float(data["norm"]["eps"])
        norm = lambda base, name: PartSpec("rmsnorm", base, {"size": width, "eps": eps, "weight_name": name})
        layers = []
        for i, entry in enumerate(data["layers"]):
            owner = self._owner(data["layers"], i)
            source = None if owner == i else owner
            layer = data["layers"][owner]                    # a layer that uses another's tensors is described by it
            base = f"l{owner}."
            parts = {"mixer": self._mixer(layer["type"], layer["mixer"], base + "mix.", i),
                     "mixer_norm": norm(base, "norm1"), "mixer_post_norm": norm(base, "norm1b")}
            mlp = layer.get("mlp")
            if mlp is not None:
                parts["feed_forward"] = PartSpec("swiglu", base + "mlp.", {
                    "hidden_size": width, "intermediate_size": int(mlp["ff"]), "activation": "gelu_tanh",
                    "gate_name": "gate", "up_name": "up", "down_name": "down"})
                parts["feed_forward_norm"] = norm(base, "norm2")
                parts["feed_forward_post_norm"] = norm(base, "norm2b")
            layers.append(LayerSpec(PartSpec("sandwich_residual", base, {}), parts,
                                    weights_of=None if source is None else int(source)))
        scale = float((data.get("embedding") or {}).get("scale", 1.0))
        return ModelSpec(
            architecture=self.architecture,
            vocab_size=self.vocab_size,
            hidden_size=width,
            max_positions=self.max_positions,
            embedding=PartSpec("token_embedding", "", {"vocab_size": self.vocab_size, "hidden_size": width,
                                                       "weight_name": "embed", "scale": scale}),
            layers=tuple(layers),
            order=tuple(LayerCall(l) for l in range(len(layers))),
            final_norm=norm("final.", "norm"),
            head=PartSpec("lm_head", "", {"vocab_size": self.vocab_size, "hidden_size": width, "weight_name": "head"}),
        )
