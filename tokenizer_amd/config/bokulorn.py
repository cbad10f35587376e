"""Configuration of the Bokulorn decoder, from its config.json keys.

The file is nested: `layers` lists the layers in their order, each with its `type` (which mixer: "latent_attention",
attention over a cached latent with a rotated key part; "latent_attention_2", the same without positions and with a
gate per coordinate; "channel_delta", a gated delta rule with a decay per key channel), the mixer's sizes and constants
under `mixer` and its feed-forward under `mlp` (null: the layer has none; `kind` "moe").  A layer with `weights_of`: j
has no tensors of its own and runs with layer j's, keeping a cache or state of its own.  `embedding.scale`, `norm.eps`,
`vocab` and `width` hold for the whole model.  Every size and constant a model may choose is read from here; nothing is
assumed equal between layers.
"""
from __future__ import annotations

import dataclasses
from typing import Any

from .base import ConfigError, ModelConfig
from .napadra import _number


@dataclasses.dataclass(frozen=True)
class BokulornConfig(ModelConfig):
    vocab: int
    width: int
    norm: dict
    layers: list
    embedding: dict | None = None
    max_positions: int = 1 << 20      # positions are not bounded by the design: the bound is this engine's own

    MIXERS = ("latent_attention", "latent_attention_2", "channel_delta")

    def validate(self) -> None:
        for key in ("vocab", "width", "max_positions"):
            if getattr(self, key) <= 0:
                raise ConfigError(f"{key} must be positive, found {getattr(self, key)}")
        _number("norm", self.norm, "eps", float, positive=False)
        if self.embedding is not None:
            _number("embedding", self.embedding, "scale", float)
        if not isinstance(self.layers, list) or not self.layers:
            raise ConfigError("config.json: `layers` must be a list with at least one layer")
        for index, layer in enumerate(self.layers):
            where = f"layers[{index}]"
            if not isinstance(layer, dict) or layer.get("type") not in self.MIXERS:
                raise ConfigError(f"config.json: {where}.type must be one of {', '.join(self.MIXERS)}")
            mixer = layer.get("mixer")
            for key in ("heads", "dim", "vdim"):
                _number(f"{where}.mixer", mixer, key)
            if layer["type"] == "channel_delta":
                kv_heads = _number(f"{where}.mixer", mixer, "kv_heads")
                if mixer["heads"] % kv_heads:
                    raise ConfigError(f"{where}: {mixer['heads']} heads is not a multiple of {kv_heads} query/key heads")
                _number(f"{where}.mixer", mixer, "conv")
            else:
                for key in ("q_rank", "kv_rank"):
                    _number(f"{where}.mixer", mixer, key)
                _number(f"{where}.mixer", mixer, "scale", float)
                if layer["type"] == "latent_attention":
                    rot_dim = _number(f"{where}.mixer", mixer, "rot_dim")
                    dims = _number(f"{where}.mixer.rot", mixer.get("rot"), "dims")
                    _number(f"{where}.mixer.rot", mixer.get("rot"), "base", float)
                    if dims != rot_dim or dims % 2:
                        raise ConfigError(f"{where}.mixer: the rotation covers the whole rotated part, an even number "
                                          f"of coordinates; found rot.dims {dims} and rot_dim {rot_dim}")
            mlp = layer.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind") != "moe":
                    raise ConfigError(f"config.json: {where}.mlp.kind must be moe")
                _number(f"{where}.mlp.expert", mlp.get("expert"), "ff")
                experts = _number(f"{where}.mlp.router", mlp.get("router"), "experts")
                top = _number(f"{where}.mlp.router", mlp.get("router"), "top")
                if top > experts:
                    raise ConfigError(f"{where}.mlp.router: top {top} of {experts} experts")
                groups = mlp["router"].get("groups")
                if groups is not None:
                    count = _number(f"{where}.mlp.router.groups", groups, "count")
                    keep = _number(f"{where}.mlp.router.groups", groups, "keep")
                    if experts % count or keep > count or keep * (experts // count) < top:
                        raise ConfigError(f"{where}.mlp.router.groups: {count} groups of {experts} experts, {keep} kept, "
                                          f"{top} experts a token")
            source = layer.get("weights_of")
            if source is not None:
                if isinstance(source, bool) or not isinstance(source, int) or not 0 <= source < len(self.layers) \
                        or source == index:
                    raise ConfigError(f"{where}.weights_of must name another layer, found {source!r}")
        for index in range(len(self.layers)):
            self.weight_owner(index)

    @property
    def eps(self) -> float:
        return float(self.norm["eps"])

    @property
    def embedding_scale(self) -> float:
        return float(self.embedding["scale"]) if self.embedding else 1.0

    def weight_owner(self, index: int) -> int:
        """The layer whose tensors layer `index` runs with (itself, unless it names another)."""
        seen = set()
        while self.layers[index].get("weights_of") is not None:
            if index in seen:
                raise ConfigError(f"layers[{index}].weights_of leads back to itself")
            seen.add(index)
            index = int(self.layers[index]["weights_of"])
        return index

    def to_dict(self) -> dict[str, Any]:
        out = super().to_dict()
        out.pop("architectures")
        out.pop("max_positions")
        return {"architecture": self.architecture, **out}
