"""Configuration of the Zomavik decoder, from its config.json keys.

The file is nested: `layers` lists the layers in their order, each with its `type` (which mixer: "parallel", an
attention and a selective scan side by side on the same input, under `mixer.left` and `mixer.right` with the weights
`mixer.left_scale` and `mixer.right_scale` of their sum), and its feed-forward under `mlp` (null: the layer has none;
`kind` "dense" or "moe").  `loop` (start, stop, times) names a run of layers that is gone through several times;
`embedding.scale`, `logit_scale`, `logit_softcap`, `norm.eps`, `vocab` and `width` hold for the whole model.  Every
size and constant a model may choose is read from here; nothing is assumed equal between layers.
"""
from __future__ import annotations

import dataclasses
from typing import Any

from .base import ConfigError, ModelConfig
from .napadra import _number


@dataclasses.dataclass(frozen=True)
class ZomavikConfig(ModelConfig):
    vocab: int
    width: int
    norm: dict
    layers: list
    embedding: dict | None = None
    loop: dict | None = None
    logit_scale: float | None = None
    logit_softcap: float | None = None
    max_positions: int = 1 << 20      # positions are not bounded by the design: the bound is this engine's own

    MIXERS = ("parallel",)

    def validate(self) -> None:
        for key in ("vocab", "width", "max_positions"):
            if getattr(self, key) <= 0:
                raise ConfigError(f"{key} must be positive, found {getattr(self, key)}")
        _number("norm", self.norm, "eps", float, positive=False)
        if self.embedding is not None:
            _number("embedding", self.embedding, "scale", float)
        for key in ("logit_scale", "logit_softcap"):
            if getattr(self, key) is not None and not getattr(self, key) > 0:
                raise ConfigError(f"{key} must be positive, found {getattr(self, key)}")
        if not isinstance(self.layers, list) or not self.layers:
            raise ConfigError("config.json: `layers` must be a list with at least one layer")
        for index, layer in enumerate(self.layers):
            where = f"layers[{index}]"
            if not isinstance(layer, dict) or layer.get("type") not in self.MIXERS:
                raise ConfigError(f"config.json: {where}.type must be one of {', '.join(self.MIXERS)}")
            mixer = layer.get("mixer")
            if not isinstance(mixer, dict):
                raise ConfigError(f"config.json: {where}.mixer is missing")
            for key in ("left_scale", "right_scale"):
                _number(f"{where}.mixer", mixer, key, float, positive=False)
            left, right = mixer.get("left"), mixer.get("right")
            for key in ("heads", "kv_heads", "dim", "vdim"):
                _number(f"{where}.mixer.left", left, key)
            if left["heads"] % left["kv_heads"]:
                raise ConfigError(f"{where}: {left['heads']} query heads is not a multiple of {left['kv_heads']} kv heads")
            _number(f"{where}.mixer.left", left, "scale", float)
            if left.get("softcap") is not None:
                _number(f"{where}.mixer.left", left, "softcap", float)
            rot = left.get("rot")
            if rot is not None:
                dims = _number(f"{where}.mixer.left.rot", rot, "dims", positive=False)
                _number(f"{where}.mixer.left.rot", rot, "base", float)
                if dims % 2 or not 0 <= dims <= left["dim"]:
                    raise ConfigError(f"{where}.mixer.left.rot.dims must be even and at most the head size, found {dims}")
            for key in ("inner", "state", "dt_rank", "conv"):
                _number(f"{where}.mixer.right", right, key)
            mlp = layer.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind") not in ("dense", "moe"):
                    raise ConfigError(f"config.json: {where}.mlp.kind must be dense or moe")
                if mlp["kind"] == "dense":
                    _number(f"{where}.mlp", mlp, "ff")
                else:
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
                            raise ConfigError(f"{where}.mlp.router.groups: {count} groups of {experts} experts, {keep} "
                                              f"kept, {top} experts a token")
                    if mlp.get("shared") is not None:
                        _number(f"{where}.mlp.shared", mlp["shared"], "ff")
        if self.loop is not None:
            start = _number("loop", self.loop, "start", positive=False)
            stop = _number("loop", self.loop, "stop", positive=False)
            _number("loop", self.loop, "times")
            if not 0 <= start < stop <= len(self.layers):
                raise ConfigError(f"loop: layers {start}..{stop} of {len(self.layers)}")

    @property
    def eps(self) -> float:
        return float(self.norm["eps"])

    @property
    def embedding_scale(self) -> float:
        return float(self.embedding["scale"]) if self.embedding else 1.0

    def run_order(self) -> list[tuple[int, bool]]:
        """(layer, whether a pass through the repeated run starts in front of it), in the order the layers run."""
        n = len(self.layers)
        if self.loop is None:
            return [(index, False) for index in range(n)]
        start, stop, times = int(self.loop["start"]), int(self.loop["stop"]), int(self.loop["times"])
        order = [(index, False) for index in range(start)]
        for _ in range(times):
            order += [(index, index == start) for index in range(start, stop)]
        return order + [(index, False) for index in range(stop, n)]

    def to_dict(self) -> dict[str, Any]:
        out = super().to_dict()
        out.pop("architectures")
        out.pop("max_positions")
        return {"architecture": self.architecture, **out}
