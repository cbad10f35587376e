"""Two mixers side by side on the same input."""
from __future__ import annotations

import dataclasses

import torch

from .base import MIXERS, Mixer, Runtime, ScaledSum
from .model import _named_back, _renamed, _strip
from .spec import CacheNeed, MixerSpec, TensorSpec


@MIXERS.register("side_by_side")
class SideBySide(Mixer):
    """a * left(h) + b * right(h): two mixers of any registered kinds read the same input (options `left`, `right`: their
    `MixerSpec`; `left_scale` a, `right_scale` b).  Their tensors lie under `left.` and `right.`; at most one of them
    keeps pages and at most one keeps state in the request's slot, and the layer's need of the cache is both together.
    The two outputs are handed on as the terms of a `ScaledSum`, so the weights are applied in float32 where the sum
    joins the stream."""

    SIDES = ("left", "right")

    def __init__(self, spec: MixerSpec, tensors: dict[str, torch.Tensor], runtime: Runtime):
        self.spec, self.runtime = spec, runtime
        self.parts, self.factors = [], []
        for side in self.SIDES:
            inner: MixerSpec = spec.options[side]
            own = _named_back(_strip(side, tensors), inner.tensor_names)
            self.parts.append(MIXERS.get(inner.kind)(inner, own, runtime))
            self.factors.append(float(spec.options.get(f"{side}_scale", 1.0)))
        self.graph_safe = all(getattr(part, "graph_safe", False) for part in self.parts)

    @staticmethod
    def tensor_specs(spec: MixerSpec) -> dict[str, TensorSpec]:
        out = {}
        for side in SideBySide.SIDES:
            inner: MixerSpec = spec.options[side]
            for name, tensor in _renamed(MIXERS.get(inner.kind).tensor_specs(inner), inner.tensor_names).items():
                out[f"{side}.{name}" if name else side] = tensor
        return out

    @staticmethod
    def cache_need(spec: MixerSpec) -> CacheNeed:
        needs = [MIXERS.get(spec.options[side].kind).cache_need(spec.options[side]) for side in SideBySide.SIDES]
        paged = [need for need in needs if need.kind != "none"]
        stateful = [need for need in needs if need.state_shape is not None]
        if len(paged) > 1 or len(stateful) > 1 or any(need.block_state_shape is not None for need in needs):
            raise ValueError("of two mixers side by side at most one keeps pages and at most one keeps state")
        need = paged[0] if paged else CacheNeed()
        if stateful:
            need = dataclasses.replace(need, state_shape=stateful[0].state_shape, state_dtype=stateful[0].state_dtype)
        return need

    def forward(self, x, ctx, cache):
        ops = self.runtime.ops
        out = ScaledSum(ops)
        for part, factor in zip(self.parts, self.factors):
            out = out.plus(ScaledSum.of(ops, part.forward(x, ctx, cache)).scaled_by(None, factor))
        return out
