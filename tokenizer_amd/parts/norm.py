"""RMSNorm over the last axis, fused with the residual add that precedes it."""
from __future__ import annotations

import torch

from .base import NORMS, Norm, NormedDelta, NormFold, Repeatable, Runtime, ScaledSum, SumDelta
from .spec import NormSpec, TensorSpec


@NORMS.register("rmsnorm")
class RMSNorm(Norm):
    """y = x / sqrt(mean(x^2) + eps) * weight (qwen-infer/src/model.rs:594-599), in float32.  The weight is the
    tensor `weight` under the norm's prefix, or (option `tensor_name`) another name there; the empty name is the
    tensor that the prefix itself names.  Option `offset` c: the stored tensor lies around zero and the scale is
    c + weight (formed once, in float32).  A delta that is itself still to be normalised (`NormedDelta`) is
    normalised, scaled and added in the same kernel; so are the two terms of a `SumDelta` (two sub-layers that read
    the same normalised rows) and the weighted terms of a `ScaledSum`."""
    graph_safe = True


    def __init__(self, spec: NormSpec, tensors: dict[str, torch.Tensor], runtime: Runtime):
        self.size, self.eps = spec.size, float(spec.eps)
        self.weight = tensors[spec.options.get("tensor_name", "weight")]
        offset = float(spec.options.get("offset") or 0.0)
        if offset:
            self.weight = (self.weight.to(torch.float32) + offset).contiguous()
        self.runtime = runtime

    @staticmethod
    def tensor_specs(spec: NormSpec) -> dict[str, TensorSpec]:
        # (A weight that is stored around zero is drawn around zero.)
        return {spec.options.get("tensor_name", "weight"): TensorSpec((spec.size,), role="vector",
                                                                      init="near_zero" if spec.options.get("offset") else "ones")}

    def fold(self):
        return NormFold(self.weight, self.eps)

    def repeatable(self):
        return Repeatable(("rmsnorm", self.size, self.eps), (self.weight,))

    def apply(self, residual, delta, rows=None):
        n_rows = residual.shape[0] if rows is None else rows.numel()
        out = torch.empty((n_rows, self.size), dtype=self.runtime.dtype, device=residual.device)
        if isinstance(delta, SumDelta):
            return self.runtime.ops.add_pair_rmsnorm(residual, delta.first, delta.second, self.weight, self.eps, out, rows,
                                                     store_residual=rows is None)
        if isinstance(delta, ScaledSum):
            return self.runtime.ops.add_terms_rmsnorm(residual, delta.terms, self.weight, self.eps, out, rows,
                                                      store_residual=rows is None)
        if isinstance(delta, NormedDelta):
            if delta.side is not None:
                done = delta.side.fused(residual, delta, self.weight, self.eps, out, rows)
                if done is not None:
                    return done
                delta = delta.side.settle(residual, delta)
            return self.runtime.ops.norm_add_rmsnorm(residual, delta.rows, delta.weight, delta.eps, self.weight, self.eps,
                                                     out, rows, store_residual=rows is None)
        return self.runtime.ops.add_rmsnorm(residual, delta, self.weight, self.eps, out, rows,
                                            store_residual=rows is None)


@NORMS.register("rmsnorm_scalar")
class ScalarRMSNorm(RMSNorm):
    """y = x / sqrt(mean(x^2) + eps) * g with one number g for every coordinate: the tensor that the norm's prefix
    itself names, of shape [].  `gain` is that number (float32 [1]) for kernels that take it so; `weight` repeats
    it over the row for the kernels of the norm above, which this norm then shares (its `fold()` too)."""
    graph_safe = True

    def __init__(self, spec: NormSpec, tensors: dict[str, torch.Tensor], runtime: Runtime):
        self.size, self.eps, self.runtime = spec.size, float(spec.eps), runtime
        self.gain = tensors[""].reshape(1).to(torch.float32).contiguous()
        self.weight = self.gain.expand(spec.size).contiguous()

    @staticmethod
    def tensor_specs(spec: NormSpec) -> dict[str, TensorSpec]:
        return {"": TensorSpec((), init="ones", role="vector")}

    def repeatable(self):
        return Repeatable(("rmsnorm_scalar", self.size, self.eps), (self.weight, self.gain))
