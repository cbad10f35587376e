"""Arrangements of norms, mixer and feed-forward around the residual stream."""
from __future__ import annotations

import torch

from .base import BLOCKS, Block, NormedDelta, Repeatable, ScaledSum, SumDelta, as_tensor, repeatable_of
from .spec import TensorSpec


@BLOCKS.register("pre_norm")
class PreNormBlock(Block):
    """x + mixer(norm1(x)), then + feed_forward(norm2(.)) (qwen-infer/src/model.rs:615-622).

    The residual stream is float32.  Each sub-layer's output is handed on as a pending `delta`
    so that the add fuses into the next norm; a part that added its output itself hands on None.
    A sub-layer that the layer does not have (None) is passed over.
    """
    graph_safe = True


    def __init__(self, mixer_norm, mixer, feed_forward_norm, feed_forward):
        self.mixer_norm, self.mixer = mixer_norm, mixer
        self.feed_forward_norm, self.feed_forward = feed_forward_norm, feed_forward

    def repeatable(self, cache):
        """The layer's library calls depend on its four parts and on which pages it reads and writes."""
        parts = [repeatable_of(part) for part in (self.mixer_norm, self.mixer, self.feed_forward_norm, self.feed_forward)]
        if any(part is None for part in parts) or cache.state is not None:
            return None
        return Repeatable(("pre_norm", cache.group, cache.writes) + tuple(part.constants for part in parts),
                          sum((part.tensors for part in parts), ()) + (cache.k_pages, cache.v_pages))

    def forward(self, residual, delta, ctx, cache):
        if self.mixer is not None:
            delta = self.mixer.forward_normed(residual, delta, self.mixer_norm, ctx, cache)
        if self.feed_forward is not None:
            delta = self.feed_forward.forward_normed(residual, delta, self.feed_forward_norm, ctx)
        return delta


@BLOCKS.register("parallel")
class ParallelBlock(Block):
    """x + (mixer(h) + feed_forward(h)) with h = norm(x): one norm, and both sub-layers read its output.  The mixer's
    norm is the layer's norm (a feed-forward norm in the layer's spec names the same tensor and is not used).  The two
    outputs are handed on together (`SumDelta`): the next layer's norm adds them to each other and to the float32
    stream and normalises the sum in one kernel.  A layer without a feed-forward hands the mixer's output on alone."""
    graph_safe = True

    def __init__(self, mixer_norm, mixer, feed_forward_norm, feed_forward):
        if mixer is None:
            raise ValueError("a parallel layer has a mixer; its norm is the layer's norm")
        self.mixer_norm, self.mixer = mixer_norm, mixer
        self.feed_forward_norm, self.feed_forward = feed_forward_norm, feed_forward

    def forward(self, residual, delta, ctx, cache):
        h = self.mixer_norm.apply(residual, delta)
        mixed = self.mixer.forward(h, ctx, cache)
        if self.feed_forward is None:
            return mixed
        return SumDelta(self.mixer.runtime.ops, mixed, self.feed_forward.forward(h, ctx))


@BLOCKS.register("parallel_scaled")
class ScaledParallelBlock(Block):
    """x + (s1 * mixer(norm1(x)) + s2 * feed_forward(norm2(x))): two norms of the same x, one for each sub-layer, and
    (option `layer_scale`) a learned scale per coordinate on each output (the block's own tensors `ls1`, `ls2` [width]).
    The outputs are handed on as the terms of a `ScaledSum`: the next norm weights and adds them to the float32 stream
    and normalises the sum in one kernel.  Where both norms are of the form x / sqrt(mean(x^2) + eps) * w, that kernel
    also gives both normalised copies of the row at once.  A mixer may itself hand back a `ScaledSum` (two mixers
    side by side): its terms join the layer's.  A layer without a feed-forward hands the mixer's terms on alone."""
    graph_safe = True

    @staticmethod
    def tensor_specs(layer) -> dict:
        width, out = int(layer.options["width"]), {}
        if layer.options.get("layer_scale"):
            out["ls1"] = TensorSpec((width,), init="ones", role="vector")
            if layer.feed_forward is not None:
                out["ls2"] = TensorSpec((width,), init="ones", role="vector")
        return out

    def __init__(self, mixer_norm, mixer, feed_forward_norm, feed_forward, layer, tensors, runtime):
        if mixer is None:
            raise ValueError("a parallel layer has a mixer")
        self.mixer_norm, self.mixer = mixer_norm, mixer
        self.feed_forward_norm, self.feed_forward = feed_forward_norm, feed_forward
        self.runtime = runtime
        scaled = bool(layer.options.get("layer_scale"))
        self.mixer_scale = tensors["ls1"].to(torch.float32).contiguous() if scaled else None
        self.ff_scale = tensors["ls2"].to(torch.float32).contiguous() if scaled and feed_forward is not None else None

    def _normed(self, residual, delta):
        """Both sub-layers' inputs from the stream and what is still to be added to it."""
        if self.feed_forward is None:
            return self.mixer_norm.apply(residual, delta), None
        ops = self.runtime.ops
        first, second = self.mixer_norm.fold(), self.feed_forward_norm.fold()
        if first is not None and second is not None and hasattr(ops, "add_terms_rmsnorm") \
                and (delta is None or isinstance(delta, (ScaledSum, torch.Tensor))):
            shape = (residual.shape[0], residual.shape[1])
            h1 = torch.empty(shape, dtype=self.runtime.dtype, device=residual.device)
            h2 = torch.empty(shape, dtype=self.runtime.dtype, device=residual.device)
            ops.add_terms_rmsnorm(residual, ScaledSum.of(ops, delta).terms, first.weight, first.eps, h1,
                                  weight2=second.weight, eps2=second.eps, out2=h2)
            return h1, h2
        h1 = self.mixer_norm.apply(residual, delta)
        return h1, self.feed_forward_norm.apply(residual, None)

    def forward(self, residual, delta, ctx, cache):
        ops = self.runtime.ops
        h1, h2 = self._normed(residual, delta)
        out = ScaledSum.of(ops, self.mixer.forward(h1, ctx, cache)).scaled_by(self.mixer_scale)
        if self.feed_forward is not None:
            out = out.plus(ScaledSum.of(ops, self.feed_forward.forward(h2, ctx)).scaled_by(self.ff_scale))
        return out


@BLOCKS.register("sandwich_norm")
class SandwichNormBlock(Block):
    """x + norm_b(mixer(norm(x))), then + norm_b'(feed_forward(norm'(.))): every sub-layer is normalised before and
    behind (RMS norms with weights; the ones behind are the block's own tensors `norm1b`, `norm2b`), and behind the
    feed-forward the layer may add an input made from the token itself (option `side_dim` > 0): with e the layer's
    slice [side_offset, side_offset + side_dim) of the token's row in the shared table `side_table`,
    y = proj(gelu_tanh(gate x) * e), x + y / sqrt(mean(y^2) + eps) * side.norm (tensors `side.gate` [side_dim, width],
    `side.proj` [width, side_dim], `side.norm` [width]).

    The stream is float32.  A sub-layer's output is handed on as a `NormedDelta`: the norm that takes it next brings
    it to unit RMS, scales it, adds it to the stream and normalises the sum in one kernel.
    """
    graph_safe = True

    @staticmethod
    def tensor_specs(layer) -> dict:
        width, out = int(layer.options["width"]), {}
        if layer.mixer is not None:
            out["norm1b"] = TensorSpec((width,), init="ones", role="vector")
        if layer.feed_forward is not None:
            out["norm2b"] = TensorSpec((width,), init="ones", role="vector")
        side = int(layer.options.get("side_dim") or 0)
        if side:
            out.update({"side.gate": TensorSpec((side, width)), "side.proj": TensorSpec((width, side)),
                        "side.norm": TensorSpec((width,), init="ones", role="vector"),
                        "/" + layer.options["side_table"]: TensorSpec((int(layer.options["vocab"]),
                                                                       int(layer.options["side_width"])))})
        return out

    def __init__(self, mixer_norm, mixer, feed_forward_norm, feed_forward, layer, tensors, runtime):
        self.mixer_norm, self.mixer = mixer_norm, mixer
        self.feed_forward_norm, self.feed_forward = feed_forward_norm, feed_forward
        self.runtime, self.eps = runtime, float(layer.options["eps"])
        self.width = int(layer.options["width"])
        self.after_mixer = tensors["norm1b"] if mixer is not None else None
        self.after_feed_forward = tensors["norm2b"] if feed_forward is not None else None
        self.side_dim = int(layer.options.get("side_dim") or 0)
        if self.side_dim:
            self.side_offset = int(layer.options["side_offset"])
            self.side_table = tensors["/" + layer.options["side_table"]]
            self.side_gate, self.side_proj, self.side_norm = tensors["side.gate"], tensors["side.proj"], tensors["side.norm"]
            # The bfloat16 products read eight elements of K at a time: a narrower token input is filled up with
            # zero rows of the gate and zero columns of the projection.
            fill = (-self.side_dim) % 8 if runtime.dtype == torch.bfloat16 else 0
            if fill:
                self.side_gate = torch.cat([self.side_gate, self.side_gate.new_zeros((fill, self.width))], dim=0).contiguous()
                self.side_proj = torch.cat([self.side_proj, self.side_proj.new_zeros((self.width, fill))], dim=1).contiguous()

    def forward(self, residual, delta, ctx, cache):
        ops = self.runtime.ops
        if self.mixer is not None:
            mixed = self.mixer.forward(self.mixer_norm.apply(residual, delta), ctx, cache)
            delta = NormedDelta(ops, mixed, self.after_mixer, self.eps)
        if self.feed_forward is not None:
            out = self.feed_forward.forward(self.feed_forward_norm.apply(residual, delta), ctx)
            delta = NormedDelta(ops, out, self.after_feed_forward, self.eps)
        if self.side_dim:
            if isinstance(delta, NormedDelta) and delta.side is None:
                delta.side = _TokenInput(self, ctx.token_ids)     # whoever takes the term next adds the token input behind it
            else:                                   # what a block of another kind handed on: a plain sum, or nothing
                delta = _TokenInput(self, ctx.token_ids).settle(residual, delta)
        return delta


class _TokenInput:
    """A sandwich block's token input of one step, still to be added behind the block's last term."""

    def __init__(self, block: SandwichNormBlock, token_ids):
        self.block, self.token_ids = block, token_ids

    def fused(self, residual, delta, weight, eps, out, rows):
        """The term's norm and add, the token input and the norm `weight` in one kernel; None if the kernel library
        has none for these sizes."""
        block = self.block
        run = getattr(block.runtime.ops, "norm_side_norm", None)
        if run is None or out.dtype != delta.rows.dtype:
            return None
        return run(residual, delta.rows, delta.weight, delta.eps, block.side_gate, block.side_proj, block.side_norm,
                   block.eps, block.side_table, self.token_ids, block.side_offset, block.side_dim, weight, eps, out, rows)

    def settle(self, residual, delta) -> NormedDelta:
        """Step by step: the stream as it stands behind the term (stored back), the gate's product, the gate, the
        projection; returns the token input as a term of its own."""
        block = self.block
        ops = block.runtime.ops
        rows = torch.empty((residual.shape[0], block.width), dtype=block.runtime.dtype, device=residual.device)
        if isinstance(delta, NormedDelta):
            ops.norm_add_rmsnorm(residual, delta.rows, delta.weight, delta.eps, None, 0.0, rows)
        else:
            ops.norm_add_rmsnorm(residual, None if delta is None else as_tensor(delta), None, 0.0, None, 0.0, rows)
        gate = ops.linear(rows, block.side_gate)
        gated = torch.empty_like(gate)
        ops.side_gate(gate, block.side_table, self.token_ids, block.side_offset, block.side_dim, gated)
        return NormedDelta(ops, ops.linear(gated, block.side_proj), block.side_norm, block.eps)
