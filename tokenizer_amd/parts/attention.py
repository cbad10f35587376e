"""Grouped-query attention over the paged cache."""
from __future__ import annotations

import math

import torch

from .base import can_fuse_decode as _can_fuse
from .base import MIXERS, POSITIONS, Mixer, Repeatable, Runtime, repeatable_of
from .spec import CacheNeed, MixerSpec, PositionSpec, TensorSpec


@MIXERS.register("gqa_attention")
class GQAttention(Mixer):
    """q/k/v projections (optional bias), position encoding, causal attention with an optional
    window over the request's pages, output projection.

    Order of operations as qwen-infer/src/model.rs:279-328 and 397-414: keys are stored after
    the position encoding, values as projected; kv head g serves query heads g*r..(g+1)*r-1
    (model.rs:571-580); scores are scaled by 1/sqrt(d) after the product; a key is visible when
    key <= query and, with a window w, key + w >= query (model.rs:119-129).
    The three projection matrices are joined into one at load time so one product makes q, k and v.

    Options of the spec, each on its own: `value_dim` (value heads of another size than the key heads), `chunk`
    (a query sees only the keys of its own run of `chunk` positions, runs counted from position 0 of the
    sequence), `distance_bias` b (head h's score loses 2^(-b (h+1) / n_heads) for every position between query
    and key), `sink` (tensor `sink`, one number per head, joins the softmax's denominator as exp(sink): no key,
    no value, not scaled, no bias) and `own_kv` False (no key and value projections: the layer reads the pages
    of the layer it is pointed at and writes nothing).  Scores, bias and weights are float32 in every kernel.

    A second family of options runs through `_run_extended` (any of them, or a position encoding of kind
    `rope_partial`, takes the layer there): `differential` c (every head has two score maps, each a softmax of its
    own over the same values: q and k projections are twice as tall, laid out head by head as [map 1, map 2];
    o = a1 - lambda a2 with lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + c, one number for the layer from the tensors
    `lq1`, `lk1`, `lq2`, `lk2` [d]; o is brought to unit RMS over the head's values, without a weight, and
    multiplied by 1 - c), `keep_first` n (under a window, keys at positions below n stay visible to every later
    query, at their true positions), `qk_norm` "whole" (an RMS norm with weights `q_norm` [n_heads d] / `k_norm`
    [n_kv d] over all query rows at once and over all key rows at once, before the rotation) and `head_gate`
    (head h's output times sigmoid(W_g x)_h, W_g = `gate_proj.weight` [n_heads, hidden], read from the mixer's
    input; the gate's rows ride in the joined projection) and `softcap` c (a scaled score s becomes c tanh(s / c)
    before the softmax); `sink` joins these too.  For the kernels the maps of differential heads are
    heads of their own: the query rows are reordered at load time to (kv head, map, head within the group), so
    that map m of kv head g is key head 2 g + m in the ordinary grouping, and key heads 2 g and 2 g + 1 read
    value head g (`value_heads`).
    """
    graph_safe = True


    def __init__(self, spec: MixerSpec, tensors: dict[str, torch.Tensor], runtime: Runtime):
        self.spec, self.runtime = spec, runtime
        self.n_q, self.n_kv, self.d = spec.n_heads, spec.n_kv_heads, spec.head_dim
        self.dv = spec.value_dim or spec.head_dim
        self.own_kv = spec.own_kv
        self.extended = self._is_extended(spec)
        if self.extended:
            self._build_extended(spec, tensors, runtime)
            return
        joined = ("q_proj", "k_proj", "v_proj") if spec.own_kv else ("q_proj",)
        self.w_qkv = torch.cat([tensors[f"{name}.weight"] for name in joined], dim=0).contiguous()
        self.b_qkv = None
        if spec.qkv_bias:
            self.b_qkv = torch.cat([tensors[f"{name}.bias"] for name in joined], dim=0).contiguous()
        self.chunk = spec.chunk
        self.slopes = None
        if spec.distance_bias is not None:
            self.slopes = torch.tensor([2.0 ** (-float(spec.distance_bias) * (h + 1) / self.n_q) for h in range(self.n_q)],
                                       dtype=torch.float32, device=runtime.device)
        self.sinks = tensors["sink"].to(torch.float32).contiguous() if spec.sink else None
        # What the kernels written for the plain form (equal head sizes, every earlier key visible up to a window,
        # a softmax over the keys alone) do not compute.
        self.extras = dict(value_dim=self.dv, chunk=self.chunk, slopes=self.slopes, sinks=self.sinks)
        self.plain = (self.dv == self.d and self.chunk is None and self.slopes is None and self.sinks is None
                      and self.own_kv)
        self.w_o = tensors["o_proj.weight"]
        self.b_o = tensors.get("o_proj.bias") if spec.out_bias else None
        self.scale = float(spec.scale) if spec.scale is not None else 1.0 / math.sqrt(self.d)
        self.window = spec.window
        position = spec.position or PositionSpec("none")
        self.position = POSITIONS.get(position.kind)(position, runtime)
        self.graph_safe = bool(getattr(self.position, "graph_safe", False))

    @staticmethod
    def _is_extended(spec: MixerSpec) -> bool:
        return (spec.differential is not None or bool(spec.keep_first) or spec.qk_norm is not None or spec.head_gate
                or spec.softcap is not None or (spec.position is not None and spec.position.kind == "rope_partial"))

    def _build_extended(self, spec: MixerSpec, tensors: dict[str, torch.Tensor], runtime: Runtime) -> None:
        if not spec.own_kv or spec.chunk is not None or spec.distance_bias is not None or spec.out_bias:
            raise ValueError("differential maps, kept first keys, normalised projections, head gates, capped scores and "
                             "the partial rotation do not combine with chunks, distance bias, borrowed keys or an output bias")
        if spec.sink and spec.differential is not None:
            raise ValueError("a sink belongs to one softmax a head, not to the two maps of a differential head")
        if spec.softcap is not None and not spec.softcap > 0:
            raise ValueError(f"a cap on the scores is positive, found {spec.softcap}")
        if spec.qk_norm not in (None, "whole"):
            raise ValueError(f"qk_norm {spec.qk_norm!r}: known is \"whole\"")
        H, G, d, dv, hidden = self.n_q, self.n_kv, self.d, self.dv, spec.hidden_size
        self.maps = 2 if spec.differential is not None else 1
        self.group = H // G
        q, k, v = tensors["q_proj.weight"], tensors["k_proj.weight"], tensors["v_proj.weight"]

        def by_kv_head(rows):           # [H, maps, d, ...] -> (kv head, map, head within the group)
            tail = rows.shape[1:]
            return rows.reshape(G, self.group, self.maps, d, *tail).transpose(1, 2).reshape(H * self.maps * d, *tail)

        joined = [by_kv_head(q) if self.maps > 1 else q, k, v]
        self.gate_offset = sum(part.shape[0] for part in joined)
        if spec.head_gate:
            joined.append(tensors["gate_proj.weight"])
        # (Rows of the joined product in eights: the matrix-core attention kernels read a row sixteen bytes at a time.)
        fill = (-sum(part.shape[0] for part in joined)) % 8 if runtime.dtype == torch.bfloat16 else 0
        if fill:
            joined.append(q.new_zeros((fill, hidden)))
        self.w_qkv = torch.cat(joined, dim=0).contiguous()
        self.b_qkv = None
        if spec.qkv_bias:
            bias = [by_kv_head(tensors["q_proj.bias"]) if self.maps > 1 else tensors["q_proj.bias"],
                    tensors["k_proj.bias"], tensors["v_proj.bias"]]
            bias.append(bias[0].new_zeros((H if spec.head_gate else 0) + fill))
            self.b_qkv = torch.cat(bias, dim=0).contiguous()
        self.lam = None
        if spec.differential is not None:
            pair = lambda a, b: torch.exp((tensors[a].to(torch.float32) * tensors[b].to(torch.float32)).sum())
            self.lam = (pair("lq1", "lk1") - pair("lq2", "lk2") + float(spec.differential)).reshape(1).contiguous()
            self.out_scale = 1.0 - float(spec.differential)
        self.q_norm = by_kv_head(tensors["q_norm"]).to(torch.float32).contiguous() if spec.qk_norm else None
        self.k_norm = tensors["k_norm"].to(torch.float32).contiguous() if spec.qk_norm else None
        self.head_gate, self.eps = spec.head_gate, float(spec.eps)
        # (A sink and a cap on the scores are handed to the attention kernels only where a layer has them.)
        self.more = {}
        if spec.sink:
            self.more["sinks"] = tensors["sink"].to(torch.float32).contiguous()
        if spec.softcap is not None:
            self.more["softcap"] = float(spec.softcap)
        self.w_o, self.b_o = tensors["o_proj.weight"], None
        self.scale = float(spec.scale) if spec.scale is not None else 1.0 / math.sqrt(d)
        self.window = spec.window
        self.keep_first = int(spec.keep_first) if spec.window is not None else 0
        position = spec.position
        if position is None or position.kind == "none":      # nothing turns: the same kernel with no coordinates to rotate
            position = PositionSpec("rope_partial", head_dim=d, theta=1.0, options={"dims": 0})
        if position.kind != "rope_partial":
            raise ValueError(f"these options store keys through the partial rotation's kernel, not {position.kind!r}")
        self.position = POSITIONS.get(position.kind)(position, runtime)
        self.plain = False

    @staticmethod
    def tensor_specs(spec: MixerSpec) -> dict[str, TensorSpec]:
        q_out, kv_out, hidden = spec.n_heads * spec.head_dim, spec.n_kv_heads * spec.head_dim, spec.hidden_size
        dv = spec.value_dim or spec.head_dim
        if spec.differential is not None:
            q_out, kv_out = 2 * q_out, 2 * kv_out
        out = {"q_proj.weight": TensorSpec((q_out, hidden)), "o_proj.weight": TensorSpec((hidden, spec.n_heads * dv))}
        if spec.own_kv:
            out.update({"k_proj.weight": TensorSpec((kv_out, hidden)),
                        "v_proj.weight": TensorSpec((spec.n_kv_heads * dv, hidden))})
        if spec.qkv_bias:
            out["q_proj.bias"] = TensorSpec((q_out,), role="vector")
            if spec.own_kv:
                out.update({"k_proj.bias": TensorSpec((kv_out,), role="vector"),
                            "v_proj.bias": TensorSpec((spec.n_kv_heads * dv,), role="vector")})
        if spec.sink:
            out["sink"] = TensorSpec((spec.n_heads,), role="vector", std=1.0)
        if spec.out_bias:
            out["o_proj.bias"] = TensorSpec((hidden,), role="vector")
        if spec.differential is not None:
            for name in ("lq1", "lk1", "lq2", "lk2"):
                out[name] = TensorSpec((spec.head_dim,), role="vector", std=0.1)
        if spec.qk_norm is not None:
            out["q_norm"] = TensorSpec((q_out,), init="ones", role="vector")
            out["k_norm"] = TensorSpec((kv_out,), init="ones", role="vector")
        if spec.head_gate:
            out["gate_proj.weight"] = TensorSpec((spec.n_heads, hidden))
        return out

    @staticmethod
    def cache_need(spec: MixerSpec) -> CacheNeed:
        if not spec.own_kv:
            return CacheNeed()                  # it reads the pages of the layer it is pointed at
        kind = "full" if spec.window is None else "window"
        if spec.differential is not None:       # a key head per map; the maps of a head read the same value head
            return CacheNeed(kind=kind, n_kv_heads=2 * spec.n_kv_heads, head_dim=spec.head_dim, window=spec.window,
                             value_dim=spec.value_dim or 0, n_value_heads=spec.n_kv_heads)
        return CacheNeed(kind=kind, n_kv_heads=spec.n_kv_heads, head_dim=spec.head_dim, window=spec.window,
                         value_dim=spec.value_dim or 0, keep_first=int(spec.keep_first) if spec.window is not None else 0)

    def repeatable(self):
        position = repeatable_of(self.position)
        if position is None or not self.plain or self.extended:
            return None
        return Repeatable(("gqa_attention", self.n_q, self.n_kv, self.d, self.scale, self.window, position.constants),
                          (self.w_qkv, self.b_qkv, self.w_o, self.b_o) + position.tensors)

    def forward_normed(self, residual, delta, norm, ctx, cache):
        """Decode batches of few bfloat16 rows: norm + q/k/v product + bias + rotation + cache write in one
        kernel, attention, then the output product added straight into the residual stream."""
        ops = self.runtime.ops
        if self.extended:
            return self._run_extended(norm.apply(residual, delta), ctx, cache)
        # The norm and the position encoding say themselves whether they have the form the fused kernels compute.
        fold = norm.fold() if delta is None else None
        behind = self.position.epilogue() if fold is not None else None
        fused = (behind is not None and self.d % 32 == 0 and cache.group is not None and self.plain
                 and _can_fuse(ops, residual, self.runtime.dtype))
        if not fused:
            # The output is handed on as a delta: an output product whose K is cut over workgroups may stay in
            # parts, and the norm that takes it next adds them in its own kernel.
            return self._run(norm.apply(residual, delta), ctx, cache, pending=getattr(ops, "takes_pending", False))
        if getattr(ops, "fold_norm", lambda hidden: True)(residual.shape[1]):
            rows, norm_weight = residual, fold.weight
        else:                       # a wide model: the norm's own kernel once, not again in every workgroup
            rows, norm_weight = norm.apply(residual, None), None
        q = ops.fused_norm_qkv_rope(rows, norm_weight, fold.eps, self.w_qkv, self.b_qkv, ctx.positions,
                                    behind.cos_sin, ctx.slots[cache.group] if cache.writes else None,
                                    cache.k_pages, cache.v_pages, self.n_q, self.n_kv, self.d)
        mixed = torch.empty((q.shape[0], self.n_q * self.d), dtype=q.dtype, device=q.device)
        ops.paged_attention(q, mixed, cache.k_pages, cache.v_pages, ctx.positions, ctx.entry_of_token,
                            ctx.block_tables[cache.group], self.n_q, self.n_kv, self.d, self.window,
                            self.scale, max_position=ctx.max_position, batch=ctx)
        ops.linear_add(mixed, self.w_o, self.b_o, residual)
        return None

    def forward(self, x, ctx, cache):
        if self.extended:
            return self._run_extended(x, ctx, cache)
        return self._run(x, ctx, cache, pending=False)

    def _run_extended(self, x, ctx, cache):
        """One product for queries, keys, values and head gates; bias, the projections' norms, the rotation and the
        store in one kernel; attention with every map a head of its own; the maps' difference or the gate; the
        output product."""
        ops = self.runtime.ops
        heads, key_heads = self.n_q * self.maps, self.n_kv * self.maps
        qkv = ops.linear(x, self.w_qkv, self.b_qkv)           # bias joins the float accumulator
        self.position.encode_and_store(qkv, None, heads, key_heads, self.d, ctx, cache, value_dim=self.dv,
                                       value_heads=self.n_kv, q_norm=self.q_norm, k_norm=self.k_norm, eps=self.eps)
        mixed = torch.empty((x.shape[0], heads * self.dv), dtype=x.dtype, device=x.device)
        ops.paged_attention(qkv, mixed, cache.k_pages, cache.v_pages, ctx.positions, ctx.entry_of_token,
                            ctx.block_tables[cache.group], heads, key_heads, self.d, self.window, self.scale,
                            max_position=ctx.max_position, batch=ctx, value_dim=self.dv, keep_first=self.keep_first,
                            value_heads=self.n_kv, **self.more)
        if self.maps > 1:
            out = torch.empty((x.shape[0], self.n_q * self.dv), dtype=x.dtype, device=x.device)
            ops.differential_heads(mixed, self.lam, self.eps, self.out_scale, self.n_q, self.group, self.dv, out)
            mixed = out
        if self.head_gate:
            ops.sigmoid_head_gate(mixed, qkv, self.gate_offset, self.n_q, self.dv)
        return ops.linear(mixed, self.w_o)

    def _run(self, x, ctx, cache, pending: bool):
        ops = self.runtime.ops
        can = getattr(ops, "can_rope_store", None)
        behind = None
        # (The projection with the store in its epilogue does not care what the attention behind it does with
        # chunks, slopes or sinks: it needs heads of one size and keys and values of the layer's own.)
        even = self.own_kv and self.dv == self.d and self.d % 32 == 0 and cache.group is not None
        if can and can(x.shape[0], self.runtime.dtype, self.w_qkv.numel()) and even:
            behind = self.position.epilogue()
        elif even and not self.plain and _can_fuse(ops, x, self.runtime.dtype) and x.shape[1] % 8 == 0:
            behind = self.position.epilogue()       # up to sixteen normalised rows: the fused decode projection
        if behind is not None:
            # A few dozen rows: bias, rotation and the cache write ride in the projection's epilogue.
            qkv = ops.fused_norm_qkv_rope(x, None, 0.0, self.w_qkv, self.b_qkv, ctx.positions, behind.cos_sin,
                                          ctx.slots[cache.group] if cache.writes else None, cache.k_pages,
                                          cache.v_pages, self.n_q, self.n_kv, self.d)
        else:
            qkv = ops.linear(x, self.w_qkv, self.b_qkv)   # bias joins the float accumulator
            if self.plain:
                self.position.encode_and_store(qkv, None, self.n_q, self.n_kv, self.d, ctx, cache)
            elif self.own_kv:
                self.position.encode_and_store(qkv, None, self.n_q, self.n_kv, self.d, ctx, cache, value_dim=self.dv)
            else:                               # queries alone: encoded in place, nothing to store
                self.position.encode_and_store(qkv, None, self.n_q, 0, self.d, ctx, cache, value_dim=self.dv)
        mixed = torch.empty((x.shape[0], self.n_q * self.dv), dtype=x.dtype, device=x.device)
        if self.plain:
            ops.paged_attention(qkv, mixed, cache.k_pages, cache.v_pages, ctx.positions, ctx.entry_of_token,
                                ctx.block_tables[cache.group], self.n_q, self.n_kv, self.d, self.window,
                                self.scale, max_position=ctx.max_position, batch=ctx)
        else:
            ops.paged_attention(qkv, mixed, cache.k_pages, cache.v_pages, ctx.positions, ctx.entry_of_token,
                                ctx.block_tables[cache.group], self.n_q, self.n_kv, self.d, self.window,
                                self.scale, max_position=ctx.max_position, batch=ctx, **self.extras)
        return ops.linear(mixed, self.w_o, self.b_o, pending=True) if pending else ops.linear(mixed, self.w_o, self.b_o)
