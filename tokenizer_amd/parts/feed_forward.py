"""Dense gated feed-forward."""
from __future__ import annotations

import torch

from .base import can_fuse_decode as _can_fuse
from .base import FEED_FORWARDS, FeedForward, Repeatable, Runtime
from .spec import FeedForwardSpec, TensorSpec


@FEED_FORWARDS.register("gated_dense")
class GatedDense(FeedForward):
    """down(act(gate(x)) * up(x)) without biases (qwen-infer/src/model.rs:245-249).

    gate and up are joined into one matrix at load time; the activation and the product with
    `up` run in float32 in one kernel.
    """
    graph_safe = True


    def __init__(self, spec: FeedForwardSpec, tensors: dict[str, torch.Tensor], runtime: Runtime):
        if spec.activation not in ("silu", "capped_swish", "gelu_tanh"):
            raise ValueError(f"gated_dense knows the activations silu, gelu_tanh and capped_swish, not {spec.activation!r}")
        self.spec, self.runtime = spec, runtime
        self.gelu = spec.activation == "gelu_tanh"     # 0.5 g (1 + tanh(sqrt(2/pi) (g + 0.044715 g^3))) in place of silu
        # capped_swish: g' = min(g, limit), u' = clamp(u, -limit, limit); g' * sigmoid(alpha g') * (u' + shift).
        # (silu is alpha 1, no limit, shift 0, and keeps the kernels written for it.)
        self.act = None
        if spec.activation == "capped_swish":
            limit = float("inf") if spec.act_limit is None else float(spec.act_limit)
            self.act = (float(spec.act_alpha), limit, float(spec.act_up_shift))
            self.act_numbers = torch.tensor(self.act, dtype=torch.float32, device=runtime.device)   # for kernels that read them
        gate, up, down = tensors["gate_proj.weight"], tensors["up_proj.weight"], tensors["down_proj.weight"]
        # The bfloat16 products read eight elements of K at a time.  An inner width that is no multiple of
        # eight is filled up with zero rows of gate and up and zero columns of down: act(0) * 0 = 0 meets a
        # zero weight, so every sum keeps its terms and gains only zeros.
        fill = (-spec.intermediate_size) % 8 if runtime.dtype == torch.bfloat16 else 0
        if fill:
            rows = gate.new_zeros((fill, gate.shape[1]))
            gate, up = torch.cat([gate, rows], dim=0), torch.cat([up, rows], dim=0)
            down = torch.cat([down, down.new_zeros((down.shape[0], fill))], dim=1).contiguous()
        self.w_gate_up = torch.cat([gate, up], dim=0).contiguous()
        self.w_down = down

    @staticmethod
    def tensor_specs(spec: FeedForwardSpec) -> dict[str, TensorSpec]:
        return {"gate_proj.weight": TensorSpec((spec.intermediate_size, spec.hidden_size)),
                "up_proj.weight": TensorSpec((spec.intermediate_size, spec.hidden_size)),
                "down_proj.weight": TensorSpec((spec.hidden_size, spec.intermediate_size))}

    def repeatable(self):
        if self.gelu:
            return None
        return Repeatable(("gated_dense", self.act), (self.w_gate_up, self.w_down))

    def forward_normed(self, residual, delta, norm, ctx):
        """Decode batches of few bfloat16 rows: norm + gate/up product + activation in one kernel, then the
        down product added straight into the residual stream."""
        ops = self.runtime.ops
        fold = norm.fold() if delta is None else None      # the norm says whether it has the form the kernel computes
        if fold is None or self.act is not None or self.gelu or not _can_fuse(ops, residual, self.runtime.dtype):
            # The output is handed on as a delta: a down product whose K is cut over workgroups may stay in
            # parts, and the norm that takes it next adds them in its own kernel.
            return self._run(norm.apply(residual, delta), pending=getattr(ops, "takes_pending", False))
        if getattr(ops, "fold_norm", lambda hidden: True)(residual.shape[1]):
            act = ops.fused_norm_gated(residual, fold.weight, fold.eps, self.w_gate_up)
        else:                       # a wide model: the norm's own kernel once, not again in every workgroup
            act = ops.fused_norm_gated(norm.apply(residual, None), None, fold.eps, self.w_gate_up)
        ops.linear_add(act, self.w_down, None, residual)
        return None

    def forward(self, x, ctx):
        return self._run(x, pending=False)

    def _run(self, x, pending: bool):
        ops = self.runtime.ops
        if self.gelu:
            act = ops.linear_silu_gate(x, self.w_gate_up, act="gelu_tanh")
        elif self.act is None:
            act = ops.linear_silu_gate(x, self.w_gate_up)
        elif _can_fuse(ops, x, self.runtime.dtype) and x.shape[1] % 8 == 0:
            # Up to sixteen normalised rows: the fused decode product with the capped activation in its epilogue.
            act = ops.fused_norm_gated(x, None, 0.0, self.w_gate_up, act=self.act_numbers)
        else:
            act = ops.linear_silu_gate(x, self.w_gate_up, act=self.act)
        return ops.linear(act, self.w_down, pending=True) if pending else ops.linear(act, self.w_down)


@FEED_FORWARDS.register("plain_dense")
class PlainDense(FeedForward):
    """down(act(up(x))) without a gate branch and without biases; `activation` "relu2" is max(z, 0)^2 (computed in
    float32 from what the first product leaves).  Tensors `up` [inner, hidden], `down` [hidden, inner]."""
    graph_safe = True

    def __init__(self, spec: FeedForwardSpec, tensors: dict[str, torch.Tensor], runtime: Runtime):
        if spec.activation != "relu2":
            raise ValueError(f"plain_dense knows the activation relu2, not {spec.activation!r}")
        self.spec, self.runtime = spec, runtime
        up, down = tensors["up"], tensors["down"]
        # (The bfloat16 products read K in eights: an inner width that is no multiple of eight is filled up with zero
        # rows of up and zero columns of down.)
        fill = (-spec.intermediate_size) % 8 if runtime.dtype == torch.bfloat16 else 0
        if fill:
            up = torch.cat([up, up.new_zeros((fill, up.shape[1]))], dim=0).contiguous()
            down = torch.cat([down, down.new_zeros((down.shape[0], fill))], dim=1).contiguous()
        self.w_up, self.w_down = up, down

    @staticmethod
    def tensor_specs(spec: FeedForwardSpec) -> dict[str, TensorSpec]:
        return {"up": TensorSpec((spec.intermediate_size, spec.hidden_size)),
                "down": TensorSpec((spec.hidden_size, spec.intermediate_size))}

    def forward(self, x, ctx):
        ops = self.runtime.ops
        up = ops.linear(x, self.w_up)
        act = torch.empty_like(up)
        ops.relu2(up, act)
        return ops.linear(act, self.w_down)


@FEED_FORWARDS.register("routed_experts")
class RoutedExperts(FeedForward):
    """A mixture of `n_experts` small gated feed-forwards (tensors `e<j>.gate|up|down`, inner width
    `intermediate_size`, silu, no biases), of which every token uses the `top_k` with the largest router logits
    (`router` [n_experts, hidden]; the logits are float32 sums), weighted by the softmax over the chosen logits alone;
    an optional shared expert (`shared.gate|up|down`, inner width `shared_size`) runs for every token and is added.

    All experts' gate and up matrices are one matrix, and all down matrices one matrix along K, so a step is two
    products whatever the routing: between them a kernel turns gate and up into weight * silu(gate) * up for the
    experts a token chose and into zero for the others (the shared expert counts as chosen with weight 1), and the
    second product then adds the chosen experts' outputs up in its own sum.  That multiplies every token with every
    expert, which is right while the weights bound the step (few rows: every expert is read anyway).  Steps with
    `GROUPED_FROM` or more (token, expert) pairs in bfloat16 sort the pairs by expert on the device into tiles of rows
    that belong to one expert each, multiply every tile with its expert's matrices alone, and add a token's experts
    up at the end (the shared expert runs as a dense one).  Either way the routing stays on the device, so the step's
    launches do not depend on it.

    Two options of the spec change what an expert and the router are, each on its own.  `gated` False: an expert is
    down(act(up(x))) with tensors `e<j>.up|down` alone, and `activation` "relu2" is max(z, 0)^2; all experts' up
    matrices are one matrix, and the kernel between the two products leaves weight * act(up) for chosen experts and
    zero for the others.  `router` "sigmoid": scores s = sigmoid(logit); an expert's choice score is s + `correction`
    (a tensor, one number an expert); with `n_groups` the experts form that many equal groups of neighbours, a group is
    worth the sum of its two largest choice scores, and only experts of the `keep_groups` best groups can be chosen
    (the others count as minus infinity); the `top_k` largest choice scores are chosen and weighted by their s over
    the chosen's sum (+ 1e-20).  `router` "softmax_all": the same with s = softmax over all experts and no correction;
    `group_worth` "max": a group is worth its largest choice score.  `shared_gate`: the shared expert's output times
    sigmoid(W_sg x), one number a token (tensor `shared.sg` [1, hidden]; its row rides behind the router's rows, so
    the gate's logit is a float32 sum of the same product).  Logits, scores and weights are float32.
    """
    graph_safe = True
    GROUPED_FROM = 1024        # (token, expert) pairs from which the sorted form runs

    def __init__(self, spec: FeedForwardSpec, tensors: dict[str, torch.Tensor], runtime: Runtime):
        if (spec.activation, spec.gated) not in (("silu", True), ("relu2", False)):
            raise ValueError(f"routed_experts knows gated silu experts and ungated relu2 experts, not "
                             f"{'gated' if spec.gated else 'ungated'} {spec.activation!r}")
        if not 0 < spec.top_k <= spec.n_experts:
            raise ValueError(f"{spec.top_k} of {spec.n_experts} experts")
        if spec.router not in ("softmax", "sigmoid", "softmax_all"):
            raise ValueError(f"router {spec.router!r}: known are softmax, sigmoid and softmax_all")
        if spec.group_worth not in ("top2", "max"):
            raise ValueError(f"group_worth {spec.group_worth!r}: known are top2 and max")
        self.spec, self.runtime = spec, runtime
        self.n_experts, self.top_k = spec.n_experts, spec.top_k
        self.inner, self.shared = spec.intermediate_size, spec.shared_size
        self.gated, self.sigmoid = spec.gated, spec.router == "sigmoid"
        self.scored = spec.router in ("sigmoid", "softmax_all")      # chosen by scores, weighted by them over their sum
        if not self.gated and self.shared:
            raise ValueError("ungated experts have no shared expert here")
        self.shared_gate = bool(spec.shared_gate) and bool(self.shared)
        if self.shared_gate and not self.scored:
            raise ValueError("the shared expert's gate rides in the scored routers' logits")
        self.w_router = tensors["router"]
        if self.shared_gate:          # the gate's row behind the experts' rows: its logit comes out of the same product
            self.w_router = torch.cat([self.w_router, tensors["shared.sg"].reshape(1, -1)], dim=0).contiguous()
        if self.scored:
            self.correction = tensors["correction"].to(torch.float32).contiguous() if self.sigmoid else None
            self.n_groups, self.keep_groups = int(spec.n_groups), int(spec.keep_groups)
            if self.n_groups and (self.n_experts % self.n_groups or not 0 < self.keep_groups <= self.n_groups
                                  or self.keep_groups * (self.n_experts // self.n_groups) < self.top_k):
                raise ValueError(f"{self.n_groups} groups of {self.n_experts} experts, {self.keep_groups} kept, {self.top_k} a token")
        names = [f"e{j}" for j in range(self.n_experts)] + (["shared"] if self.shared else [])
        gate_up, down = [], []
        for name in names:
            gate_up += [tensors[f"{name}.gate"], tensors[f"{name}.up"]] if self.gated else [tensors[f"{name}.up"]]
            down.append(tensors[f"{name}.down"])
        self.total = self.n_experts * self.inner + self.shared           # columns between the two products
        fill = (-self.total) % 8 if runtime.dtype == torch.bfloat16 else 0     # the second product reads K in eights
        if fill:
            down.append(down[0].new_zeros((spec.hidden_size, fill)))
        self.w_gate_up = torch.cat(gate_up, dim=0).contiguous()
        self.w_down = torch.cat(down, dim=1).contiguous()
        self.columns = self.total + fill
        # For the sorted form: the shared expert's matrices by themselves (views of the joined gate/up rows; its down
        # columns as a matrix of their own).
        self.groupable = (runtime.dtype == torch.bfloat16 and self.inner % 8 == 0 and spec.hidden_size % 8 == 0
                          and self.shared % 8 == 0 and self.n_experts <= 256)
        if self.groupable and self.shared:
            self.w_shared_gate_up = self.w_gate_up[self.n_experts * 2 * self.inner:]
            self.w_shared_down = self.w_down[:, self.n_experts * self.inner:self.n_experts * self.inner + self.shared].contiguous()

    @staticmethod
    def tensor_specs(spec: FeedForwardSpec) -> dict[str, TensorSpec]:
        out = {"router": TensorSpec((spec.n_experts, spec.hidden_size), std=0.5)}
        if spec.router == "sigmoid":
            out["correction"] = TensorSpec((spec.n_experts,), role="vector", std=0.2)
        if spec.shared_gate and spec.shared_size:
            out["shared.sg"] = TensorSpec((1, spec.hidden_size), std=0.5)
        sizes = [(f"e{j}", spec.intermediate_size) for j in range(spec.n_experts)]
        if spec.shared_size:
            sizes.append(("shared", spec.shared_size))
        for name, inner in sizes:
            if spec.gated:
                out[f"{name}.gate"] = TensorSpec((inner, spec.hidden_size))
            out.update({f"{name}.up": TensorSpec((inner, spec.hidden_size)), f"{name}.down": TensorSpec((spec.hidden_size, inner))})
        return out

    def forward(self, x, ctx):
        ops = self.runtime.ops
        chosen = torch.empty((x.shape[0], self.top_k), dtype=torch.int32, device=x.device)
        weights = torch.empty((x.shape[0], self.top_k), dtype=torch.float32, device=x.device)
        shared_weight = None
        if self.sigmoid and not self.shared_gate and self.spec.group_worth == "top2":
            fused = getattr(ops, "route_rows_sigmoid", None)   # few rows: the router's product and the choice in one kernel
            if (fused is None or x.shape[0] > ops.ROUTE_ROWS_FUSED
                    or not fused(x, self.w_router, self.correction, self.n_groups, self.keep_groups, chosen, weights)):
                ops.route_sigmoid(ops.linear(x, self.w_router, out_dtype=torch.float32), self.correction, self.n_groups,
                                  self.keep_groups, chosen, weights)
        elif self.scored:
            if self.shared_gate:
                shared_weight = torch.empty((x.shape[0],), dtype=torch.float32, device=x.device)
            kind = dict(softmax=not self.sigmoid, group_max=self.spec.group_worth == "max", gate=shared_weight)
            fused = getattr(ops, "route_rows_scores", None)    # few rows: the router's product and the choice in one kernel
            if (fused is None or x.shape[0] > ops.ROUTE_ROWS_FUSED
                    or not fused(x, self.w_router, self.correction, self.n_experts, self.n_groups, self.keep_groups, chosen,
                                 weights, **kind)):
                ops.route_scores(ops.linear(x, self.w_router, out_dtype=torch.float32), self.correction, self.n_experts,
                                 self.n_groups, self.keep_groups, chosen, weights, **kind)
        else:
            fused = getattr(ops, "route_rows", None)      # the router's product and the choice in one kernel, where there is one
            if fused is None or not fused(x, self.w_router, chosen, weights):
                ops.route_top(ops.linear(x, self.w_router, out_dtype=torch.float32), chosen, weights)
        if self.groupable and x.shape[0] * self.top_k >= self.GROUPED_FROM and hasattr(ops, "grouped_linear"):
            return self._sorted(x, chosen, weights, shared_weight)
        gate_up = ops.linear(x, self.w_gate_up)
        act = torch.empty((x.shape[0], self.columns), dtype=x.dtype, device=x.device)
        if self.gated and shared_weight is not None:
            ops.expert_gate(gate_up, chosen, weights, self.n_experts, self.inner, self.shared, act, shared_weight=shared_weight)
        elif self.gated:
            ops.expert_gate(gate_up, chosen, weights, self.n_experts, self.inner, self.shared, act)
        else:
            ops.expert_act(gate_up, chosen, weights, self.n_experts, self.inner, act)
        return ops.linear(act, self.w_down)

    def _sorted(self, x, chosen, weights, shared_weight=None):
        """Tiles of rows that belong to one expert each: gate/up, the activation, down, then a token's experts added up."""
        ops = self.runtime.ops
        hidden, inner = x.shape[1], self.inner
        bm = 128 if x.shape[0] * self.top_k >= 2048 * max(1, self.n_experts // 8) else 64
        slot_of, row_of, tile_expert = ops.expert_slots(chosen, self.n_experts, bm)
        wide = (2 if self.gated else 1) * inner          # an expert's rows of the joined first matrix
        gate_up = ops.grouped_linear(x, row_of, tile_expert, bm, self.w_gate_up, wide * hidden, wide, hidden, torch.bfloat16)
        act = torch.empty((gate_up.shape[0], inner), dtype=x.dtype, device=x.device)
        if self.gated:
            ops.silu_gate(gate_up, act)
        else:
            ops.relu2(gate_up, act)
        rows = ops.grouped_linear(act, None, tile_expert, bm, self.w_down, inner, hidden, inner, torch.float32)
        shared = None
        if self.shared:
            shared = ops.linear(ops.linear_silu_gate(x, self.w_shared_gate_up), self.w_shared_down)
        out = torch.empty((x.shape[0], hidden), dtype=x.dtype, device=x.device)
        if shared_weight is not None:
            return ops.expert_combine(rows, slot_of, weights, shared, out, shared_weight=shared_weight)
        return ops.expert_combine(rows, slot_of, weights, shared, out)
