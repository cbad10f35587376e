"""Gated delta rule with a decay per key channel, short convolutions, and its state in the request's slot."""
from __future__ import annotations

import torch

from .base import MIXERS, Mixer, Runtime
from .spec import CacheNeed, MixerSpec, TensorSpec


@MIXERS.register("gated_delta")
class GatedDelta(Mixer):
    """With h the mixer's input, H = `n_heads`, G = `n_kv_heads` query/key heads of d, value heads of dv:
    q = W_q h, k = W_k h [G d], v = W_v h [H dv]; each passes a short causal convolution over time, channel by channel
    (`<name>.conv` [channels, taps], the last column the current token's, zeros before a sequence's start) and silu;
    q and k become unit vectors per head, x / sqrt(sum(x^2) + `unit_eps`), q times d^(-1/2); head i reads q/k head
    i // (H / G).  beta = sigmoid(W_b h) [H]; decay g = exp(-exp(A_log_i) * softplus(W_a2 (W_a1 h) + dt_bias)) [H, d],
    one number per head and key channel.  Per head, with the state S [d, dv] (zero at a sequence's start):
    S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q  (the read-out sees the token's own write).
    o is brought to unit RMS per head (`eps`), times `norm` [dv], times sigmoid(W_g2 (W_g1 h)) [H dv], then W_o.

    The layer's per-request state (float32, `CacheNeed.state_shape`) is one row a slot: [H d dv (S, per head [d, dv]) |
    (taps - 1) (2 G d + H dv) (the convolutions' last inputs, oldest first)], read as zeros by a step that starts at
    position 0.  Unit vectors, beta, softplus, the decays, the recurrence and the head norm are float32 in every
    dtype; the decay's pre-activation comes out of its product in float32.
    Tensors: q, q.conv, k, k.conv, v, v.conv, b, a1, a2, A_log, dt_bias, g1, g2, norm, o.
    """
    graph_safe = True

    def __init__(self, spec: MixerSpec, tensors: dict[str, torch.Tensor], runtime: Runtime):
        self.spec, self.runtime = spec, runtime
        H, G, d, dv = spec.n_heads, spec.n_kv_heads, spec.head_dim, spec.value_dim or spec.head_dim
        self.heads, self.groups, self.d, self.dv, self.taps = H, G, d, dv, int(spec.conv_taps)
        self.eps, self.unit_eps = float(spec.eps), float(spec.options.get("unit_eps", 1e-6))
        self.channels = 2 * G * d + H * dv
        # One product for q, k, v, beta and the two narrow projections; every part starts at a multiple of eight
        # columns, filled up with rows of zeros.
        parts, self.offsets, at = [], {}, 0
        for name in ("q", "k", "v", "b", "a1", "g1"):
            weight = tensors[name]
            self.offsets[name] = at
            fill = (-weight.shape[0]) % 8
            parts.append(weight if not fill else torch.cat([weight, weight.new_zeros((fill, weight.shape[1]))], dim=0))
            at += weight.shape[0] + fill
        if tensors["a2"].shape[1] != tensors["a1"].shape[0] or tensors["g2"].shape[1] != tensors["g1"].shape[0]:
            raise ValueError("the narrow projections' two matrices do not fit each other")
        self.w_in = torch.cat(parts, dim=0).contiguous()
        self.low_a, self.low_g = tensors["a1"].shape[0], tensors["g1"].shape[0]
        self.w_a2 = self._filled_k(tensors["a2"])
        self.w_g2 = self._filled_k(tensors["g2"])
        self.conv = torch.cat([tensors["q.conv"], tensors["k.conv"], tensors["v.conv"]], dim=0).to(torch.float32).contiguous()
        self.dt_bias = tensors["dt_bias"].to(torch.float32).contiguous()
        self.neg_rate = (-torch.exp(tensors["A_log"].to(torch.float32))).contiguous()          # -exp(A_log), per head
        self.norm = tensors["norm"].to(torch.float32).repeat(H).contiguous()                  # one weight for every head
        self.w_o = tensors["o"]

    @staticmethod
    def _filled_k(weight: torch.Tensor) -> torch.Tensor:
        """The matrix with its K filled up to a multiple of eight with zero columns (its input's columns there are
        the zeros that the joined product's fill rows leave)."""
        fill = (-weight.shape[1]) % 8
        return weight if not fill else torch.cat([weight, weight.new_zeros((weight.shape[0], fill))], dim=1).contiguous()

    @staticmethod
    def tensor_specs(spec: MixerSpec) -> dict[str, TensorSpec]:
        H, G, d, dv, hidden = spec.n_heads, spec.n_kv_heads, spec.head_dim, spec.value_dim or spec.head_dim, spec.hidden_size
        low = int(spec.options.get("low_rank") or max(8, d // 2))     # (no configuration key: the file's tensors say)
        taps = int(spec.conv_taps)
        return {"q": TensorSpec((G * d, hidden)), "q.conv": TensorSpec((G * d, taps), role="vector", std=0.5),
                "k": TensorSpec((G * d, hidden)), "k.conv": TensorSpec((G * d, taps), role="vector", std=0.5),
                "v": TensorSpec((H * dv, hidden)), "v.conv": TensorSpec((H * dv, taps), role="vector", std=0.5),
                "b": TensorSpec((H, hidden)), "A_log": TensorSpec((H,), role="vector", std=0.5),
                "norm": TensorSpec((dv,), init="ones", role="vector"),
                "a1": TensorSpec((-1, hidden), free_size=low), "a2": TensorSpec((H * d, -1), free_size=low),
                "dt_bias": TensorSpec((H * d,), role="vector", std=0.5),
                "g1": TensorSpec((-1, hidden), free_size=low), "g2": TensorSpec((H * dv, -1), free_size=low), "o": TensorSpec((hidden, H * dv))}

    @staticmethod
    def state_size(spec: MixerSpec) -> int:
        H, G, d, dv = spec.n_heads, spec.n_kv_heads, spec.head_dim, spec.value_dim or spec.head_dim
        return H * d * dv + (int(spec.conv_taps) - 1) * (2 * G * d + H * dv)

    @staticmethod
    def cache_need(spec: MixerSpec) -> CacheNeed:
        return CacheNeed(kind="none", state_shape=(GatedDelta.state_size(spec),))

    def forward(self, x, ctx, cache):
        ops = self.runtime.ops
        if cache.state is None:
            raise ValueError("the recurrent mixer needs its state in the request's slot")
        H, d, dv = self.heads, self.d, self.dv
        n_tokens = x.shape[0]
        rows = ops.linear(x, self.w_in)
        memory = H * d * dv
        fresh = torch.empty((n_tokens, self.channels), dtype=x.dtype, device=x.device)
        # (q, k and v channels lie at their parts' offsets in the joined product's rows and side by side behind it.)
        ops.short_conv_silu(rows, (self.offsets["q"], self.offsets["k"], self.offsets["v"]),
                            (self.groups * d, self.groups * d, H * dv), self.conv, cache.state, memory, ctx.cu_q,
                            ctx.first_position, ctx.state_slots, ctx.entry_of_token, fresh)
        low_a = rows[:, self.offsets["a1"]:self.offsets["a1"] + self.w_a2.shape[1]]
        low_g = rows[:, self.offsets["g1"]:self.offsets["g1"] + self.w_g2.shape[1]]
        decay = ops.linear(low_a, self.w_a2, self.dt_bias, out_dtype=torch.float32)       # the bias joins the float sum
        gate = ops.linear(low_g, self.w_g2)
        read = torch.empty((n_tokens, H * dv), dtype=torch.float32, device=x.device)
        ops.delta_scan(fresh, decay, self.neg_rate, rows, self.offsets["b"], cache.state, ctx.cu_q, ctx.first_position,
                       ctx.state_slots, read, H, self.groups, d, dv, self.unit_eps)
        mixed = torch.empty((n_tokens, H * dv), dtype=x.dtype, device=x.device)
        ops.head_norm_gate(read, self.norm, gate, 0, self.eps, H, dv, mixed)
        return ops.linear(mixed, self.w_o)
