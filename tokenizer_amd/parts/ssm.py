"""Selective scan: a diagonal linear recurrence per channel whose step sizes, inputs and read-outs depend on the token."""
from __future__ import annotations

import torch

from .base import MIXERS, Mixer, Runtime
from .spec import CacheNeed, MixerSpec, TensorSpec


@MIXERS.register("selective_scan")
class SelectiveScan(Mixer):
    """With h the mixer's input, C = `inner_size` channels, N = `state_dim`, R = `dt_rank`, K = `conv_taps`:
    [x | z] = W_in h (C each); x passes a short causal convolution over time, channel by channel (`conv` [C, K] with
    bias `conv.b`, the last column the current token's, zeros before a sequence's start) and silu.  [dt | B | C] = W_x x
    (R, N, N); the step size of channel c is d_c = softplus(W_dt dt + `dt.b`)_c; A = -exp(`A_log`) [C, N].  Per
    channel c and state n, with S zero at a sequence's start:
        S[c, n] <- exp(d_c A[c, n]) S[c, n] + d_c x_c B_n;   y_c = sum_n S[c, n] C_n + D_c x_c,
    then y * silu(z) and W_o.

    The layer's per-request state (float32, `CacheNeed.state_shape`) is one row a slot: [C N (S, per channel N numbers) |
    (K - 1) C (the convolution's last inputs, oldest first)], read as zeros by a step that starts at position 0.  Step
    sizes (softplus of a float32 sum with the bias in it), exponentials, the recurrence and the read-out are float32 in
    every dtype; x, B, C and z are what their products and the convolution leave in the compute dtype.
    Tensors: in, conv, conv.b, x, dt, dt.b, A_log, D, o.
    """
    graph_safe = True

    def __init__(self, spec: MixerSpec, tensors: dict[str, torch.Tensor], runtime: Runtime):
        self.spec, self.runtime = spec, runtime
        self.inner, self.n, self.rank, self.taps = int(spec.inner_size), int(spec.state_dim), int(spec.dt_rank), int(spec.conv_taps)
        if min(self.inner, self.n, self.rank, self.taps) <= 0:
            raise ValueError("a selective scan needs channels, state, a step-size rank and at least one tap")
        eights = runtime.dtype == torch.bfloat16          # the bfloat16 products read K in eights, rows in eights
        self.w_in = tensors["in"]
        self.conv = tensors["conv"].to(torch.float32).contiguous()
        self.conv_bias = tensors["conv.b"].to(torch.float32).contiguous()
        w_x, w_dt = tensors["x"], tensors["dt"]
        # The narrow product's rows are filled up with zero rows to a multiple of eight, and the step sizes' matrix
        # with zero columns: it then reads the first eights of a narrow row, and what lies there beyond the R numbers
        # (the start of B) meets zeros.
        fill = (-w_x.shape[0]) % 8 if eights else 0
        self.w_x = w_x if not fill else torch.cat([w_x, w_x.new_zeros((fill, w_x.shape[1]))], dim=0).contiguous()
        fill = (-self.rank) % 8 if eights else 0
        self.w_dt = w_dt if not fill else torch.cat([w_dt, w_dt.new_zeros((w_dt.shape[0], fill))], dim=1).contiguous()
        self.dt_bias = tensors["dt.b"].to(torch.float32).contiguous()
        self.neg_rate = (-torch.exp(tensors["A_log"].to(torch.float32))).contiguous()      # A [C, N]
        self.skip = tensors["D"].to(torch.float32).contiguous()
        self.w_o = tensors["o"]

    @staticmethod
    def tensor_specs(spec: MixerSpec) -> dict[str, TensorSpec]:
        C, N, R, K, hidden = spec.inner_size, spec.state_dim, spec.dt_rank, spec.conv_taps, spec.hidden_size
        return {"in": TensorSpec((2 * C, hidden)), "conv": TensorSpec((C, K), role="vector", std=0.5),
                "conv.b": TensorSpec((C,), role="vector", std=0.2), "x": TensorSpec((R + 2 * N, C)),
                "dt": TensorSpec((C, R), std=0.1), "dt.b": TensorSpec((C,), role="vector", std=0.5),
                "A_log": TensorSpec((C, N), role="vector", std=0.5), "D": TensorSpec((C,), init="ones", role="vector"),
                "o": TensorSpec((hidden, C))}

    @staticmethod
    def state_size(spec: MixerSpec) -> int:
        return spec.inner_size * spec.state_dim + (int(spec.conv_taps) - 1) * spec.inner_size

    @staticmethod
    def cache_need(spec: MixerSpec) -> CacheNeed:
        return CacheNeed(kind="none", state_shape=(SelectiveScan.state_size(spec),))

    def forward(self, x, ctx, cache):
        ops = self.runtime.ops
        if cache.state is None:
            raise ValueError("the recurrent mixer needs its state in the request's slot")
        C, N, R = self.inner, self.n, self.rank
        n_tokens = x.shape[0]
        rows = ops.linear(x, self.w_in)                                  # [T, 2 C]: x | z
        fresh = torch.empty((n_tokens, C), dtype=x.dtype, device=x.device)
        ops.short_conv_silu(rows, (0,), (C,), self.conv, cache.state, C * N, ctx.cu_q, ctx.first_position,
                            ctx.state_slots, ctx.entry_of_token, fresh, bias=self.conv_bias)
        low = ops.linear(fresh, self.w_x)                                # [T, R + 2 N (+ fill)]: dt | B | C
        pre = ops.linear(low[:, :self.w_dt.shape[1]], self.w_dt, self.dt_bias, out_dtype=torch.float32)   # the bias joins the float sum
        gated = torch.empty((n_tokens, C), dtype=x.dtype, device=x.device)
        ops.selective_scan(fresh, pre, self.neg_rate, low, R, R + N, self.skip, rows, C, cache.state, ctx.cu_q,
                           ctx.first_position, ctx.state_slots, gated, C, N)
        return ops.linear(gated, self.w_o)
