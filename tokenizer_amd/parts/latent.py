"""Attention over a cached latent (multi-head latent attention) in its absorbed form."""
from __future__ import annotations

import torch

from .base import MIXERS, Mixer, Runtime
from .position import scaled_rates
from .spec import CacheNeed, MixerSpec, TensorSpec


@MIXERS.register("latent_attention")
class LatentAttention(Mixer):
    """Queries through a normalised latent, keys and values from one normalised latent a token that all heads share.

    With h the mixer's input, r = `kv_rank`, d = `head_dim`, e = `rot_dim`, dv = `value_dim`:
    c_q = norm(W_dq h) (weight `dq.norm`), q = W_uq c_q laid out head by head as [d plain | e rotated];
    W_dkv h has r + e rows: c = norm(first r) (weight `dkv.norm`), the last e (not normalised) are one key part that is
    rotated and shared by all heads; head i: k_i = W_uk,i c, v_i = W_uv,i c,
    score = (q_i,plain . k_i + rot(q_i,rot) . rot(k_rot)) * scale, causal softmax, o_i = sum of weights * v_i; the gate
    (`head_gate`: sigmoid of one number a head; `element_gate`: of one number a coordinate of the joined heads, both
    projected from h by `g`), then W_o.  The rotation pairs coordinate j with j + e/2 and turns the pair at position p by
    p * base^(-2j/e) (option `rot_base`; angles, sine and cosine in float32).

    Only c and the rotated key part are cached, and nothing is ever expanded from them: since
    q_i,plain . (W_uk,i c) = (W_uk,i^T q_i,plain) . c, a head's query is taken into the latent's space (a product per
    head with W_uk,i^T), the cache is read as ONE key head of r + e coordinates [c | rot(k_rot)] that all query heads
    share, the same rows serve as values, and a head's r leading output coordinates go through W_uv,i afterwards:
    sum_j w_j (W_uv,i c_j) = W_uv,i (sum_j w_j c_j).  So the paged attention kernels of the grouped-query mixer run it
    as they are (n_kv = 1, head size r + e), for prompts, portions and single tokens alike, and a token costs the
    cache r + e numbers a layer whatever the number of heads.  Scores and weights are float32 there.

    Tensors: dq, dq.norm, uq, dkv, dkv.norm, uk, uv, g, o.
    """
    graph_safe = True

    def __init__(self, spec: MixerSpec, tensors: dict[str, torch.Tensor], runtime: Runtime):
        if spec.head_gate == spec.element_gate:
            raise ValueError("latent attention has a gate a head or a gate a coordinate")
        self.spec, self.runtime = spec, runtime
        H, d, dv, r, e = spec.n_heads, spec.head_dim, spec.value_dim or spec.head_dim, spec.kv_rank, spec.rot_dim
        self.heads, self.d, self.dv, self.rank, self.rot, self.q_rank = H, d, dv, r, e, spec.q_rank
        self.key_dim = r + e                         # what a token's row of the cache holds
        self.eps, self.scale = float(spec.eps), float(spec.scale)
        if e % 2:
            raise ValueError(f"a rotation over {e} coordinates")
        # One product for the two down-projections and the gate; every part starts at a multiple of eight columns
        # (sixteen bytes in bfloat16), filled up with rows of zeros.
        parts, self.offsets, at = [], {}, 0
        for name in ("dq", "dkv", "g"):
            weight = tensors[name]
            self.offsets[name] = at
            fill = (-weight.shape[0]) % 8
            parts.append(weight if not fill else torch.cat([weight, weight.new_zeros((fill, weight.shape[1]))], dim=0))
            at += weight.shape[0] + fill
        self.w_in = torch.cat(parts, dim=0).contiguous()
        self.q_norm = tensors["dq.norm"].to(torch.float32).contiguous()
        self.kv_norm = tensors["dkv.norm"].to(torch.float32).contiguous()
        self.w_uq = tensors["uq"]
        # W_uk,i^T as the matrix of a product out = x W^T: [H, r, d]; W_uv,i as it is: [H, dv, r].
        self.w_absorb = tensors["uk"].reshape(H, d, r).transpose(1, 2).contiguous()
        self.w_uv = tensors["uv"].reshape(H, dv, r).contiguous()
        self.w_o = tensors["o"]
        self.rates = scaled_rates(float(spec.options.get("rot_base", 1.0)), e, None).to(runtime.device).contiguous() if e else None

    @staticmethod
    def tensor_specs(spec: MixerSpec) -> dict[str, TensorSpec]:
        H, d, dv, hidden = spec.n_heads, spec.head_dim, spec.value_dim or spec.head_dim, spec.hidden_size
        gate_rows = H if spec.head_gate else H * dv
        return {"dq": TensorSpec((spec.q_rank, hidden)), "dq.norm": TensorSpec((spec.q_rank,), init="ones", role="vector"),
                "uq": TensorSpec((H * (d + spec.rot_dim), spec.q_rank)),
                "dkv": TensorSpec((spec.kv_rank + spec.rot_dim, hidden)),
                "dkv.norm": TensorSpec((spec.kv_rank,), init="ones", role="vector"),
                "uk": TensorSpec((H * d, spec.kv_rank)), "uv": TensorSpec((H * dv, spec.kv_rank)),
                "g": TensorSpec((gate_rows, hidden)), "o": TensorSpec((hidden, H * dv))}

    @staticmethod
    def cache_need(spec: MixerSpec) -> CacheNeed:
        # One key head of kv_rank + rot_dim coordinates; the same rows, transposed within a page, as the value head.
        return CacheNeed(kind="full", n_kv_heads=1, head_dim=spec.kv_rank + spec.rot_dim)

    def forward(self, x, ctx, cache):
        ops, H, D = self.runtime.ops, self.heads, self.key_dim
        n_tokens = x.shape[0]
        rows = ops.linear(x, self.w_in)
        latent_q = torch.empty((n_tokens, self.q_rank), dtype=x.dtype, device=x.device)
        # Both latents' norms, the rotation of the shared key part and the store of [c | rot(k_rot)] as key and as value.
        ops.latent_store(rows, self.offsets["dq"], self.q_rank, self.q_norm, self.offsets["dkv"], self.rank, self.kv_norm,
                         self.rot, self.rates, self.eps, ctx.positions, ctx.slots[cache.group] if cache.writes else None,
                         cache.k_pages, cache.v_pages, latent_q)
        q = ops.linear(latent_q, self.w_uq)                                   # [T, H (d + e)]
        absorbed = torch.empty((n_tokens, H * D), dtype=x.dtype, device=x.device)
        ops.head_linear(q, 0, self.d + self.rot, self.w_absorb, absorbed, 0, D)
        if self.rot:
            ops.rotate_tails(q, H, self.d + self.rot, self.d, self.rot, self.rates, ctx.positions, absorbed, D, self.rank)
        mixed = torch.empty((n_tokens, H * D), dtype=x.dtype, device=x.device)
        ops.paged_attention(absorbed, mixed, cache.k_pages, cache.v_pages, ctx.positions, ctx.entry_of_token,
                            ctx.block_tables[cache.group], H, 1, D, None, self.scale, max_position=ctx.max_position,
                            batch=ctx)
        out = torch.empty((n_tokens, H * self.dv), dtype=x.dtype, device=x.device)
        ops.head_linear(mixed, 0, D, self.w_uv, out, 0, self.dv)
        if self.spec.head_gate:
            ops.sigmoid_head_gate(out, rows, self.offsets["g"], H, self.dv)
        else:
            ops.sigmoid_head_gate(out, rows, self.offsets["g"], H * self.dv, 1)
        return ops.linear(out, self.w_o)
