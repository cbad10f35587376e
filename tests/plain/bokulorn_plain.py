"""Plain, slow Bokulorn decoder: whole sequences, no cache, one function per mechanism.

Written from the design's equations in this file's own notation; it shares no code with `tokenizer_amd`.
Everything runs on the CPU in the dtype given (float64 by default).  A model is a config dict (the keys of
its config.json) and a dict of tensors by name.
"""
from __future__ import annotations

import json
import math
import os

import torch


def load_folder(folder: str, dtype=torch.float64):
    from safetensors.torch import load_file
    with open(os.path.join(folder, "config.json")) as fh:
        cfg = json.load(fh)
    tensors = {k: (v if v.dtype in (torch.int32, torch.int64) else v.to(dtype))
               for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    return cfg, tensors


# ------------------------------------------------------------------ small pieces
def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x over the root of (its mean square + eps), along the last axis."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def offset_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """A norm whose stored weight lies around zero: the scale is 1 + w."""
    return unit_rms(x, eps) * (1.0 + w)


def plain_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return unit_rms(x, eps) * w


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


# ------------------------------------------------------------------ rotation
def rotate(x: torch.Tensor, positions: torch.Tensor, base: float) -> torch.Tensor:
    """x [T, ..., n]: coordinate i < n/2 and coordinate i + n/2 turn together by the angle p * base^(-2i/n)."""
    n = x.shape[-1]
    half = n // 2
    rates = torch.tensor([float(base) ** (-2.0 * i / n) for i in range(half)], dtype=x.dtype)
    angles = positions.to(x.dtype)[:, None] * rates[None, :]
    while angles.dim() < x.dim():
        angles = angles.unsqueeze(1)
    cos, sin = torch.cos(angles), torch.sin(angles)
    a, b = x[..., :half], x[..., half:]
    return torch.cat([a * cos - b * sin, b * cos + a * sin], dim=-1)


# ------------------------------------------------------------------ attention over latents
def causal_softmax_mix(scores: torch.Tensor, values: torch.Tensor) -> torch.Tensor:
    """scores [H, T, T], values [T, H, dv]: softmax over the keys at or before each query; [T, H, dv]."""
    T = scores.shape[-1]
    hidden = torch.triu(torch.ones(T, T, dtype=torch.bool), diagonal=1)
    weights = torch.softmax(scores.masked_fill(hidden, float("-inf")), dim=-1)
    return torch.einsum("hqk,khd->qhd", weights, values)


def latent_attention(h: torch.Tensor, m: dict, w: dict, eps: float, rotated: bool) -> torch.Tensor:
    """Queries through a normalised latent, keys and values from a normalised latent c shared by the heads.  With
    `rotated` every query head ends in `rot_dim` coordinates that are rotated and meet one rotated key part (the last
    rows of the key/value down-projection, not normalised) that all heads share, and the gate is one number a head;
    without, the gate has a number for every output coordinate."""
    T = h.shape[0]
    H, d, dv, rank = m["heads"], m["dim"], m["vdim"], m["kv_rank"]
    dr = int(m.get("rot_dim") or 0) if rotated else 0
    positions = torch.arange(T)
    cq = plain_norm(h @ w["dq"].T, w["dq.norm"], eps)
    q = (cq @ w["uq"].T).reshape(T, H, d + dr)
    down = h @ w["dkv"].T
    c = plain_norm(down[:, :rank], w["dkv.norm"], eps)
    k = (c @ w["uk"].T).reshape(T, H, d)
    v = (c @ w["uv"].T).reshape(T, H, dv)
    scores = torch.einsum("qhd,khd->hqk", q[..., :d], k)
    if dr:
        base = float(m["rot"]["base"])
        assert int(m["rot"]["dims"]) == dr
        q_rot = rotate(q[..., d:], positions, base)
        k_rot = rotate(down[:, rank:rank + dr], positions, base)
        scores = scores + torch.einsum("qhd,kd->hqk", q_rot, k_rot)
    o = causal_softmax_mix(scores * float(m["scale"]), v)
    gate = torch.sigmoid(h @ w["g"].T)
    o = o * gate[:, :, None] if rotated else o * gate.reshape(T, H, dv)
    return o.reshape(T, H * dv) @ w["o"].T


# ------------------------------------------------------------------ delta rule with a decay per key channel
def short_convolution(x: torch.Tensor, taps: torch.Tensor) -> torch.Tensor:
    """x [T, C], taps [C, n]: y_t = sum_j taps[:, n - 1 - j] x_(t-j), zeros before the start."""
    T, n = x.shape[0], taps.shape[1]
    padded = torch.cat([torch.zeros(n - 1, x.shape[1], dtype=x.dtype), x], dim=0)
    y = torch.zeros_like(x)
    for j in range(n):
        y = y + padded[j:j + T] * taps[:, j]
    return y


def channel_delta(h: torch.Tensor, m: dict, w: dict, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(short_convolution(h @ w["q"].T, w["q.conv"])).reshape(T, G, d)
    k = silu(short_convolution(h @ w["k"].T, w["k.conv"])).reshape(T, G, d)
    v = silu(short_convolution(h @ w["v"].T, w["v.conv"])).reshape(T, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    share = H // G
    q, k = q.repeat_interleave(share, dim=1), k.repeat_interleave(share, dim=1)     # head h reads q/k head h // share
    beta = torch.sigmoid(h @ w["b"].T)                                               # [T, H]
    step = softplus((h @ w["a1"].T) @ w["a2"].T + w["dt_bias"]).reshape(T, H, d)
    decay = torch.exp(-torch.exp(w["A_log"])[None, :, None] * step)                   # [T, H, d]
    S = torch.zeros(H, d, dv, dtype=h.dtype)
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for t in range(T):
        S = decay[t][:, :, None] * S
        u = beta[t][:, None] * (v[t] - torch.einsum("hdv,hd->hv", S, k[t]))
        S = S + k[t][:, :, None] * u[:, None, :]
        out[t] = torch.einsum("hdv,hd->hv", S, q[t])
    out = unit_rms(out, eps) * w["norm"]
    gate = torch.sigmoid((h @ w["g1"].T) @ w["g2"].T).reshape(T, H, dv)
    return (out * gate).reshape(T, H * dv) @ w["o"].T


# ------------------------------------------------------------------ routed feed-forward
def route(h: torch.Tensor, r: dict, w: dict):
    """Which experts each row uses and with what weights: (chosen [T, top], weights [T, top])."""
    E, top = int(r["experts"]), int(r["top"])
    s = torch.sigmoid(h @ w["router"].T)
    choice = s + w["correction"]
    groups = r.get("groups")
    if groups:
        count, keep = int(groups["count"]), int(groups["keep"])
        per = E // count
        grouped = choice.reshape(-1, count, per)
        worth = torch.topk(grouped, min(2, per), dim=-1).values.sum(-1)
        best = torch.topk(worth, keep, dim=-1).indices
        allowed = torch.zeros_like(worth, dtype=torch.bool).scatter_(1, best, True)
        choice = grouped.masked_fill(~allowed[:, :, None], float("-inf")).reshape(-1, E)
    chosen = torch.topk(choice, top, dim=-1).indices
    picked = torch.gather(s, 1, chosen)
    return chosen, picked / (picked.sum(-1, keepdim=True) + 1e-20)


def routed_feed_forward(h: torch.Tensor, mlp: dict, w: dict) -> torch.Tensor:
    chosen, weights = route(h, mlp["router"], w)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, a in zip(chosen[t].tolist(), weights[t]):
            inner = torch.relu(w[f"e{e}.up"] @ h[t]) ** 2
            out[t] = out[t] + a * (w[f"e{e}.down"] @ inner)
    return out


# ------------------------------------------------------------------ the model
def sub(tensors: dict, prefix: str) -> dict:
    lead = prefix + "."
    return {k[len(lead):]: v for k, v in tensors.items() if k.startswith(lead)}


def weight_owner(cfg: dict, index: int) -> int:
    seen = set()
    while cfg["layers"][index].get("weights_of") is not None and index not in seen:
        seen.add(index)
        index = int(cfg["layers"][index]["weights_of"])
    return index


def forward(cfg: dict, tensors: dict, ids: list[int], layers_out: list | None = None) -> torch.Tensor:
    """Logits [T, vocab] of the whole sequence `ids`; `layers_out` collects the stream behind every layer."""
    eps = float(cfg["norm"]["eps"])
    x = tensors["embed"][torch.tensor(ids)] * float(cfg["embedding"]["scale"])
    for index, layer in enumerate(cfg["layers"]):
        own = f"l{weight_owner(cfg, index)}"
        h = offset_norm(x, tensors[f"{own}.norm1"], eps)
        m, w = layer["mixer"], sub(tensors, f"{own}.mix")
        if layer["type"] == "latent_attention":
            y = latent_attention(h, m, w, eps, rotated=True)
        elif layer["type"] == "latent_attention_2":
            y = latent_attention(h, m, w, eps, rotated=False)
        elif layer["type"] == "channel_delta":
            y = channel_delta(h, m, w, eps)
        else:
            raise ValueError(layer["type"])
        if layer.get("mlp") is not None:
            y = y + routed_feed_forward(h, layer["mlp"], sub(tensors, f"{own}.mlp"))
        x = x + y
        if layers_out is not None:
            layers_out.append(x.clone())
    return offset_norm(x, tensors["final.norm"], eps) @ tensors["head"].T


def greedy_generate(cfg: dict, tensors: dict, prompt, n_new: int) -> list[int]:
    """The first maximum of the last position's logits, appended and run again from the start, `n_new` times."""
    ids, out = list(prompt), []
    for _ in range(n_new):
        logits = forward(cfg, tensors, ids)[-1]
        out.append(int(torch.argmax(logits)))
        ids.append(out[-1])
    return out
