"""Plain, slow Zomavik decoder: whole sequences, no cache, one function per mechanism.

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
def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * w


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def cap(z: torch.Tensor, limit: float) -> torch.Tensor:
    """limit * tanh(z / limit): the identity near zero, never beyond +-limit."""
    return limit * torch.tanh(z / limit)


# ------------------------------------------------------------------ rotation
def rotate_leading(x: torch.Tensor, positions: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """x [T, heads, n]: of the first `dims` coordinates, i < dims/2 and i + dims/2 turn together by the angle
    p * base^(-2i/dims); the coordinates from `dims` on stay."""
    half = dims // 2
    if half == 0:
        return x
    rates = torch.tensor([float(base) ** (-2.0 * i / dims) for i in range(half)], dtype=x.dtype)
    angles = positions.to(x.dtype)[:, None, None] * rates[None, None, :]
    cos, sin = torch.cos(angles), torch.sin(angles)
    a, b = x[..., :half], x[..., half:dims]
    return torch.cat([a * cos - b * sin, b * cos + a * sin, x[..., dims:]], dim=-1)


# ------------------------------------------------------------------ the attention side
def capped_sink_attention(h: torch.Tensor, m: dict, w: dict) -> torch.Tensor:
    """Causal attention whose scores are capped and whose softmax has one more term exp(sink) per head in its
    denominator, token by token and head by head."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    positions = torch.arange(T)
    q = (h @ w["q"].T + w["q.b"]).reshape(T, H, d)
    k = (h @ w["k"].T + w["k.b"]).reshape(T, G, d)
    v = (h @ w["v"].T + w["v.b"]).reshape(T, G, dv)
    rot = m.get("rot")
    if rot:
        q = rotate_leading(q, positions, int(rot["dims"]), float(rot["base"]))
        k = rotate_leading(k, positions, int(rot["dims"]), float(rot["base"]))
    out = torch.zeros((T, H, dv), dtype=h.dtype)
    for head in range(H):
        g = head // (H // G)
        for t in range(T):
            s = (k[:t + 1, g] @ q[t, head]) * float(m["scale"])
            if m.get("softcap") is not None:
                s = cap(s, float(m["softcap"]))
            sink = w["sink"][head]
            top = torch.maximum(s.max(), sink)
            e = torch.exp(s - top)
            out[t, head] = (e[:, None] * v[:t + 1, g]).sum(0) / (e.sum() + torch.exp(sink - top))
    return out.reshape(T, H * dv) @ w["o"].T


# ------------------------------------------------------------------ the recurrent side
def causal_taps(x: torch.Tensor, taps: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """x [T, C], taps [C, K]: y_t = bias + sum_j taps[:, K-1-j] x_{t-j}, inputs before the start are zero."""
    T, K = x.shape[0], taps.shape[1]
    y = bias.expand(T, -1).clone()
    for j in range(K):
        if j < T:
            y[j:] = y[j:] + x[:T - j] * taps[:, K - 1 - j]
    return y


def selective_scan(h: torch.Tensor, m: dict, w: dict) -> torch.Tensor:
    T = h.shape[0]
    inner, n, rank = m["inner"], m["state"], m["dt_rank"]
    both = h @ w["in"].T
    x, z = both[:, :inner], both[:, inner:]
    x = silu(causal_taps(x, w["conv"], w["conv.b"]))
    low = x @ w["x"].T
    step = softplus(low[:, :rank] @ w["dt"].T + w["dt.b"])                # [T, inner]
    B, C = low[:, rank:rank + n], low[:, rank + n:rank + 2 * n]
    A = -torch.exp(w["A_log"])                                             # [inner, n]
    S = torch.zeros((inner, n), dtype=h.dtype)
    y = torch.zeros((T, inner), dtype=h.dtype)
    for t in range(T):
        S = torch.exp(step[t][:, None] * A) * S + (step[t] * x[t])[:, None] * B[t][None, :]
        y[t] = S @ C[t] + w["D"] * x[t]
    return (y * silu(z)) @ w["o"].T


def side_by_side(h: torch.Tensor, m: dict, w: dict) -> torch.Tensor:
    left = capped_sink_attention(h, m["left"], sub(w, "left"))
    right = selective_scan(h, m["right"], sub(w, "right"))
    return float(m["left_scale"]) * left + float(m["right_scale"]) * right


# ------------------------------------------------------------------ feed-forwards
def dense_feed_forward(h: torch.Tensor, w: dict) -> torch.Tensor:
    return (torch.relu(h @ w["up"].T) ** 2) @ w["down"].T


def gated_expert(h: torch.Tensor, w: dict, name: str) -> torch.Tensor:
    return w[f"{name}.down"] @ (silu(w[f"{name}.gate"] @ h) * (w[f"{name}.up"] @ h))


def route(h: torch.Tensor, router: dict, w: dict):
    """Softmax over all experts; a group is worth its best expert; the `top` best experts of the `keep` best groups,
    weighted by their scores over the chosen's sum."""
    s = torch.softmax(h @ w["router"].T, dim=-1)
    T, E = s.shape
    allowed = torch.ones_like(s, dtype=torch.bool)
    groups = router.get("groups")
    if groups:
        count, keep = int(groups["count"]), int(groups["keep"])
        worth = s.reshape(T, count, E // count).max(dim=-1).values
        kept = torch.topk(worth, keep, dim=-1).indices
        mask = torch.zeros((T, count), dtype=torch.bool)
        mask.scatter_(1, kept, True)
        allowed = mask[:, :, None].expand(T, count, E // count).reshape(T, E)
    choice = torch.where(allowed, s, torch.full_like(s, -1.0))
    chosen = torch.topk(choice, int(router["top"]), dim=-1).indices
    picked = torch.gather(s, 1, chosen)
    return chosen, picked / (picked.sum(-1, keepdim=True) + 1e-20)


def routed_feed_forward(h: torch.Tensor, mlp: dict, w: dict) -> torch.Tensor:
    chosen, weights = route(h, mlp["router"], w)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, a in zip(chosen[t].tolist(), weights[t]):
            out[t] = out[t] + a * gated_expert(h[t], w, f"e{e}")
        if mlp.get("shared"):
            out[t] = out[t] + torch.sigmoid(w["shared.sg"][0] @ h[t]) * gated_expert(h[t], w, "shared")
    return out


# ------------------------------------------------------------------ the model
def sub(tensors: dict, prefix: str) -> dict:
    lead = prefix + "."
    return {k[len(lead):]: v for k, v in tensors.items() if k.startswith(lead)}


def run_order(cfg: dict) -> list[tuple[int, bool]]:
    """(layer, whether a pass through the repeated run starts in front of it), in the order the layers run."""
    n, loop = len(cfg["layers"]), cfg.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    start, stop, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    order = [(i, False) for i in range(start)]
    for _ in range(times):
        order += [(i, i == start) for i in range(start, stop)]
    return order + [(i, False) for i in range(stop, n)]


def forward(cfg: dict, tensors: dict, ids: list[int], layers_out: list | None = None) -> torch.Tensor:
    """Logits [T, vocab] of the whole sequence `ids`; `layers_out` collects the stream behind every layer run."""
    eps = float(cfg["norm"]["eps"])
    x0 = tensors["embed"][torch.tensor(ids)] * float((cfg.get("embedding") or {}).get("scale", 1.0))
    x = x0
    for index, pass_starts in run_order(cfg):
        if pass_starts:
            x = torch.cat([x, x0], dim=-1) @ tensors["loop.in"].T
        layer, name = cfg["layers"][index], f"l{index}"
        if layer["type"] != "parallel":
            raise ValueError(layer["type"])
        y = side_by_side(rms_norm(x, tensors[f"{name}.norm1"], eps), layer["mixer"], sub(tensors, f"{name}.mix"))
        y = y * tensors[f"{name}.ls1"]
        mlp = layer.get("mlp")
        if mlp is not None:
            g = rms_norm(x, tensors[f"{name}.norm2"], eps)
            w = sub(tensors, f"{name}.mlp")
            f = dense_feed_forward(g, w) if mlp["kind"] == "dense" else routed_feed_forward(g, mlp, w)
            y = y + f * tensors[f"{name}.ls2"]
        x = x + y
        if layers_out is not None:
            layers_out.append(x.clone())
    logits = rms_norm(x, tensors["final.norm"], eps) @ tensors["head"].T * float(cfg.get("logit_scale") or 1.0)
    return cap(logits, float(cfg["logit_softcap"])) if cfg.get("logit_softcap") else logits


def greedy_generate(cfg: dict, tensors: dict, prompt, n_new: int) -> list[int]:
    """The first maximum of the last position's logits, appended and run again from the start, `n_new` times."""
    ids, out = list(prompt), []
    for _ in range(n_new):
        logits = forward(cfg, tensors, ids)[-1]
        out.append(int(torch.argmax(logits)))
        ids.append(out[-1])
    return out
