"""Zomavik as a `ModelSpec`: a decoder whose layers read two norms of the same stream, one for a mixer and one for a
feed-forward, x + (ls1 * mixer(norm1(x)) + ls2 * feed_forward(norm2(x))) with a learned scale per coordinate on each;
the mixer is an attention (biased projections, a rotation of the heads' leading coordinates, capped scores, a sink in
the softmax) and a selective scan side by side, each with a weight; the feed-forward is dense (squared ReLU, no gate)
or a mixture of gated experts chosen by their softmax scores within the best groups, with a shared expert behind a
gate of its own; a run of layers is gone through several times with the same weights (each pass with a cache and state
of its own), and every pass starts by taking the token's embedding in again through a matrix; the embedding is scaled,
the logits are scaled and capped.

Tensor names: `embed`, `head`, `final.norm`, `loop.in`; layer i's start with `l<i>.`: `norm1`, `norm2`, `ls1`, `ls2`,
`mix.left.*` (q, k, v with `.b`, sink, o), `mix.right.*` (in, conv, conv.b, x, dt, dt.b, A_log, D, o), `mlp.*` (up|down,
or e<j>.gate|up|down, router, shared.gate|up|down|sg).
"""
from __future__ import annotations

from ..config.registry import register_architecture
from ..config.zomavik import ZomavikConfig
from ..parts.spec import FeedForwardSpec, LayerSpec, MixerSpec, ModelSpec, NormSpec, PositionSpec, ScheduleEntry

_ATTENTION_NAMES = (("q_proj.weight", "q"), ("k_proj.weight", "k"), ("v_proj.weight", "v"), ("o_proj.weight", "o"),
                    ("q_proj.bias", "q.b"), ("k_proj.bias", "k.b"), ("v_proj.bias", "v.b"), ("sink", "sink"))


def _attention(raw: dict, width: int, eps: float, max_positions: int) -> MixerSpec:
    rot = raw.get("rot") or {}
    position = PositionSpec("rope_partial", head_dim=raw["dim"], theta=float(rot.get("base", 1.0)),
                            max_positions=max_positions, options={"dims": int(rot.get("dims") or 0)})
    return MixerSpec("gqa_attention", hidden_size=width, n_heads=raw["heads"], n_kv_heads=raw["kv_heads"],
                     head_dim=raw["dim"], value_dim=raw["vdim"], scale=float(raw["scale"]), qkv_bias=True, sink=True,
                     softcap=None if raw.get("softcap") is None else float(raw["softcap"]), eps=eps, position=position,
                     tensor_names=_ATTENTION_NAMES)


def _scan(raw: dict, width: int) -> MixerSpec:
    return MixerSpec("selective_scan", hidden_size=width, inner_size=int(raw["inner"]), state_dim=int(raw["state"]),
                     dt_rank=int(raw["dt_rank"]), conv_taps=int(raw["conv"]))


def _feed_forward(mlp: dict | None, width: int) -> FeedForwardSpec | None:
    if mlp is None:
        return None
    if mlp["kind"] == "dense":
        return FeedForwardSpec("plain_dense", hidden_size=width, intermediate_size=mlp["ff"], activation="relu2", gated=False)
    router, groups = mlp["router"], mlp["router"].get("groups") or {}
    shared = int((mlp.get("shared") or {}).get("ff") or 0)
    return FeedForwardSpec("routed_experts", hidden_size=width, intermediate_size=mlp["expert"]["ff"], activation="silu",
                           n_experts=router["experts"], top_k=router["top"], shared_size=shared, shared_gate=bool(shared),
                           router="softmax_all", n_groups=int(groups.get("count") or 0),
                           keep_groups=int(groups.get("keep") or 0), group_worth="max")


def zomavik_spec(cfg: ZomavikConfig) -> ModelSpec:
    width, eps = cfg.width, cfg.eps
    norm = NormSpec("rmsnorm", width, eps, options={"tensor_name": ""})     # the weight is the tensor the prefix names
    layers = []
    for index, layer in enumerate(cfg.layers):
        prefix, raw = f"l{index}", layer["mixer"]
        mixer = MixerSpec("side_by_side", hidden_size=width,
                          options={"left": _attention(raw["left"], width, eps, cfg.max_positions),
                                   "right": _scan(raw["right"], width),
                                   "left_scale": float(raw["left_scale"]), "right_scale": float(raw["right_scale"])})
        feed_forward = _feed_forward(layer.get("mlp"), width)
        layers.append(LayerSpec(
            block="parallel_scaled", mixer=mixer, feed_forward=feed_forward, mixer_norm=norm,
            feed_forward_norm=None if feed_forward is None else norm, mixer_prefix=f"{prefix}.mix",
            feed_forward_prefix=f"{prefix}.mlp", mixer_norm_prefix=f"{prefix}.norm1",
            feed_forward_norm_prefix=f"{prefix}.norm2", prefix=prefix, options={"width": width, "layer_scale": True}))
    # A layer that runs several times keeps keys, values and state of each pass apart: the first pass has the layer's
    # own cache unit, every further pass a unit of its own.  The passes' starts are where the frame takes the token in again.
    schedule, extra, seen, starts = [], [], set(), []
    for index, pass_starts in cfg.run_order():
        if pass_starts:
            starts.append(len(schedule))
        if index in seen:
            schedule.append(ScheduleEntry(index, unit=len(cfg.layers) + len(extra)))
            extra.append(index)
        else:
            schedule.append(ScheduleEntry(index))
            seen.add(index)
    options = {"head_scale": cfg.logit_scale, "head_cap": cfg.logit_softcap}
    if starts:
        options["pass_input"] = {"tensor": "loop.in", "before": tuple(starts)}
    return ModelSpec(
        architecture=cfg.architecture, vocab_size=cfg.vocab, hidden_size=width, max_positions=cfg.max_positions,
        embedding_name="embed", layers=tuple(layers), schedule=tuple(schedule), final_norm=norm,
        final_norm_prefix="final.norm", tied_head=False, head_name="head", extra_cache_units=tuple(extra),
        embedding_scale=cfg.embedding_scale, options=options)


register_architecture("Zomavik", ZomavikConfig, zomavik_spec)
