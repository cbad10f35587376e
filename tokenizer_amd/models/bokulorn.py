"""Bokulorn as a `ModelSpec`: a decoder whose layers read one norm (its weight stored around zero) for a mixer and a
routed feed-forward side by side, x + (mixer(norm(x)) + feed_forward(norm(x))); three mixers (attention over a cached
latent with a rotated key part that all heads share and a gate per head; the same without positions and with a gate per
coordinate; a gated delta rule with a decay per key channel, short convolutions and its state in the request's slot);
experts without a gate branch (squared ReLU) chosen by sigmoid scores with a correction and a limit to the best groups;
layers that run with another layer's tensors and a cache or state of their own; a scaled embedding.

Tensor names: `embed`, `head`, `final.norm`; layer i's start with `l<i>.`: `norm1`, `mix.*` (the mixer's), `mlp.*`
(e<j>.up|down, router, correction).
"""
from __future__ import annotations

from ..config.bokulorn import BokulornConfig
from ..config.registry import register_architecture
from ..parts.spec import FeedForwardSpec, LayerSpec, MixerSpec, ModelSpec, NormSpec, ScheduleEntry


def _mixer(kind: str, raw: dict, width: int, eps: float) -> MixerSpec:
    if kind == "channel_delta":
        return MixerSpec("gated_delta", hidden_size=width, n_heads=raw["heads"], n_kv_heads=raw["kv_heads"],
                         head_dim=raw["dim"], value_dim=raw["vdim"], conv_taps=int(raw["conv"]), eps=eps,
                         options={"unit_eps": 1e-6})
    rotated = kind == "latent_attention"
    rot = raw.get("rot") or {}
    return MixerSpec("latent_attention", hidden_size=width, n_heads=raw["heads"], n_kv_heads=1, head_dim=raw["dim"],
                     value_dim=raw["vdim"], scale=float(raw["scale"]), q_rank=raw["q_rank"], kv_rank=raw["kv_rank"],
                     rot_dim=int(raw["rot_dim"]) if rotated else 0, head_gate=rotated, element_gate=not rotated,
                     eps=eps, options={"rot_base": float(rot.get("base", 1.0))})


def bokulorn_spec(cfg: BokulornConfig) -> ModelSpec:
    width, eps = cfg.width, cfg.eps
    # The weight is the tensor the prefix names, and the scale is one more than it.
    norm = NormSpec("rmsnorm", width, eps, options={"tensor_name": "", "offset": 1.0})
    owners = sorted({cfg.weight_owner(index) for index in range(len(cfg.layers))})
    place = {index: at for at, index in enumerate(owners)}        # a layer with tensors of its own -> its place in `layers`
    layers = []
    for index in owners:
        layer, prefix = cfg.layers[index], f"l{index}"
        mlp = layer.get("mlp")
        feed_forward = None
        if mlp is not None:
            router, groups = mlp["router"], mlp["router"].get("groups") or {}
            feed_forward = FeedForwardSpec("routed_experts", hidden_size=width, intermediate_size=mlp["expert"]["ff"],
                                           activation="relu2", gated=False, n_experts=router["experts"], top_k=router["top"],
                                           router="sigmoid", n_groups=int(groups.get("count") or 0),
                                           keep_groups=int(groups.get("keep") or 0))
        layers.append(LayerSpec(
            block="parallel", mixer=_mixer(layer["type"], layer["mixer"], width, eps), feed_forward=feed_forward,
            mixer_norm=norm, feed_forward_norm=None if mlp is None else norm, mixer_prefix=f"{prefix}.mix",
            feed_forward_prefix=f"{prefix}.mlp", mixer_norm_prefix=f"{prefix}.norm1",
            feed_forward_norm_prefix=f"{prefix}.norm1", prefix=prefix))
    # A layer that runs with another layer's tensors keeps keys, values and state of its own: a cache unit behind
    # the units of the layers that own tensors.
    schedule, extra = [], []
    for index in range(len(cfg.layers)):
        owner = cfg.weight_owner(index)
        if owner == index:
            schedule.append(ScheduleEntry(place[index]))
        else:
            schedule.append(ScheduleEntry(place[owner], unit=len(layers) + len(extra)))
            extra.append(place[owner])
    return ModelSpec(
        architecture=cfg.architecture, vocab_size=cfg.vocab, hidden_size=width, max_positions=cfg.max_positions,
        embedding_name="embed", layers=tuple(layers), schedule=tuple(schedule), final_norm=norm,
        final_norm_prefix="final.norm", tied_head=False, head_name="head", extra_cache_units=tuple(extra),
        embedding_scale=cfg.embedding_scale)


register_architecture("Bokulorn", BokulornConfig, bokulorn_spec)
