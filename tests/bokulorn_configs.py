"""Tiny Bokulorn configurations for the tests, and their model folders.  They differ in every size and constant and in
the order of their layers; head counts and groupings, key, value and latent sizes, rotated coordinates, taps, expert
counts and groups take values that make nothing equal by accident (and some the values 1 and 0)."""
import os

import torch


def _delta(heads, kv_heads, dim, vdim, conv):
    return "channel_delta", {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}


def _rotated(heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, base):
    return "latent_attention", {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank,
                                "kv_rank": kv_rank, "scale": scale, "rot": {"dims": rot_dim, "base": base}}


def _unrotated(heads, dim, vdim, q_rank, kv_rank, scale):
    return "latent_attention_2", {"heads": heads, "dim": dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
                                  "scale": scale}


def _moe(experts, top, ff, count, keep):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top,
                                                            "groups": {"count": count, "keep": keep}}}


def _layer(kind_mixer, mlp=None, weights_of=None):
    out = {"type": kind_mixer[0], "mixer": kind_mixer[1], "mlp": mlp}
    if weights_of is not None:
        out["weights_of"] = weights_of
    return out


def _model(vocab, width, eps, scale, layers):
    return {"architecture": "Bokulorn", "vocab": vocab, "width": width, "norm": {"eps": eps},
            "embedding": {"scale": scale}, "layers": layers}


_A = [_delta(4, 2, 16, 24, 4), _rotated(4, 16, 8, 24, 24, 40, 0.3, 10000.0), _unrotated(2, 32, 16, 32, 32, 0.2)]
_B = [_rotated(3, 10, 6, 14, 20, 22, 0.35, 300.0), _delta(3, 3, 12, 14, 2), _unrotated(3, 6, 10, 12, 18, 0.4)]
_C = [_unrotated(4, 16, 64, 64, 96, 0.25), _rotated(2, 32, 16, 32, 48, 64, 0.18, 500000.0), _delta(4, 1, 64, 32, 5)]
_D = [_delta(2, 1, 20, 8, 1), _rotated(1, 24, 2, 40, 16, 30, 0.2, 100.0)]

BOKULORN = {
    # name: (config.json keys, weight seed)
    # All three mixers; layers 3 and 4 run with the tensors of layers 0 and 1 and a state and cache of their own; a layer
    # without feed-forward; two of three groups kept.
    "A": (_model(211, 64, 1e-5, 8.0, [
        _layer(_A[0], _moe(6, 2, 24, 3, 2)), _layer(_A[1], _moe(4, 1, 20, 2, 1)), _layer(_A[2]),
        _layer(_A[0], _moe(6, 2, 24, 3, 2), weights_of=0), _layer(_A[1], _moe(4, 1, 20, 2, 1), weights_of=1)]), 3),
    # Sizes that are no multiples of eight anywhere; as many query/key heads as heads; two taps; groups of one expert, all
    # kept; a layer that names a layer which names another.
    "B": (_model(97, 52, 2e-6, 3.5, [
        _layer(_B[0], _moe(5, 1, 10, 5, 5)), _layer(_B[1], _moe(6, 3, 14, 2, 2)), _layer(_B[2], _moe(4, 2, 12, 1, 1)),
        _layer(_B[1], _moe(6, 3, 14, 2, 2), weights_of=1), _layer(_B[1], _moe(6, 3, 14, 2, 2), weights_of=3)]), 8),
    # Latents and heads in sixteens (the sizes the matrix-core kernels take), attention first, one query/key head for
    # four heads, five taps, one of two groups kept.
    "C": (_model(180, 128, 1e-6, 11.3, [
        _layer(_C[0], _moe(8, 3, 32, 2, 1)), _layer(_C[1], _moe(8, 2, 16, 4, 3)), _layer(_C[2], _moe(12, 4, 24, 3, 2)),
        _layer(_C[0], _moe(8, 3, 32, 2, 1), weights_of=0)]), 21),
    # One tap (no convolution state), one head, a rotation of one pair, no layer with another's tensors, a scale of 1.
    "D": (_model(120, 40, 1e-6, 1.0, [_layer(_D[0], _moe(3, 1, 16, 3, 1)), _layer(_D[1])]), 34),
}


def write_model(raw: dict, seed: int, folder: str, sharpen: float = 5.0, router: float = 6.0) -> str:
    """A model folder from the random-weights mode, with its matrices made `sharpen` times larger, so that attention
    weights are peaked and the recurrent layer's gates, decays and step sizes move over their whole ranges: a key too
    many or too few, a lost state or a convolution that forgets its last inputs then moves the logits by much more than
    rounding does.  The routers are decisive (`router` times the drawn weights, far from the near ties that rounding
    tips), with corrections large enough to change the choice; the embedding is of the size of what the layers add."""
    import tokenizer_amd as ta
    from safetensors.torch import load_file, save_file
    from tokenizer_amd.config import BokulornConfig

    ta.write_random_model(BokulornConfig.from_dict(raw), seed, folder, norm_spread=0.3)
    path = os.path.join(folder, "model.safetensors")
    tensors = load_file(path)
    for name, tensor in tensors.items():
        if name == "embed":
            tensors[name] = (tensor.float() * 50.0 / float(raw["embedding"]["scale"])).to(torch.bfloat16)
        elif name.endswith(".router"):
            tensors[name] = (tensor.float() * router).to(torch.bfloat16)
        elif name.endswith((".a2", ".g2")):
            tensors[name] = (tensor.float() * 4 * sharpen).to(torch.bfloat16)
        elif tensor.dim() == 2 and name != "head" and not name.endswith(".conv"):
            tensors[name] = (tensor.float() * sharpen).to(torch.bfloat16)
    save_file(tensors, path)
    return folder


def random_config(seed: int) -> dict:
    """A Bokulorn configuration drawn from a seed: the number and order of layers, the three mixers, head counts and
    groupings, key, value and latent sizes (some in sixteens, some odd multiples of two), rotated coordinates, taps,
    routed feed-forwards with groups, layers without one, layers that run with another layer's tensors."""
    import random
    rng = random.Random(seed)
    width = rng.choice([32, 40, 64, 72, 96, 128])
    layers = []
    for _ in range(rng.randint(1, 4)):
        kind = rng.choice(["channel_delta", "latent_attention", "latent_attention_2"])
        dim = rng.choice([8, 12, 16, 16, 32, 32, 48, 64])
        vdim = dim if rng.random() < 0.5 else rng.choice([8, 10, 16, 24, 40])
        if kind == "channel_delta":
            kv_heads = rng.choice([1, 1, 2, 3])
            mixer = _delta(kv_heads * rng.choice([1, 2, 4]), kv_heads, dim, vdim, rng.choice([1, 2, 3, 4, 6]))
        else:
            heads = rng.choice([1, 2, 3, 4, 6])
            q_rank, kv_rank = rng.choice([8, 12, 16, 24, 40]), rng.choice([8, 16, 22, 32, 48, 64, 96])
            scale = rng.choice([dim ** -0.5, 0.2, 0.35])
            if kind == "latent_attention":
                rot_dim = rng.choice([2, 4, 8, 16, 16, 32])
                mixer = _rotated(heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, rng.choice([100.0, 10000.0, 500000.0]))
            else:
                mixer = _unrotated(heads, dim, vdim, q_rank, kv_rank, scale)
        mlp = None
        if rng.random() < 0.8:
            count = rng.choice([1, 2, 3, 4])
            per = rng.choice([1, 2, 3, 4])
            keep = rng.randint(1, count)
            mlp = _moe(count * per, rng.randint(1, min(4, keep * per)), rng.choice([8, 10, 16, 24, 32]), count, keep)
        layers.append(_layer(mixer, mlp))
    for _ in range(rng.randint(0, 3)):
        source = rng.randrange(len(layers))
        layers.insert(rng.randint(source + 1, len(layers)), {**layers[source], "weights_of": None})
    # (The inserted layers name their sources by index once every layer has its place.)
    placed = []
    for index, layer in enumerate(layers):
        if "weights_of" in layer and layer["weights_of"] is None:
            like = [j for j, other in enumerate(layers) if "weights_of" not in other and other["mixer"] is layer["mixer"]]
            layer = {**layer, "weights_of": like[0]}
        placed.append(layer)
    return _model(rng.choice([61, 128, 200, 333]), width, rng.choice([1e-6, 1e-5]), rng.choice([1.0, 5.0, width ** 0.5]), placed)
