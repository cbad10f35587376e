"""Tiny Zomavik configurations for the tests, and their model folders.  They differ in every size and constant and in
the order of their layers; head counts and groupings, key and value sizes, rotated coordinates, channels, state sizes,
step-size ranks, taps, expert counts and groups take values that make nothing equal by accident (and some the values 1
and 0)."""
import os

import torch


def _left(heads, kv_heads, dim, vdim, dims, base, scale, softcap):
    out = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
           "rot": {"dims": dims, "base": base}}
    if softcap is not None:
        out["softcap"] = softcap
    return out


def _right(inner, state, dt_rank, conv):
    return {"inner": inner, "state": state, "dt_rank": dt_rank, "conv": conv}


def _mixer(left, right, left_scale, right_scale):
    return {"left": left, "right": right, "left_scale": left_scale, "right_scale": right_scale}


def _dense(ff):
    return {"kind": "dense", "ff": ff}


def _moe(experts, top, ff, count=None, keep=None, shared=None):
    router = {"experts": experts, "top": top}
    if count is not None:
        router["groups"] = {"count": count, "keep": keep}
    out = {"kind": "moe", "expert": {"ff": ff}, "router": router}
    if shared is not None:
        out["shared"] = {"ff": shared}
    return out


def _layer(mixer, mlp=None):
    return {"type": "parallel", "mixer": mixer, "mlp": mlp}


def _model(vocab, width, eps, layers, scale=None, loop=None, logit_scale=None, logit_softcap=None):
    out = {"architecture": "Zomavik", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if scale is not None:
        out["embedding"] = {"scale": scale}
    if loop is not None:
        out["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    if logit_scale is not None:
        out["logit_scale"] = logit_scale
    if logit_softcap is not None:
        out["logit_softcap"] = logit_softcap
    return out


_A = [_mixer(_left(4, 2, 16, 24, 8, 10000.0, 0.3, 20.0), _right(48, 5, 3, 4), 0.7, 0.4),
      _mixer(_left(2, 1, 32, 16, 32, 500.0, 0.2, 8.0), _right(40, 9, 6, 3), 0.3, 1.1)]
_B = [_mixer(_left(3, 3, 10, 14, 6, 300.0, 0.35, 5.0), _right(36, 7, 5, 2), 1.2, 0.8),
      _mixer(_left(6, 2, 6, 10, 0, 100.0, 0.4, None), _right(20, 3, 2, 5), 0.5, 0.5)]
_C = [_mixer(_left(4, 1, 64, 64, 32, 500000.0, 0.125, 28.0), _right(128, 16, 8, 4), 0.65, 0.45),
      _mixer(_left(8, 2, 32, 32, 32, 10000.0, 0.18, 12.0), _right(256, 24, 16, 3), 0.9, 0.2)]
_D = [_mixer(_left(1, 1, 24, 40, 2, 100.0, 0.2, 3.0), _right(16, 1, 1, 1), 1.0, 1.0)]
_E = [_mixer(_left(5, 5, 12, 6, 10, 2000.0, 0.29, 7.0), _right(30, 11, 3, 3), 0.8, 0.6),
      _mixer(_left(2, 1, 18, 22, 18, 50.0, 0.24, 40.0), _right(54, 20, 7, 4), 0.45, 0.9)]

ZOMAVIK = {
    # name: (config.json keys, weight seed)
    # A dense layer, two kinds of routed layers (with a shared expert and groups; without either) and a layer without
    # feed-forward; layers 1 and 2 run twice.
    "A": (_model(211, 64, 1e-5, [
        _layer(_A[0], _dense(40)), _layer(_A[1], _moe(6, 2, 24, 3, 2, shared=16)), _layer(_A[0], _moe(4, 1, 20)),
        _layer(_A[1])], scale=8.0, loop=(1, 3, 2), logit_scale=0.5, logit_softcap=9.0), 3),
    # Sizes that are no multiples of eight anywhere; as many key heads as heads; two and five taps; no rotation in one
    # layer and no cap on its scores; nothing repeated, the logits as they are; groups of one expert, all kept.
    "B": (_model(97, 52, 2e-6, [
        _layer(_B[0], _moe(5, 1, 10, 5, 5, shared=6)), _layer(_B[1], _dense(30)), _layer(_B[0], _moe(6, 3, 14, 2, 2))],
        scale=3.5), 8),
    # Heads in sixteens with values as wide as keys (the sizes the matrix-core kernels take), one key head for four;
    # the first layer alone runs three times; one of two and two of four groups kept.
    "C": (_model(180, 128, 1e-6, [
        _layer(_C[0], _moe(8, 3, 32, 2, 1, shared=32)), _layer(_C[1], _moe(8, 2, 16, 4, 2, shared=8)),
        _layer(_C[0], _dense(96))], scale=11.3, loop=(0, 1, 3), logit_scale=2.0, logit_softcap=25.0), 21),
    # One tap (no convolution state), one head, a rotation of one pair, one number of state, a step-size rank of one,
    # weights of 1 on both sides, an embedding as it is, a run that is gone through once, scaled logits without a cap.
    # A width that is no multiple of four under a repeated run (the pass's input is a row of twice that width), an odd
    # vocabulary, the whole model gone through twice, seven experts without groups, twenty numbers of state.
    "E": (_model(131, 50, 1e-5, [_layer(_E[0], _moe(7, 3, 18, shared=10)), _layer(_E[1], _dense(34)), _layer(_E[0])],
                 scale=6.0, loop=(0, 3, 2), logit_scale=1.5, logit_softcap=12.0), 55),
    "D": (_model(120, 40, 1e-6, [_layer(_D[0], _moe(3, 1, 16, 3, 1)), _layer(_D[0], _dense(24))], loop=(0, 2, 1),
                 logit_scale=0.7), 34),
}


def write_model(raw: dict, seed: int, folder: str, sharpen: float = 5.0, router: float = 6.0) -> str:
    """A model folder from the random-weights mode, with its matrices made `sharpen` times larger, so that attention
    weights are peaked and the recurrent side's step sizes and gates move over their ranges: a key too many or too few,
    a lost state or a convolution that forgets its last inputs then moves the logits by much more than rounding does.
    The routers are decisive (`router` times the drawn weights, far from the near ties that rounding tips); the
    embedding is of the size of what the layers add; layer scales and sinks are spread."""
    import tokenizer_amd as ta
    from safetensors.torch import load_file, save_file
    from tokenizer_amd.config import ZomavikConfig

    ta.write_random_model(ZomavikConfig.from_dict(raw), seed, folder, norm_spread=0.3)
    path = os.path.join(folder, "model.safetensors")
    tensors = load_file(path)
    scale = float((raw.get("embedding") or {}).get("scale", 1.0))
    for name, tensor in tensors.items():
        if name == "embed":
            tensors[name] = (tensor.float() * 50.0 / scale).to(torch.bfloat16)
        elif name == "loop.in":
            tensors[name] = (tensor.float() * 25.0).to(torch.bfloat16)
        elif name.endswith((".router", ".sg")):
            tensors[name] = (tensor.float() * router).to(torch.bfloat16)
        elif name.endswith(".right.dt"):
            tensors[name] = (tensor.float() * 2 * sharpen).to(torch.bfloat16)
        elif tensor.dim() == 2 and name != "head" and not name.endswith((".conv", ".A_log")):
            tensors[name] = (tensor.float() * sharpen).to(torch.bfloat16)
    save_file(tensors, path)
    return folder


def random_config(seed: int) -> dict:
    """A Zomavik configuration drawn from a seed: the number of layers, head counts and groupings, key and value sizes
    (some in sixteens and equal, some odd multiples of two), rotated coordinates, channels, state sizes, ranks, taps,
    dense and routed feed-forwards with and without groups and shared experts, layers without one, a repeated run."""
    import random
    rng = random.Random(seed)
    width = rng.choice([32, 40, 64, 72, 96, 128])
    layers = []
    for _ in range(rng.randint(1, 4)):
        dim = rng.choice([8, 12, 16, 16, 32, 32, 48, 64])
        vdim = dim if rng.random() < 0.5 else rng.choice([8, 10, 16, 24, 40])
        kv_heads = rng.choice([1, 1, 2, 3])
        left = _left(kv_heads * rng.choice([1, 2, 4]), kv_heads, dim, vdim, rng.choice([0, 2, dim // 2 // 2 * 2, dim]),
                     rng.choice([100.0, 10000.0, 500000.0]), rng.choice([dim ** -0.5, 0.2, 0.35]),
                     rng.choice([None, 4.0, 18.0, 50.0]))
        right = _right(rng.choice([16, 24, 40, 64, 100]), rng.choice([1, 4, 8, 11, 16, 24, 40]), rng.choice([1, 3, 8, 12]),
                       rng.choice([1, 2, 3, 4, 6]))
        mixer = _mixer(left, right, rng.choice([0.55, 0.7, 1.0]), rng.choice([0.4, 0.45, 1.3]))
        kind = rng.random()
        if kind < 0.2:
            mlp = None
        elif kind < 0.45:
            mlp = _dense(rng.choice([8, 20, 32, 50]))
        else:
            count, per = rng.choice([1, 2, 3, 4]), rng.choice([1, 2, 3, 4])
            keep = rng.randint(1, count)
            grouped = rng.random() < 0.7
            top = rng.randint(1, min(4, keep * per if grouped else count * per))
            mlp = _moe(count * per, top, rng.choice([8, 10, 16, 24, 32]), count if grouped else None,
                       keep if grouped else None, rng.choice([None, 8, 12, 16]))
        layers.append(_layer(mixer, mlp))
    loop = None
    if rng.random() < 0.7:
        start = rng.randrange(len(layers))
        loop = (start, rng.randint(start + 1, len(layers)), rng.randint(1, 3))
    return _model(rng.choice([61, 128, 200, 333]), width, rng.choice([1e-6, 1e-5]), layers,
                  scale=rng.choice([None, 5.0, width ** 0.5]), loop=loop, logit_scale=rng.choice([None, 0.3, 1.5]),
                  logit_softcap=rng.choice([None, 10.0, 35.0]))
