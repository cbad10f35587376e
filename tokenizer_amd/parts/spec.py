"""Descriptions of a model as data: parts, layers and the order they run in.

An architecture turns its configuration into a `ModelSpec`.  Nothing below
knows any architecture: every size and constant is a field, every part is named
by a `kind` that the part registries resolve, and the run order is a list of
`ScheduleEntry`, which may name a layer twice or point a layer at another
layer's cache.
"""
from __future__ import annotations

import dataclasses
from typing import Any


@dataclasses.dataclass(frozen=True)
class TensorSpec:
    """One tensor a part needs from the weight file.

    `init` says how the random-weights mode fills it: "normal" (N(0, std)),
    "ones", "zeros" or "eye" (the identity matrix).  `role` says how it is kept in memory: "matrix" tensors
    feed matrix products and are held in the compute dtype, "vector" tensors
    (norm scales, biases) are small and held in float32, "table" tensors are
    integer tables kept as int32, "keep" tensors stay as the file stores them.
    A -1 in `shape` is a size that only the file gives (no configuration key names it): the loader takes what it
    finds there, and the random-weights mode writes `free_size`.
    """
    shape: tuple[int, ...]
    init: str = "normal"
    std: float = 0.02
    role: str = "matrix"
    free_size: int = 0

    def fits(self, shape) -> bool:
        shape = tuple(shape)
        return len(shape) == len(self.shape) and all(want in (-1, found) for want, found in zip(self.shape, shape))

    def drawn_shape(self) -> tuple[int, ...]:
        return tuple(self.free_size if size == -1 else size for size in self.shape)


@dataclasses.dataclass(frozen=True)
class CacheNeed:
    """What a mixer asks of the cache manager for one layer.

    kind "full": keys and values of every position, in pages.
    kind "window": only the last `window` + 1 positions are ever read; pages
    wholly behind the window are given back.
    kind "none": no pages.
    `state_shape`: per-request state of fixed size kept in a slot, or None.
    `value_dim`: size of a value head where it differs from the key heads' `head_dim` (0: the same).
    `block_state_shape`: per-request state that the block around the mixer keeps in the same slot (the last
    token's normalised row, for a token shift), or None; always float32.
    `keep_first`: with a window, the first so many positions of a sequence stay readable for every later query.
    `n_value_heads`: the number of value heads where it is not the number of key heads (several key heads, the
    maps of one differential head, read the same values).
    """
    kind: str = "none"
    n_kv_heads: int = 0
    head_dim: int = 0
    window: int | None = None
    state_shape: tuple[int, ...] | None = None
    state_dtype: str = "float32"
    value_dim: int = 0
    block_state_shape: tuple[int, ...] | None = None
    keep_first: int = 0           # kind "window": the pages of the first so many positions are never given back
    n_value_heads: int = 0        # value heads where several key heads read one value head (0: as many as key heads)

    @property
    def v_dim(self) -> int:
        return self.value_dim or self.head_dim

    @property
    def v_heads(self) -> int:
        return self.n_value_heads or self.n_kv_heads

    def page_key(self) -> tuple:
        """Layers with equal keys share one group of pages and one block table."""
        return (self.kind, self.n_kv_heads, self.head_dim, self.window, self.v_dim, self.keep_first, self.v_heads)


@dataclasses.dataclass(frozen=True)
class NormSpec:
    kind: str
    size: int
    eps: float
    options: dict[str, Any] = dataclasses.field(default_factory=dict, hash=False, compare=False)


@dataclasses.dataclass(frozen=True)
class PositionSpec:
    """Position encoding applied to queries and keys inside a mixer."""
    kind: str                     # "rope_half_split", "none", ...
    head_dim: int = 0
    theta: float = 0.0
    max_positions: int = 0
    options: dict[str, Any] = dataclasses.field(default_factory=dict, hash=False, compare=False)


@dataclasses.dataclass(frozen=True)
class MixerSpec:
    kind: str                     # "gqa_attention", ...
    hidden_size: int
    n_heads: int = 0
    n_kv_heads: int = 0
    head_dim: int = 0
    qkv_bias: bool = False
    out_bias: bool = False
    window: int | None = None
    scale: float | None = None    # None = 1/sqrt(head_dim)
    position: PositionSpec | None = None
    value_dim: int | None = None  # size of a value head (None = head_dim)
    chunk: int | None = None      # a query sees only keys of its own run of `chunk` positions, counted from 0
    distance_bias: float | None = None   # b: head h's scores lose 2^(-b (h+1) / n_heads) per position of distance
    sink: bool = False            # a learned number per head joins the softmax's denominator
    own_kv: bool = True           # False: no key/value projections; the layer reads the cache it is pointed at
    gate_cap: float | None = None  # recurrent mixers: the cap on the gates' pre-activations
    eps: float = 0.0              # mixers with a norm of their own inside
    keep_first: int = 0           # with a window: keys at positions below this stay visible to every later query
    differential: float | None = None   # c: two score maps per head over the same values, o = a1 - lambda a2 with
    #                               lambda = exp(lq1.lk1) - exp(lq2.lk2) + c, o brought to unit RMS per head, times 1 - c
    qk_norm: str | None = None    # "whole": RMS norm with a weight over all query rows at once (and all key rows), before rotation
    head_gate: bool = False       # each head's output times sigmoid of one number projected from the mixer's input
    q_rank: int = 0               # latent attention: width of the normalised latent the queries are projected up from
    kv_rank: int = 0              # latent attention: width of the normalised latent that keys and values are projected
    #                               up from (the latent is what the cache keeps, with the rotated key part behind it)
    rot_dim: int = 0              # latent attention: coordinates at the end of every query head that are rotated and meet
    #                               one rotated key part shared by all heads (0: no positions at all)
    element_gate: bool = False    # the mixer's output times sigmoid of a projection of its input, coordinate by coordinate
    conv_taps: int = 0            # recurrent mixers: taps of the short causal convolution over q, k and v (0: none)
    softcap: float | None = None  # c: a score (scaled, biased) becomes c tanh(score / c) before the softmax
    inner_size: int = 0           # selective scan: channels of the recurrence
    state_dim: int = 0            # selective scan: numbers of state a channel keeps
    dt_rank: int = 0              # selective scan: width of the narrow projection the step sizes are made from
    tensor_names: tuple[tuple[str, str], ...] = ()   # (part's name, file's name) where a file names tensors otherwise
    options: dict[str, Any] = dataclasses.field(default_factory=dict, hash=False, compare=False)


@dataclasses.dataclass(frozen=True)
class FeedForwardSpec:
    kind: str                     # "gated_dense", ...
    hidden_size: int
    intermediate_size: int = 0
    activation: str = "silu"      # "silu", "gelu_tanh", or "capped_swish" with the three numbers below
    act_alpha: float = 1.0        # g * sigmoid(alpha g)
    act_limit: float | None = None  # g is cut at +limit, the other branch at +-limit
    act_up_shift: float = 0.0     # added to the other branch before the product
    n_experts: int = 0            # routed feed-forwards: experts of `intermediate_size`, of which a token uses `top_k`
    top_k: int = 0
    shared_size: int = 0          # inner width of an expert that every token uses (0: none)
    gated: bool = True            # experts are down(act(gate) * up); False: down(act(up)), tensors `up` and `down` alone
    router: str = "softmax"       # "softmax": the largest logits, weighted by the softmax over the chosen; "sigmoid":
    #                               scores s = sigmoid(logit), chosen by s + `correction` (a tensor, one number an
    #                               expert), weighted by s over the chosen's sum; "softmax_all": scores s = softmax
    #                               over all experts, chosen by s, weighted by s over the chosen's sum
    n_groups: int = 0             # "sigmoid": experts form so many equal groups of neighbours (0: no groups) ...
    keep_groups: int = 0          # ... of which only the best so many (by the sum of a group's two largest choice
    #                               scores) can be chosen from
    group_worth: str = "top2"     # what a group is worth: "top2" (the sum of its two largest choice scores) or "max"
    shared_gate: bool = False     # the shared expert's output times sigmoid of one number projected from the input
    #                               (tensor `shared.sg` [1, hidden])
    tensor_names: tuple[tuple[str, str], ...] = ()
    options: dict[str, Any] = dataclasses.field(default_factory=dict, hash=False, compare=False)


@dataclasses.dataclass(frozen=True)
class LayerSpec:
    """One layer: which block arrangement, which parts, and their tensor name prefixes.

    Either sub-layer may be absent (None for the part and for its norm; at least one is there): a layer of a
    mixer alone, or of a feed-forward alone.  Since the schedule is a list of layers, any chain of sub-layers
    (two mixers before one feed-forward, say) is a run of such layers.
    """
    block: str                    # "pre_norm", ...
    mixer: MixerSpec | None
    feed_forward: FeedForwardSpec | None
    mixer_norm: NormSpec | None
    feed_forward_norm: NormSpec | None
    mixer_prefix: str = ""
    feed_forward_prefix: str = ""
    mixer_norm_prefix: str = ""
    feed_forward_norm_prefix: str = ""
    prefix: str = ""              # of the tensors that belong to the block itself (blocks that have any)
    options: dict[str, Any] = dataclasses.field(default_factory=dict, hash=False, compare=False)   # the block's own constants

    def __post_init__(self):
        if self.mixer is None and self.feed_forward is None:
            raise ValueError("a layer needs a mixer or a feed-forward")
        for part, norm, what in ((self.mixer, self.mixer_norm, "mixer"),
                                 (self.feed_forward, self.feed_forward_norm, "feed-forward")):
            if (part is None) != (norm is None):
                raise ValueError(f"a layer's {what} and its norm are there together or not at all")


@dataclasses.dataclass(frozen=True)
class ScheduleEntry:
    """Run `layer`; its mixer uses the cache of `cache_of` (default: its own).

    A layer that reads another layer's cache writes nothing into it.  `unit`: the run has a cache of its own under
    this number instead of the layer's (a layer that runs several times with the same weights and keeps keys,
    values and state of each run apart): units 0..n_layers-1 are the layers' own, `ModelSpec.extra_cache_units`
    lists the further ones, each by the layer whose need it repeats.
    """
    layer: int
    cache_of: int | None = None
    unit: int | None = None

    def cache_unit(self) -> int:
        if self.unit is not None:
            return self.unit
        return self.layer if self.cache_of is None else self.cache_of


@dataclasses.dataclass(frozen=True)
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden_size: int
    max_positions: int
    embedding_name: str
    layers: tuple[LayerSpec, ...]
    schedule: tuple[ScheduleEntry, ...]
    final_norm: NormSpec
    final_norm_prefix: str
    tied_head: bool
    head_name: str                # used when the head is not tied
    embedding_std: float = 0.02
    embedding_scale: float = 1.0  # the embedding's rows are multiplied by this on their way into the stream
    frame: str = "decoder"        # what stands around the layers (`parts.base.FRAMES`)
    extra_cache_units: tuple[int, ...] = ()   # cache unit n_layers + i repeats the need of layer extra_cache_units[i]
    options: dict[str, Any] = dataclasses.field(default_factory=dict, hash=False, compare=False)   # the frame's own constants
