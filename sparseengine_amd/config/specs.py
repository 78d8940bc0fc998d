"""Architecture-neutral description of a model: which parts each layer is made of, with every
size and constant as a field, and the order in which layers run.

An architecture module turns its own ``config.json`` keys into a ``ModelSpec``; the model builder
knows only these specs.  Each spec class carries a ``kind`` string that the part registries use
to find the implementing class, so a new kind of part is a new spec class plus one registration.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, ClassVar


@dataclass(frozen=True)
class NormSpec:
    kind: ClassVar[str] = "rms"
    eps: float = 1e-6


@dataclass(frozen=True)
class RotarySpec:
    """Rotation of the first ``rotary_dim`` dims of every head; ``pairing`` 'neox' pairs
    ``(d, d + rotary_dim/2)``.  ``scaling`` is the sorted item tuple of a rope_scaling dict."""
    kind: ClassVar[str] = "rotary"
    rotary_dim: int = 0
    theta: float = 10000.0
    max_position: int = 0
    pairing: str = "neox"
    scaling: tuple | None = None


@dataclass(frozen=True)
class NoPositionSpec:
    kind: ClassVar[str] = "none"


@dataclass(frozen=True)
class AttentionSpec:
    """Causal grouped-query attention over a paged key/value cache."""
    kind: ClassVar[str] = "gqa_attention"
    num_heads: int = 0
    num_kv_heads: int = 0
    head_dim: int = 0
    scale: float = 1.0
    qk_norm: str = "none"          # "none" | "flat" (one RMS statistic per token over all heads) | "per_head" (one per token and head)
    qk_norm_eps: float = 1e-6
    window: int | None = None       # keys further back than this are not read (None: all keys)
    position: Any = field(default_factory=NoPositionSpec)
    kv_page_size: int | None = None  # tokens per cache page of this layer's group (None: the engine's)


@dataclass(frozen=True)
class MoESpec:
    """Routed SwiGLU experts."""
    kind: ClassVar[str] = "moe"
    num_experts: int = 0
    top_k: int = 0
    intermediate_size: int = 0
    scoring: str = "sigmoid"        # "sigmoid" | "softmax"
    selection_bias: bool = True     # a per-expert bias added for selection only
    norm_topk_prob: bool = True
    routed_scaling_factor: float = 1.0
    activation: str = "silu"


@dataclass(frozen=True)
class DenseMLPSpec:
    """Gated feed-forward ``down(act(gate x) * up x)`` without routing."""
    kind: ClassVar[str] = "dense_mlp"
    intermediate_size: int = 0
    activation: str = "silu"


@dataclass(frozen=True)
class LayerSpec:
    """One layer: how mixer and feed-forward are arranged (``block``) and what they are."""
    mixer: Any
    feed_forward: Any
    norm: NormSpec = field(default_factory=NormSpec)
    block: str = "prenorm"


@dataclass(frozen=True)
class ScheduleEntry:
    """One position of the run order.  ``layer`` indexes ``ModelSpec.layers``; a layer may appear
    more than once.  ``cache_from`` names an earlier position whose cache this one reads instead
    of keeping one of its own."""
    layer: int
    cache_from: int | None = None


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    hidden_size: int
    vocab_size: int
    layers: tuple[LayerSpec, ...]
    schedule: tuple[ScheduleEntry, ...]
    final_norm: NormSpec
    max_position: int
    tie_word_embeddings: bool = False
    # (name, value) pairs for an architecture's own model class (``Architecture.model_factory``): constants of
    # the model's two ends that the generic decoder does not have (an embedding multiplier, a logit scale)
    constants: tuple[tuple[str, float], ...] = ()

    def __post_init__(self):
        for pos, entry in enumerate(self.schedule):
            if not 0 <= entry.layer < len(self.layers):
                raise ValueError(f"schedule position {pos} names layer {entry.layer}, "
                                 f"but there are {len(self.layers)} layers")
            if entry.cache_from is not None:
                if not 0 <= entry.cache_from < pos:
                    raise ValueError(f"schedule position {pos} reads the cache of position "
                                     f"{entry.cache_from}, which does not run before it")
                if self.schedule[entry.cache_from].cache_from is not None:
                    raise ValueError(f"schedule position {pos} reads the cache of position "
                                     f"{entry.cache_from}, which has no cache of its own")


def default_schedule(num_layers: int) -> tuple[ScheduleEntry, ...]:
    return tuple(ScheduleEntry(i) for i in range(num_layers))
