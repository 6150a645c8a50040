"""Architecture-neutral description of a decoder model.

A model is a list of layers, each put together from parts (norm, mixer,
feed-forward, position encoding), and a *schedule*: the order in which the
layers run.  Every size and constant is a field of a spec, so one model may use
different mixers and feed-forwards in different layers, and a new part only has
to define a spec dataclass with a ``kind`` string and register a builder for it
(see ``parts.registry``).

The specs are plain data: they can be built on a machine without a GPU and are
what the cache manager, the weight loader and the random-weights writer read.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional, Tuple


@dataclass(frozen=True)
class RMSNormSpec:
    """y = x * rsqrt(mean(x^2) + eps) * w over the last dimension."""
    eps: float
    kind: str = "rmsnorm"


@dataclass(frozen=True)
class RopeSpec:
    """Half-split rotary position encoding over ``rotary_dim`` features.

    Angles are ``position * theta ** (-2 i / rotary_dim)``; the pair of feature
    ``i`` is feature ``i + rotary_dim / 2``.
    """
    theta: float
    rotary_dim: int
    max_positions: int
    kind: str = "rope_half"


@dataclass(frozen=True)
class AttentionSpec:
    """Grouped-query attention over a paged key/value cache.

    ``window`` is None for attention over all earlier keys, or the number of
    most recent keys (the query's own position included) that a query sees.
    ``qk_norm_eps`` is None when queries and keys are not normalised per head.
    """
    num_heads: int
    num_kv_heads: int
    head_dim: int
    scale: float
    qkv_bias: bool = False
    qk_norm_eps: Optional[float] = None
    window: Optional[int] = None
    position: Optional[object] = None  # a position-encoding spec, e.g. RopeSpec
    kind: str = "paged_attention"


@dataclass(frozen=True)
class SwiGLUSpec:
    """down(silu(gate(x)) * up(x)), no biases."""
    intermediate_size: int
    kind: str = "swiglu"


@dataclass(frozen=True)
class LayerSpec:
    """One pre-norm residual block: x += mixer(norm(x)); x += ffn(norm(x)).

    ``prefix`` is the checkpoint name prefix of the layer's tensors
    (for instance ``model.layers.3``).
    """
    prefix: str
    mixer_norm: object
    mixer: object
    ffn_norm: object
    ffn: object
    kind: str = "prenorm_block"
    # checkpoint names of the four parts inside ``prefix``, in the order of the fields above
    part_names: Tuple[str, str, str, str] = ("input_layernorm", "self_attn", "post_attention_layernorm", "mlp")


@dataclass(frozen=True)
class ScheduleEntry:
    """One run of a layer.

    ``layer`` indexes ``ModelSpec.layers`` (a layer may appear in several
    entries: its weights are shared, each entry has a cache of its own).
    ``cache_from`` is None, or the index of an earlier schedule entry whose
    cache this run reads instead of writing one of its own.
    """
    layer: int
    cache_from: Optional[int] = None


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden_size: int
    layers: Tuple[LayerSpec, ...]
    schedule: Tuple[ScheduleEntry, ...]
    final_norm: object
    embed_name: str
    final_norm_name: str
    head_name: str
    tie_head: bool
    max_positions: int
    eos_token_ids: Tuple[int, ...] = field(default_factory=tuple)
    # optional parts around the layers: a spec with a ``kind`` (and a ``prefix`` for its tensors' names)
    stream_prologue: Optional[object] = None   # changes the stream right after the embedding
    logit_epilogue: Optional[object] = None    # changes the logits after the head

    def validate(self) -> None:
        if not self.layers:
            raise ValueError("a model needs at least one layer")
        for i, entry in enumerate(self.schedule):
            if not 0 <= entry.layer < len(self.layers):
                raise ValueError(f"schedule entry {i} names layer {entry.layer}, "
                                 f"the model has {len(self.layers)}")
            if entry.cache_from is not None:
                if not 0 <= entry.cache_from < i:
                    raise ValueError(f"schedule entry {i} reads the cache of entry "
                                     f"{entry.cache_from}, which does not run before it")
                if self.schedule[entry.cache_from].cache_from is not None:
                    raise ValueError(f"schedule entry {i} reads the cache of entry "
                                     f"{entry.cache_from}, which has no cache of its own")
