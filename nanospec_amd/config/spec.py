"""Typed descriptions of a model as data: which parts each layer is made of, with every size
and constant as a field, and the order in which the layers run.

A ``ModelSpec`` is what an architecture's configuration is turned into (see
``config/registry.py``); ``parts/`` builds the runnable model from it.  No part reads an
architecture's configuration: it sees only its own spec.  A spec class carries a ``kind``
string; ``parts/registry.py`` maps (role, kind) to the class that implements it, so a new
mixer, feed-forward, norm or position encoding is one spec dataclass plus one implementation
registered under a new kind.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import ClassVar


@dataclass(frozen=True)
class RMSNormSpec:
    """y = w * x / sqrt(mean(x^2) + eps) over the last axis."""

    kind: ClassVar[str] = "rmsnorm"
    dim: int
    eps: float


@dataclass(frozen=True)
class RopeSpec:
    """Rotary position encoding over the first ``rotary_dim`` elements of a head; pair j is elements j and
    j + rotary_dim/2 (``interleaved``: 2j and 2j + 1).  ``scaling`` is None or the llama3 frequency scaling as
    (factor, low_freq_factor, high_freq_factor, original_max_position_embeddings).  ``cos_sin_factor`` multiplies
    cosine and sine."""

    kind: ClassVar[str] = "rope"
    rotary_dim: int
    theta: float
    scaling: tuple[float, float, float, int] | None = None
    max_positions: int | None = None  # None = unbounded
    interleaved: bool = False
    cos_sin_factor: float = 1.0


@dataclass(frozen=True)
class NoPositionSpec:
    kind: ClassVar[str] = "none"


@dataclass(frozen=True)
class AttentionSpec:
    """Soft-max attention over a key/value cache with grouped query heads.  ``window`` = 0 sees
    all earlier keys; ``window`` = w sees the last w positions (its own included)."""

    kind: ClassVar[str] = "attention"
    hidden: int
    heads: int
    kv_heads: int
    head_dim: int
    position: object  # a position spec (RopeSpec, NoPositionSpec, ...)
    softmax_scale: float  # multiplies q.k before the soft-max
    window: int = 0


@dataclass(frozen=True)
class SwiGLUSpec:
    """down(silu(gate(x)) * up(x)), dense, no bias."""

    kind: ClassVar[str] = "swiglu"
    hidden: int
    intermediate: int


@dataclass(frozen=True)
class PreNormBlockSpec:
    """x = x + mixer(norm1(x)); x = x + feed_forward(norm2(x)).  ``prefix`` is the layer's
    tensor-name prefix in the checkpoint, e.g. ``model.layers.3.``; the four names that follow it are the
    architecture's own and are appended to it: the two norms' weight tensors and the prefixes under which
    the mixer and the feed-forward find their tensors (None: the part's ``kind`` and a dot)."""

    kind: ClassVar[str] = "prenorm"
    prefix: str
    mixer_norm: object
    mixer: object
    ffn_norm: object
    ffn: object
    mixer_norm_name: str = "mixer_norm.weight"
    mixer_prefix: str | None = None
    ffn_norm_name: str = "ffn_norm.weight"
    ffn_prefix: str | None = None


@dataclass(frozen=True)
class LayerCall:
    """One entry of the run order.  ``layer`` indexes ``ModelSpec.layers`` (a layer may be named
    by several entries: its weights are used again, each entry with a cache of its own).
    ``cache_from`` names an EARLIER entry of the run order whose cache this entry reads instead
    of writing one of its own."""

    layer: int
    cache_from: int | None = None


@dataclass(frozen=True)
class ModelSpec:
    vocab_size: int
    hidden: int
    embed_name: str  # tensor name of the [vocab, hidden] table
    layers: tuple  # block specs
    run_order: tuple[LayerCall, ...]
    final_norm: object
    final_norm_name: str
    head_name: str  # tensor name of the [vocab, hidden] output matrix
    tie_head: bool  # a missing head tensor is the embedding table
    eos_token_ids: tuple[int, ...] = field(default_factory=tuple)
    # what an architecture may do at the two ends of the stack; the defaults do nothing and launch nothing
    embed_scale: float = 1.0  # the embedding rows are multiplied by this as they enter the stream
    logit_scale: float = 1.0  # the head's 32-bit logits are multiplied by this ...
    logit_softcap: float = 0.0  # ... and then, if > 0, become softcap * tanh(logit / softcap)

    def __post_init__(self) -> None:
        for pos, call in enumerate(self.run_order):
            if not 0 <= call.layer < len(self.layers):
                raise ValueError(f"run order entry {pos} names layer {call.layer}, but there are {len(self.layers)} layers")
            if call.cache_from is not None:
                if not 0 <= call.cache_from < pos:
                    raise ValueError(f"run order entry {pos} reads the cache of entry {call.cache_from}, which is not an earlier entry")
                if self.run_order[call.cache_from].cache_from is not None:
                    raise ValueError(f"run order entry {pos} reads the cache of entry {call.cache_from}, which has no cache of its own")
