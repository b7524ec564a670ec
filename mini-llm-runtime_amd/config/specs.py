"""Typed descriptions of a model, independent of any architecture.

An architecture's configuration (for instance `Qwen3Config`) turns its config.json keys into
a `ModelSpec`: a list of layers, each put together from part specs (norm, mixer,
feed-forward), and a schedule that says in which order the layers run and whose cache each
run uses.  The parts registry builds the parts from these specs; no part sees the
architecture's name.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional, Tuple


@dataclass(frozen=True)
class NormSpec:
    kind: str                 # key in the norm registry, e.g. "rmsnorm"
    size: int
    eps: float


@dataclass(frozen=True)
class PositionSpec:
    kind: str                 # key in the position registry, e.g. "rope_split_half"
    dim: int                  # rotated width (the head size here)
    base: float


@dataclass(frozen=True)
class AttentionSpec:
    kind: str                 # key in the mixer registry, e.g. "gqa_attention"
    hidden: int
    q_heads: int
    kv_heads: int
    head_dim: int
    scale: float              # factor on q.k before the softmax
    qk_norm: Optional[NormSpec] = None      # per-head norm of q and k before the rotation
    position: Optional[PositionSpec] = None
    window: Optional[int] = None            # keys seen: positions in (p - window, p]; None = all


@dataclass(frozen=True)
class MlpSpec:
    kind: str                 # key in the feed-forward registry, e.g. "swiglu"
    hidden: int
    intermediate: int
    activation: str = "silu"


@dataclass(frozen=True)
class LayerSpec:
    kind: str                 # key in the block registry, e.g. "prenorm"
    norm1: NormSpec
    mixer: object             # any mixer spec with a `kind`
    norm2: NormSpec
    ffn: object               # any feed-forward spec with a `kind`


@dataclass(frozen=True)
class LayerRun:
    """One entry of the run order: run `layer`'s weights against cache entry `cache`.
    `write_cache=False` reads what another run wrote into that entry."""
    layer: int
    cache: int
    write_cache: bool = True


@dataclass(frozen=True)
class EmbedSpec:
    kind: str                 # key in the embed registry, e.g. "token_embedding"
    vocab_size: int
    hidden: int


@dataclass(frozen=True)
class HeadSpec:
    kind: str                 # key in the head registry, e.g. "linear_head"
    vocab_size: int
    hidden: int
    tied: bool = False        # no tensor of its own: the embedding's table


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden: int
    layers: Tuple[LayerSpec, ...]
    schedule: Tuple[LayerRun, ...]
    final_norm: NormSpec
    tie_embeddings: bool
    max_positions: int
    eos_token_ids: Tuple[int, ...] = field(default_factory=tuple)
    embed: Optional[object] = None      # any embed spec with a `kind`; None: a plain table [vocab_size, hidden]
    head: Optional[object] = None       # any head spec with a `kind`; None: a plain projection, tied as `tie_embeddings` says

    def embed_spec(self):
        return self.embed if self.embed is not None else EmbedSpec("token_embedding", self.vocab_size, self.hidden)

    def head_spec(self):
        return self.head if self.head is not None else HeadSpec("linear_head", self.vocab_size, self.hidden,
                                                                self.tie_embeddings)
