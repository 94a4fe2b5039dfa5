"""A model as data: what each layer is made of, and the order in which layers run.

A plan holds no tensors and no code.  Each spec names a part by `kind` (looked up in
the part registries of `parts.base`) and carries every size and constant that part
needs, so no part ever asks which model it is in.  The run list is data too: it may
name a layer twice, or let a run read the cache that another run writes.
"""

from dataclasses import dataclass
from typing import Any, Optional


@dataclass(frozen=True)
class NormSpec:
    kind: str  # "rmsnorm"
    size: int
    eps: float


@dataclass(frozen=True)
class RotarySpec:
    """Rotary position encoding of a head's first `rotary_dim` coordinates.
    kind "rope_half": pairs are (i, i + rotary_dim/2)."""

    kind: str
    rotary_dim: int
    theta: float


@dataclass(frozen=True)
class AttentionSpec:
    """Grouped-query softmax attention over a paged cache."""

    kind: str  # "attention"
    hidden_size: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    scale: float  # multiplies q.k before the softmax
    qk_norm: Optional[NormSpec]  # per-head norm of q and k before the rotation, or None
    position: Optional[RotarySpec]  # applied to q and k, or None
    window: int = 0  # > 0: a query at p sees keys p-window+1..p only; 0: all keys


@dataclass(frozen=True)
class GatedMLPSpec:
    """Dense gated feed-forward: down(act(gate(x)) * up(x))."""

    kind: str  # "gated_mlp"
    hidden_size: int
    intermediate_size: int
    activation: str  # "silu"


@dataclass(frozen=True)
class BlockSpec:
    """One layer: a mixer and a feed-forward with their norms, and how they are arranged.
    arrangement "prenorm": x += mixer(norm(x)); x += ffn(norm(x))."""

    arrangement: str
    mixer: Any
    mixer_norm: NormSpec
    ffn: Any
    ffn_norm: NormSpec


@dataclass(frozen=True)
class Run:
    """One entry of the run list: execute layer `layer`.

    cache: id of the cache this run's mixer uses (None: a cache of its own, named after
           the run's index).  Two runs with the same id share one cache.
    writes: whether this run stores what it computes into that cache; a run that only
           reads another run's cache sets this to False.
    """

    layer: int
    cache: Optional[int] = None
    writes: bool = True


@dataclass(frozen=True)
class ModelPlan:
    vocab_size: int
    hidden_size: int
    layers: tuple  # of BlockSpec
    run: tuple  # of Run
    final_norm: NormSpec
    tied_head: bool
    max_positions: int
    embedding_scale: float = 1.0  # multiplies the embedding rows as they enter the stream
    logit_scale: float = 1.0  # multiplies the head's output
    logit_softcap: float = 0.0  # > 0: logits = cap * tanh(logits / cap), after the scale

    def cache_id(self, run_index: int) -> int:
        r = self.run[run_index]
        return run_index if r.cache is None else r.cache


def sequential_run(num_layers: int) -> tuple:
    """Every layer once, in order, each with a cache of its own."""
    return tuple(Run(i) for i in range(num_layers))
