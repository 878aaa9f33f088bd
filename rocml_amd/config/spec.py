"""Architecture-neutral description of a decoder: parts, blocks, run order.

A ``ModelSpec`` is what an architecture's configuration is turned into before
anything is built.  It names every size and constant of every part, layer by
layer, so that no part needs to know which model it belongs to, and the order
in which layers run is a list of its own (``schedule``).  The reference fixes
all of this in one struct for one architecture (rocml/src/config.rs:32-54) and
keeps its constants in code (docs/multiarch-audit.md lists them as gaps 1-8);
here they are fields.

A part's spec is any object with a ``kind`` attribute; ``kind`` selects the
builder in ``rocml_amd.parts.registry``.  The dataclasses below are the specs of
the parts this library ships.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Optional, Tuple


@dataclass(frozen=True)
class NormSpec:
    """Root-mean-square norm over the last ``size`` values with a gain vector."""
    size: int
    eps: float
    kind: str = "rmsnorm"


@dataclass(frozen=True)
class RopeSpec:
    """Rotary position encoding with NEOX pairing ``(i, i + rot_dim/2)`` over the
    first ``rot_dim`` values of a head; ``theta`` is the frequency base."""
    head_dim: int
    rot_dim: int
    theta: float
    kind: str = "rope_neox"


@dataclass(frozen=True)
class AttentionSpec:
    """Softmax attention with grouped key/value heads over a cache.

    ``window`` is ``None`` for full causal attention, else the number of most
    recent positions (the query's own included) a query may see.  ``qk_norm`` is
    the per-head norm of queries and keys before rotation, or ``None``."""
    hidden: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    scale: float
    window: Optional[int] = None
    qk_norm: Optional[NormSpec] = None
    position: Optional[RopeSpec] = None
    kind: str = "attention"


@dataclass(frozen=True)
class GatedMlpSpec:
    """Dense gated feed-forward: ``down(act(gate(x)) * up(x))``."""
    hidden: int
    intermediate: int
    activation: str = "silu"
    kind: str = "gated_mlp"


@dataclass(frozen=True)
class TokenTableSpec:
    """The model's input: a row of a ``[vocab, hidden]`` table per token, times ``scale``."""
    vocab: int
    hidden: int
    scale: float = 1.0
    kind: str = "token_table"


@dataclass(frozen=True)
class NormLinearHeadSpec:
    """The model's output: a norm of the wanted rows of the residual stream, then their
    product with a ``[vocab, hidden]`` matrix; ``tied``: that matrix is the input's table."""
    vocab: int
    hidden: int
    norm: NormSpec
    tied: bool
    kind: str = "norm_linear"


@dataclass(frozen=True)
class BlockSpec:
    """One layer: a mixer and a feed-forward with their norms.

    ``arrangement`` names how they are wired; ``pre_norm`` is
    ``x += mixer(norm(x)); x += ffn(norm(x))``."""
    mixer: Any
    ffn: Any
    mixer_norm: NormSpec
    ffn_norm: NormSpec
    arrangement: str = "pre_norm"


@dataclass(frozen=True)
class ScheduleEntry:
    """One execution of a layer.  ``layer`` indexes ``ModelSpec.layers`` (a layer
    may appear in several entries and then runs its weights again with a cache
    line of its own).  ``reads_cache_of`` names an earlier entry of the schedule
    whose cache line this execution reads instead of writing its own."""
    layer: int
    reads_cache_of: Optional[int] = None


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    vocab: int
    hidden: int
    layers: Tuple[BlockSpec, ...]
    schedule: Tuple[ScheduleEntry, ...]
    final_norm: NormSpec
    tie_lm_head: bool
    max_positions: int
    embed_scale: float = 1.0
    eos_token_ids: Tuple[int, ...] = ()     # generation stops at any of these unless told otherwise
    # The parts at the model's two ends, chosen by ``kind`` like every other part.  None: the token
    # table and the norm-then-matrix head that the fields above describe.
    embedding: Any = None
    head: Any = None

    def embedding_spec(self) -> Any:
        return self.embedding if self.embedding is not None else \
            TokenTableSpec(self.vocab, self.hidden, self.embed_scale)

    def head_spec(self) -> Any:
        return self.head if self.head is not None else \
            NormLinearHeadSpec(self.vocab, self.hidden, self.final_norm, self.tie_lm_head)

    def validate(self) -> None:
        from ..errors import ConfigError
        if not self.layers:
            raise ConfigError("a model needs at least one layer")
        for i, entry in enumerate(self.schedule):
            if not 0 <= entry.layer < len(self.layers):
                raise ConfigError(f"schedule entry {i} names layer {entry.layer}, "
                                  f"the model has {len(self.layers)}")
            src = entry.reads_cache_of
            if src is not None:
                if not 0 <= src < i:
                    raise ConfigError(f"schedule entry {i} reads the cache of entry {src}, "
                                      "which does not run before it")
                if self.schedule[src].reads_cache_of is not None:
                    raise ConfigError(f"schedule entry {i} reads the cache of entry {src}, "
                                      "which has no cache line of its own")


def default_schedule(n_layers: int) -> Tuple[ScheduleEntry, ...]:
    """Every layer once, in order, each with its own cache line."""
    return tuple(ScheduleEntry(layer=i) for i in range(n_layers))
