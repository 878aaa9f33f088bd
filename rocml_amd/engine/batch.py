"""What one step of the engine works on: the tokens of a batch, packed.

The reference's two entry points take one sequence and an implicit position
(rocml/src/forward/chunk_forward.rs:62, rocml/src/forward/mod.rs:236).  A step here
takes several sequences with unequal numbers of new tokens; they are packed one after
another, and every token carries its sequence and its absolute position, so rotation,
cache append and the causal bound need nothing else.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Optional, Sequence

import numpy as np
import torch

from .workspace import Workspace


@dataclass
class StepEntry:
    """New tokens of one sequence and the places among them whose logits are wanted."""
    slot: int
    tokens: Sequence[int]
    want: Sequence[int] = ()


@dataclass
class StepContext:
    n_tokens: int
    n_seqs: int
    token_ids: torch.Tensor      # [T] int32
    token_seq: torch.Tensor      # [T] int32: index of the token's sequence in this step
    token_pos: torch.Tensor      # [T] int32: absolute position
    cu_seqlens: torch.Tensor     # [B + 1] int32: where each sequence's tokens start
    seq_lens: torch.Tensor       # [B] int32: sequence length after this step
    seq_slots: torch.Tensor      # [B] int32: cache slot of each sequence
    max_new: int                 # most new tokens of any sequence
    max_len: int                 # longest sequence after this step
    new_counts: Sequence[int]    # new tokens of each sequence (host)
    workspace: Workspace
    memo: Dict = field(default_factory=dict)
    block_tables: Dict = field(default_factory=dict)   # cache group name -> [B, width] int32
    want_rows: Optional[torch.Tensor] = None           # token rows whose logits are wanted

    @property
    def is_decode(self) -> bool:
        return self.max_new == 1


def pack_step(slots: Sequence[int], starts: Sequence[int], tokens: Sequence[Sequence[int]]):
    """Host arrays of a packed step: ids, sequence index and position per token, offsets,
    final lengths."""
    counts = np.asarray([len(t) for t in tokens], dtype=np.int32)
    total = int(counts.sum())
    cu = np.zeros(len(tokens) + 1, dtype=np.int32)
    np.cumsum(counts, out=cu[1:])
    ids = np.fromiter((t for toks in tokens for t in toks), dtype=np.int32, count=total)
    seq = np.repeat(np.arange(len(tokens), dtype=np.int32), counts)
    first = np.asarray(starts, dtype=np.int32)
    # position of a token = its sequence's start + its place among the sequence's new tokens
    pos = np.arange(total, dtype=np.int32) - np.repeat(cu[:-1], counts) + np.repeat(first, counts)
    lens = first + counts
    return ids, seq, pos, cu, lens, np.asarray(slots, dtype=np.int32)
