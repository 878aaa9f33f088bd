"""The model's input: one row of the embedding table per token, in 32-bit
(rocml-kernels/kernels/embedding.hip:10-27; rocml/src/forward/chunk_forward.rs:96-103)."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import ops
from ..config.spec import TokenTableSpec
from .base import BuildContext, Embedding, ParamSpec
from .registry import register_embedding


class TokenTable(Embedding):
    prompt_graph_safe = True

    def __init__(self, spec: TokenTableSpec, ctx: BuildContext):
        self.vocab = spec.vocab
        self.hidden = spec.hidden
        self.scale = float(spec.scale)
        self.table: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {"weight": ParamSpec((self.vocab, self.hidden))}

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.table = tensors["weight"]

    def shared_matrix(self) -> Optional[torch.Tensor]:
        return self.table

    def forward(self, step, x: torch.Tensor) -> None:
        ops.embed_gather(self.table, step.token_ids, x, self.scale)


register_embedding("token_table", TokenTable)
