"""The model's output: the norm of the rows whose logits are wanted, then their product with
the output matrix (rocml/src/forward/chunk_forward.rs:170-184 does both for the last row only).
A tied output matrix is the embedding's table itself, one buffer
(rocml/src/weights/mod.rs:48-62 loads it twice)."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import ops
from ..config.spec import NormLinearHeadSpec
from ..errors import ConfigError
from .base import BuildContext, Head, ParamSpec
from .registry import build_norm, register_head


class NormLinearHead(Head):
    takes_pending = True

    def __init__(self, spec: NormLinearHeadSpec, ctx: BuildContext):
        self.vocab = spec.vocab
        self.hidden = spec.hidden
        self.tied = bool(spec.tied)
        self.dtype = ctx.dtype
        self.norm = build_norm(spec.norm, ctx)
        self.matrix: Optional[torch.Tensor] = None
        self.graph_safe = getattr(self.norm, "graph_safe", True)
        self.prompt_graph_safe = getattr(self.norm, "prompt_graph_safe", False)

    def param_specs(self) -> Dict[str, ParamSpec]:
        specs = {f"final_norm.{name}": p for name, p in self.norm.param_specs().items()}
        if not self.tied:
            specs["lm_head.weight"] = ParamSpec((self.vocab, self.hidden))
        return specs

    def bind(self, tensors: Dict[str, torch.Tensor], shared: Optional[torch.Tensor] = None) -> None:
        prefix = "final_norm."
        self.norm.bind({k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)})
        if self.tied:
            if shared is None or tuple(shared.shape) != (self.vocab, self.hidden):
                raise ConfigError("a tied output matrix needs an embedding with a [vocab, hidden] table")
            self.matrix = shared
        else:
            self.matrix = tensors["lm_head.weight"]

    def step_matrix_elements(self) -> int:
        return self.vocab * self.hidden

    def activation_bytes(self, n_wanted: int) -> int:
        size = 2 if self.dtype == torch.bfloat16 else 4
        return n_wanted * (self.hidden * size + self.vocab * 4)

    def forward(self, step, x: torch.Tensor, want_rows: torch.Tensor, n_want: int) -> torch.Tensor:
        ws = step.workspace
        xn = ws.get("head.xn", (n_want, self.hidden), self.dtype)
        if getattr(self.norm, "fuses_pending", False):
            self.norm.forward(x, xn, rows=want_rows, pending=ws.take_pending(x))
        else:
            ws.flush_pending()
            self.norm.forward(x, xn, rows=want_rows)
        logits = ws.get("head.logits", (n_want, self.vocab), torch.float32)
        ops.gemm(xn, self.matrix, logits, workspace=ws.scratch())
        return logits


register_head("norm_linear", NormLinearHead)
