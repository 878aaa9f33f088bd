"""Root-mean-square norm: ``y = x / sqrt(mean(x^2) + eps) * gain`` in 32-bit
(rocml-kernels/kernels/rmsnorm.hip:18-42); reads the 32-bit residual stream and writes
the activation type."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import ops
from ..config.spec import NormSpec
from .base import BuildContext, Norm, NormHint, ParamSpec
from .registry import register_norm


class RMSNorm(Norm):
    prompt_graph_safe = True

    def __init__(self, spec: NormSpec, ctx: BuildContext):
        self.size = spec.size
        self.eps = float(spec.eps)
        self.gain: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {"weight": ParamSpec((self.size,), role="gain", init="gain")}

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.gain = tensors["weight"]

    fuses_pending = True      # forward() can add a deferred product's partial sums to x itself

    def prescale_hint(self) -> Optional[NormHint]:
        return None if self.gain is None else NormHint(self.gain, self.eps, self.size)

    def forward(self, x: torch.Tensor, out: torch.Tensor, rows: Optional[torch.Tensor] = None,
                pending: Optional[torch.Tensor] = None) -> None:
        ops.rmsnorm(x, self.gain, self.eps, out, rows, partials=pending)


register_norm("rmsnorm", RMSNorm)
