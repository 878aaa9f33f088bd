"""Dense gated feed-forward: ``y = down(act(gate(x)) * up(x))`` with no bias
(rocml/src/forward/ffn.rs:36-107, rocml-kernels/kernels/silu_mul.hip:12-20).  Gate and up
are one product over the concatenated weight; the residual sum is the down product's
epilogue."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import ops
from ..config.spec import GatedMlpSpec
from ..errors import ConfigError
from .base import BuildContext, FeedForward, ParamSpec
from .registry import register_feed_forward
from .residual import stream


class GatedMlp(FeedForward):
    adds_only = True
    prompt_graph_safe = True

    def __init__(self, spec: GatedMlpSpec, ctx: BuildContext):
        if spec.activation != "silu":
            raise ConfigError(f"activation {spec.activation!r} is not supported (silu only)")
        self.spec = spec
        self.dtype = ctx.dtype
        self.w_gate_up: Optional[torch.Tensor] = None
        self.w_down: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        s = self.spec
        return {"gate_proj.weight": ParamSpec((s.intermediate, s.hidden)),
                "up_proj.weight": ParamSpec((s.intermediate, s.hidden)),
                "down_proj.weight": ParamSpec((s.hidden, s.intermediate))}

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        # Rows in (gate_j, up_j) pairs: the product's epilogue then has both halves of an
        # output in one lane and applies the activation to its 32-bit sums.
        gate, up = tensors["gate_proj.weight"], tensors["up_proj.weight"]
        self.w_gate_up = torch.stack([gate, up], dim=1).reshape(2 * gate.shape[0], gate.shape[1]).contiguous()
        self.w_down = tensors["down_proj.weight"]
        self.fused = self.dtype == torch.bfloat16 and self.spec.hidden % 8 == 0

    def activation_bytes(self, n_tokens: int) -> int:
        s = self.spec
        size = 2 if self.dtype == torch.bfloat16 else 4
        fused = self.dtype == torch.bfloat16 and s.hidden % 8 == 0
        return n_tokens * s.intermediate * (size + (0 if fused else 8))

    def takes_row_scale(self, step) -> bool:
        # the gated epilogue of the few-rows products applies it
        return self.w_gate_up is not None and self.fused and step.n_tokens <= ops.ROW_SCALE_MAX_ROWS

    def forward(self, step, xn, x_accum) -> None:
        s = self.spec
        n = step.n_tokens
        ws = step.workspace
        h = ws.get("mlp.h", (n, s.intermediate), self.dtype)
        if self.fused:
            ops.gemm(xn, self.w_gate_up, h, workspace=ws.scratch(), epilogue="swiglu", row_scale=stream(step).row_scale)
        else:
            if stream(step).row_scale is not None:
                raise ConfigError("the feed-forward was handed an input without its norm's scale in a step it cannot scale")
            gate_up = ws.get("mlp.gate_up", (n, 2 * s.intermediate), torch.float32)
            ops.gemm(xn, self.w_gate_up, gate_up, workspace=ws.scratch())
            ops.swiglu(gate_up, h, interleaved=True)
        stream(step).add_product(h, self.w_down, x_accum)


register_feed_forward("gated_mlp", GatedMlp)
