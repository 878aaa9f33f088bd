"""Arrangement of a mixer and a feed-forward into one layer.

``pre_norm`` is the reference's wiring (rocml/src/forward/chunk_forward.rs:107-135):
``x += mixer(norm(x))``, then ``x += ffn(norm(x))``; the residual stream ``x`` stays
32-bit and the normalised copy has the activation type."""
from __future__ import annotations

from typing import Dict

import torch

from ..config.spec import BlockSpec
from .base import BuildContext, ParamSpec, Part
from .registry import build_feed_forward, build_mixer, build_norm, register_block


class PreNormBlock(Part):
    def __init__(self, spec: BlockSpec, ctx: BuildContext):
        self.dtype = ctx.dtype
        self.hidden = spec.mixer_norm.size
        self.children = {"mixer_norm": build_norm(spec.mixer_norm, ctx),
                         "mixer": build_mixer(spec.mixer, ctx),
                         "ffn_norm": build_norm(spec.ffn_norm, ctx),
                         "ffn": build_feed_forward(spec.ffn, ctx)}
        self.mixer_norm = self.children["mixer_norm"]
        self.mixer = self.children["mixer"]
        self.ffn_norm = self.children["ffn_norm"]
        self.ffn = self.children["ffn"]
        self.graph_safe = all(getattr(c, "graph_safe", True) for c in self.children.values())

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {f"{name}.{p}": spec for name, child in self.children.items()
                for p, spec in child.param_specs().items()}

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        for name, child in self.children.items():
            prefix = name + "."
            child.bind({k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)})

    def cache_request(self):
        return self.mixer.cache_request()

    def flops(self, new_counts, starts) -> int:
        return self.mixer.flops(new_counts, starts) + self.ffn.flops(new_counts, starts)

    def activation_bytes(self, n_tokens: int) -> int:
        size = 2 if self.dtype == torch.bfloat16 else 4
        return n_tokens * self.hidden * size + self.mixer.activation_bytes(n_tokens) + self.ffn.activation_bytes(n_tokens)

    takes_pending = True      # forward() may be handed a stream that still lacks deferred sums

    def forward(self, step, x: torch.Tensor, cache, owns_cache: bool) -> None:
        ws = step.workspace
        xn = ws.get("block.xn", tuple(x.shape), self.dtype)
        self._norm(step, self.mixer_norm, x, xn)
        if not getattr(self.mixer, "adds_only", False):
            ws.flush_pending()
        self.mixer.forward(step, xn, x, cache, owns_cache)
        self._norm(step, self.ffn_norm, x, xn)
        if not getattr(self.ffn, "adds_only", False):
            ws.flush_pending()
        self.ffn.forward(step, xn, x)

    @staticmethod
    def _norm(step, norm, x, xn) -> None:
        """A part may leave the last step of its residual sum (adding split-K partial sums
        to x) to the norm that reads x next; a norm that cannot do that gets x completed."""
        ws = step.workspace
        if getattr(norm, "fuses_pending", False):
            norm.forward(x, xn, pending=ws.take_pending(x))
        else:
            ws.flush_pending()
            norm.forward(x, xn)


register_block("pre_norm", PreNormBlock)
