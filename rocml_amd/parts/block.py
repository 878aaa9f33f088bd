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
from .residual import stream


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
        self.prompt_graph_safe = all(getattr(c, "prompt_graph_safe", False) for c in self.children.values())

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
    takes_next_norm = True    # forward() accepts the hint of the norm that reads the stream after it

    def entry_hint(self, step):
        """The norm this block reads the residual stream with first, for the product that completes
        the stream before it, if the block's mixer can apply the norm's scale itself in this step."""
        return self._hint(step, self.mixer_norm, self.mixer)

    def forward(self, step, x: torch.Tensor, cache, owns_cache: bool, next_norm=None) -> None:
        """``next_norm``: the hint of the norm that reads ``x`` after this block (``entry_hint`` of
        the block that runs next), or None."""
        ws = step.workspace
        rs = stream(step)
        xn, rs.row_scale = self._norm(step, self.mixer_norm, x)
        if not getattr(self.mixer, "adds_only", False):
            ws.flush_pending()
        rs.next_norm = self._hint(step, self.ffn_norm, self.ffn)
        self.mixer.forward(step, xn, x, cache, owns_cache)
        rs.next_norm = None
        xn, rs.row_scale = self._norm(step, self.ffn_norm, x)
        if not getattr(self.ffn, "adds_only", False):
            ws.flush_pending()
        rs.next_norm = next_norm
        self.ffn.forward(step, xn, x)
        rs.next_norm = None
        rs.row_scale = None

    @staticmethod
    def _hint(step, norm, consumer):
        takes = getattr(consumer, "takes_row_scale", None)
        hint = getattr(norm, "prescale_hint", None)
        if takes is None or hint is None or not takes(step):
            return None
        return hint()

    def _norm(self, step, norm, x):
        """The norm's output and what is left to apply to it (None: nothing).  A part may leave the
        last step of its residual sum (adding split-K partial sums to x) to the norm that reads x
        next, or have prepared the norm's output itself; a norm that can use neither gets x
        completed."""
        ws = step.workspace
        gain = getattr(norm, "gain", None)
        prepared = stream(step).take_prescaled(x, gain) if gain is not None else None
        if prepared is not None:
            return prepared
        xn = ws.get("block.xn", tuple(x.shape), self.dtype)
        if getattr(norm, "fuses_pending", False):
            norm.forward(x, xn, pending=ws.take_pending(x))
        else:
            ws.flush_pending()
            norm.forward(x, xn)
        return xn, None


register_block("pre_norm", PreNormBlock)
