"""How parts add to the 32-bit residual stream, and what a norm finds prepared for it.

The residual sum is the epilogue of a part's last product (the reference adds in a kernel of
its own, rocml/src/forward/ffn.rs:88-107, attention.rs:237-244).  Two things can ride on that
product, both knowledge of the parts and none of the engine's:

* the product may be cut along K and its partial sums left for the next norm to add (the
  workspace's deferred sums);
* when the block has said which norm reads the stream next (``next_norm``) and the consumer of
  that norm's output can apply a row scale itself, the product is completed by one kernel that
  also writes ``bfloat16(x * gain)`` and the sums of squares of ``x``; the norm kernel then
  disappears and the consumer finds ``row_scale`` set.

One ``ResidualStream`` lives as long as a step (in ``step.memo``); blocks and parts reach it
with ``stream(step)``.
"""
from __future__ import annotations

from typing import Optional

import torch

from .. import ops
from .base import NormHint

_KEY = "residual_stream"


class ResidualStream:
    def __init__(self, workspace):
        self.workspace = workspace
        # the norm that will read the stream next, if its consumer can apply the norm's scale itself
        # (set by the block around a part's forward)
        self.next_norm: Optional[NormHint] = None
        # set around a part's forward: its input lacks this scale (an ``ops.RowScale``)
        self.row_scale = None
        self._prescaled = None

    def add_product(self, a: torch.Tensor, w: torch.Tensor, target: torch.Tensor) -> None:
        """``target += a @ w.T``.  The product may leave partial sums to the next norm
        (``workspace.take_pending``), or have prepared that norm (``take_prescaled``)."""
        ws = self.workspace
        hint = self.next_norm
        self._prescaled = None
        if hint is not None and target.dtype == torch.float32 and hint.width == target.shape[1] \
                and ops.gemm_residual_prescale_pays(a, w):
            ws.flush_pending()
            rows = target.shape[0]
            xg = ws.get("residual.prepared", tuple(target.shape), torch.bfloat16)
            parts = (target.shape[1] + ops.PRESCALE_TILE - 1) // ops.PRESCALE_TILE
            ssq = ws.get("residual.ssq", (rows, parts), torch.float32)
            ops.gemm_residual_prescale(a, w, target, hint.gain, xg, ssq)
            self._prescaled = (target.data_ptr(), hint.gain.data_ptr(), xg, ops.RowScale(ssq, hint.eps, hint.width))
            return
        splits = ops.gemm(a, w, target, accumulate=True, workspace=ws.scratch(), defer=True)
        if splits:
            ws.set_pending(target, splits)

    def take_prescaled(self, target: torch.Tensor, gain: torch.Tensor):
        """``(operand, row scale)`` if the last ``add_product`` into ``target`` prepared the norm
        with this ``gain``; None otherwise (``target`` is complete then, or has pending sums)."""
        hit, self._prescaled = self._prescaled, None
        if hit is None or hit[0] != target.data_ptr() or hit[1] != gain.data_ptr():
            return None
        return hit[2], hit[3]


def stream(step) -> ResidualStream:
    """The step's residual stream helper (made on first use)."""
    found = step.memo.get(_KEY)
    if found is None:
        found = step.memo[_KEY] = ResidualStream(step.workspace)
    return found
