"""Named activation buffers that live across steps.

The reference preallocates one set of activation buffers for a token and one for a
chunk of up to 512 tokens (rocml/src/forward/scratch.rs:11-69,
rocml/src/forward/chunk_scratch.rs:29-110).  Here a buffer is asked for by name and
shape; it is allocated at the largest size seen and handed out as a view, so a step
allocates nothing once sizes have settled and addresses stay fixed for graph replay.
``generation`` counts reallocations: a recorded graph is valid only for the
generation it was recorded in.
"""
from __future__ import annotations

import math
from typing import Dict, Tuple

import torch


class Workspace:
    SCRATCH_BYTES = 128 << 20

    def __init__(self, device, scratch_bytes: int = SCRATCH_BYTES):
        self.device = device
        self._buffers: Dict[str, torch.Tensor] = {}
        self._views: Dict[tuple, torch.Tensor] = {}     # (name, type, shape) -> the view handed out last time
        self.generation = 0
        self._scratch_bytes = scratch_bytes
        self._scratch = None
        self._pending = None

    def get(self, name: str, shape: Tuple[int, ...], dtype: torch.dtype) -> torch.Tensor:
        # (a step asks for the same few views over and over; building one costs as much as a launch)
        view = self._views.get((name, dtype, shape))
        if view is not None:
            return view
        n = math.prod(shape)
        key = f"{name}/{dtype}"
        buf = self._buffers.get(key)
        if buf is None or buf.numel() < n:
            buf = torch.empty(max(n, 1), dtype=dtype, device=self.device)
            self._buffers[key] = buf
            self.generation += 1
            self._views = {k: v for k, v in self._views.items() if (k[0], k[1]) != (name, dtype)}
        view = buf[:n].view(shape)
        if len(self._views) < 4096:
            self._views[(name, dtype, shape)] = view
        return view

    def scratch(self) -> torch.Tensor:
        """Device memory kernels may use for partial results of one launch.  Partial sums
        that a deferred product left there are added to their target first."""
        if self._scratch is None:
            self._scratch = torch.empty(self._scratch_bytes, dtype=torch.uint8, device=self.device)
            self.generation += 1
        self.flush_pending()
        return self._scratch

    # -- deferred split-K sums --------------------------------------------------------------
    # A product that was split along K and whose result is to be added to a tensor may leave
    # its partial sums in the scratch memory; the next kernel that reads the tensor (a norm)
    # adds them itself.  Whoever needs the scratch memory or the tensor before that calls
    # flush_pending, which runs the addition as a kernel of its own.
    def set_pending(self, target: torch.Tensor, n_splits: int) -> None:
        self.flush_pending()
        self._pending = (target, n_splits)

    def _partials(self) -> torch.Tensor:
        target, n_splits = self._pending
        n = n_splits * target.numel()
        return self._scratch[:n * 4].view(torch.float32).view(n_splits, target.shape[0], target.shape[1])

    def take_pending(self, target: torch.Tensor):
        """The partial sums waiting for ``target`` (``[splits, rows, n]``), which the caller
        now adds itself; None if there are none."""
        if self._pending is None:
            return None
        if self._pending[0].data_ptr() != target.data_ptr():
            self.flush_pending()
            return None
        partials = self._partials()
        self._pending = None
        return partials

    def flush_pending(self) -> None:
        if self._pending is not None:
            from .. import ops
            partials = self._partials()
            target = self._pending[0]
            self._pending = None
            ops.splitk_reduce(partials, target, accumulate=True)

    def drop_pending(self) -> None:
        self._pending = None

    def bytes(self) -> int:
        total = sum(b.numel() * b.element_size() for b in self._buffers.values())
        return total + (0 if self._scratch is None else self._scratch.numel())
