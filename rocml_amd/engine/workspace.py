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
    def __init__(self, device, scratch_bytes: int = 64 << 20):
        self.device = device
        self._buffers: Dict[str, torch.Tensor] = {}
        self.generation = 0
        self._scratch_bytes = scratch_bytes
        self._scratch = None

    def get(self, name: str, shape: Tuple[int, ...], dtype: torch.dtype) -> torch.Tensor:
        n = math.prod(shape)
        key = f"{name}/{dtype}"
        buf = self._buffers.get(key)
        if buf is None or buf.numel() < n:
            buf = torch.empty(max(n, 1), dtype=dtype, device=self.device)
            self._buffers[key] = buf
            self.generation += 1
        return buf[:n].view(shape)

    def scratch(self) -> torch.Tensor:
        """Device memory kernels may use for partial results of one launch."""
        if self._scratch is None:
            self._scratch = torch.empty(self._scratch_bytes, dtype=torch.uint8, device=self.device)
            self.generation += 1
        return self._scratch

    def bytes(self) -> int:
        total = sum(b.numel() * b.element_size() for b in self._buffers.values())
        return total + (0 if self._scratch is None else self._scratch.numel())
