"""Rotary position encoding with NEOX pairing (rocml-kernels/kernels/rope.hip:18-33):
``f_i = theta^(-2i/rot_dim)``, angle ``pos * f_i``, pair ``(i, i + rot_dim/2)``.  The part
owns the frequencies and prepares one cos/sin table per step from the step's token
positions; every mixer with the same spec shares it."""
from __future__ import annotations

import torch

from .. import ops
from ..config.spec import RopeSpec
from ..errors import ConfigError
from .base import BuildContext, PositionEncoding
from .registry import register_position


class RopeNeox(PositionEncoding):
    prompt_graph_safe = True

    def __init__(self, spec: RopeSpec, ctx: BuildContext):
        if spec.rot_dim % 2 != 0 or not 0 < spec.rot_dim <= spec.head_dim:
            raise ConfigError(f"rotary width {spec.rot_dim} must be even and at most the head size {spec.head_dim}")
        self.spec = spec
        self.rot_dim = spec.rot_dim
        half = spec.rot_dim // 2
        inv = [float(spec.theta) ** (-2.0 * i / spec.rot_dim) for i in range(half)]
        self.inv_freq = torch.tensor(inv, dtype=torch.float64, device=ctx.device)

    def tables(self, step):
        key = ("rope", self.spec)
        hit = step.memo.get(key)
        if hit is None:
            half = self.rot_dim // 2
            cos = step.workspace.get(f"rope.cos.{id(self)}", (step.n_tokens, half), torch.float32)
            sin = step.workspace.get(f"rope.sin.{id(self)}", (step.n_tokens, half), torch.float32)
            ops.rope_table(step.token_pos, self.inv_freq, cos, sin)
            hit = (cos, sin)
            step.memo[key] = hit
        return hit


register_position("rope_neox", RopeNeox)
