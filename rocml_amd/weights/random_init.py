"""Random weights from a configuration and a seed, and the writer of a model folder.

The reference has no random weights; the rules are the benchmark configurations':
matrices and the embedding table N(0, 0.02), norm gains 1 or 1 + N(0, 0.02).  Every
tensor has a generator of its own, seeded by the seed and the tensor's name, so the
values do not depend on the order or on which other tensors exist.
"""
from __future__ import annotations

import hashlib
import json
import os
from typing import Dict, Iterator, Tuple

import torch

from ..parts.base import ParamSpec

STD = 0.02


def _tensor_seed(seed: int, name: str) -> int:
    digest = hashlib.sha256(f"{seed}:{name}".encode("utf-8")).digest()
    return int.from_bytes(digest[:8], "little")


# The draws are the same bits on the CPU and on the GPU: element i of a tensor is a function of
# (seed, tensor name, i) made of operations that every device computes exactly.  A counter-based
# generator (splitmix64: a 64-bit counter times the golden-ratio increment, then two rounds of
# xor-shift and multiply, all in wrapping 64-bit integers) gives 32 bits per element; the upper
# 16 pick a cell of the inverse normal distribution function, tabulated once on the CPU, the
# lower 16 a place inside the cell, by one multiplication and one addition in 64-bit floating
# point.  The distribution is the normal one with its density made piecewise constant on 65,536
# cells of equal probability and its tails cut near 5 standard deviations.
_CELLS = 1 << 16
_CHUNK = 1 << 26
_table_cache: Dict[str, torch.Tensor] = {}


def _signed(v: int) -> int:
    v &= (1 << 64) - 1
    return v - (1 << 64) if v >= (1 << 63) else v


def _lsr(x: torch.Tensor, n: int) -> torch.Tensor:
    return (x >> n) & ((1 << (64 - n)) - 1)


def _quantile_table(device) -> torch.Tensor:
    key = str(device)
    if key not in _table_cache:
        edges = torch.arange(_CELLS + 1, dtype=torch.float64) / _CELLS
        edges[0], edges[-1] = 1.0 / (_CELLS * 64), 1.0 - 1.0 / (_CELLS * 64)
        _table_cache[key] = torch.special.ndtri(edges).to(device)
    return _table_cache[key]


def standard_normal(n: int, stream: int, device="cpu") -> torch.Tensor:
    """``n`` draws of stream ``stream`` (any 64-bit integer) as 64-bit floats on ``device``."""
    table = _quantile_table(device)
    out = torch.empty(n, dtype=torch.float64, device=device)
    for start in range(0, n, _CHUNK):
        stop = min(n, start + _CHUNK)
        z = torch.arange(start + 1, stop + 1, dtype=torch.int64, device=device)
        z = z * _signed(0x9E3779B97F4A7C15) + _signed(stream)
        z = (z ^ _lsr(z, 30)) * _signed(0xBF58476D1CE4E5B9)
        z = (z ^ _lsr(z, 27)) * _signed(0x94D049BB133111EB)
        z = z ^ _lsr(z, 31)
        cell = _lsr(z, 48)
        inside = (_lsr(z, 32) & (_CELLS - 1)).to(torch.float64)
        inside = (inside + 0.5) * (1.0 / _CELLS)
        low = table[cell]
        width = table[cell + 1] - low
        out[start:stop] = low + width * inside
    return out


def random_tensor(name: str, spec: ParamSpec, seed: int, dtype: torch.dtype, norm_jitter: bool,
                  device="cpu") -> torch.Tensor:
    """The tensor called ``name`` for ``seed``: drawn on ``device``, the same values on any device,
    rounded once to ``dtype``."""
    n = 1
    for d in spec.shape:
        n *= d

    def normal() -> torch.Tensor:
        return (standard_normal(n, _tensor_seed(seed, name), device) * STD).to(torch.float32).view(spec.shape)

    if spec.init == "normal":
        t = normal()
    elif spec.init == "gain":
        t = torch.ones(spec.shape, dtype=torch.float32, device=device)
        if norm_jitter:
            t += normal()
    elif spec.init == "zeros":
        t = torch.zeros(spec.shape, dtype=torch.float32, device=device)
    else:
        raise ValueError(f"unknown init rule {spec.init!r}")
    if spec.role == "int_table":
        return t.to(torch.int32)
    return t.to(dtype)


def random_tensors(param_specs: Dict[str, ParamSpec], names: Dict[str, str], seed: int,
                   dtype: torch.dtype, norm_jitter: bool, device="cpu") -> Iterator[Tuple[str, torch.Tensor]]:
    """Yields ``(checkpoint name, tensor)``; the seed is tied to the checkpoint name."""
    for internal, spec in param_specs.items():
        ckpt = names[internal]
        yield ckpt, random_tensor(ckpt, spec, seed, dtype, norm_jitter, device)


def write_model_dir(path: str, config: Dict, seed: int, dtype: torch.dtype = torch.bfloat16,
                    norm_jitter: bool = True, device="cpu") -> str:
    """Writes ``config.json`` and ``model.safetensors`` for ``config`` (config.json's
    dictionary) with random weights; returns ``path``.  ``device`` is where the values are
    drawn (they are the same anywhere; a GPU draws a large model in seconds)."""
    from safetensors.torch import save_file
    from ..config import architecture_of
    from ..engine.model import DecoderModel
    arch = architecture_of(config)
    cfg = arch.read_config(config)
    spec = arch.to_spec(cfg)
    model = DecoderModel(spec, torch.float32, device="meta")
    names = arch.checkpoint_names(spec)
    tensors = {name: t.cpu() for name, t in random_tensors(model.param_specs(), names, seed, dtype, norm_jitter, device)}
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w", encoding="utf-8") as f:
        json.dump(cfg.to_dict() if hasattr(cfg, "to_dict") else config, f, indent=2)
    save_file(tensors, os.path.join(path, "model.safetensors"), metadata={"format": "pt"})
    return path
