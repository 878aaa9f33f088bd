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
    return int.from_bytes(digest[:8], "little") & ((1 << 63) - 1)


def random_tensor(name: str, spec: ParamSpec, seed: int, dtype: torch.dtype, norm_jitter: bool,
                  device="cpu") -> torch.Tensor:
    """The tensor called ``name`` for ``seed``: drawn in 32-bit on ``device``, then cast.
    The CPU and the GPU draw different values for the same seed; files are written on the CPU."""
    gen = torch.Generator(device=device)
    gen.manual_seed(_tensor_seed(seed, name))
    if spec.init == "normal":
        t = torch.empty(spec.shape, dtype=torch.float32, device=device).normal_(0.0, STD, generator=gen)
    elif spec.init == "gain":
        t = torch.ones(spec.shape, dtype=torch.float32, device=device)
        if norm_jitter:
            t += torch.empty(spec.shape, dtype=torch.float32, device=device).normal_(0.0, STD, generator=gen)
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
                    norm_jitter: bool = True) -> str:
    """Writes ``config.json`` and ``model.safetensors`` for ``config`` (config.json's
    dictionary) with random weights; returns ``path``."""
    from safetensors.torch import save_file
    from ..config import architecture_of
    from ..engine.model import DecoderModel
    arch = architecture_of(config)
    cfg = arch.read_config(config)
    spec = arch.to_spec(cfg)
    model = DecoderModel(spec, torch.float32, device="meta")
    names = arch.checkpoint_names(spec)
    tensors = dict(random_tensors(model.param_specs(), names, seed, dtype, norm_jitter))
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w", encoding="utf-8") as f:
        json.dump(cfg.to_dict() if hasattr(cfg, "to_dict") else config, f, indent=2)
    save_file(tensors, os.path.join(path, "model.safetensors"), metadata={"format": "pt"})
    return path
