"""Loads a model folder: config.json picks the architecture, tensors come from
safetensors by name.

The reference reads each tensor by name, checks rank and shape, and fails on the first
problem (rocml/src/weights/mod.rs:36-76,82-120; rocml/src/weights/layer.rs:39-63).  Here
all names and shapes are checked before anything is read, and one error lists every
missing tensor, every tensor the model does not use and every wrong shape.  Types:
operands of matrix products are held in the compute type (bfloat16 or float32), gain
vectors in 32-bit, integer tables as int32; a file tensor that is 32-bit already is not
rounded when the compute type is float32, and bfloat16 widens to float32 exactly.
"""
from __future__ import annotations

import json
import os
from typing import Dict, List, Optional

import torch

from ..config import architecture_of, read_config_json
from ..engine.model import DecoderModel, compute_dtype
from ..errors import WeightsError
from ..parts.base import ParamSpec

_FLOAT_FILE_TYPES = ("F64", "F32", "F16", "BF16")
_INT_FILE_TYPES = ("I64", "I32", "I16", "I8", "U8")


def _shard_files(path: str) -> List[str]:
    single = os.path.join(path, "model.safetensors")
    index = os.path.join(path, "model.safetensors.index.json")
    if os.path.isfile(single):
        return [single]
    if os.path.isfile(index):
        with open(index, "r", encoding="utf-8") as f:
            files = sorted(set(json.load(f)["weight_map"].values()))
        missing = [n for n in files if not os.path.isfile(os.path.join(path, n))]
        if missing:
            raise WeightsError(f"{path}: the index names files that are not there: {', '.join(missing)}")
        return [os.path.join(path, n) for n in files]
    raise WeightsError(f"{path}: neither model.safetensors nor model.safetensors.index.json exists")


def check_tensors(expected: Dict[str, ParamSpec], names: Dict[str, str],
                  found: Dict[str, tuple]) -> None:
    """``found`` maps checkpoint names to ``(shape, file dtype)``.  Raises one
    ``WeightsError`` listing everything that does not fit."""
    problems: List[str] = []
    wanted = {names[k]: (k, spec) for k, spec in expected.items()}
    missing = sorted(n for n in wanted if n not in found)
    unexpected = sorted(n for n in found if n not in wanted)
    if missing:
        problems.append("missing tensors: " + ", ".join(missing))
    if unexpected:
        problems.append("unexpected tensors: " + ", ".join(unexpected))
    for ckpt, (internal, spec) in sorted(wanted.items()):
        if ckpt not in found:
            continue
        shape, ftype = found[ckpt]
        if tuple(shape) != tuple(spec.shape):
            problems.append(f"wrong shape: {ckpt} is {list(shape)}, the model needs {list(spec.shape)}")
        allowed = _INT_FILE_TYPES if spec.role == "int_table" else _FLOAT_FILE_TYPES
        if ftype not in allowed:
            problems.append(f"wrong type: {ckpt} is stored as {ftype}, expected one of {', '.join(allowed)}")
    if problems:
        raise WeightsError("the checkpoint does not fit the model:\n  " + "\n  ".join(problems))


def load_model(path: str, dtype="bfloat16", device="cuda") -> DecoderModel:
    """Builds the model that ``path/config.json`` names and binds the folder's weights."""
    from safetensors import safe_open
    raw = read_config_json(path)
    arch = architecture_of(raw)
    cfg = arch.read_config(raw)
    spec = arch.to_spec(cfg)
    model = DecoderModel(spec, compute_dtype(dtype), device=device)
    model.config = cfg
    expected = model.param_specs()
    names = arch.checkpoint_names(spec)
    files = _shard_files(path)
    where: Dict[str, str] = {}
    found: Dict[str, tuple] = {}
    for file in files:
        with safe_open(file, framework="pt", device="cpu") as f:
            for name in f.keys():
                sl = f.get_slice(name)
                found[name] = (tuple(sl.get_shape()), sl.get_dtype())
                where[name] = file
    check_tensors(expected, names, found)
    tensors: Dict[str, torch.Tensor] = {}
    by_file: Dict[str, List[str]] = {}
    for internal in expected:
        by_file.setdefault(where[names[internal]], []).append(internal)
    for file, internals in by_file.items():
        with safe_open(file, framework="pt", device="cpu") as f:
            for internal in internals:
                t = f.get_tensor(names[internal])
                tensors[internal] = t.to(device=model.device, dtype=model.storage_dtype(expected[internal])).contiguous()
    model.bind(tensors)
    return model


def random_model(config: Dict, seed: int, dtype="bfloat16", device="cuda", norm_jitter: bool = False,
                 n_layers: Optional[int] = None) -> DecoderModel:
    """A model with random weights drawn on the device, without a file; the values are the ones
    ``write_model_dir`` writes for the same configuration and seed."""
    from .random_init import random_tensor
    if n_layers is not None:
        config = dict(config, num_hidden_layers=n_layers)
    arch = architecture_of(config)
    cfg = arch.read_config(config)
    spec = arch.to_spec(cfg)
    model = DecoderModel(spec, compute_dtype(dtype), device=device)
    model.config = cfg
    names = arch.checkpoint_names(spec)
    tensors = {}
    for internal, p in model.param_specs().items():
        tensors[internal] = random_tensor(names[internal], p, seed, model.storage_dtype(p), norm_jitter,
                                          device=model.device)
    model.bind(tensors)
    return model
