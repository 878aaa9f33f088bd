"""Catalog of named models and the rule that tells a name from a folder.

The reference keeps a compiled-in table of checkpoints with a default context
and a sampling preset each (rocml/src/registry/catalog.rs:25-37,216-258) and
resolves ``--model`` as a path if it looks like one, else as a catalog name,
listing all names when it is unknown (rocml/src/registry/mod.rs:42-84,123-127).
Here an entry carries the whole configuration, so a model with random weights
needs no file.  Sizes of the 8B, 14B and 32B entries are the ones the
benchmark configurations name; the two tiny entries are the test models.  The
reference's other dense names (0.6B, 1.7B, 4B; rocml/src/registry/catalog.rs:216-248)
come without sizes in its files, which read them from each checkpoint: the sizes
here are the ones published with those checkpoints and nothing in the reference
pins them.
"""
from __future__ import annotations

import os
from dataclasses import dataclass
from typing import Dict, List, Optional

from ..errors import UnknownModelError
from ..sampling.params import SamplingParams

# Sampling preset the reference attaches to every dense Qwen3 entry
# (rocml/src/registry/catalog.rs:44-51).
QWEN_THINKING_SAMPLING = SamplingParams(temperature=0.6, top_k=20, top_p=0.95)

DEFAULT_CTX = 4096


@dataclass(frozen=True)
class ModelEntry:
    name: str
    config: Dict
    default_ctx: int = DEFAULT_CTX
    sampling: Optional[SamplingParams] = None
    init_norm_jitter: bool = False   # norm gains 1 + N(0, 0.02) instead of 1


def _qwen3(vocab, hidden, inter, layers, heads, kv_heads, head_dim, theta, eps, tied, max_pos):
    return {"architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "vocab_size": vocab,
            "hidden_size": hidden, "intermediate_size": inter, "num_hidden_layers": layers,
            "num_attention_heads": heads, "num_key_value_heads": kv_heads, "head_dim": head_dim,
            "rope_theta": theta, "rms_norm_eps": eps, "tie_word_embeddings": tied,
            "max_position_embeddings": max_pos, "hidden_act": "silu", "attention_bias": False}


CATALOG: List[ModelEntry] = [
    ModelEntry("tiny-a", _qwen3(256, 64, 128, 2, 4, 2, 16, 10000.0, 1e-6, True, 128),
               default_ctx=128, init_norm_jitter=True),
    ModelEntry("tiny-b", _qwen3(384, 96, 224, 3, 6, 2, 32, 1000000.0, 1e-5, False, 512),
               default_ctx=512, init_norm_jitter=True),
    ModelEntry("qwen3-0.6b", _qwen3(151936, 1024, 3072, 28, 16, 8, 128, 1000000.0, 1e-6, True, 40960),
               sampling=QWEN_THINKING_SAMPLING),
    ModelEntry("qwen3-1.7b", _qwen3(151936, 2048, 6144, 28, 16, 8, 128, 1000000.0, 1e-6, True, 40960),
               sampling=QWEN_THINKING_SAMPLING),
    ModelEntry("qwen3-4b", _qwen3(151936, 2560, 9728, 36, 32, 8, 128, 1000000.0, 1e-6, True, 40960),
               sampling=QWEN_THINKING_SAMPLING),
    ModelEntry("qwen3-8b", _qwen3(151936, 4096, 12288, 36, 32, 8, 128, 1000000.0, 1e-6, False, 40960),
               sampling=QWEN_THINKING_SAMPLING),
    ModelEntry("qwen3-14b", _qwen3(151936, 5120, 17408, 40, 40, 8, 128, 1000000.0, 1e-6, False, 40960),
               sampling=QWEN_THINKING_SAMPLING),
    ModelEntry("qwen3-32b", _qwen3(151936, 5120, 25600, 64, 64, 8, 128, 1000000.0, 1e-6, False, 40960),
               sampling=QWEN_THINKING_SAMPLING),
]

_BY_NAME = {e.name: e for e in CATALOG}


def register_model(entry: ModelEntry) -> None:
    """Adds a named configuration (of any registered architecture) to the catalog."""
    if entry.name in _BY_NAME:
        raise ValueError(f"the catalog already has a model called {entry.name!r}")
    CATALOG.append(entry)
    _BY_NAME[entry.name] = entry


def catalog_names() -> List[str]:
    from .registry import load_plugins
    load_plugins()
    return [e.name for e in CATALOG]


def looks_like_path(name_or_path: str) -> bool:
    """A folder with config.json, or anything with a path separator, is a path
    (rocml/src/registry/mod.rs:123-127 has the same rule for files)."""
    return (os.sep in name_or_path or name_or_path.startswith(".")
            or os.path.isdir(name_or_path))


@dataclass(frozen=True)
class Resolved:
    path: Optional[str]          # model folder, if --model was one
    entry: Optional[ModelEntry]  # catalog entry, if --model was a name


def resolve(name_or_path: str) -> Resolved:
    from .registry import load_plugins
    load_plugins()
    if looks_like_path(name_or_path):
        if not os.path.isfile(os.path.join(name_or_path, "config.json")):
            raise UnknownModelError(f"{name_or_path!r} is not a model folder (no config.json in it)")
        return Resolved(path=name_or_path, entry=None)
    if name_or_path not in _BY_NAME:
        raise UnknownModelError(
            f"unknown model {name_or_path!r}; known names: {', '.join(catalog_names())}; "
            "or give a folder with config.json and model.safetensors")
    return Resolved(path=None, entry=_BY_NAME[name_or_path])
