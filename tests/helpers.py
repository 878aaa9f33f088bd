"""Shared pieces of the tests: tiny configurations, model folders in temporary
directories, and drivers that run a trace through the engine."""
from __future__ import annotations

import json
import os
from typing import Dict, List, Sequence

import numpy as np
import torch

from rocml_amd.config.catalog import CATALOG

_BY_NAME = {e.name: e for e in CATALOG}

TINY_A = dict(_BY_NAME["tiny-a"].config)
TINY_B = dict(_BY_NAME["tiny-b"].config)
# Differs from A and B in every size: 5 heads with groups of one, a head size of 48, a width
# and a vocabulary that are no power of two, a window in the first of its two layers.
TINY_C = {"architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "vocab_size": 301,
          "hidden_size": 80, "intermediate_size": 176, "num_hidden_layers": 2,
          "num_attention_heads": 5, "num_key_value_heads": 5, "head_dim": 48,
          "rope_theta": 500000.0, "rms_norm_eps": 3e-6, "tie_word_embeddings": False,
          "max_position_embeddings": 1024, "hidden_act": "silu", "attention_bias": False,
          "sliding_window": 24, "layer_types": ["sliding_attention", "full_attention"]}
# Four heads in groups of four sharing one key/value head, a window of 70 that crosses a
# page of the cache, more layers.
TINY_D = {"architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "vocab_size": 515,
          "hidden_size": 72, "intermediate_size": 200, "num_hidden_layers": 4,
          "num_attention_heads": 4, "num_key_value_heads": 1, "head_dim": 64,
          "rope_theta": 20000.0, "rms_norm_eps": 2e-5, "tie_word_embeddings": True,
          "max_position_embeddings": 2048, "hidden_act": "silu", "attention_bias": False,
          "sliding_window": 70,
          "layer_types": ["full_attention", "sliding_attention", "full_attention", "sliding_attention"]}

# Sizes that fit none of the fast kernels' rules: a width of 92 and an intermediate size of 150
# (no multiple of 8), a head size of 112 (a step of 16, no multiple of 32), three query heads on
# one key/value head, an odd vocabulary.
TINY_E = {"architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "vocab_size": 257,
          "hidden_size": 92, "intermediate_size": 150, "num_hidden_layers": 2,
          "num_attention_heads": 3, "num_key_value_heads": 1, "head_dim": 112,
          "rope_theta": 1234.5, "rms_norm_eps": 1e-4, "tie_word_embeddings": False,
          "max_position_embeddings": 300, "hidden_act": "silu", "attention_bias": False}

# Wide enough (K of 2048 and more) for the products of a prompt to be cut along K, with the halves
# left to the next norm or to the q/k kernel.
TINY_F = {"architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "vocab_size": 300,
          "hidden_size": 2048, "intermediate_size": 2112, "num_hidden_layers": 2,
          "num_attention_heads": 8, "num_key_value_heads": 2, "head_dim": 32,
          "rope_theta": 10000.0, "rms_norm_eps": 1e-6, "tie_word_embeddings": True,
          "max_position_embeddings": 512, "hidden_act": "silu", "attention_bias": False}

# A head size of 96 (one and a half waves wide where a kernel takes a thread per value) with
# eight query heads on each key/value head, three layers.
TINY_G = {"architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "vocab_size": 1000,
          "hidden_size": 128, "intermediate_size": 176, "num_hidden_layers": 3,
          "num_attention_heads": 16, "num_key_value_heads": 2, "head_dim": 96,
          "rope_theta": 10000.0, "rms_norm_eps": 1e-6, "tie_word_embeddings": False,
          "max_position_embeddings": 512, "hidden_act": "silu", "attention_bias": False}

# A head size of 128 on three key/value heads of two query heads each, no window: in bfloat16 the
# decode steps of this one (and of D) take the attention kernel that reads the projection itself.
TINY_H = {"architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "vocab_size": 777,
          "hidden_size": 88, "intermediate_size": 120, "num_hidden_layers": 2,
          "num_attention_heads": 6, "num_key_value_heads": 3, "head_dim": 128,
          "rope_theta": 1000000.0, "rms_norm_eps": 1e-6, "tie_word_embeddings": False,
          "max_position_embeddings": 1024, "hidden_act": "silu", "attention_bias": False}

TINY = {"A": (TINY_A, 0), "B": (TINY_B, 1), "C": (TINY_C, 2), "D": (TINY_D, 3), "E": (TINY_E, 4), "F": (TINY_F, 5),
        "G": (TINY_G, 22), "H": (TINY_H, 23)}


def make_model_dir(tmp_path, config: Dict, seed: int, dtype=torch.float32) -> str:
    from rocml_amd.weights import write_model_dir
    path = os.path.join(str(tmp_path), f"model_{seed}_{str(dtype).split('.')[-1]}")
    return write_model_dir(path, config, seed, dtype=dtype, norm_jitter=True)


def read_weights(path: str) -> Dict[str, torch.Tensor]:
    from safetensors.torch import load_file
    return load_file(os.path.join(path, "model.safetensors"))


def read_config(path: str) -> Dict:
    with open(os.path.join(path, "config.json")) as f:
        return json.load(f)


def random_tokens(n: int, vocab: int, seed: int) -> List[int]:
    rng = np.random.default_rng(seed)
    return [int(t) for t in rng.integers(0, vocab, size=n)]


def rel_to_max(got: torch.Tensor, ref: torch.Tensor) -> float:
    """Largest absolute difference over the largest absolute reference value."""
    ref = ref.to(torch.float64)
    return float((got.to(torch.float64) - ref).abs().max() / ref.abs().max())


def per_position(got: torch.Tensor, ref: torch.Tensor) -> float:
    """The worst position's largest absolute difference over that position's largest absolute
    reference value: a fault at one place is not hidden by large logits elsewhere."""
    ref = ref.to(torch.float64)
    diff = (got.to(torch.float64) - ref).abs().amax(dim=-1)
    return float((diff / ref.abs().amax(dim=-1)).max())


def run_whole(engine, tokens: Sequence[int]) -> torch.Tensor:
    """One request alone, whole: logits at every position, [T, V] on the CPU."""
    from rocml_amd.engine import StepEntry
    slot = engine.new_sequence()
    logits = engine.step([StepEntry(slot, list(tokens), list(range(len(tokens))))]).cpu()
    engine.release(slot)
    return logits


def run_tail_by_one(engine, tokens: Sequence[int], tail: int) -> torch.Tensor:
    """Prefix in one step, then the last ``tail`` tokens one by one; logits at every position."""
    from rocml_amd.engine import StepEntry
    slot = engine.new_sequence()
    n = len(tokens)
    head = n - min(tail, n - 1)
    out = [engine.step([StepEntry(slot, list(tokens[:head]), list(range(head)))]).cpu()]
    for i in range(head, n):
        out.append(engine.step([StepEntry(slot, [tokens[i]], [0])]).cpu())
    engine.release(slot)
    return torch.cat(out)


def run_batch(engine, prompts: Sequence[Sequence[int]], n_prefill: Sequence[int]) -> List[torch.Tensor]:
    """A batch of sequences that start together: sequence ``i`` brings its first
    ``n_prefill[i]`` tokens in the first step and one token in each later step until it
    has none left, when it leaves the batch and its slot is given back.  Returns logits at
    every position of every sequence."""
    from rocml_amd.engine import StepEntry
    slots = [engine.new_sequence() for _ in prompts]
    got: List[List[torch.Tensor]] = [[] for _ in prompts]
    entries = [StepEntry(slots[i], list(p[:n_prefill[i]]), list(range(n_prefill[i])))
               for i, p in enumerate(prompts)]
    logits = engine.step(entries).cpu()
    at = 0
    for i in range(len(prompts)):
        got[i].append(logits[at:at + n_prefill[i]])
        at += n_prefill[i]
    fed = list(n_prefill)
    live = list(range(len(prompts)))
    for i in list(live):
        if fed[i] == len(prompts[i]):
            engine.release(slots[i])
            live.remove(i)
    while live:
        entries = [StepEntry(slots[i], [prompts[i][fed[i]]], [0]) for i in live]
        logits = engine.step(entries).cpu()
        for row, i in enumerate(live):
            got[i].append(logits[row:row + 1])
            fed[i] += 1
        for i in list(live):
            if fed[i] == len(prompts[i]):
                engine.release(slots[i])
                live.remove(i)
    return [torch.cat(g) for g in got]
