"""Typed configuration of the dense Qwen3 decoder, read from config.json.

The reference reads the same quantities from GGUF metadata, all required, and
validates them (rocml/src/config.rs:57-131): every size nonzero, the number of
query heads a multiple of the number of key/value heads, an even head size.
``head_dim`` is a key of its own and is never derived from ``hidden / heads``
(rocml/src/config.rs:70).  Here the keys are config.json's.
"""
from __future__ import annotations

import json
import math
import os
from dataclasses import dataclass, field, asdict
from typing import Dict, Optional, Tuple

from ..errors import ConfigError, UnsupportedArchitectureError
from .spec import (AttentionSpec, BlockSpec, GatedMlpSpec, ModelSpec, NormSpec, RopeSpec,
                   default_schedule)

ARCHITECTURE = "Qwen3ForCausalLM"

_REQUIRED_INT = ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                 "num_attention_heads", "num_key_value_heads", "head_dim",
                 "max_position_embeddings")
_REQUIRED_FLOAT = ("rope_theta", "rms_norm_eps")
_LAYER_TYPES = ("full_attention", "sliding_attention")


@dataclass(frozen=True)
class Qwen3Config:
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    max_position_embeddings: int
    rope_theta: float
    rms_norm_eps: float
    tie_word_embeddings: bool = False
    hidden_act: str = "silu"
    sliding_window: Optional[int] = None
    layer_types: Optional[Tuple[str, ...]] = None
    eos_token_id: Optional[Tuple[int, ...]] = None
    architectures: Tuple[str, ...] = field(default=(ARCHITECTURE,))

    # ---- reading ---------------------------------------------------------
    @classmethod
    def from_dict(cls, raw: Dict) -> "Qwen3Config":
        archs = raw.get("architectures")
        if not archs or archs[0] != ARCHITECTURE:
            raise UnsupportedArchitectureError(
                f"config.json names architecture {archs!r}; this class reads {ARCHITECTURE!r}")
        values = {}
        for key in _REQUIRED_INT:
            if key not in raw:
                raise ConfigError(f"config.json lacks the required key {key!r}")
            v = raw[key]
            if isinstance(v, bool) or not isinstance(v, int):
                raise ConfigError(f"config.json key {key!r} must be an integer, found {v!r}")
            values[key] = v
        for key in _REQUIRED_FLOAT:
            if key not in raw:
                raise ConfigError(f"config.json lacks the required key {key!r}")
            v = raw[key]
            if isinstance(v, bool) or not isinstance(v, (int, float)):
                raise ConfigError(f"config.json key {key!r} must be a number, found {v!r}")
            values[key] = float(v)
        values["tie_word_embeddings"] = bool(raw.get("tie_word_embeddings", False))
        values["hidden_act"] = raw.get("hidden_act", "silu")
        if raw.get("attention_bias", False):
            raise ConfigError("attention_bias=true is not supported: the projections have no bias")
        if raw.get("rope_scaling") is not None:
            raise ConfigError("rope_scaling is not supported: the rotation has no scaling factors")
        layer_types = raw.get("layer_types")
        window = raw.get("sliding_window")
        if layer_types is None and raw.get("use_sliding_window", False):
            # Older files give a boundary instead of a list: layers from
            # max_window_layers on slide.
            if "max_window_layers" not in raw:
                raise ConfigError("use_sliding_window=true needs layer_types or max_window_layers")
            first = raw["max_window_layers"]
            layer_types = ["sliding_attention" if i >= first else "full_attention"
                           for i in range(values["num_hidden_layers"])]
        if layer_types is not None:
            values["layer_types"] = tuple(layer_types)
            if any(t == "sliding_attention" for t in layer_types):
                values["sliding_window"] = window
        eos = raw.get("eos_token_id")
        if eos is not None:
            # one id or a list of them; generation stops at any of them
            ids = list(eos) if isinstance(eos, (list, tuple)) else [eos]
            for t in ids:
                if isinstance(t, bool) or not isinstance(t, int) or not 0 <= t < values["vocab_size"]:
                    raise ConfigError(f"config.json key 'eos_token_id' must name token ids below vocab_size, found {eos!r}")
            values["eos_token_id"] = tuple(ids)
        cfg = cls(**values)
        cfg.validate()
        return cfg

    @classmethod
    def from_json(cls, path: str) -> "Qwen3Config":
        if os.path.isdir(path):
            path = os.path.join(path, "config.json")
        with open(path, "r", encoding="utf-8") as f:
            try:
                raw = json.load(f)
            except json.JSONDecodeError as e:
                raise ConfigError(f"{path} is not valid JSON: {e}") from e
        return cls.from_dict(raw)

    def to_dict(self) -> Dict:
        d = asdict(self)
        d["architectures"] = list(self.architectures)
        d["model_type"] = "qwen3"
        d["attention_bias"] = False
        if self.layer_types is None:
            d.pop("layer_types")
            d.pop("sliding_window")
        else:
            d["layer_types"] = list(self.layer_types)
            # the older pair of keys that says the same for files read by the boundary: layers
            # from max_window_layers on slide (when the sliding layers are the trailing ones)
            sliding = [t == "sliding_attention" for t in self.layer_types]
            d["use_sliding_window"] = any(sliding)
            if any(sliding) and sliding == sorted(sliding):
                d["max_window_layers"] = sliding.index(True)
        if self.eos_token_id is None:
            d.pop("eos_token_id")
        else:
            d["eos_token_id"] = list(self.eos_token_id) if len(self.eos_token_id) > 1 else self.eos_token_id[0]
        return d

    # ---- rules -----------------------------------------------------------
    def validate(self) -> None:
        for key in _REQUIRED_INT:
            if getattr(self, key) <= 0:
                raise ConfigError(f"{key} must be positive, found {getattr(self, key)}")
        if self.num_attention_heads % self.num_key_value_heads != 0:
            raise ConfigError(
                f"num_attention_heads {self.num_attention_heads} is not a multiple of "
                f"num_key_value_heads {self.num_key_value_heads} (grouped heads need it)")
        if self.head_dim % 2 != 0:
            raise ConfigError(f"head_dim {self.head_dim} must be even (rotation pairs i with i+D/2)")
        if self.rope_theta <= 0 or not math.isfinite(self.rope_theta):
            raise ConfigError(f"rope_theta must be positive and finite, found {self.rope_theta}")
        if self.rms_norm_eps <= 0 or not math.isfinite(self.rms_norm_eps):
            raise ConfigError(f"rms_norm_eps must be positive and finite, found {self.rms_norm_eps}")
        if self.hidden_act != "silu":
            raise ConfigError(f"hidden_act {self.hidden_act!r} is not supported (silu only)")
        if self.layer_types is not None:
            if len(self.layer_types) != self.num_hidden_layers:
                raise ConfigError(f"layer_types has {len(self.layer_types)} entries for "
                                  f"{self.num_hidden_layers} layers")
            for t in self.layer_types:
                if t not in _LAYER_TYPES:
                    raise ConfigError(f"layer type {t!r} is not one of {_LAYER_TYPES}")
            if "sliding_attention" in self.layer_types:
                if not isinstance(self.sliding_window, int) or self.sliding_window <= 0:
                    raise ConfigError("sliding_attention layers need a positive sliding_window")

    # ---- derived ---------------------------------------------------------
    @property
    def q_dim(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_dim(self) -> int:
        return self.num_key_value_heads * self.head_dim

    def n_params(self) -> int:
        h, i, v = self.hidden_size, self.intermediate_size, self.vocab_size
        per_layer = (self.q_dim * h + 2 * self.kv_dim * h + h * self.q_dim + 2 * self.head_dim
                     + 2 * h + 3 * i * h)
        head = 0 if self.tie_word_embeddings else v * h
        return v * h + self.num_hidden_layers * per_layer + h + head

    def layer_window(self, layer: int) -> Optional[int]:
        if self.layer_types is None or self.layer_types[layer] == "full_attention":
            return None
        return self.sliding_window

    def to_model_spec(self) -> ModelSpec:
        """The architecture as parts.  Pre-norm blocks; attention with per-head
        q/k norm that shares the model's eps (rocml/src/forward/attention.rs:105-123),
        rotation over the whole head, ``scale = 1/sqrt(head_dim)``
        (rocml/src/forward/attention.rs:160); SwiGLU feed-forward
        (rocml/src/forward/ffn.rs:36-107); final norm; optional tied output matrix."""
        head_norm = NormSpec(size=self.head_dim, eps=self.rms_norm_eps)
        rope = RopeSpec(head_dim=self.head_dim, rot_dim=self.head_dim, theta=self.rope_theta)
        hidden_norm = NormSpec(size=self.hidden_size, eps=self.rms_norm_eps)
        layers = []
        for i in range(self.num_hidden_layers):
            mixer = AttentionSpec(hidden=self.hidden_size, n_heads=self.num_attention_heads,
                                  n_kv_heads=self.num_key_value_heads, head_dim=self.head_dim,
                                  scale=1.0 / math.sqrt(self.head_dim),
                                  window=self.layer_window(i), qk_norm=head_norm, position=rope)
            ffn = GatedMlpSpec(hidden=self.hidden_size, intermediate=self.intermediate_size,
                               activation=self.hidden_act)
            layers.append(BlockSpec(mixer=mixer, ffn=ffn, mixer_norm=hidden_norm,
                                    ffn_norm=hidden_norm))
        spec = ModelSpec(architecture=ARCHITECTURE, vocab=self.vocab_size, hidden=self.hidden_size,
                         layers=tuple(layers), schedule=default_schedule(self.num_hidden_layers),
                         final_norm=hidden_norm, tie_lm_head=self.tie_word_embeddings,
                         max_positions=self.max_position_embeddings,
                         eos_token_ids=self.eos_token_id or ())
        spec.validate()
        return spec


def checkpoint_names(spec: ModelSpec) -> Dict[str, str]:
    """Internal parameter name -> tensor name in the checkpoint.

    The reference loads the same roles under GGUF names
    (rocml/src/weights/mod.rs:41-62, rocml/src/weights/layer.rs:39-63); the
    safetensors names are the ones its notes use for the original checkpoint
    (.claude/CLAUDE.md:365): ``self_attn.{q,k,v,o}_proj``, ``q_norm``, ``k_norm``,
    ``input_layernorm``, ``post_attention_layernorm``, ``mlp.{gate,up,down}_proj``."""
    names = {"embed.weight": "model.embed_tokens.weight",
             "final_norm.weight": "model.norm.weight"}
    if not spec.tie_lm_head:
        names["lm_head.weight"] = "lm_head.weight"
    for i in range(len(spec.layers)):
        src = f"model.layers.{i}."
        dst = f"layers.{i}."
        names[dst + "mixer_norm.weight"] = src + "input_layernorm.weight"
        names[dst + "ffn_norm.weight"] = src + "post_attention_layernorm.weight"
        for p in ("q", "k", "v", "o"):
            names[dst + f"mixer.{p}_proj.weight"] = src + f"self_attn.{p}_proj.weight"
        names[dst + "mixer.q_norm.weight"] = src + "self_attn.q_norm.weight"
        names[dst + "mixer.k_norm.weight"] = src + "self_attn.k_norm.weight"
        for p in ("gate", "up", "down"):
            names[dst + f"ffn.{p}_proj.weight"] = src + f"mlp.{p}_proj.weight"
    return names
