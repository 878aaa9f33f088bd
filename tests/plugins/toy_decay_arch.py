"""A toy architecture that lives outside the package: a configuration class with keys of its
own, a mixer with a state of fixed size per sequence, its own tensor names.  Importing the
module registers all of it; the command line and the replay program learn of it through the
environment variable ROCML_AMD_PLUGINS and are otherwise unchanged.  It is no model of anyone's:
layers alternate between a decaying running sum and the library's attention.

The module also holds the plain implementation the tests compare with.
"""
from __future__ import annotations

import math
from dataclasses import asdict, dataclass
from typing import Dict, List, Sequence

import torch

from rocml_amd import ops
from rocml_amd.config import Architecture, register_architecture
from rocml_amd.config.spec import (AttentionSpec, BlockSpec, GatedMlpSpec, ModelSpec, NormSpec, RopeSpec,
                                   default_schedule)
from rocml_amd.errors import ConfigError
from rocml_amd.parts import Mixer, ParamSpec, StateRequest, register_mixer

ARCHITECTURE = "ToyDecayLM"


@dataclass(frozen=True)
class DecaySpec:
    hidden: int
    width: int
    decay: float
    kind: str = "toy_decay"


class DecayMixer(Mixer):
    """state <- decay * state + W_in x; out = W_out state.  The state lives in the cache's
    fixed-size region of the sequence's slot and is advanced once per token, in order.  A decode
    step (one token per sequence) is made of device work only, so the engine may record it."""

    def __init__(self, spec: DecaySpec, ctx):
        self.spec = spec
        self.dtype = ctx.dtype

    def param_specs(self) -> Dict[str, ParamSpec]:
        s = self.spec
        return {"in_proj.weight": ParamSpec((s.width, s.hidden)), "out_proj.weight": ParamSpec((s.hidden, s.width))}

    def bind(self, tensors) -> None:
        self.w_in, self.w_out = tensors["in_proj.weight"], tensors["out_proj.weight"]

    def cache_request(self):
        return StateRequest((self.spec.width,))

    def forward(self, step, xn, x_accum, cache, owns_cache) -> None:
        ws = step.workspace
        n, width = step.n_tokens, self.spec.width
        u = ws.get("toy.u", (n, width), torch.float32)
        ops.gemm(xn, self.w_in, u)
        states = ws.get("toy.states", (n, width), torch.float32)        # the state after each token
        if step.is_decode:
            slots = cache.slots.long()
            new = cache.state.index_select(0, slots) * self.spec.decay + u
            cache.state.index_copy_(0, slots, new)
            states.copy_(new)
        else:
            slots = cache.slots.cpu().tolist()
            cu = step.cu_seqlens.cpu().tolist()
            for b, slot in enumerate(slots):
                state = cache.state[slot]
                for t in range(cu[b], cu[b + 1]):
                    state.mul_(self.spec.decay).add_(u[t])
                    states[t] = state
        lowered = ws.get("toy.states_lowered", (n, width), self.dtype)
        lowered.copy_(states)
        ops.gemm(lowered, self.w_out, x_accum, accumulate=True)


register_mixer("toy_decay", DecayMixer)

_KEYS = ("toy_vocab", "toy_width", "toy_depth", "toy_state", "toy_inner", "toy_heads", "toy_head", "toy_max_len")


@dataclass(frozen=True)
class ToyConfig:
    toy_vocab: int
    toy_width: int
    toy_depth: int
    toy_state: int
    toy_inner: int
    toy_heads: int
    toy_head: int
    toy_max_len: int
    toy_decay: float
    toy_eps: float
    toy_stop: int = -1

    @classmethod
    def from_dict(cls, raw: Dict) -> "ToyConfig":
        for key in _KEYS + ("toy_decay", "toy_eps"):
            if key not in raw:
                raise ConfigError(f"config.json lacks the required key {key!r}")
        for key in _KEYS:
            if not isinstance(raw[key], int) or raw[key] <= 0:
                raise ConfigError(f"config.json key {key!r} must be a positive integer, found {raw[key]!r}")
        return cls(**{k: raw[k] for k in _KEYS}, toy_decay=float(raw["toy_decay"]), toy_eps=float(raw["toy_eps"]),
                   toy_stop=int(raw.get("toy_stop", -1)))

    def to_dict(self) -> Dict:
        return dict(asdict(self), architectures=[ARCHITECTURE])


def to_spec(cfg: ToyConfig) -> ModelSpec:
    norm = NormSpec(cfg.toy_width, cfg.toy_eps)
    ffn = GatedMlpSpec(cfg.toy_width, cfg.toy_inner)
    attention = AttentionSpec(hidden=cfg.toy_width, n_heads=cfg.toy_heads, n_kv_heads=1, head_dim=cfg.toy_head,
                              scale=1.0 / math.sqrt(cfg.toy_head), qk_norm=None,
                              position=RopeSpec(cfg.toy_head, cfg.toy_head, 10000.0))
    decay = DecaySpec(cfg.toy_width, cfg.toy_state, cfg.toy_decay)
    layers = tuple(BlockSpec(mixer=decay if i % 2 == 0 else attention, ffn=ffn, mixer_norm=norm, ffn_norm=norm)
                   for i in range(cfg.toy_depth))
    return ModelSpec(architecture=ARCHITECTURE, vocab=cfg.toy_vocab, hidden=cfg.toy_width, layers=layers,
                     schedule=default_schedule(cfg.toy_depth), final_norm=norm, tie_lm_head=True,
                     max_positions=cfg.toy_max_len, eos_token_ids=() if cfg.toy_stop < 0 else (cfg.toy_stop,))


def checkpoint_names(spec: ModelSpec) -> Dict[str, str]:
    names = {"embed.weight": "tok.weight", "final_norm.weight": "out_norm.gain"}
    for i, block in enumerate(spec.layers):
        src, dst = f"blocks.{i}.", f"layers.{i}."
        names[dst + "mixer_norm.weight"] = src + "norm_a.gain"
        names[dst + "ffn_norm.weight"] = src + "norm_b.gain"
        if block.mixer.kind == "toy_decay":
            names[dst + "mixer.in_proj.weight"] = src + "sum.in.weight"
            names[dst + "mixer.out_proj.weight"] = src + "sum.out.weight"
        else:
            for p in ("q", "k", "v", "o"):
                names[dst + f"mixer.{p}_proj.weight"] = src + f"attn.{p}.weight"
        for p in ("gate", "up", "down"):
            names[dst + f"ffn.{p}_proj.weight"] = src + f"ffn.{p}.weight"
    return names


register_architecture(Architecture(name=ARCHITECTURE, read_config=ToyConfig.from_dict, to_spec=to_spec,
                                   checkpoint_names=checkpoint_names))


# ---- the plain implementation of the toy: whole sequences, no cache ------------------------------
def plain_forward(raw: Dict, w: Dict[str, torch.Tensor], tokens: Sequence[int], rounded=lambda t: t) -> torch.Tensor:
    """Logits at every position.  ``rounded`` is applied to the matrices only (the oracle of a
    bfloat16 engine up to the activations' rounding)."""
    from tests.plain import qwen3_plain as plain
    w = {k: (rounded(v.double()) if v.dim() > 1 else v.double()) for k, v in w.items()}
    eps, t = raw["toy_eps"], len(tokens)
    x = w["tok.weight"][list(tokens)]
    for i in range(raw["toy_depth"]):
        pre = f"blocks.{i}."
        xn = plain.rmsnorm(x, w[pre + "norm_a.gain"], eps)
        if i % 2 == 0:
            state = torch.zeros(raw["toy_state"], dtype=torch.float64)
            out = []
            for r in range(t):
                state = raw["toy_decay"] * state + w[pre + "sum.in.weight"] @ xn[r]
                out.append(w[pre + "sum.out.weight"] @ state)
            x = x + torch.stack(out)
        else:
            h, d = raw["toy_heads"], raw["toy_head"]
            q = plain.rope_neox((xn @ w[pre + "attn.q.weight"].t()).reshape(t, h, d), list(range(t)), 10000.0)
            k = plain.rope_neox((xn @ w[pre + "attn.k.weight"].t()).reshape(t, 1, d), list(range(t)), 10000.0)
            v = (xn @ w[pre + "attn.v.weight"].t()).reshape(t, 1, d)
            o = plain.causal_attention(q, k, v, 1.0 / math.sqrt(d))
            x = x + o.reshape(t, h * d) @ w[pre + "attn.o.weight"].t()
        xn = plain.rmsnorm(x, w[pre + "norm_b.gain"], eps)
        x = x + plain.swiglu(xn @ w[pre + "ffn.gate.weight"].t(), xn @ w[pre + "ffn.up.weight"].t()) \
            @ w[pre + "ffn.down.weight"].t()
    return plain.rmsnorm(x, w["out_norm.gain"], eps) @ w["tok.weight"].t()


def plain_greedy(raw: Dict, w: Dict[str, torch.Tensor], prompt: Sequence[int], n_new: int) -> List[int]:
    ids, out = list(prompt), []
    for _ in range(n_new):
        nxt = int(torch.argmax(plain_forward(raw, w, ids)[-1]))
        if nxt == raw.get("toy_stop", -1):
            break
        out.append(nxt)
        ids.append(nxt)
    return out
