"""Plain, slow implementation of the dense Qwen3 decoder, whole sequences, no cache.

Written from the formulas of xmiksay/rocml (paths below are relative to the
reference checkout); it shares no code with ``rocml_amd``.  Every function
takes plain ``torch`` tensors on the CPU and computes in ``float64`` unless a
dtype is given, one function per part of the model.

Weights are a ``dict`` of tensors under the checkpoint's tensor names
(``model.layers.N.self_attn.q_proj.weight`` ...); the configuration is a plain
``dict`` with config.json's keys.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence

import torch


def embedding(table: torch.Tensor, ids: Sequence[int]) -> torch.Tensor:
    """``x[t, :] = table[ids[t], :]`` with no scaling
    (rocml-kernels/kernels/embedding.hip:6-18, rocml/src/forward/mod.rs:271-277)."""
    return torch.stack([table[int(i)] for i in ids])


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, rounded_before_scale=None) -> torch.Tensor:
    """Per row: ``inv = 1/sqrt(sum(x^2)/n + eps)``, ``y_i = x_i * inv * w_i``; the
    gain multiplies directly, there is no ``1 + w``
    (rocml-kernels/kernels/rmsnorm.hip:18-42).  ``rounded_before_scale`` (for the oracle of an
    engine that stores ``x * w`` in low precision and applies the row's scale to the sums of
    the product that follows) is applied to ``x * w``; the result is the same number otherwise."""
    n = x.shape[-1]
    mean_sq = (x * x).sum(dim=-1, keepdim=True) / n
    inv = 1.0 / torch.sqrt(mean_sq + eps)
    if rounded_before_scale is not None:
        return rounded_before_scale(x * weight) * inv
    return x * inv * weight


def rope_neox(x: torch.Tensor, positions: Sequence[int], theta: float) -> torch.Tensor:
    """NEOX rotary embedding over the full head: for ``i < D/2``,
    ``f_i = theta^(-2i/D)``, ``a = pos * f_i`` and the pair ``(i, i + D/2)``
    is rotated by ``a`` (rocml-kernels/kernels/rope.hip:18-33).

    ``x`` is ``[tokens, heads, D]``; ``positions[t]`` is token ``t``'s absolute
    position (rocml/src/forward/attention.rs:125-140)."""
    tokens, heads, d = x.shape
    half = d // 2
    # angles in float64 whatever the type of x: a = pos * theta^(-2i/D), one row per token
    inv_freq = torch.tensor([theta ** (-2.0 * i / d) for i in range(half)], dtype=torch.float64)
    angle = torch.tensor([float(p) for p in positions], dtype=torch.float64)[:, None] * inv_freq[None, :]
    c = torch.cos(angle).to(x.dtype)[:, None, :]
    s = torch.sin(angle).to(x.dtype)[:, None, :]
    x0, x1 = x[:, :, :half], x[:, :, half:2 * half]
    out = x.clone()
    out[:, :, :half] = x0 * c - x1 * s
    out[:, :, half:2 * half] = x0 * s + x1 * c
    return out


def _same(t: torch.Tensor) -> torch.Tensor:
    return t


def round_bfloat16(t: torch.Tensor) -> torch.Tensor:
    """The nearest bfloat16 value (ties to even), kept in the tensor's own type."""
    return t.to(torch.bfloat16).to(t.dtype)


def causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                     scale: float, window: Optional[int] = None, rounded=_same) -> torch.Tensor:
    """Causal softmax attention of one whole sequence with grouped heads.

    ``q`` is ``[T, Hq, D]``, ``k`` and ``v`` are ``[T, Hkv, D]``.  Query head
    ``h`` uses kv head ``h // (Hq/Hkv)`` (rocml-kernels/kernels/attn_decode.hip:22-30);
    ``s_j = (q . k_j) * scale`` with the scale applied after the dot product and the
    token at position ``p`` sees ``j in [0, p]``
    (rocml-kernels/kernels/attn_prefill.hip:121,167-190); ``out = softmax(s) @ v``
    (rocml-kernels/kernels/attn_decode.hip:227-254 give the same sum after merging).
    ``window`` (not in the reference, which has full attention only) restricts
    the keys to the last ``window`` positions ``[p - window + 1, p]``.
    ``rounded`` is applied to the unnormalised probabilities ``e^(s - max)`` that multiply the
    values; their sum, which divides the result, is taken before rounding (a low-precision
    second product with full-precision statistics)."""
    t_len, hq, d = q.shape
    hkv = k.shape[1]
    group = hq // hkv
    out = torch.zeros_like(q)
    place = torch.arange(t_len)
    seen = place[None, :] <= place[:, None]                  # row p sees columns j <= p
    if window is not None:
        seen &= place[None, :] > place[:, None] - window     # ... and j >= p - window + 1
    for h in range(hq):
        kv = h // group
        scores = (q[:, h] @ k[:, kv].T) * scale
        scores = scores.masked_fill(~seen, float("-inf"))
        e = torch.exp(scores - scores.max(dim=-1, keepdim=True).values)   # 0 where a key is not seen
        out[:, h] = (rounded(e) @ v[:, kv]) / e.sum(dim=-1, keepdim=True)
    return out


def swiglu(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """``h = g / (1 + exp(-g)) * u`` (rocml-kernels/kernels/silu_mul.hip:12-20)."""
    return gate / (1.0 + torch.exp(-gate)) * up


def linear(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """``y = x @ W^T`` for a ``[out, in]`` row-major weight, no bias
    (rocml-kernels/kernels/gemv_f16.hip:8-36, rocml/src/weights/mod.rs:78-98)."""
    return x @ weight.t()


def attention_block(x: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str, cfg: dict,
                    positions: Sequence[int], window: Optional[int], rounded=_same, rounded_probs=None) -> torch.Tensor:
    """One layer's attention sub-block on the normalised input
    (rocml/src/forward/attention_chunk.rs:97-256,316-330): three projections
    without bias, per-head RMSNorm of q and k with one ``[D]`` gain each and the
    model's eps, rotary embedding of q and k, causal attention with
    ``scale = 1/sqrt(D)`` (rocml/src/forward/attention.rs:160), output projection.
    ``rounded`` is applied where a low-precision engine stores a tensor: q, k and v as the
    attention reads them and the attention's output; ``rounded_probs`` (the same unless given)
    to the probabilities, which only an engine whose second product runs in low precision rounds."""
    hq = cfg["num_attention_heads"]
    hkv = cfg["num_key_value_heads"]
    d = cfg["head_dim"]
    eps = cfg["rms_norm_eps"]
    t_len = x.shape[0]
    q = linear(x, w[prefix + "self_attn.q_proj.weight"]).reshape(t_len, hq, d)
    k = linear(x, w[prefix + "self_attn.k_proj.weight"]).reshape(t_len, hkv, d)
    v = linear(x, w[prefix + "self_attn.v_proj.weight"]).reshape(t_len, hkv, d)
    q = rmsnorm(q, w[prefix + "self_attn.q_norm.weight"], eps)
    k = rmsnorm(k, w[prefix + "self_attn.k_norm.weight"], eps)
    q = rounded(rope_neox(q, positions, cfg["rope_theta"]))
    k = rounded(rope_neox(k, positions, cfg["rope_theta"]))
    o = rounded(causal_attention(q, k, rounded(v), 1.0 / math.sqrt(d), window,
                                 rounded if rounded_probs is None else rounded_probs))
    return linear(o.reshape(t_len, hq * d), w[prefix + "self_attn.o_proj.weight"])


def mlp_block(x: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str, rounded=_same) -> torch.Tensor:
    """Gated feed-forward on the normalised input
    (rocml/src/forward/ffn.rs:36-107): ``down(silu(gate(x)) * up(x))``; ``rounded`` is
    applied to the gated activation, the one tensor a low-precision engine stores here."""
    g = linear(x, w[prefix + "mlp.gate_proj.weight"])
    u = linear(x, w[prefix + "mlp.up_proj.weight"])
    return linear(rounded(swiglu(g, u)), w[prefix + "mlp.down_proj.weight"])


def layer_windows(cfg: dict) -> List[Optional[int]]:
    """Window of each layer from config.json: ``layer_types`` names each layer
    ``full_attention`` or ``sliding_attention`` (the latter uses
    ``sliding_window``).  The reference runs full attention in every layer
    (docs/multiarch-audit.md gap 1); without ``layer_types`` so does this."""
    n = cfg["num_hidden_layers"]
    kinds = cfg.get("layer_types")
    if not kinds:
        return [None] * n
    return [cfg["sliding_window"] if kind == "sliding_attention" else None for kind in kinds]


def forward(cfg: dict, weights: Dict[str, torch.Tensor], tokens: Sequence[int],
            dtype: torch.dtype = torch.float64, first_position: int = 0, rounded=_same,
            last: Optional[int] = None, rounded_probs=None, ffn_norm_rounds_before_scale: bool = False) -> torch.Tensor:
    """Logits ``[T, V]`` at every position of one whole sequence.

    Pre-norm residual blocks (rocml/src/forward/chunk_forward.rs:96-135):
    ``x += attn(rmsnorm(x))``; ``x += mlp(rmsnorm(x))``; then the final norm and
    the output matrix, which is the embedding table when the checkpoint has no
    ``lm_head.weight`` (rocml/src/weights/mod.rs:48-62,
    rocml/src/forward/mod.rs:342-380).  ``first_position`` shifts every position
    (used by the shift-invariance test only).  ``rounded`` (``round_bfloat16`` for the oracle
    of a bfloat16 engine) is applied to every tensor such an engine holds in low precision:
    the matrices, the normalised activations that feed a product, q, k, v, the probabilities,
    the attention's output and the gated activation; the residual stream, the norms'
    statistics, the rotation, the softmax statistics and all sums stay in ``dtype``.
    ``rounded_probs`` replaces it for the probabilities alone (``lambda t: t`` for an engine
    whose attention multiplies probabilities and values in full precision).
    ``ffn_norm_rounds_before_scale``: the norm before the feed-forward stores ``x * gain`` in
    low precision and the row's scale reaches the gate and up sums unrounded."""
    w = {name: (rounded(t.to(dtype)) if t.dim() > 1 else t.to(dtype)) for name, t in weights.items()}
    eps = cfg["rms_norm_eps"]
    positions = [first_position + t for t in range(len(tokens))]
    windows = layer_windows(cfg)
    x = embedding(w["model.embed_tokens.weight"], tokens)
    for layer in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{layer}."
        xn = rounded(rmsnorm(x, w[p + "input_layernorm.weight"], eps))
        x = x + attention_block(xn, w, p, cfg, positions, windows[layer], rounded, rounded_probs)
        if ffn_norm_rounds_before_scale:
            xn = rmsnorm(x, w[p + "post_attention_layernorm.weight"], eps, rounded_before_scale=rounded)
        else:
            xn = rounded(rmsnorm(x, w[p + "post_attention_layernorm.weight"], eps))
        x = x + mlp_block(xn, w, p, rounded)
    if last is not None:            # logits of the last positions only (a large vocabulary)
        x = x[-last:]
    xn = rounded(rmsnorm(x, w["model.norm.weight"], eps))
    head = w["lm_head.weight"] if "lm_head.weight" in w else w["model.embed_tokens.weight"]
    return linear(xn, head)


def greedy(cfg: dict, weights: Dict[str, torch.Tensor], prompt: Sequence[int], n_new: int,
           stop: Sequence[int] = ()) -> List[int]:
    """Greedy continuation by recomputing the whole sequence for every token;
    the first maximum wins (rocml/src/sample.rs:172-182) and a stop token ends
    the sequence without being emitted (rocml/src/generate/resumed.rs:215-219)."""
    ids = list(prompt)
    out: List[int] = []
    for _ in range(n_new):
        logits = forward(cfg, weights, ids)[-1]
        nxt = int(torch.argmax(logits))
        if nxt in stop:
            break
        out.append(nxt)
        ids.append(nxt)
    return out
