"""Softmax attention with grouped key/value heads over the paged cache.

Order of work as in the reference's layer (rocml/src/forward/attention_chunk.rs:97-330):
projections without bias, per-head norm of q and k, rotation, append to the cache, causal
attention with the scale applied after the dot product, output projection, residual sum.
Here q, k and v come from one product over the concatenated weight, norm + rotation +
append are one kernel, and the residual sum is the output product's epilogue.  Head
counts, head size, scale, window, the optional norm and the optional position encoding
are the spec's, nothing is fixed here.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import ops
from ..config.spec import AttentionSpec
from ..errors import ConfigError
from .base import BuildContext, KVCacheRequest, Mixer, ParamSpec
from .registry import build_position, register_mixer
from .residual import stream


class Attention(Mixer):
    adds_only = True
    FUSED_PREFILL_MIN_TOKENS = 1024

    def __init__(self, spec: AttentionSpec, ctx: BuildContext):
        if spec.n_heads % spec.n_kv_heads != 0:
            raise ConfigError(f"{spec.n_heads} query heads are not a multiple of {spec.n_kv_heads} key/value heads")
        if spec.qk_norm is not None and spec.qk_norm.size != spec.head_dim:
            raise ConfigError("the per-head norm must span the head size")
        if spec.qk_norm is not None and spec.qk_norm.kind != "rmsnorm":
            # the norm of q and k runs inside the rotation and attention kernels, which know one kind
            raise ConfigError(f"the per-head norm must be of kind 'rmsnorm', got {spec.qk_norm.kind!r}")
        if spec.window is not None and spec.window <= 0:
            raise ConfigError(f"window must be positive, got {spec.window}")
        self.spec = spec
        self.dtype = ctx.dtype
        self.n_cus = ops.cu_count(ctx.device)
        self.q_dim = spec.n_heads * spec.head_dim
        self.kv_dim = spec.n_kv_heads * spec.head_dim
        self.position = build_position(spec.position, ctx) if spec.position is not None else None
        self.pairing = getattr(self.position, "pairing", "halves")
        if self.pairing not in ops.ROPE_PAIRINGS:
            raise ConfigError(f"unknown rotation pairing {self.pairing!r}; known: {sorted(ops.ROPE_PAIRINGS)}")
        # (what may be recorded as a graph: the attention's own launches always, its position
        # encoding's if that part says so)
        self.graph_safe = self.position is None or getattr(self.position, "graph_safe", True)
        self.prompt_graph_safe = self.graph_safe and (self.position is None or getattr(self.position, "prompt_graph_safe", False))
        self.w_qkv: Optional[torch.Tensor] = None
        self.w_o: Optional[torch.Tensor] = None
        self.q_gain: Optional[torch.Tensor] = None
        self.k_gain: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        s = self.spec
        specs = {"q_proj.weight": ParamSpec((self.q_dim, s.hidden)),
                 "k_proj.weight": ParamSpec((self.kv_dim, s.hidden)),
                 "v_proj.weight": ParamSpec((self.kv_dim, s.hidden)),
                 "o_proj.weight": ParamSpec((s.hidden, self.q_dim))}
        if s.qk_norm is not None:
            specs["q_norm.weight"] = ParamSpec((s.head_dim,), role="gain", init="gain")
            specs["k_norm.weight"] = ParamSpec((s.head_dim,), role="gain", init="gain")
        return specs

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        # One [Q + 2 KV, hidden] matrix: q rows first, so a layer that only reads another
        # layer's cache multiplies by the leading Q rows.
        self.w_qkv = torch.cat([tensors["q_proj.weight"], tensors["k_proj.weight"],
                                tensors["v_proj.weight"]], dim=0).contiguous()
        self.w_o = tensors["o_proj.weight"]
        if self.spec.qk_norm is not None:
            self.q_gain = tensors["q_norm.weight"]
            self.k_gain = tensors["k_norm.weight"]

    def flops(self, new_counts, starts) -> int:
        # the products with the weights, and 4 * heads * head size per query and key it sees
        keys = 0
        w = self.spec.window
        for n, s0 in zip(new_counts, starts):
            if w is None:
                keys += n * s0 + n * (n + 1) // 2
            else:
                keys += sum(min(s0 + i + 1, w) for i in range(n))
        return 2 * sum(new_counts) * self.matrix_elements() + 4 * self.spec.n_heads * self.spec.head_dim * keys

    def activation_bytes(self, n_tokens: int) -> int:
        size = 2 if self.dtype == torch.bfloat16 else 4
        rot = 0 if self.position is None else 2 * n_tokens * (self.position.rot_dim // 2) * 4
        return n_tokens * ((self.q_dim + 2 * self.kv_dim) * 4 + 2 * self.q_dim * size) + rot

    def _fused_decode(self, step) -> bool:
        rot = None if self.position is None else self.position.rot_dim
        return step.max_new == 1 and ops.attention_decode_fusable(
            self.dtype, self.spec.n_heads, self.spec.n_kv_heads, self.spec.head_dim, ops.FUSED_DECODE_PAGE, rot, self.pairing)

    def _fused_prefill(self, step, cache) -> bool:
        """Whether the prompt kernel prepares its queries itself: it pays from about a thousand
        tokens on (the preparation lengthens every attention block by some 6 us, the norm-and-rotation
        kernel's q rows cost 8 us per thousand tokens at 32 heads of 128)."""
        rot = None if self.position is None else self.position.rot_dim
        return (step.max_new > 1 and step.n_tokens >= self.FUSED_PREFILL_MIN_TOKENS
                and step.cu_seqlens is not None and self.dtype == torch.bfloat16
                and ops.attention_prefill_fusable(cache.k.dtype, self.spec.head_dim, cache.k.shape[2], rot, self.pairing))

    def takes_row_scale(self, step) -> bool:
        # only the decode kernel that reads the projection's sums itself applies a scale to them
        return self._fused_decode(step)

    def cache_request(self) -> KVCacheRequest:
        return KVCacheRequest(self.spec.n_kv_heads, self.spec.head_dim, self.spec.window)

    def _decode_splits(self, step, cache) -> int:
        """Splits of the key range in a decode step: enough blocks to fill the chip, at most one
        per page the block table has room for.  It depends on the step's shape only, never on
        the sequences' lengths, so a recorded step can be replayed as they grow."""
        if step.max_new != 1:
            return 0
        return ops.decode_splits(step.n_tokens * self.spec.n_kv_heads, self.n_cus, min(cache.block_table.shape[1], 64))

    def forward(self, step, xn, x_accum, cache, owns_cache: bool) -> None:
        s = self.spec
        n = step.n_tokens
        ws = step.workspace
        rows = self.q_dim + 2 * self.kv_dim if owns_cache else self.q_dim
        qkv = ws.get("attn.qkv", (n, rows), torch.float32)
        scratch = ws.scratch()
        # (the decode kernel that reads the projection adds four partial sums in one trip to memory
        # and further ones one after the other: K is cut into few pieces for it)
        splits = ops.gemm(xn, self.w_qkv[:rows], qkv, workspace=scratch, defer=True,
                          max_splits=ops.FUSED_DECODE_SPLITS if self._fused_decode(step) else 0)
        if splits:      # the product's split-K partial sums; the next kernel adds them
            qkv = scratch[:splits * n * rows * 4].view(torch.float32).view(splits, n, rows)
        cos = sin = None
        rot = 0
        if self.position is not None:
            cos, sin = self.position.tables(step)
            rot = self.position.rot_dim
        eps = s.qk_norm.eps if s.qk_norm is not None else 1.0
        o = ws.get("attn.o", (n, self.q_dim), self.dtype)
        if self._fused_decode(step) and cache.k.dtype == self.dtype and cache.k.shape[2] == ops.FUSED_DECODE_PAGE:
            # One token per sequence: norm, rotation, append and attention in one launch, straight
            # from the projection.  The attention's own partial results go behind the projection's.
            used = (splits * n * rows * 4 + 255) // 256 * 256 if splits else 0
            # (a step of one token per sequence numbers its tokens as its sequences)
            ops.attention_decode_fused(qkv, o, cache.k, cache.v, cache.block_table, None, step.token_pos,
                                       s.n_heads, s.n_kv_heads, s.head_dim, s.scale, self.q_gain, self.k_gain, eps,
                                       cos, sin, write_kv=owns_cache, window=s.window, workspace=scratch[used:],
                                       max_len=step.max_len, n_splits=self._decode_splits(step, cache),
                                       row_scale=stream(step).row_scale)
        else:
            if stream(step).row_scale is not None:
                raise ConfigError("the attention was handed an input without its norm's scale in a step it cannot scale")
            if not splits and self._fused_prefill(step, cache):
                # A prompt step: keys and values are prepared and appended, the attention kernel
                # prepares its queries from the projection itself.
                if owns_cache:
                    ops.qk_norm_rope_append(qkv, s.n_heads, s.n_kv_heads, s.head_dim, self.q_gain, self.k_gain, eps,
                                            cos, sin, rot, None, cache.k, cache.v, cache.block_table, step.token_seq,
                                            step.token_pos, write_kv=True, pairing=self.pairing)
                ops.attention_prefill_fused(qkv, o, cache.k, cache.v, cache.block_table, step.token_pos, s.n_heads,
                                            s.n_kv_heads, s.head_dim, s.scale, self.q_gain, eps, cos, sin, s.window,
                                            step.cu_seqlens, step.new_counts, max_len=step.max_len)
            else:
                q = ws.get("attn.q", (n, self.q_dim), self.dtype)
                ops.qk_norm_rope_append(qkv, s.n_heads, s.n_kv_heads, s.head_dim, self.q_gain, self.k_gain, eps,
                                        cos, sin, rot, q, cache.k, cache.v, cache.block_table, step.token_seq,
                                        step.token_pos, write_kv=owns_cache, n_splits=max(splits, 1), pairing=self.pairing)
                ops.attention(q, o, cache.k, cache.v, cache.block_table, step.token_seq, step.token_pos,
                              s.n_heads, s.n_kv_heads, s.head_dim, s.scale, s.window, workspace=ws.scratch(),
                              cu_seqlens=step.cu_seqlens, max_new=step.max_new, q_counts=step.new_counts,
                              max_len=step.max_len, n_splits=self._decode_splits(step, cache))
        stream(step).add_product(o, self.w_o, x_accum)


register_mixer("attention", Attention)
