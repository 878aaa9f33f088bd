"""Interfaces of the parts a decoder is put together from.

The reference writes each layer as one function over one struct of weights
(rocml/src/forward/attention.rs:30-249, rocml/src/forward/ffn.rs:17-111).  Here a
layer is assembled from parts that know nothing about the model around them:

* every part declares its parameters (``param_specs``) and receives them as device
  tensors (``bind``);
* a **mixer** moves information between the tokens of a sequence and may ask for
  storage in the cache (``cache_request``): keys and values, or a state of fixed size;
* a **feed-forward** works on each token alone;
* a **norm** maps the 32-bit residual stream to the activation type;
* a **position encoding** prepares per-step tables that mixers share;
* an **embedding** turns the step's token ids into the first residual stream, and a **head**
  turns the wanted rows of the last one into logits.

Mixers and feed-forwards add their result into the 32-bit residual stream they are
handed (``x_accum``), which lets a product's epilogue do the residual sum.  A part whose
last product was split along K may leave the final addition of the partial sums to the
norm that reads ``x_accum`` next (``step.workspace.set_pending``).  Nobody else has to know:
the stream is completed (``flush_pending``) before it is handed to a norm that cannot add the
sums itself (no ``fuses_pending``), to a mixer or feed-forward that does not declare
``adds_only`` (that it only ever adds into ``x_accum`` and never reads it), and to a block
arrangement that does not declare ``takes_pending``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

import torch


@dataclass(frozen=True)
class ParamSpec:
    """Shape and role of one parameter.

    ``matrix``: an operand of a matrix product, held in the model's compute type.
    ``gain``: a small vector used in 32-bit arithmetic, always held in 32-bit.
    ``int_table``: integers, held as int32.
    ``init`` names how random weights are drawn: ``normal`` is N(0, 0.02), ``gain`` is 1
    (or 1 + N(0, 0.02) when jitter is asked for), ``zeros`` is 0."""
    shape: Tuple[int, ...]
    role: str = "matrix"
    init: str = "normal"


@dataclass(frozen=True)
class BuildContext:
    dtype: torch.dtype          # compute type: torch.bfloat16 or torch.float32
    device: torch.device


@dataclass(frozen=True)
class KVCacheRequest:
    """Keys and values per position: ``window`` is None when all positions are kept."""
    n_kv_heads: int
    head_dim: int
    window: Optional[int] = None


@dataclass(frozen=True)
class StateRequest:
    """A per-sequence state of fixed shape, zero when a sequence starts."""
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


class Part:
    # False: forward() waits for the GPU or works on the host (reads a tensor back, loops over
    # tokens), so a decode step with this part cannot be recorded and replayed as a graph
    graph_safe = True
    # True: the same holds for a step that brings several tokens per sequence: given the
    # sequences' token counts and first positions, forward() launches the same device work every
    # time and touches nothing on the host, so a short prompt step of a shape seen before may be
    # replayed too.  A part has to say so itself.
    prompt_graph_safe = False

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {}

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        """Receives the tensors named by ``param_specs``, already on the device and in
        the type their role asks for."""

    def matrix_elements(self) -> int:
        """Elements of the part's matrices (what a step multiplies each token with)."""
        total = 0
        for p in self.param_specs().values():
            if p.role == "matrix":
                n = 1
                for d in p.shape:
                    n *= d
                total += n
        return total

    def flops(self, new_counts, starts) -> int:
        """Floating-point operations of a step in which sequence ``b`` brings ``new_counts[b]``
        tokens on top of ``starts[b]`` cached ones: two per token and matrix element unless the
        part knows better."""
        return 2 * sum(new_counts) * self.matrix_elements()

    def activation_bytes(self, n_tokens: int) -> int:
        """Bytes of workspace buffers the part asks for in a step of ``n_tokens`` tokens; what
        the cache leaves free beside itself is sized with it."""
        return 0


@dataclass(frozen=True)
class NormHint:
    """A norm of the kind ``x / sqrt(mean(x^2) + eps) * gain`` over ``width`` values, as the
    producer of ``x`` needs to know it to prepare the norm's output."""
    gain: torch.Tensor
    eps: float
    width: int


class Norm(Part):
    fuses_pending = False     # True: forward() takes ``pending`` partial sums and adds them to x itself

    def prescale_hint(self) -> Optional[NormHint]:
        """What the product that completes the residual stream needs to prepare this norm's output
        up to the rows' scale; None if the norm is not of that kind."""
        return None

    def forward(self, x: torch.Tensor, out: torch.Tensor, rows: Optional[torch.Tensor] = None) -> None:
        raise NotImplementedError


class PositionEncoding(Part):
    """What the attention part asks of it: an attribute ``rot_dim`` (the leading width of a head
    that is rotated, even) and ``tables(step)`` returning ``(cos, sin)``, two 32-bit tensors
    ``[tokens, rot_dim / 2]`` for the step's ``token_pos``; the pair of a head that is rotated by
    the angle whose cosine and sine stand in column ``i`` is ``(i, i + rot_dim / 2)`` with
    ``pairing = "halves"`` and ``(2 i, 2 i + 1)`` with ``pairing = "neighbours"``."""
    pairing = "halves"

    def tables(self, step: Any) -> Any:
        """Per-step tables for the step's token positions; computed once a step (``step.memo``
        is a dictionary that lives as long as the step)."""
        raise NotImplementedError


class Mixer(Part):
    adds_only = False     # True: forward() never reads x_accum, it only adds into it

    def takes_row_scale(self, step: Any) -> bool:
        """Whether, in this step, forward() can take its input as ``bfloat16(x * gain)`` with the
        norm's row scale still to be applied (``parts.residual.stream(step).row_scale``, an
        ``ops.RowScale``) instead of
        the normed input."""
        return False

    def cache_request(self) -> Optional[Any]:
        return None

    def forward(self, step: Any, xn: torch.Tensor, x_accum: torch.Tensor, cache: Any,
                owns_cache: bool) -> None:
        """Adds the mixer's output for the step's tokens into ``x_accum`` (32-bit,
        ``[tokens, hidden]``).  ``cache`` is the view of the cache line this execution
        uses; with ``owns_cache`` false it belongs to another execution and is read only."""
        raise NotImplementedError


class FeedForward(Part):
    adds_only = False     # True: forward() never reads x_accum, it only adds into it

    def takes_row_scale(self, step: Any) -> bool:
        """As ``Mixer.takes_row_scale``."""
        return False

    def forward(self, step: Any, xn: torch.Tensor, x_accum: torch.Tensor) -> None:
        raise NotImplementedError


class Embedding(Part):
    def shared_matrix(self) -> Optional[torch.Tensor]:
        """The ``[vocab, hidden]`` table a head may use as its output matrix (tied weights), or
        None if the embedding has no such table."""
        return None

    def forward(self, step: Any, x: torch.Tensor) -> None:
        """Writes the residual stream's first value for the step's tokens into ``x`` (32-bit,
        ``[tokens, hidden]``)."""
        raise NotImplementedError


class Head(Part):
    takes_pending = False     # True: forward() may be handed a stream that still lacks deferred sums

    def bind(self, tensors: Dict[str, torch.Tensor], shared: Optional[torch.Tensor] = None) -> None:
        """``shared``: the embedding's table, for a head whose output matrix is tied to it."""

    def step_matrix_elements(self) -> int:
        """Elements of the matrices a step reads for its wanted rows (a tied table counts: the
        head reads all of it, the embedding only the step's rows)."""
        return self.matrix_elements()

    def flops(self, n_wanted: int) -> int:
        return 2 * n_wanted * self.step_matrix_elements()

    def activation_bytes(self, n_wanted: int) -> int:
        return 0

    def forward(self, step: Any, x: torch.Tensor, want_rows: torch.Tensor, n_want: int) -> torch.Tensor:
        """32-bit logits ``[n_want, vocab]`` of the token rows of ``x`` named by ``want_rows``."""
        raise NotImplementedError
