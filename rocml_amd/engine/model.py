"""A decoder built from a ``ModelSpec``: an embedding part, the layers in schedule order and a
head part.  It holds no sizes of its own and no knowledge of any architecture; the data flow
is the reference's (rocml/src/forward/chunk_forward.rs:96-184): embedding, blocks, then the
head (norm and output product) only for the rows whose logits are wanted.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..cache import Cache
from ..cache.cache import HEADROOM_BYTES
from ..config.spec import ModelSpec
from ..errors import ConfigError
from ..parts import BuildContext, ParamSpec, build_block, build_embedding, build_head
from .batch import StepContext
from .workspace import Workspace

RUNTIME_BYTES = 256 << 20      # kept free for the runtime, code objects and the sampler beside the activations

_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32,
           torch.bfloat16: torch.bfloat16, torch.float32: torch.float32}


def compute_dtype(name) -> torch.dtype:
    if name not in _DTYPES:
        raise ConfigError(f"compute type must be bfloat16 or float32, got {name!r}")
    return _DTYPES[name]


class DecoderModel:
    def __init__(self, spec: ModelSpec, dtype, device="cuda"):
        spec.validate()
        self.spec = spec
        self.dtype = compute_dtype(dtype)
        self.device = torch.device(device)
        ctx = BuildContext(dtype=self.dtype, device=self.device)
        self.embedding = build_embedding(spec.embedding_spec(), ctx)
        self.blocks = [build_block(b, ctx) for b in spec.layers]
        self.head = build_head(spec.head_spec(), ctx)
        self.bound = False
        # whether a decode step may be recorded as a graph: every part must say so
        self.graph_safe = all(getattr(part, "graph_safe", True)
                              for part in [self.embedding, self.head] + self.blocks)
        # ... and a short prompt step of a shape seen before
        self.prompt_graph_safe = self.graph_safe and all(getattr(part, "prompt_graph_safe", False)
                                                         for part in [self.embedding, self.head] + self.blocks)

    @property
    def embed(self) -> Optional[torch.Tensor]:
        """The embedding's table (None before weights are bound or if it has none)."""
        return self.embedding.shared_matrix() if self.bound else None

    @property
    def lm_head(self) -> Optional[torch.Tensor]:
        return getattr(self.head, "matrix", None)

    # -- parameters --------------------------------------------------------------------
    def param_specs(self) -> Dict[str, ParamSpec]:
        """Embedding parameters under ``embed.``, a layer's under ``layers.<i>.``, the head's under
        the names it gives them."""
        specs = {f"embed.{name}": p for name, p in self.embedding.param_specs().items()}
        for i, block in enumerate(self.blocks):
            for name, p in block.param_specs().items():
                specs[f"layers.{i}.{name}"] = p
        specs.update(self.head.param_specs())
        return specs

    def storage_dtype(self, p: ParamSpec) -> torch.dtype:
        return {"matrix": self.dtype, "gain": torch.float32, "int_table": torch.int32}[p.role]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.embedding.bind({k[len("embed."):]: v for k, v in tensors.items() if k.startswith("embed.")})
        for i, block in enumerate(self.blocks):
            prefix = f"layers.{i}."
            block.bind({k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)})
        self.head.bind({k: tensors[k] for k in self.head.param_specs()}, shared=self.embedding.shared_matrix())
        self.bound = True

    def weight_bytes(self) -> int:
        total = 0
        for name, p in self.param_specs().items():
            n = 1
            for d in p.shape:
                n *= d
            total += n * torch.empty((), dtype=self.storage_dtype(p)).element_size()
        return total

    def n_params(self) -> int:
        total = 0
        for p in self.param_specs().values():
            n = 1
            for d in p.shape:
                n *= d
            total += n
        return total

    def step_weight_bytes(self) -> int:
        """Bytes of weights a step has to read once: every layer as often as the schedule runs
        it and the head's matrices; of the embedding only the step's rows, which are not
        counted (a tied table is read as the head's matrix)."""
        per_layer = []
        for block in self.blocks:
            n = 0
            for p in block.param_specs().values():
                e = 1
                for d in p.shape:
                    e *= d
                n += e * torch.empty((), dtype=self.storage_dtype(p)).element_size()
            per_layer.append(n)
        size = torch.empty((), dtype=self.dtype).element_size()
        return sum(per_layer[e.layer] for e in self.spec.schedule) + self.head.step_matrix_elements() * size

    def step_flops(self, new_counts, starts, n_wanted: int) -> int:
        """Floating-point operations of a step: the layers in schedule order and the head for
        the wanted rows."""
        total = sum(self.blocks[e.layer].flops(new_counts, starts) for e in self.spec.schedule)
        return total + self.head.flops(n_wanted)

    # -- cache -------------------------------------------------------------------------
    def cache_requests(self) -> List[Optional[object]]:
        """What each schedule entry needs of the cache (None if it reads another's)."""
        return [None if e.reads_cache_of is not None else self.blocks[e.layer].cache_request()
                for e in self.spec.schedule]

    def activation_bytes(self, n_tokens: int, n_wanted: int) -> int:
        """Bytes of activations and scratch memory a step of ``n_tokens`` tokens with ``n_wanted``
        rows of logits asks the workspace for: the residual stream, the largest layer's buffers
        (layers share theirs), the wanted rows and their logits, and the scratch memory."""
        per_layer = max(b.activation_bytes(n_tokens) for b in self.blocks)
        return (n_tokens * self.spec.hidden * 4 + per_layer + self.head.activation_bytes(n_wanted)
                + Workspace.SCRATCH_BYTES)

    def new_cache(self, max_tokens: int, max_seqs: Optional[int] = None,
                  step_tokens: Optional[int] = None) -> Cache:
        """The cache for this model.  ``step_tokens`` (the most tokens a piece of a step brings)
        sizes what is left free beside the cache: the reference's 768 MiB
        (rocml/src/budget/mod.rs:37) cover its pieces of 512 tokens, a longer piece needs more."""
        free = None
        if torch.device(self.device).type == "cuda":
            # what the driver reports as free, and what torch holds without using it
            free = torch.cuda.mem_get_info(self.device)[0] + \
                torch.cuda.memory_reserved(self.device) - torch.cuda.memory_allocated(self.device)
        headroom = HEADROOM_BYTES
        if step_tokens is not None:
            wanted = max_seqs if max_seqs is not None else 64
            headroom = max(headroom, self.activation_bytes(step_tokens, wanted) + RUNTIME_BYTES)
        return Cache(self.cache_requests(), max_tokens, self.dtype, self.device, max_seqs=max_seqs,
                     free_bytes=free, step_tokens=step_tokens, headroom=headroom)

    # -- forward -----------------------------------------------------------------------
    def forward(self, step: StepContext, cache: Cache, block_tables: Dict[str, torch.Tensor],
                want_rows: Optional[torch.Tensor], n_want: int) -> Optional[torch.Tensor]:
        """Runs the step's tokens through every schedule entry; returns 32-bit logits
        ``[n_want, vocab]`` for the token rows in ``want_rows`` (None if none are wanted)."""
        s = self.spec
        ws = step.workspace
        ws.drop_pending()
        x = ws.get("model.x", (step.n_tokens, s.hidden), torch.float32)
        self.embedding.forward(step, x)
        for i, entry in enumerate(s.schedule):
            owner = i if entry.reads_cache_of is None else entry.reads_cache_of
            view = None
            if cache.has_line(owner):
                group, line = cache.line(owner)
                view = group.view(line, step)
            block = self.blocks[entry.layer]
            if not getattr(block, "takes_pending", False):
                ws.flush_pending()
            # the block that runs next may let this block's last product prepare its first norm
            following = self.blocks[s.schedule[i + 1].layer] if i + 1 < len(s.schedule) else None
            hint = None
            if getattr(block, "takes_next_norm", False) and hasattr(following, "entry_hint"):
                hint = following.entry_hint(step)
            if hint is not None:
                block.forward(step, x, view, owner == i, next_norm=hint)
            else:
                block.forward(step, x, view, owner == i)
        if n_want == 0:
            ws.drop_pending()
            return None
        if not getattr(self.head, "takes_pending", False):
            ws.flush_pending()
        return self.head.forward(step, x, want_rows, n_want)
