"""The step function: a batch of sequences, their new tokens, logits at wanted places.

One entry point replaces the reference's pair ``forward_chunk`` / ``forward_token``
(rocml/src/forward/chunk_forward.rs:62-189, rocml/src/forward/mod.rs:246-387): a step
runs exactly the tokens it is given, as one packed batch, on top of what earlier steps
left in the cache, and returns 32-bit logits only for the rows that were asked for
(the reference computes the last row only, chunk_forward.rs:143-184).  A sequence that
would pass the model's positions is an error, never a truncation
(rocml/src/forward/mod.rs:253-258).  Long steps are cut into pieces of at most
``max_step_tokens`` tokens internally, as the reference cuts prompts at 512
(chunk_forward.rs:41-52); the cut is invisible because every piece reads the cache.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import numpy as np
import torch

from ..cache import Cache
from ..errors import CacheFullError, ContextOverflowError, RocmlError
from .. import profile
from .batch import StepContext, StepEntry, pack_step
from .model import DecoderModel
from .workspace import Workspace


def _bucket(n: int) -> int:
    b = 1
    while b < n:
        b *= 2
    return b


class Engine:
    def __init__(self, model: DecoderModel, max_tokens: int, max_seqs: Optional[int] = None,
                 max_step_tokens: int = 8192, use_graphs: bool = True):
        if not model.bound:
            raise RocmlError("the model has no weights bound")
        self.model = model
        if max_step_tokens < 1:
            raise RocmlError("max_step_tokens must be at least 1")
        self.max_step_tokens = max_step_tokens
        self.cache: Cache = model.new_cache(max_tokens, max_seqs, step_tokens=max_step_tokens)
        self.workspace = Workspace(model.device)
        self.steps_run = 0
        self.use_graphs = use_graphs and model.graph_safe
        self.max_graph_batch = 256
        self.max_graph_prompt_tokens = 1024     # prompt steps of at most so many tokens may be recorded
        self.max_prompt_graphs = 32
        self._graphs: Dict[tuple, tuple] = {}

    # -- sequences -----------------------------------------------------------------------
    def new_sequence(self) -> int:
        return self.cache.new_sequence()

    def release(self, slot: int) -> None:
        self.cache.free_sequence(slot)

    def length(self, slot: int) -> int:
        return self.cache.length(slot)

    # -- the step ------------------------------------------------------------------------
    def step(self, entries: Sequence[StepEntry], device_ids: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
        """Runs the entries' tokens; returns ``[n_wanted, vocab]`` 32-bit logits on the
        device in the order of the entries and of their ``want`` lists, or None when
        nothing is wanted.  The result is a buffer of the engine and holds until the next
        step.  ``device_ids`` (int32 on the device, one per entry, every entry bringing one
        token): the token ids are taken from there instead of from the entries, whose tokens
        only stand for their number; for ids that a sampler has just drawn and the host has not
        seen yet."""
        spec = self.model.spec
        if not entries:
            return None
        if device_ids is not None:
            if any(len(e.tokens) != 1 for e in entries) or device_ids.numel() != len(entries) \
                    or device_ids.dtype != torch.int32 or not device_ids.is_cuda:
                raise RocmlError("ids on the device go with one token per entry: int32, one per entry")
        slots = [e.slot for e in entries]
        if len(set(slots)) != len(slots):
            raise RocmlError("a sequence appears twice in one step")
        starts, new_lens = [], []
        counts = [len(e.tokens) for e in entries]
        if min(counts) == 0:
            raise RocmlError("a step entry needs at least one token")
        # one look at all ids together; the entry at fault is searched for only when there is one
        flat = np.fromiter((t for e in entries for t in e.tokens), dtype=np.int64, count=sum(counts))
        if int(flat.min()) < 0 or int(flat.max()) >= spec.vocab:
            bad = int(flat[(flat < 0) | (flat >= spec.vocab)][0])
            raise RocmlError(f"token id {bad} is outside the vocabulary of {spec.vocab}")
        for e, n in zip(entries, counts):
            if not self.cache.slots.is_live(e.slot):
                raise RocmlError(f"slot {e.slot} is not a live sequence")
            for w in e.want:
                if not 0 <= int(w) < n:
                    raise RocmlError(f"wanted place {w} is outside the entry's {n} tokens")
            start = self.cache.length(e.slot)
            if start + n > spec.max_positions:
                raise ContextOverflowError(
                    f"sequence would reach {start + n} positions; the model has "
                    f"{spec.max_positions}")
            starts.append(start)
            new_lens.append(start + n)
        # The step as pieces of at most max_step_tokens tokens (a sequence may straddle pieces).
        # Pages are reserved piece by piece, and a piece is committed before the next runs, so a
        # group with a window gives pages back while a long prompt passes through it; the whole
        # plan is checked against the free pages first, so a step is never left half run for want
        # of pages.  (Any other failure inside a piece, a kernel's refusal say, leaves the pieces
        # before it committed: the caller then releases the step's sequences, as the generation
        # loop does.)
        total = sum(counts)
        n_want_total = sum(len(e.want) for e in entries)
        pieces = None
        if total > self.max_step_tokens:
            pieces = self.plan_pieces(counts)
            short = self.cache.fits([[(entries[i].slot, starts[i] + hi) for i, _, hi in piece] for piece in pieces])
            if short is not None:
                raise CacheFullError(short)
        if pieces is None:             # one piece: its reservation is all or nothing by itself
            self.cache.reserve(slots, new_lens)
            logits = self._run_piece(slots, starts, [list(e.tokens) for e in entries],
                                     [list(e.want) for e in entries], device_ids)
            self.cache.commit(slots, new_lens)
            self.steps_run += 1
            return logits

        result = None
        if n_want_total:
            result = torch.empty((n_want_total, spec.vocab), dtype=torch.float32, device=self.model.device)
        want_base = np.cumsum([0] + [len(e.want) for e in entries])
        self.cache.reserve(slots, new_lens, which="kept")
        for piece in pieces:
            p_slots, p_starts, p_tokens, p_want, p_dest = [], [], [], [], []
            for i, lo, hi in piece:
                e = entries[i]
                wanted = [(k, w - lo) for k, w in enumerate(e.want) if lo <= w < hi]
                p_slots.append(e.slot)
                p_starts.append(starts[i] + lo)
                p_tokens.append(list(e.tokens[lo:hi]))
                p_want.append([w for _, w in wanted])
                p_dest.extend(int(want_base[i]) + k for k, _ in wanted)
            p_lens = [s + len(t) for s, t in zip(p_starts, p_tokens)]
            self.cache.reserve(p_slots, p_lens, which="windowed")
            # (ids on the device come one per entry, so a piece's entries are a run of them)
            p_ids = None if device_ids is None else device_ids[piece[0][0]:piece[0][0] + len(piece)]
            logits = self._run_piece(p_slots, p_starts, p_tokens, p_want, p_ids)
            if logits is not None:
                result[torch.as_tensor(p_dest, device=self.model.device)] = logits
            self.cache.commit(p_slots, p_lens)
        self.steps_run += 1
        return result

    def plan_pieces(self, counts: Sequence[int]) -> List[List[tuple]]:
        """How a step whose entries bring ``counts`` tokens is cut: a list of pieces, each a list
        of ``(entry, first token, one past the last token)`` in the order of the entries."""
        pieces: List[List[tuple]] = []
        done = [0] * len(counts)
        while any(d < c for d, c in zip(done, counts)):
            room = self.max_step_tokens
            piece = []
            for i, c in enumerate(counts):
                left = c - done[i]
                if left == 0 or room == 0:
                    continue
                take = min(left, room)
                piece.append((i, done[i], done[i] + take))
                done[i] += take
                room -= take
            pieces.append(piece)
        return pieces

    def _run_piece(self, slots: List[int], starts: List[int], tokens: List[List[int]],
                   want: List[List[int]], device_ids: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
        ids, seq, pos, cu, lens, slot_arr = pack_step(slots, starts, tokens)
        want_rows = np.asarray([int(cu[b]) + w for b, ws_ in enumerate(want) for w in ws_], dtype=np.int32)
        width = _bucket(self.cache.table_width(slots))
        tables = [self.cache.block_table(g, slots, width) for g in self.cache.kv_groups]
        # One upload for all integer tables of the step.
        parts = [ids, seq, pos, cu, lens, slot_arr, want_rows] + [t.reshape(-1) for t in tables]
        host = np.concatenate(parts) if parts else np.zeros(0, np.int32)
        meta = self.workspace.get("step.meta", (max(host.size, 1),), torch.int32)
        meta[:host.size].copy_(torch.from_numpy(host))
        if device_ids is not None:
            meta[:ids.size].copy_(device_ids)           # the ids lead the table
        max_new = max(len(t) for t in tokens)
        n_want = int(want_rows.size)

        def context() -> StepContext:
            views, at = [], 0
            for p in parts:
                views.append(meta[at:at + p.size])
                at += p.size
            d_ids, d_seq, d_pos, d_cu, d_lens, d_slots, d_want = views[:7]
            block_tables: Dict[str, torch.Tensor] = {}
            for g, v in zip(self.cache.kv_groups, views[7:]):
                block_tables[g.name] = v.view(len(slots), width)
            step = StepContext(n_tokens=int(ids.size), n_seqs=len(slots), token_ids=d_ids, token_seq=d_seq,
                               token_pos=d_pos, cu_seqlens=d_cu, seq_lens=d_lens, seq_slots=d_slots,
                               max_new=max_new, max_len=int(lens.max()),
                               new_counts=tuple(len(t) for t in tokens),
                               workspace=self.workspace)
            step.block_tables = block_tables
            step.want_rows = d_want if n_want else None
            return step

        def run(step: StepContext) -> Optional[torch.Tensor]:
            return self.model.forward(step, self.cache, step.block_tables, step.want_rows, n_want)

        profile.set_phase("decode" if max_new == 1 else "prefill")
        # (a profiler times single launches: no recorded graph while one is active)
        if not self.use_graphs or len(slots) > self.max_graph_batch or profile.active() is not None:
            return run(context())
        # Steps of one shape run from a recorded graph: the launches of a step are the same every
        # time, only the integer tables change, and those lie at fixed addresses.  A decode step's
        # shape is its number of sequences; a prompt step's is every sequence's number of tokens
        # and first position (short prompts only: a long one keeps the GPU busy far longer than
        # the host needs to launch it).  A shape runs plainly the first time (kernels set
        # themselves up, buffers reach their size), is recorded the second time, and replayed
        # from then on.
        if max_new == 1:
            key = (len(slots), n_want, width)
        elif self.model.prompt_graph_safe and int(ids.size) <= self.max_graph_prompt_tokens:
            key = ("prompt", tuple(len(t) for t in tokens), tuple(starts), n_want, width)
        else:
            return run(context())
        entry = self._graphs.get(key)
        if entry is not None and entry[0] != self.workspace.generation:
            entry = None                      # a buffer moved: the recorded addresses are stale
        if entry is None:
            result = run(context())
            self._remember(key, (self.workspace.generation, None, None))
            return result
        generation, graph, result = entry
        if graph is None:
            graph = torch.cuda.CUDAGraph()
            step = context()
            with torch.cuda.graph(graph):
                result = run(step)
            if self.workspace.generation != generation:
                # recording allocated a buffer after all; run plainly and start over
                del self._graphs[key]
                return run(context())
            self._remember(key, (generation, graph, result))
        graph.replay()
        return result

    def _remember(self, key, entry) -> None:
        """Keeps a shape's graph; of the prompt shapes only the ``max_prompt_graphs`` seen last."""
        self._graphs.pop(key, None)
        self._graphs[key] = entry                      # (a dict keeps insertion order: last seen last)
        if key[0] == "prompt":
            prompts = [k for k in self._graphs if k[0] == "prompt"]
            for k in prompts[:max(0, len(prompts) - self.max_prompt_graphs)]:
                del self._graphs[k]
