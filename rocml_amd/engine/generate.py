"""The generation loop: batches of unequal prompts, stop tokens, sequences that end
earlier, and as many batches one after another as there are requests.

Per sequence the flow is the reference's (rocml/src/generate/resumed.rs:193-233): the
prompt in one step, then sample, stop on a stop token without emitting it, emit, and run
the token.  Around it, which the reference does not have: requests are taken in order
into a batch while slots and cache pages for their prompt and their whole output are
free; the batch starts together; a sequence that ends leaves the batch and gives its
slot back; when the batch is empty the next one starts.  The loop decides on token ids
only and talks to the model through a small backend, so its decisions can be tested
without a GPU.
"""
from __future__ import annotations

import time
from dataclasses import dataclass, field
from typing import FrozenSet, List, Optional, Sequence

from ..errors import CacheFullError, RocmlError
from ..sampling.params import SamplingParams
from ..sampling.sampler import SequenceSampling


@dataclass
class Request:
    prompt: Sequence[int]
    max_new_tokens: int = 64
    params: SamplingParams = field(default_factory=SamplingParams)
    stop_tokens: FrozenSet[int] = frozenset()


@dataclass
class Result:
    tokens: List[int]
    finish_reason: str            # "stop", "length", "context" or "empty"
    prompt_tokens: int


@dataclass
class GenerateStats:
    """Token counts and seconds of the two phases (rocml/src/generate/mod.rs:27-51)."""
    prompt_tokens: int = 0
    generated_tokens: int = 0
    prompt_seconds: float = 0.0
    decode_seconds: float = 0.0
    batches: int = 0
    decode_steps: int = 0

    def prompt_tok_s(self) -> float:
        return self.prompt_tokens / self.prompt_seconds if self.prompt_seconds > 0 else 0.0

    def decode_tok_s(self) -> float:
        return self.generated_tokens / self.decode_seconds if self.decode_seconds > 0 else 0.0


class EngineBackend:
    """The loop's view of the engine and the sampler.

    With ``run_ahead`` (the default) the backend does not let the GPU wait for the host between
    decode steps: as soon as the sampler has been launched it launches the next step for the same
    sequences, with the token ids taken from the sampler's output on the device, and only then
    waits for the ids to reach the host.  When the loop then asks for that step it is running
    already; a sequence that the loop ended meanwhile (a stop token, a limit) was run one token
    too far, which nobody sees: its row is dropped and its slot is released."""

    def __init__(self, engine, sampler=None, run_ahead: bool = True):
        from ..sampling.sampler import DeviceSampler
        self.engine = engine
        self.sampler = sampler or DeviceSampler(engine.model.device)
        self.max_positions = engine.model.spec.max_positions
        self.run_ahead = run_ahead and hasattr(self.sampler, "sample_start")
        self._row_slots: Optional[List[int]] = None     # the slots whose logits the last step returned, row by row
        self._ahead = None                              # (slots, logits, slots still live, ids drawn) of a step launched ahead

    def can_admit(self, lengths: Sequence[int], prompts: Optional[Sequence[int]] = None) -> bool:
        """Whether new sequences with prompts of ``prompts`` tokens that will grow to ``lengths``
        fit the free slots and pages: the prompt step as the engine would cut it, then a token
        at a time (a group with a window is counted by its window, not by the final length)."""
        cache = self.engine.cache
        if len(lengths) > cache.slots.n_free:
            return False
        prompts = list(lengths) if prompts is None else list(prompts)
        keys = [("new", i) for i in range(len(lengths))]
        pieces = [[(keys[i], hi) for i, _, hi in piece] for piece in self.engine.plan_pieces(prompts)]
        return cache.fits(pieces, final=list(zip(keys, lengths))) is None

    def new_sequence(self) -> int:
        return self.engine.new_sequence()

    def release(self, slot: int) -> None:
        self.engine.release(slot)
        if self._ahead is not None:
            self._ahead[2].discard(slot)        # the slot may come back as another sequence

    def step(self, slots: Sequence[int], tokens: Sequence[Sequence[int]]):
        from .batch import StepEntry
        slots = list(slots)
        ahead, self._ahead = self._ahead, None
        covered = set() if ahead is None else set(slots) & ahead[2]
        if covered and (len(covered) != len(slots) or any(len(t) != 1 for t in tokens)):
            # some of these sequences are one token further already: running them again would
            # advance them twice
            raise RocmlError("a step was launched ahead for sequences %s; the next step must continue them all "
                             "with the one token each that was drawn" % sorted(covered))
        if covered:
            # the step is running already, with the tokens the sampler drew
            drawn = ahead[3]
            for s, t in zip(slots, tokens):
                if s in drawn and int(t[0]) != drawn[s]:
                    raise RocmlError(f"sequence {s} was run ahead with token {drawn[s]}, not {int(t[0])}")
            self._row_slots = slots
            if slots == ahead[0]:
                return ahead[1]
            import torch
            rows = torch.tensor([ahead[0].index(s) for s in slots], dtype=torch.int64, device=ahead[1].device)
            return ahead[1].index_select(0, rows)
        self._row_slots = slots
        return self.engine.step([StepEntry(s, list(t), [len(t) - 1]) for s, t in zip(slots, tokens)])

    def sample(self, logits, seqs: Sequence[SequenceSampling], may_continue: Optional[Sequence[bool]] = None) -> List[int]:
        """``may_continue[b]``: whether sequence ``b`` goes on after this token unless it is a
        stop token (the loop knows the limits); only those are run ahead."""
        if not self.run_ahead or self._row_slots is None or len(self._row_slots) != len(seqs):
            return self.sampler.sample(logits, seqs)
        from .batch import StepEntry
        started = self.sampler.sample_start(logits, seqs)
        rows = [b for b in range(len(seqs)) if may_continue is None or may_continue[b]]
        self._ahead = None
        if rows:
            slots = [self._row_slots[b] for b in rows]
            ids = started[0]
            if len(rows) != len(seqs):
                import torch
                ids = ids.index_select(0, torch.tensor(rows, dtype=torch.int64, device=ids.device))
            try:
                # those sequences one token further, as if none of them drew a stop token; refused (a
                # full cache) it changes nothing and the loop goes on step by step
                ahead = self.engine.step([StepEntry(s, [0], [0]) for s in slots], device_ids=ids)
                self._ahead = (slots, ahead, set(slots), {})
            except RocmlError:
                self._ahead = None
        drawn = self.sampler.finish(started)
        if self._ahead is not None:
            self._ahead[3].update((self._row_slots[b], int(drawn[b])) for b in rows)
        return drawn

    def synchronize(self) -> None:
        import torch
        if torch.device(self.engine.model.device).type == "cuda":
            torch.cuda.synchronize()


@dataclass
class _Live:
    index: int
    request: Request
    slot: int
    sampling: SequenceSampling
    out: List[int] = field(default_factory=list)
    released: bool = False


class Generator:
    def __init__(self, backend, max_batch: int = 64):
        if max_batch < 1:
            raise RocmlError("max_batch must be at least 1")
        self.backend = backend
        self.max_batch = max_batch
        self.stats = GenerateStats()
        import inspect
        self._hints = "may_continue" in inspect.signature(backend.sample).parameters
        # called with the number of decode steps run so far after each of them: a place for a
        # benchmark to take its times without a loop of its own
        self.on_step = None
        # called as on_token(request index, token id) for every token as it is drawn, in the order
        # of the batch (the reference hands every piece to a callback as it is decoded,
        # rocml/src/generate/mod.rs:67-85)
        self.on_token = None

    def _final_length(self, r: Request) -> int:
        return min(len(r.prompt) + r.max_new_tokens, self.backend.max_positions)

    def _take_batch(self, requests: Sequence[Request], first: int) -> int:
        """Number of requests, from ``first`` on, that start together."""
        lengths: List[int] = []
        prompts: List[int] = []
        n = 0
        while first + n < len(requests) and n < self.max_batch:
            r = requests[first + n]
            if len(r.prompt) == 0:
                if n == 0:
                    return 0      # handled alone by the caller
                break
            if not self.backend.can_admit(lengths + [self._final_length(r)], prompts + [len(r.prompt)]):
                break
            lengths.append(self._final_length(r))
            prompts.append(len(r.prompt))
            n += 1
        if n == 0:
            raise CacheFullError(f"request {first} does not fit the cache even alone "
                                 f"({self._final_length(requests[first])} positions)")
        return n

    def run(self, requests: Sequence[Request]) -> List[Result]:
        # every request is looked at before the first batch starts: a request that can never run
        # must not cost the results of those before it
        for i, r in enumerate(requests):
            if len(r.prompt) > self.backend.max_positions:
                raise RocmlError(f"request {i}: a prompt of {len(r.prompt)} tokens exceeds the "
                                 f"model's {self.backend.max_positions} positions")
        results: List[Optional[Result]] = [None] * len(requests)
        at = 0
        while at < len(requests):
            n = self._take_batch(requests, at)
            if n == 0:
                # An empty prompt gives no logits and so no token
                # (rocml/src/forward/chunk_forward.rs:38-40, rocml/src/generate/resumed.rs:215).
                results[at] = Result([], "empty", 0)
                at += 1
                continue
            self._run_batch(requests, at, n, results)
            at += n
        return results  # type: ignore[return-value]

    def _run_batch(self, requests, first: int, n: int, results) -> None:
        be = self.backend
        live: List[_Live] = []
        try:
            for i in range(n):
                r = requests[first + i]
                live.append(_Live(first + i, r, be.new_sequence(), SequenceSampling.start(r.params, first + i, r.prompt)))
            self._decode_batch(live, results)
        finally:
            # whatever ended the batch, its sequences give their slots and pages back
            for s in live:
                if not s.released:
                    s.released = True
                    be.release(s.slot)

    def _decode_batch(self, live: List[_Live], results) -> None:
        be = self.backend
        self.stats.batches += 1
        t0 = time.perf_counter()
        logits = be.step([s.slot for s in live], [list(s.request.prompt) for s in live])
        be.synchronize()
        t1 = time.perf_counter()
        self.stats.prompt_seconds += t1 - t0
        self.stats.prompt_tokens += sum(len(s.request.prompt) for s in live)
        running = list(live)
        while running:
            if self._hints:
                # (a backend that runs ahead of the host wants to know who certainly ends here)
                goes_on = [len(s.out) + 1 < s.request.max_new_tokens
                           and len(s.request.prompt) + len(s.out) + 1 < be.max_positions for s in running]
                drawn = be.sample(logits, [s.sampling for s in running], may_continue=goes_on)
            else:
                drawn = be.sample(logits, [s.sampling for s in running])
            still: List[_Live] = []
            for s, tok in zip(running, drawn):
                reason = None
                if s.request.max_new_tokens <= 0:
                    reason = "length"
                elif tok in s.request.stop_tokens:
                    reason = "stop"          # not emitted (rocml/src/generate/resumed.rs:217-219)
                else:
                    s.out.append(tok)
                    s.sampling.history.append(tok)
                    self.stats.generated_tokens += 1
                    if self.on_token is not None:
                        self.on_token(s.index, tok)
                    if len(s.out) >= s.request.max_new_tokens:
                        reason = "length"
                    elif len(s.request.prompt) + len(s.out) >= be.max_positions:
                        reason = "context"
                if reason is None:
                    still.append(s)
                else:
                    results[s.index] = Result(s.out, reason, len(s.request.prompt))
                    s.released = True
                    be.release(s.slot)
            running = still
            if running:
                logits = be.step([s.slot for s in running], [[s.out[-1]] for s in running])
                self.stats.decode_steps += 1
                if self.on_step is not None:
                    self.on_step(self.stats.decode_steps)
        be.synchronize()
        self.stats.decode_seconds += time.perf_counter() - t1
