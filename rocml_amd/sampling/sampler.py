"""Draws the next token of every sequence of a batch on the device.

The order of operations is the reference's host sampler (rocml/src/sample.rs:90-166):
repeat penalty over the last ``repeat_penalty_window`` tokens of prompt and output,
greedy when the temperature is not positive, else temperature, top-k, softmax, top-p and
a draw with one uniform number from the sequence's own xorshift64* stream
(rocml/src/sample.rs:56-83).  Logits stay on the device; only the drawn ids come back.
Where candidates tie exactly at the k-th value the lowest ids are kept, top-p keeps all
tokens as probable as the last one it needs, and the draw walks the vocabulary in id
order (the reference walks it in order of probability): the distribution is the same,
the token drawn for a given uniform number may differ.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional, Sequence

import numpy as np
import torch

from .. import ops
from .params import Rng, SamplingParams, sequence_seed


@dataclass
class SequenceSampling:
    """Sampling state of one sequence: its parameters, random stream and history."""
    params: SamplingParams
    rng: Rng
    history: List[int] = field(default_factory=list)

    @staticmethod
    def start(params: SamplingParams, index: int, prompt: Sequence[int]) -> "SequenceSampling":
        return SequenceSampling(params, Rng(sequence_seed(params.seed, index)), list(prompt))


class DeviceSampler:
    def __init__(self, device):
        self.device = torch.device(device)
        self._work: Optional[torch.Tensor] = None
        self._argmax_work: Optional[torch.Tensor] = None
        # the parameters of a call travel in one pinned buffer and one copy (32-bit words, floats
        # and integers side by side), the drawn ids come back through another
        self._stage: Optional[torch.Tensor] = None
        self._stage_dev: Optional[torch.Tensor] = None
        self._ids_host: Optional[torch.Tensor] = None

    def _ids(self, out: torch.Tensor) -> List[int]:
        return self.finish(self._start_copy(out))

    def _start_copy(self, out: torch.Tensor):
        batch = out.numel()
        if self._ids_host is None or self._ids_host.numel() < batch:
            self._ids_host = torch.empty(max(batch, 64), dtype=torch.int32, pin_memory=True)
        host = self._ids_host[:batch]
        host.copy_(out, non_blocking=True)
        done = torch.cuda.Event()
        done.record(torch.cuda.current_stream(self.device))
        return out, host, done

    def finish(self, started) -> List[int]:
        """Waits for the ids of ``sample_start`` to reach the host and returns them."""
        _, host, done = started
        done.synchronize()
        return host.tolist()

    def sample(self, logits: torch.Tensor, seqs: Sequence[SequenceSampling]) -> List[int]:
        """``logits`` is ``[B, V]`` 32-bit on the device, row ``b`` for ``seqs[b]``.  Returns
        the drawn ids and appends them to nothing: the caller decides what a token means."""
        return self.finish(self.sample_start(logits, seqs))

    def sample_start(self, logits: torch.Tensor, seqs: Sequence[SequenceSampling]):
        """Launches the sampling and the copy of the drawn ids to the host without waiting for
        either; ``finish`` waits.  The first element of what it returns is the ids on the device
        (int32 ``[B]``), which work launched meanwhile may read."""
        batch, vocab = logits.shape
        assert batch == len(seqs)
        out = torch.empty(batch, dtype=torch.int32, device=self.device)
        if all(s.params.is_greedy() and not s.params.penalty_active() for s in seqs):
            if self._argmax_work is None or self._argmax_work.numel() < batch * ops.ARGMAX_WORK_WORDS:
                self._argmax_work = torch.empty(max(batch, 64) * ops.ARGMAX_WORK_WORDS, dtype=torch.int32, device=self.device)
            ops.argmax(logits, out, self._argmax_work)
            return self._start_copy(out)
        if self._work is None or self._work.numel() < logits.numel():
            self._work = torch.empty(logits.numel(), dtype=torch.float32, device=self.device)
        window = max([s.params.repeat_penalty_window for s in seqs if s.params.penalty_active()] + [1])
        words = batch * (6 + window)
        if self._stage is None or self._stage.numel() < words:
            self._stage = torch.empty(2 * words, dtype=torch.int32, pin_memory=True)
            self._stage_dev = torch.empty(2 * words, dtype=torch.int32, device=self.device)
        stage = self._stage[:words].numpy()
        stage[:] = 0
        temperature, uniform, top_p, penalty = (stage[i * batch:(i + 1) * batch].view(np.float32) for i in range(4))
        top_k, hist_len = stage[4 * batch:5 * batch], stage[5 * batch:6 * batch]
        hist = stage[6 * batch:].reshape(batch, window)
        top_p[:] = -1.0
        for b, s in enumerate(seqs):
            p = s.params
            if p.penalty_active():
                recent = s.history[-p.repeat_penalty_window:] if p.repeat_penalty_window > 0 else []
                penalty[b] = p.repeat_penalty
                hist[b, :len(recent)] = recent
                hist_len[b] = len(recent)
            if p.is_greedy():
                continue
            temperature[b] = p.temperature
            top_k[b] = 0 if p.top_k is None else max(1, int(p.top_k))
            top_p[b] = -1.0 if p.top_p is None else min(max(float(p.top_p), 0.0), 1.0)
            uniform[b] = s.rng.next_f32()
        # every drawing sequence with a small top-k: the selection may run on slices of the row
        drawing = top_k[temperature > 0]
        small_k = int(drawing.max()) if drawing.size and drawing.min() >= 1 and drawing.max() <= ops.SAMPLE_SMALL_K else 0
        dev = self._stage_dev[:words]
        dev.copy_(self._stage[:words], non_blocking=True)
        floats = dev[:4 * batch].view(torch.float32)
        ops.sample(logits, self._work, floats[:batch], floats[batch:2 * batch], out,
                   top_k=dev[4 * batch:5 * batch], top_p=floats[2 * batch:3 * batch],
                   penalty=floats[3 * batch:4 * batch], history=dev[6 * batch:].view(batch, window),
                   history_len=dev[5 * batch:6 * batch], small_k=small_k)
        return self._start_copy(out)
