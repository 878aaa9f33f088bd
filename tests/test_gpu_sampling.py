"""The sampling kernels against the reference's rules (rocml/src/sample.rs:90-202), written
out plainly here: penalty, greedy on temperature <= 0, temperature, top-k, softmax, top-p,
draw.  Its own tests fix the cases: temperature 0 and top_k = 1 are argmax, draws stay inside
the top-k set and the nucleus, a seed repeats its draws (rocml/src/sample.rs:214-295)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from rocml_amd import ops  # noqa: E402
from rocml_amd.sampling import DeviceSampler, SamplingParams, SequenceSampling  # noqa: E402


def candidates(logits, temperature, top_k, top_p, penalty=None, history=(), window=64):
    """Probabilities (float64, 0 outside the candidate set) after every filter."""
    v = np.asarray(logits, dtype=np.float64).copy()
    if penalty:
        for t in list(history)[-window:]:
            v[t] = v[t] / penalty if v[t] > 0 else v[t] * penalty
    if temperature <= 0:
        p = np.zeros_like(v)
        p[int(np.argmax(v))] = 1.0
        return p
    v = v / temperature
    keep = np.ones(len(v), dtype=bool)
    if top_k is not None and top_k < len(v):
        order = np.lexsort((np.arange(len(v)), -v))      # by value descending, then by index
        keep[:] = False
        keep[order[:max(1, top_k)]] = True
    p = np.where(keep, np.exp(v - v[keep].max()), 0.0)
    if top_p is not None and top_p < 1.0:
        order = np.argsort(-p, kind="stable")
        cum = np.cumsum(p[order])
        cut = int(np.searchsorted(cum, top_p * p.sum() - 1e-12)) + 1
        last = p[order[cut - 1]]
        p = np.where(p >= last, p, 0.0)                    # ties with the last one stay
    return p


def test_argmax_takes_the_first_maximum():
    logits = torch.randn(5, 1000)
    logits[0, 17] = logits[0, 400] = 9.0                   # a tie: the lower id wins
    logits[1, 999] = 9.0
    logits[2, 0] = 9.0
    logits[3] = 1.0
    out = torch.empty(5, dtype=torch.int32, device="cuda")
    ops.argmax(logits.cuda(), out)
    assert out.cpu().tolist() == [17, 999, 0, 0, int(logits[4].argmax())]
    # long rows take the two-stage path: the first maximum still wins, across pieces too
    long = torch.randn(3, 151936)
    long[0, 5000] = long[0, 140000] = 50.0
    long[1, 151935] = 50.0
    work = torch.empty(3 * ops.ARGMAX_WORK_WORDS, dtype=torch.int32, device="cuda")
    out = torch.empty(3, dtype=torch.int32, device="cuda")
    ops.argmax(long.cuda(), out, work)
    assert out.cpu().tolist() == [5000, 151935, int(long[2].argmax())]


def _draw(logits, params_list, us, histories=None):
    sampler = DeviceSampler("cuda:0")
    seqs = []
    for i, p in enumerate(params_list):
        s = SequenceSampling.start(p, i, histories[i] if histories else [])

        class Fixed:                                       # a stream that returns the given number
            def __init__(self, u):
                self.u = u

            def next_f32(self):
                return self.u
        s.rng = Fixed(us[i])
        seqs.append(s)
    return sampler.sample(logits.cuda(), seqs)


def test_temperature_zero_and_top_k_one_are_argmax():
    g = torch.Generator().manual_seed(0)
    logits = torch.randn(4, 517, generator=g)
    want = logits.argmax(dim=1).tolist()
    assert _draw(logits, [SamplingParams()] * 4, [0.3] * 4) == want
    assert _draw(logits, [SamplingParams(temperature=0.8, top_k=1)] * 4, [0.1, 0.5, 0.9, 0.999]) == want
    mixed = [SamplingParams(), SamplingParams(temperature=1.0, top_k=1), SamplingParams(temperature=-1.0), SamplingParams()]
    assert _draw(logits, mixed, [0.7] * 4) == want


@pytest.mark.parametrize("params", [
    SamplingParams(temperature=0.7), SamplingParams(temperature=1.3, top_k=20),
    SamplingParams(temperature=0.6, top_k=20, top_p=0.95), SamplingParams(temperature=1.0, top_p=0.5),
    SamplingParams(temperature=0.9, top_k=5, repeat_penalty=1.3), SamplingParams(temperature=2.0, top_p=0.0)])
def test_draws_follow_the_filtered_distribution(params):
    g = torch.Generator().manual_seed(1)
    vocab, batch = 1531, 64
    logits = torch.randn(1, vocab, generator=g) * 2.5
    history = [int(t) for t in torch.randint(0, vocab, (80,), generator=g)] + [int(logits.argmax())]
    p = candidates(logits[0].numpy(), params.temperature, params.top_k, params.top_p,
                   params.repeat_penalty, history, params.repeat_penalty_window)
    cum = np.cumsum(p)
    us = [(i + 0.37) / batch for i in range(batch)]
    got = _draw(logits.expand(batch, vocab).contiguous(), [params] * batch, us, [history] * batch)
    for u, tok in zip(us, got):
        assert p[tok] > 0, f"token {tok} is outside the candidate set"
        t = u * cum[-1]
        lo = cum[tok] - p[tok]
        assert lo - 1e-4 * cum[-1] <= t <= cum[tok] + 1e-4 * cum[-1], (u, tok)
    if params.top_k:
        assert len(set(got)) <= params.top_k
    if params.top_p == 0.0:
        assert len(set(got)) == 1                          # the nucleus keeps at least one token


@pytest.mark.parametrize("vocab", [700, 5000, 151936, 300001])
@pytest.mark.parametrize("params", [
    SamplingParams(temperature=0.9, top_k=1), SamplingParams(temperature=0.9, top_k=7, top_p=0.8),
    SamplingParams(temperature=1.4, top_k=64, top_p=0.97, repeat_penalty=1.3),
    SamplingParams(temperature=1.4, top_k=65, top_p=0.97, repeat_penalty=1.3)])
def test_small_top_k_on_slices_of_the_row(vocab, params):
    """A top-k of at most 64 is selected on slices of the vocabulary and merged by one wave, 65
    by the kernel that walks whole rows: both against the plain rule, at vocabularies of one
    slice, of a few, of many, and beyond the size where the slices grow."""
    g = torch.Generator().manual_seed(vocab % 97)
    batch = 32
    logits = torch.randn(1, vocab, generator=g) * 2.0
    logits[0, vocab - 1] = logits[0].max() + 0.5          # the last token of the last slice is a candidate
    history = [int(t) for t in logits[0].topk(12).indices] * 2 + [int(t) for t in torch.randint(0, vocab, (30,), generator=g)]
    p = candidates(logits[0].numpy(), params.temperature, params.top_k, params.top_p,
                   params.repeat_penalty, history, params.repeat_penalty_window)
    cum = np.cumsum(p)
    us = [(i + 0.61) / batch for i in range(batch)]
    got = _draw(logits.expand(batch, vocab).contiguous(), [params] * batch, us, [history] * batch)
    for u, tok in zip(us, got):
        assert p[tok] > 0, f"token {tok} is outside the candidate set"
        t = u * cum[-1]
        assert cum[tok] - p[tok] - 1e-4 * cum[-1] <= t <= cum[tok] + 1e-4 * cum[-1], (u, tok)
    assert len(set(got)) <= params.top_k


def test_ties_at_the_kth_value_keep_the_lowest_ids():
    logits = torch.full((1, 300), -5.0)
    logits[0, [10, 50, 90, 130]] = 2.0                      # four equal candidates, k = 2
    got = set(_draw(logits.expand(32, 300).contiguous(), [SamplingParams(temperature=1.0, top_k=2)] * 32,
                    [(i + 0.5) / 32 for i in range(32)]))
    assert got == {10, 50}


def test_the_two_zeros_tie():
    """-0.0 and +0.0 are one value: among them the lowest ids are kept, whatever their signs."""
    logits = torch.full((1, 200), -3.0)
    zeros = [4, 9, 20, 33, 61, 150]
    logits[0, zeros] = torch.tensor([-0.0, 0.0, -0.0, 0.0, 0.0, -0.0])
    got = set(_draw(logits.expand(32, 200).contiguous(), [SamplingParams(temperature=1.3, top_k=3)] * 32,
                    [(i + 0.5) / 32 for i in range(32)]))
    assert got == {4, 9, 20}
    logits[logits < -1] = -30.0
    got = set(_draw(logits.expand(32, 200).contiguous(), [SamplingParams(temperature=1.3, top_k=50, top_p=0.5)] * 32,
                    [(i + 0.5) / 32 for i in range(32)]))
    assert got == set(zeros)                                # ties with the nucleus' last value stay


def test_penalty_changes_the_greedy_choice():
    logits = torch.zeros(1, 50)
    logits[0, 7], logits[0, 9] = 3.0, 2.9
    assert _draw(logits, [SamplingParams(repeat_penalty=1.5)], [0.0], [[7]]) == [9]
    assert _draw(logits, [SamplingParams(repeat_penalty=1.5)], [0.0], [[7] + [1] * 64]) == [7]   # outside the window
    assert _draw(logits, [SamplingParams(repeat_penalty=1.0)], [0.0], [[7]]) == [7]


def test_penalty_with_a_long_history_in_a_large_vocabulary():
    """More flagged tokens than the kernel sets aside for later, and a history longer than its
    copy in LDS: the penalised maximum and the draws must still be the plain rule's."""
    g = torch.Generator().manual_seed(5)
    vocab, window = 700001, 600
    logits = torch.randn(2, vocab, generator=g) * 2.0
    top = [int(t) for t in logits[0].topk(300).indices]           # the best tokens are all penalised
    history = top + [int(t) for t in torch.randint(0, vocab, (300,), generator=g)]
    greedy = SamplingParams(repeat_penalty=1.7, repeat_penalty_window=window)
    want = [int(np.argmax(np.where(candidates(logits[r].numpy(), 0.0, None, None, 1.7, history, window) > 0, 1, 0)))
            for r in range(2)]
    assert _draw(logits, [greedy] * 2, [0.0] * 2, [history] * 2) == want
    assert want[0] not in top[:50]
    draw = SamplingParams(temperature=0.8, top_k=40, repeat_penalty=1.7, repeat_penalty_window=window)
    p = candidates(logits[0].numpy(), 0.8, 40, None, 1.7, history, window)
    got = _draw(logits[:1].expand(16, vocab).contiguous(), [draw] * 16, [(i + 0.5) / 16 for i in range(16)], [history] * 16)
    assert all(p[t] > 0 for t in got) and len(set(got)) > 4


def test_same_seed_same_draws_and_own_stream_per_sequence():
    g = torch.Generator().manual_seed(3)
    logits = torch.randn(3, 700, generator=g)
    sampler = DeviceSampler("cuda:0")
    p = SamplingParams(temperature=1.0, seed=11)

    def run(indices):
        seqs = [SequenceSampling.start(p, i, []) for i in indices]
        rows = logits[indices].cuda()
        return [sampler.sample(rows, seqs) for _ in range(5)]
    a, b = run([0, 1, 2]), run([0, 1, 2])
    assert a == b
    alone = run([1])
    assert [step[1] for step in a] == [step[0] for step in alone]     # batching does not change a sequence's draws
