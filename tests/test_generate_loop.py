"""The generation loop's decisions with a scripted backend (no GPU): batches, stop tokens,
sequences that end earlier, slots given back and used again, limits."""
from typing import Dict, List

import pytest

from rocml_amd.engine.generate import Generator, Request
from rocml_amd.errors import CacheFullError, RocmlError
from rocml_amd.sampling import Rng, SamplingParams, sequence_seed


class Scripted:
    """Next token of a sequence = (sum of its tokens so far) % 50; counts what it is asked."""

    def __init__(self, max_positions=1000, slots=4, room=10_000):
        self.max_positions = max_positions
        self.free_slots = list(range(slots))
        self.room = room
        self.history: Dict[int, List[int]] = {}
        self.steps: List[List[int]] = []          # slots of each step
        self.step_tokens: List[List[List[int]]] = []
        self.released: List[int] = []

    def can_admit(self, lengths, prompts=None):
        return len(lengths) <= len(self.free_slots) and sum(lengths) <= self.room

    def new_sequence(self):
        s = self.free_slots.pop(0)
        self.history[s] = []
        return s

    def release(self, slot):
        assert slot in self.history, "released twice"
        del self.history[slot]
        self.released.append(slot)
        self.free_slots.insert(0, slot)

    def step(self, slots, tokens):
        assert len(set(slots)) == len(slots)
        self.steps.append(list(slots))
        self.step_tokens.append([list(t) for t in tokens])
        for s, t in zip(slots, tokens):
            self.history[s].extend(t)
        return [sum(self.history[s]) % 50 for s in slots]

    def sample(self, logits, seqs):
        return list(logits)

    def synchronize(self):
        pass


def _expected(prompt, n, stop=()):
    toks, out = list(prompt), []
    for _ in range(n):
        t = sum(toks) % 50
        if t in stop:
            return out, "stop"
        out.append(t)
        toks.append(t)
    return out, "length"


def test_unequal_prompts_end_at_different_times():
    be = Scripted()
    reqs = [Request([1, 2, 3], 5), Request([4], 2), Request([7, 7, 7, 7, 7, 7], 8), Request([9, 1], 1)]
    res = Generator(be, max_batch=4).run(reqs)
    for r, q in zip(res, reqs):
        assert (r.tokens, r.finish_reason) == _expected(q.prompt, q.max_new_tokens)
        assert r.prompt_tokens == len(q.prompt)
    assert be.steps[0] == [0, 1, 2, 3] and be.step_tokens[0] == [[1, 2, 3], [4], [7] * 6, [9, 1]]
    assert be.steps[1] == [0, 1, 2]              # the request with one new token has left
    assert be.steps[2] == [0, 2]
    assert all(len(t) == 1 for step in be.step_tokens[1:] for t in step)     # one token each afterwards
    assert len(be.steps) == 8                    # prompt step + 7 more for the longest (no step after its last token)
    assert sorted(be.released) == [0, 1, 2, 3] and not be.history


def test_stop_token_is_not_emitted_and_frees_the_slot():
    full, _ = _expected([5, 6], 10)
    stop = full[3]
    want, reason = _expected([5, 6], 10, stop=[stop])
    be = Scripted()
    res = Generator(be).run([Request([5, 6], 10, stop_tokens=frozenset([stop])), Request([1], 10)])
    assert (res[0].tokens, res[0].finish_reason) == (want, "stop") and stop not in res[0].tokens
    assert res[1].finish_reason == "length" and len(res[1].tokens) == 10
    gone = len(want) + 1                          # steps in which the first sequence took part
    assert all(0 in s for s in be.steps[:gone]) and all(0 not in s for s in be.steps[gone:])


def test_every_token_is_handed_out_as_it_is_drawn():
    """``on_token`` sees every emitted token of every request once, in the order they were drawn
    (a step's tokens in the order of the batch), and never a stop token."""
    full, _ = _expected([5, 6], 10)
    stop = full[3]
    reqs = [Request([5, 6], 10, stop_tokens=frozenset([stop])), Request([1], 4), Request([], 3), Request([2, 2], 6)]
    seen = []
    gen = Generator(Scripted(slots=2), max_batch=2)
    gen.on_token = lambda index, token: seen.append((index, token))
    res = gen.run(reqs)
    for i, r in enumerate(res):
        assert [t for j, t in seen if j == i] == r.tokens
    assert stop not in [t for j, t in seen if j == 0] and len(seen) == sum(len(r.tokens) for r in res)
    firsts = [j for j, _ in seen[:2]]
    assert firsts == [0, 1]                       # the first step's tokens in the order of the batch


def test_batches_follow_slots_and_room_and_reuse_slots():
    be = Scripted(slots=2)
    reqs = [Request([i + 1], 3) for i in range(5)]
    res = Generator(be, max_batch=8).run(reqs)
    assert [r.tokens for r in res] == [_expected(q.prompt, 3)[0] for q in reqs]
    assert sorted(be.steps[0]) == [0, 1] and sorted(be.steps[3]) == [0, 1] and len(be.steps[6]) == 1    # three batches
    assert be.released.count(0) == 3 and be.released.count(1) == 2
    be = Scripted(slots=8, room=20)               # room for prompt + output of two requests at a time
    gen = Generator(be, max_batch=8)
    gen.run([Request([1] * 4, 5)] * 5)
    assert gen.stats.batches == 3
    with pytest.raises(CacheFullError):
        Generator(Scripted(room=5)).run([Request([1] * 4, 5)])
    be = Scripted()
    Generator(be, max_batch=1).run([Request([1], 1), Request([2], 1)])
    assert [len(s) for s in be.steps] == [1, 1]


def test_limits_and_empty_prompts():
    be = Scripted(max_positions=6)
    res = Generator(be).run([Request([1, 2, 3, 4], 10), Request([], 5), Request([3], 0)])
    assert res[0].finish_reason == "context" and len(res[0].tokens) == 2      # 4 + 2 = 6 positions
    assert res[1].finish_reason == "empty" and res[1].tokens == []
    assert res[2].finish_reason == "length" and res[2].tokens == []
    with pytest.raises(RocmlError, match="positions"):
        Generator(be).run([Request([1] * 7, 1)])
    with pytest.raises(RocmlError):
        Generator(be, max_batch=0)


def test_rng_matches_the_reference_generator():
    # xorshift64* (rocml/src/sample.rs:56-83), first outputs for seed 1 computed by hand from
    # the definition: x ^= x >> 12; x ^= x << 25; x ^= x >> 27; out = x * 0x2545F4914F6CDD1D.
    r = Rng(1)
    x = 1
    x ^= x >> 12
    x ^= (x << 25) & (2 ** 64 - 1)
    x ^= x >> 27
    assert r.next_u64() == (x * 0x2545F4914F6CDD1D) % 2 ** 64
    assert Rng(0).state == 0x9E3779B97F4A7C15
    draws = [Rng(42).next_f32() for _ in range(3)]
    assert draws[0] == draws[1] == draws[2] and 0.0 <= draws[0] < 1.0
    r = Rng(7)
    vals = [r.next_f32() for _ in range(2000)]
    assert 0.45 < sum(vals) / len(vals) < 0.55 and all(v * 2 ** 24 == int(v * 2 ** 24) for v in vals)
    assert sequence_seed(5, 0) == 5 and len({sequence_seed(5, i) for i in range(100)}) == 100
    assert SamplingParams().is_greedy() and not SamplingParams(temperature=0.7).is_greedy()
    assert not SamplingParams(repeat_penalty=1.0).penalty_active() and SamplingParams(repeat_penalty=1.1).penalty_active()


def test_profile_report_rows_and_roofline_columns():
    """The per-operation report from raw records: time share, rates, analytical minimum
    t_min = max(bytes / bandwidth, flops / peak), efficiency and wasted time per row
    (rocml/src/profile/report.rs:21-75), phases apart, worklist by wasted time."""
    from rocml_amd.profile import HBM_BYTES_PER_S, build_report
    peak = 2.5e15
    records = [("decode", "product", 8_000_000_000, 1_000_000, 2.0),       # memory bound: t_min 1 ms
               ("decode", "product", 8_000_000_000, 1_000_000, 2.0),
               ("decode", "rmsnorm", 80_000, 0, 0.5),
               ("prefill", "product", 1_000, 5_000_000_000_000, 4.0)]      # compute bound: t_min 2 ms
    rep = build_report(records, peak)
    assert [p.phase for p in rep.phases] == ["prefill", "decode"]
    dec = rep.phases[1]
    assert dec.total_elapsed_ms == 4.5 and [r.label for r in dec.by_op] == ["product", "rmsnorm"]
    prod = dec.by_op[0]
    assert prod.count == 2 and prod.bytes == 16_000_000_000
    assert abs(prod.t_min_ms - 1e3 * 16e9 / HBM_BYTES_PER_S) < 1e-9 and abs(prod.efficiency - 0.5) < 1e-9
    assert abs(prod.wasted_ms - 2.0) < 1e-9 and abs(prod.gb_per_sec - 4000.0) < 1e-6
    assert abs(prod.pct_of_bandwidth_roofline - 50.0) < 1e-9 and abs(prod.pct_of_phase_time - 100 * 4 / 4.5) < 1e-9
    pre = rep.phases[0].by_op[0]
    assert abs(pre.t_min_ms - 2.0) < 1e-9 and abs(pre.pct_of_flop_roofline - 50.0) < 1e-9
    assert rep.worklist[0].startswith("decode product") or rep.worklist[0].startswith("prefill product")
    assert "t_min ms" in rep.to_human() and "report" in rep.to_json()


def test_profiler_wraps_the_launch_helpers_only_while_it_is_active():
    import torch
    from rocml_amd import ops, profile
    before = {name: getattr(ops, name) for name in ("gemm", "rmsnorm", "attention", "sample")}
    assert profile.active() is None
    with profile.OpProfiler(torch.float32) as p:
        assert profile.active() is p and ops.gemm is not before["gemm"]
        profile.set_phase("decode")
        assert p.phase == "decode"
        with pytest.raises(RuntimeError):
            profile.OpProfiler().__enter__()
    assert profile.active() is None
    assert all(getattr(ops, name) is fn for name, fn in before.items())
    profile.set_phase("prefill")                     # without a profiler: nothing to tag


# ---- the engine's backend running ahead of the host (no GPU: a scripted engine and sampler) -------
class _FakeCache:
    def __init__(self, slots):
        self.free = list(range(slots))

    class _Slots:
        def __init__(self, outer):
            self.outer = outer

        @property
        def n_free(self):
            return len(self.outer.free)

    @property
    def slots(self):
        return _FakeCache._Slots(self)

    def fits(self, pieces, final=None):
        return None


class _FakeEngine:
    """Next-token rule of ``Scripted``; a step may take its ids from a tensor 'on the device'."""

    def __init__(self, slots=4, max_positions=1000):
        import types
        self.model = types.SimpleNamespace(spec=types.SimpleNamespace(max_positions=max_positions), device="cpu")
        self.cache = _FakeCache(slots)
        self.history = {}
        self.steps = []

    def plan_pieces(self, counts):
        return [[(i, 0, c) for i, c in enumerate(counts)]]

    def new_sequence(self):
        s = self.cache.free.pop(0)
        self.history[s] = []
        return s

    def release(self, slot):
        del self.history[slot]
        self.cache.free.insert(0, slot)

    def step(self, entries, device_ids=None):
        import torch
        self.steps.append(([e.slot for e in entries], device_ids is not None))
        rows = []
        for i, e in enumerate(entries):
            toks = [int(device_ids[i])] if device_ids is not None else list(e.tokens)
            if len(self.history[e.slot]) + len(toks) > self.model.spec.max_positions:
                raise RocmlError("context")
            self.history[e.slot].extend(toks)
            rows.append([float(sum(self.history[e.slot]) % 50)])
        return torch.tensor(rows)


class _FakeSampler:
    def sample(self, logits, seqs):
        return self.finish(self.sample_start(logits, seqs))

    def sample_start(self, logits, seqs):
        import torch
        ids = logits[:, 0].to(torch.int32)
        return ids, ids.clone(), None

    def finish(self, started):
        return started[1].tolist()


@pytest.mark.parametrize("run_ahead", [True, False])
def test_the_backend_may_run_ahead_of_the_host_without_changing_a_token(run_ahead):
    from rocml_amd.engine.generate import EngineBackend
    reqs = [Request([1, 2, 3], 5), Request([4], 2, stop_tokens=frozenset({9})), Request([7] * 6, 8), Request([9, 1], 1),
            Request([5, 6], 10, stop_tokens=frozenset(_expected([5, 6], 10)[0][3:4])),
            Request([3], 4), Request([8], 3), Request([2], 6)]               # prompts of one token on slots used before
    want = Generator(Scripted(), max_batch=3).run(reqs)
    engine = _FakeEngine(slots=3)
    got = Generator(EngineBackend(engine, sampler=_FakeSampler(), run_ahead=run_ahead), max_batch=3).run(reqs)
    assert [(r.tokens, r.finish_reason) for r in got] == [(r.tokens, r.finish_reason) for r in want]
    assert not engine.history and sorted(engine.cache.free) == [0, 1, 2]
    ahead = [slots for slots, from_device in engine.steps if from_device]
    assert bool(ahead) == run_ahead
    if run_ahead:
        # a sequence is only run ahead when it may go on: the only tokens run for nothing are
        # those behind a stop token (one request above stops on one)
        ran = sum(len(s) for s in ahead)
        useful = sum(len(r.tokens) - 1 for r in want if r.tokens)          # every token but the last is run through the model
        assert useful <= ran <= useful + 2


def test_running_ahead_stops_at_the_models_last_position():
    from rocml_amd.engine.generate import EngineBackend
    engine = _FakeEngine(slots=2, max_positions=6)
    got = Generator(EngineBackend(engine, sampler=_FakeSampler()), max_batch=2).run([Request([1, 2, 3], 10), Request([4], 3)])
    want = Generator(Scripted(max_positions=6), max_batch=2).run([Request([1, 2, 3], 10), Request([4], 3)])
    assert [(r.tokens, r.finish_reason) for r in got] == [(r.tokens, r.finish_reason) for r in want]
    assert got[0].finish_reason == "context" and all(len(h) <= 6 for h in engine.history.values())


def test_a_step_that_does_not_continue_the_one_launched_ahead_is_refused():
    """After sampling with run-ahead the sequences are one token further already: a next step for
    only some of them with others beside, or with another token than the one drawn, would advance
    them twice or feed them something they were not run with; the backend says so."""
    import torch
    from rocml_amd.engine.generate import EngineBackend
    from rocml_amd.sampling import SamplingParams
    from rocml_amd.sampling.sampler import SequenceSampling

    def start():
        engine = _FakeEngine(slots=3)
        backend = EngineBackend(engine, sampler=_FakeSampler())
        slots = [backend.new_sequence() for _ in range(3)]
        logits = backend.step(slots[:2], [[1, 2], [3]])
        seqs = [SequenceSampling(SamplingParams.greedy(), None, []) for _ in range(2)]
        drawn = backend.sample(logits, seqs, [True, True])
        return backend, slots, drawn

    backend, slots, drawn = start()
    assert backend.step(slots[:2], [[drawn[0]], [drawn[1]]]).shape[0] == 2        # the step that was launched
    backend, slots, drawn = start()
    assert backend.step(slots[1:2], [[drawn[1]]]).shape[0] == 1                   # a subset: its rows are picked
    backend, slots, drawn = start()
    with pytest.raises(RocmlError, match="launched ahead"):
        backend.step(slots[1:3], [[drawn[1]], [5]])                                # one ran ahead, one did not
    backend, slots, drawn = start()
    with pytest.raises(RocmlError, match="run ahead with token"):
        backend.step(slots[:2], [[drawn[0]], [drawn[1] + 1]])
    backend, slots, drawn = start()
    with pytest.raises(RocmlError, match="launched ahead"):
        backend.step(slots[:1], [[drawn[0], 4]])                                   # more than the one token
    backend, slots, drawn = start()
    backend.release(slots[0])
    backend.release(slots[1])
    s = backend.new_sequence()                                                      # a slot that ran ahead, now another sequence
    assert backend.step([s], [[1, 2, 3]]).shape[0] == 1
