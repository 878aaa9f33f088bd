"""bin/trace_run as a user runs it: a process fed JSON lines, logits files read back and
compared with the plain implementation, for whole requests, tails fed one by one and batches
of unequal lengths whose slots are used again."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from tests import helpers
from tests.plain import qwen3_plain as plain

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def replay(model_dir, dtype, out_dir, steps, max_tokens):
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model_dir, "--dtype", dtype,
           "--out", out_dir, "--max-tokens", str(max_tokens)]
    proc = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    for step in steps:
        proc.stdin.write(json.dumps(step) + "\n")
        proc.stdin.flush()
        line = proc.stdout.readline().strip()
        assert line == f"done {step['step']}", line
    proc.stdin.close()
    assert proc.wait(timeout=60) == 0


def logits_of(out_dir, step, vocab):
    return torch.from_numpy(np.fromfile(os.path.join(out_dir, f"{step}.f32"), dtype="<f4").reshape(-1, vocab))


@pytest.mark.parametrize("name,dtype,tol", [("B", "float32", 2e-5), ("B", "bfloat16", 2e-2), ("H", "bfloat16", 2e-2)])
def test_replay_whole_tail_and_batches(tmp_path, name, dtype, tol):
    cfg, seed = helpers.TINY[name]
    path = helpers.make_model_dir(tmp_path, cfg, seed, torch.float32)
    weights = helpers.read_weights(path)
    if dtype == "bfloat16":
        weights = {k: (v if v.dim() == 1 else v.to(torch.bfloat16).float()) for k, v in weights.items()}
    vocab = cfg["vocab_size"]
    prompts = {rid: helpers.random_tokens(n, vocab, 90 + i) for i, (rid, n) in enumerate([("a", 50), ("b", 7), ("c", 100)])}
    refs = {rid: plain.forward(cfg, weights, p) for rid, p in prompts.items()}
    steps, expect = [], []
    n = 0
    # each request alone and whole
    for rid, p in prompts.items():
        steps.append({"step": n, "entries": [{"id": rid + "w", "tokens": p, "want": list(range(len(p)))}], "end": [rid + "w"]})
        expect.append((n, [(rid, 0, len(p))]))
        n += 1
    # the last 32 tokens one by one
    p = prompts["a"]
    steps.append({"step": n, "entries": [{"id": "t", "tokens": p[:18], "want": [17]}], "end": []})
    expect.append((n, [("a", 17, 18)]))
    n += 1
    for i in range(18, 50):
        steps.append({"step": n, "entries": [{"id": "t", "tokens": [p[i]], "want": [0]}], "end": ["t"] if i == 49 else []})
        expect.append((n, [("a", i, i + 1)]))
        n += 1
    # two batches of unequal lengths; shorter requests end earlier; the second batch reuses what the first gave back
    for order in (["a", "b", "c"], ["c", "b", "a"]):
        cut = {rid: max(1, len(prompts[rid]) - 5 - 2 * j) for j, rid in enumerate(order)}
        steps.append({"step": n, "entries": [{"id": rid, "tokens": prompts[rid][:cut[rid]], "want": [cut[rid] - 1]}
                                             for rid in order], "end": []})
        expect.append((n, [(rid, cut[rid] - 1, cut[rid]) for rid in order]))
        n += 1
        fed = dict(cut)
        live = list(order)
        while live:
            entries = [{"id": rid, "tokens": [prompts[rid][fed[rid]]], "want": [0]} for rid in live]
            for rid in live:
                fed[rid] += 1
            ending = [rid for rid in live if fed[rid] == len(prompts[rid])]
            steps.append({"step": n, "entries": entries, "end": ending})
            expect.append((n, [(rid, fed[rid] - 1, fed[rid]) for rid in live]))
            live = [rid for rid in live if rid not in ending]
            n += 1
    # a step that wants nothing writes no file
    steps.append({"step": n, "entries": [{"id": "z", "tokens": [1, 2, 3], "want": []}], "end": ["z"]})
    out_dir = str(tmp_path / "out")
    replay(path, dtype, out_dir, steps, max_tokens=64 * 5)          # 1 + 1 + 2 pages for a, b, c, and one to spare
    assert not os.path.exists(os.path.join(out_dir, f"{n}.f32"))
    for step, rows in expect:
        got = logits_of(out_dir, step, vocab)
        want = torch.cat([refs[rid][lo:hi] for rid, lo, hi in rows])
        assert got.shape == want.shape
        assert helpers.rel_to_max(got, want) < tol, f"step {step}"
