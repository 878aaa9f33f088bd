"""Another architecture, defined under tests/plugins and registered from there: a configuration
class with keys of its own, tensor names of its own and a mixer with a state of fixed size.  Its
model folder is written, loaded, generated from through the command line and replayed through
bin/trace_run (both as processes of their own that learn of it from ROCML_AMD_PLUGINS), and
stepped through the Python entry point with recorded decode steps: nothing under rocml_amd/
knows of it."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from tests import helpers

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PLUGIN = "tests.plugins.toy_decay_arch"
TOY = {"architectures": ["ToyDecayLM"], "toy_vocab": 211, "toy_width": 64, "toy_depth": 4, "toy_state": 24,
       "toy_inner": 96, "toy_heads": 2, "toy_head": 64, "toy_max_len": 256, "toy_decay": 0.85, "toy_eps": 1e-5}


def _env():
    env = dict(os.environ)
    env["ROCML_AMD_PLUGINS"] = PLUGIN
    env["PYTHONPATH"] = ROOT + os.pathsep + env.get("PYTHONPATH", "")
    return env


@pytest.fixture(scope="module")
def toy(tmp_path_factory):
    import tests.plugins.toy_decay_arch as arch
    from rocml_amd.weights import write_model_dir
    path = write_model_dir(str(tmp_path_factory.mktemp("toy") / "model"), TOY, seed=11, dtype=torch.float32)
    return arch, path, helpers.read_config(path), helpers.read_weights(path)


def test_the_toy_architecture_loads_steps_and_generates(toy):
    from rocml_amd.api import Model
    from rocml_amd.config import known_architectures
    arch, path, raw, weights = toy
    assert "ToyDecayLM" in known_architectures() and raw["toy_state"] == 24 and "tok.weight" in weights
    a, b, c = (helpers.random_tokens(n, raw["toy_vocab"], 30 + n) for n in (40, 9, 70))
    refs = [arch.plain_forward(raw, weights, p) for p in (a, b, c)]
    for dtype, tol in (("float32", 2e-5), ("bfloat16", 2e-2)):
        rounded = (lambda t: t) if dtype == "float32" else (lambda t: t.to(torch.bfloat16).to(t.dtype))
        want = refs if dtype == "float32" else [arch.plain_forward(raw, weights, p, rounded) for p in (a, b, c)]
        model = Model.load(path, dtype=dtype, ctx=128, max_batch=3)
        engine = model.engine
        assert engine.use_graphs and len(engine.cache.state_groups) == 1 and len(engine.cache.kv_groups) == 1
        assert helpers.rel_to_max(helpers.run_whole(engine, a), want[0]) < tol
        # a slot that is handed out again starts from a zero state; decode steps are recorded and replayed
        assert helpers.rel_to_max(helpers.run_tail_by_one(engine, b, 6), want[1]) < tol
        got = helpers.run_batch(engine, [a, b, c], [30, 3, 58])
        for g, w in zip(got, want):
            assert helpers.rel_to_max(g, w) < tol
        assert any(entry[1] is not None for entry in engine._graphs.values())
        engine.cache.check()
    model = Model.load(path, dtype="float32", ctx=128, max_batch=2)
    assert [r.tokens for r in model.generate([a, b], max_new_tokens=7)] == \
        [arch.plain_greedy(raw, weights, p, 7) for p in (a, b)]


def test_the_command_line_and_the_replay_program_run_the_toy_architecture(toy, tmp_path):
    arch, path, raw, weights = toy
    prompt = helpers.random_tokens(12, raw["toy_vocab"], 5)
    cli = [sys.executable, os.path.join(ROOT, "bin", "rocml_amd"), "generate", "--model", path, "--dtype", "float32",
           "--prompt-ids", " ".join(map(str, prompt)), "-n", "6", "--ctx", "64", "--batch", "2"]
    done = subprocess.run(cli, env=_env(), capture_output=True, text=True, timeout=300)
    assert done.returncode == 0, done.stderr
    assert [int(t) for t in done.stdout.strip().splitlines()[-1].split()] == arch.plain_greedy(raw, weights, prompt, 6)
    # without the plugin the architecture is unknown, and the error says which ones are known
    plain_env = {k: v for k, v in _env().items() if k != "ROCML_AMD_PLUGINS"}
    done = subprocess.run(cli, env=plain_env, capture_output=True, text=True, timeout=300)
    assert done.returncode == 1 and "ToyDecayLM" in done.stderr and "Qwen3ForCausalLM" in done.stderr

    tokens = helpers.random_tokens(30, raw["toy_vocab"], 6)
    other = helpers.random_tokens(11, raw["toy_vocab"], 7)
    ref, ref_other = arch.plain_forward(raw, weights, tokens), arch.plain_forward(raw, weights, other)
    out_dir = str(tmp_path / "out")
    proc = subprocess.Popen([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", path, "--dtype", "float32",
                             "--out", out_dir, "--max-tokens", "256"], env=_env(), stdin=subprocess.PIPE,
                            stdout=subprocess.PIPE, text=True)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": tokens[:20], "want": [0, 19]},
                                     {"id": "b", "tokens": other[:9], "want": [8]}], "end": []}]
    for i in range(20, 30):
        entries = [{"id": "a", "tokens": [tokens[i]], "want": [0]}]
        if i - 11 < len(other):
            entries.append({"id": "b", "tokens": [other[i - 11]], "want": [0]})
        steps.append({"step": i - 19, "entries": entries, "end": ["b"] if i - 11 == len(other) - 1 else []})
    for step in steps:
        proc.stdin.write(json.dumps(step) + "\n")
        proc.stdin.flush()
        assert proc.stdout.readline().strip() == f"done {step['step']}"
    proc.stdin.close()
    assert proc.wait(timeout=60) == 0

    def logits(step):
        return torch.from_numpy(np.fromfile(os.path.join(out_dir, f"{step}.f32"), dtype="<f4").reshape(-1, raw["toy_vocab"]))
    assert helpers.rel_to_max(logits(0), torch.stack([ref[0], ref[19], ref_other[8]])) < 2e-5
    for i in range(20, 30):
        want = [ref[i]] + ([ref_other[i - 11]] if i - 11 < len(other) else [])
        assert helpers.rel_to_max(logits(i - 19), torch.stack(want)) < 2e-5, f"step {i - 19}"
