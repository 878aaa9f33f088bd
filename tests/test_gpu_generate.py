"""Generation through the Python entry point against the plain implementation: greedy
tokens, stop tokens, more requests than fit one batch (slots are used again), long
decoding, the first tokens of a sequence, seeded temperature sampling."""
import pytest
import torch

from tests import helpers
from tests.plain import qwen3_plain as plain

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    root = tmp_path_factory.mktemp("gen_models")
    out = {}
    for name, (cfg, seed) in helpers.TINY.items():
        path = helpers.make_model_dir(root, cfg, seed, torch.float32)
        out[name] = (path, helpers.read_config(path), helpers.read_weights(path))
    return out


def _load(path, dtype, **kw):
    from rocml_amd.api import Model
    return Model.load(path, dtype=dtype, **kw)


def near_tie(cfg, weights, prompt, produced, k):
    """The reference's rule for a greedy flip (rocml/tests/greedy_parity.rs:33-34,158-160):
    acceptable only where the two best logits of the plain run are within 1e-2 of each
    other, relative to the larger."""
    logits = plain.forward(cfg, weights, list(prompt) + list(produced[:k]))[-1]
    top = torch.topk(logits, 2).values
    return float((top[0] - top[1]).abs() / top[0].abs().clamp_min(1e-9)) < 1e-2


@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E"])
def test_greedy_float32_matches_token_for_token(models, name):
    path, cfg, weights = models[name]
    model = _load(path, "float32", ctx=256, max_batch=3)
    lengths = [5, 9, 13, 1, 30, 2, 64]
    prompts = [helpers.random_tokens(n, cfg["vocab_size"], 40 + i) for i, n in enumerate(lengths)]
    want = [plain.greedy(cfg, weights, p, 8) for p in prompts]
    got = model.generate(prompts, max_new_tokens=8)            # 7 requests, 3 slots: three batches
    assert [r.tokens for r in got] == want
    assert all(r.finish_reason == "length" for r in got)
    assert model.last_stats.batches == 3 and model.last_stats.generated_tokens == 56
    model.engine.cache.check()
    assert not model.engine.cache.lengths
    # a stop token ends its sequence early and is not emitted; the others go on
    stop = want[2][3]
    got = model.generate(prompts[:3], max_new_tokens=8, stop_tokens=[stop])
    for r, w, p in zip(got, want, prompts):
        ref = plain.greedy(cfg, weights, p, 8, stop=[stop])
        assert r.tokens == ref and r.finish_reason == ("stop" if len(ref) < 8 else "length")


@pytest.mark.parametrize("name", ["B", "D"])
def test_greedy_bfloat16_flips_only_at_near_ties(models, name):
    path, cfg, weights = models[name]
    rounded = {k: (v if v.dim() == 1 else v.to(torch.bfloat16).float()) for k, v in weights.items()}
    model = _load(path, "bfloat16", ctx=128, max_batch=4)
    prompts = [helpers.random_tokens(n, cfg["vocab_size"], 60 + i) for i, n in enumerate([1, 7, 16, 33])]
    got = [r.tokens for r in model.generate(prompts, max_new_tokens=12)]
    for p, g in zip(prompts, got):
        assert len(g) == 12
        w = plain.greedy(cfg, rounded, p, 12)
        if g != w:
            k = next(i for i in range(12) if g[i] != w[i])
            assert near_tie(cfg, rounded, p, w, k), f"tokens differ at {k} without a near tie: {g} vs {w}"


@pytest.mark.parametrize("dtype,tol", [("float32", 2e-5), ("bfloat16", 2e-2)])
def test_long_decoding_and_first_tokens(models, dtype, tol):
    from rocml_amd.engine import StepEntry
    path, cfg, weights = models["D"]               # window of 70: decoding crosses pages and the window's edge
    w = weights if dtype == "float32" else {k: (v if v.dim() == 1 else v.to(torch.bfloat16).float()) for k, v in weights.items()}
    model = _load(path, dtype, ctx=512, max_batch=2)
    toks = helpers.random_tokens(260, cfg["vocab_size"], 77)
    ref = plain.forward(cfg, w, toks)
    eng = model.engine
    slot = eng.new_sequence()
    rows = [eng.step([StepEntry(slot, toks[:3], [0, 1, 2])]).cpu()]
    for t in toks[3:]:
        rows.append(eng.step([StepEntry(slot, [t], [0])]).cpu())
    eng.release(slot)
    got = torch.cat(rows)
    assert helpers.rel_to_max(got, ref) < tol
    assert helpers.rel_to_max(got[:3], ref[:3]) < tol          # the first tokens of a sequence
    # one token at a time from the very first token
    slot = eng.new_sequence()
    rows = [eng.step([StepEntry(slot, [t], [0])]).cpu() for t in toks[:5]]
    eng.release(slot)
    assert helpers.rel_to_max(torch.cat(rows), ref[:5]) < tol


def test_temperature_sampling_is_seeded_and_ignores_batching(models):
    from rocml_amd.sampling import SamplingParams
    path, cfg, weights = models["B"]
    prompts = [helpers.random_tokens(n, cfg["vocab_size"], 80 + i) for i, n in enumerate([1, 7, 16, 33])]
    params = SamplingParams(temperature=0.7, seed=1)
    together = _load(path, "float32", ctx=128, max_batch=4)
    a = [r.tokens for r in together.generate(prompts, params, max_new_tokens=12)]
    b = [r.tokens for r in together.generate(prompts, params, max_new_tokens=12)]
    assert a == b
    one_by_one = _load(path, "float32", ctx=128, max_batch=1)
    c = [r.tokens for r in one_by_one.generate(prompts, params, max_new_tokens=12)]
    assert a == c                                                # batches of one draw the same tokens
    d = [r.tokens for r in together.generate(prompts, SamplingParams(temperature=0.7, seed=2), max_new_tokens=12)]
    assert a != d
    greedy = [r.tokens for r in together.generate(prompts, max_new_tokens=12)]
    assert a != greedy


def test_command_line_generate_and_models(models, capsys):
    from rocml_amd.cli import main
    path, cfg, weights = models["A"]
    prompt = helpers.random_tokens(6, cfg["vocab_size"], 5)
    rc = main(["generate", "--model", path, "--dtype", "float32", "--prompt-ids", " ".join(map(str, prompt)),
               "-n", "5", "--ctx", "64", "--batch", "2"])
    out = capsys.readouterr().out.strip().splitlines()
    assert rc == 0 and [int(t) for t in out[-1].split()] == plain.greedy(cfg, weights, prompt, 5)
    assert main(["models"]) == 0 and "qwen3-8b" in capsys.readouterr().out
    assert main(["generate", "--model", "no-such-model", "--prompt-ids", "1"]) == 1
    assert "known names" in capsys.readouterr().err


def test_command_line_profile_report(models, capsys, tmp_path):
    """--profile times every operation (steps then run launch by launch) and prints the report;
    the tokens are those of an unprofiled run; bench --profile-json writes the report."""
    import json
    from rocml_amd.cli import main
    path, cfg, weights = models["B"]
    prompt = helpers.random_tokens(9, cfg["vocab_size"], 6)
    argv = ["generate", "--model", path, "--dtype", "float32", "--prompt-ids", " ".join(map(str, prompt)),
            "-n", "6", "--ctx", "64", "--batch", "2"]
    assert main(argv) == 0
    plain_out = capsys.readouterr().out.strip().splitlines()
    assert main(argv + ["--profile"]) == 0
    out = capsys.readouterr().out.strip().splitlines()
    assert out[0] == plain_out[0] and [int(t) for t in out[0].split()] == plain.greedy(cfg, weights, prompt, 6)
    text = "\n".join(out[1:])
    assert text.startswith("prefill:") and "\ndecode:" in text
    for label in ("product", "attention", "rmsnorm", "embedding", "argmax"):
        assert label in text
    report_path = tmp_path / "report.json"
    assert main(["bench", "--model", path, "--dtype", "bfloat16", "--prompt-tokens", "20", "--decode-tokens", "4",
                 "--runs", "2", "--batch", "2", "--ctx", "64", "--json", "--profile-json", str(report_path)]) == 0
    doc = json.loads(report_path.read_text())
    phases = {p["phase"]: p for p in doc["report"]["phases"]}
    assert set(phases) == {"prefill", "decode"} and doc["bench"]["decode_tokens"] == 4
    products = [r for r in phases["decode"]["by_op"] if r["label"] == "product"][0]
    n_layers = cfg["num_hidden_layers"]
    assert products["count"] == 3 * (4 * n_layers + 1)            # four products a layer and the output, three decode steps
    assert products["elapsed_ms"] > 0 and products["t_min_ms"] > 0 and 0 < products["efficiency"]


def test_position_and_reset_through_the_entry_point(models):
    from rocml_amd.engine import StepEntry
    path, cfg, weights = models["A"]
    model = _load(path, "float32", ctx=64, max_batch=2)
    toks = helpers.random_tokens(20, cfg["vocab_size"], 3)
    ref = plain.forward(cfg, weights, toks)
    a, b = model.new_sequence(), model.new_sequence()
    model.step([StepEntry(a, toks[:7], []), StepEntry(b, toks[:3], [])])
    assert model.position(a) == 7 and model.position(b) == 3
    model.reset()
    model.engine.cache.check()
    assert not model.engine.cache.lengths
    c = model.new_sequence()                       # a slot and pages that were just given back, not cleared
    got = model.step([StepEntry(c, toks, list(range(20)))]).cpu()
    assert model.position(c) == 20 and helpers.rel_to_max(got, ref) < 2e-5


@pytest.mark.parametrize("dtype,tol", [("float32", 2e-5), ("bfloat16", 2e-2)])
def test_prompts_far_longer_than_the_window_through_the_entry_point(models, dtype, tol):
    """Config D has layers with a window of 70.  With ``max_batch`` set, their cache group is
    sized for its windows, not for whole sequences; a prompt of 1,000 tokens passes through it in
    pieces, and generation continues from what the window still holds."""
    from rocml_amd.api import LoadOptions, Model
    from rocml_amd.engine import Engine, StepEntry
    from rocml_amd.weights import load_model
    path, cfg, weights = models["D"]
    w = weights if dtype == "float32" else {k: (v if v.dim() == 1 else v.to(torch.bfloat16).float()) for k, v in weights.items()}
    long_prompt = helpers.random_tokens(1000, cfg["vocab_size"], 91)
    short_prompt = helpers.random_tokens(300, cfg["vocab_size"], 92)
    model = Model.load(path, LoadOptions(dtype=dtype, ctx=1100, max_batch=2))
    got = model.generate([long_prompt, short_prompt], max_new_tokens=6)
    refs = {}
    for g, p in zip(got, (long_prompt, short_prompt)):
        # one pass of the plain implementation over prompt and answer: every generated token must be
        # the best continuation of what stands before it (in bfloat16: or within a near tie of it)
        assert len(g.tokens) == 6 and g.finish_reason == "length"
        ref = refs[len(p)] = plain.forward(cfg, w, list(p) + g.tokens)
        for k, tok in enumerate(g.tokens):
            row = ref[len(p) - 1 + k]
            best = int(torch.argmax(row))
            if tok != best:
                top = torch.topk(row, 2).values
                assert dtype == "bfloat16" and float((top[0] - row[tok]) / top[0].abs()) < 1e-2, f"token {k}: {tok} for {best}"
    model.engine.cache.check()
    assert not model.engine.cache.lengths
    # logits, with pieces far smaller than the prompt: the windowed group is then a handful of pages
    engine = Engine(load_model(path, dtype=dtype, device="cuda:0"), max_tokens=2 * 1100, max_seqs=2, max_step_tokens=96)
    windowed = [g for g in engine.cache.kv_groups if g.window is not None][0]
    assert windowed.n_pages == 2 * 4 + 2
    ref = refs[1000]
    a, b = engine.new_sequence(), engine.new_sequence()
    places = [0, 69, 70, 71, 500, 998, 999]
    logits = engine.step([StepEntry(a, long_prompt[:999], places[:-1]), StepEntry(b, short_prompt[:10], [])]).cpu()
    assert helpers.rel_to_max(logits, ref[places[:-1]]) < tol
    logits = engine.step([StepEntry(a, [long_prompt[999]], [0]), StepEntry(b, [short_prompt[10]], [])]).cpu()
    assert helpers.rel_to_max(logits, ref[999:1000]) < tol
    engine.release(a)
    engine.release(b)
    engine.cache.check()


def test_generation_stops_at_the_models_end_of_sequence_id(models, tmp_path):
    """``eos_token_id`` of config.json (or generation_config.json) ends a sequence by default and
    is not emitted; ``ignore_eos`` and the command line's --ignore-eos go on."""
    import json
    import shutil
    from rocml_amd.cli import main
    path, cfg, weights = models["B"]
    prompt = helpers.random_tokens(9, cfg["vocab_size"], 7)
    free = plain.greedy(cfg, weights, prompt, 8)
    eos = free[3]
    cut = free[:free.index(eos)]
    with_eos = str(tmp_path / "with_eos")
    shutil.copytree(path, with_eos)
    with open(f"{with_eos}/config.json", "w") as f:
        json.dump(dict(cfg, eos_token_id=eos), f)
    model = _load(with_eos, "float32", ctx=64, max_batch=1)
    r = model.generate([prompt], max_new_tokens=8)[0]
    assert r.tokens == cut and r.finish_reason == "stop"
    assert model.generate([prompt], max_new_tokens=8, ignore_eos=True)[0].tokens == free
    in_generation_config = str(tmp_path / "generation_config")
    shutil.copytree(path, in_generation_config)
    with open(f"{in_generation_config}/generation_config.json", "w") as f:
        json.dump({"eos_token_id": [eos, next(t for t in range(cfg["vocab_size"]) if t not in free)]}, f)
    model = _load(in_generation_config, "float32", ctx=64, max_batch=1)
    assert model.generate([prompt], max_new_tokens=8)[0].tokens == cut
    assert _load(path, "float32", ctx=64, max_batch=1).generate([prompt], max_new_tokens=8)[0].tokens == free


def test_a_catalog_model_has_the_weights_its_written_folder_has(tmp_path):
    """``--model tiny-b`` draws its weights on the GPU, ``init`` writes them on the CPU: the same
    seed gives the same bits, so both generate the same tokens and hold the same tensors."""
    from rocml_amd.api import Model
    from rocml_amd.cli import main
    out = str(tmp_path / "tiny_b")
    assert main(["init", "--model", "tiny-b", "--out", out, "--weights-seed", "5", "--dtype", "float32"]) == 0
    by_name = Model.load("tiny-b", dtype="float32", seed=5, ctx=64, max_batch=2)
    from_folder = Model.load(out, dtype="float32", ctx=64, max_batch=2)
    a, b = by_name.engine.model, from_folder.engine.model
    assert torch.equal(a.embed, b.embed) and torch.equal(a.lm_head, b.lm_head)
    for x, y in zip(a.blocks, b.blocks):
        assert torch.equal(x.mixer.w_qkv, y.mixer.w_qkv) and torch.equal(x.ffn.w_down, y.ffn.w_down)
        assert torch.equal(x.mixer.q_gain, y.mixer.q_gain) and torch.equal(x.mixer_norm.gain, y.mixer_norm.gain)
    prompts = [[3, 17, 200], [5, 6, 7, 8, 9, 10, 11]]
    assert [r.tokens for r in by_name.generate(prompts, max_new_tokens=6)] == \
        [r.tokens for r in from_folder.generate(prompts, max_new_tokens=6)]
    assert not torch.equal(Model.load("tiny-b", dtype="float32", seed=6, ctx=64).engine.model.embed, a.embed)


def test_a_decode_step_cut_into_pieces_runs_the_ids_that_were_drawn(models):
    """With fewer tokens to a step than the batch has sequences every decode step runs in pieces;
    a step launched ahead of the host takes its ids from the sampler's output on the device, and
    every piece must take its own run of them."""
    from rocml_amd.engine import Engine, EngineBackend, Generator, Request
    from rocml_amd.weights import load_model
    path, cfg, weights = models["B"]
    prompts = [helpers.random_tokens(n, cfg["vocab_size"], 140 + i) for i, n in enumerate([4, 1, 9, 2, 6, 3, 5])]
    want = [plain.greedy(cfg, weights, p, 6) for p in prompts]
    for run_ahead in (True, False):
        engine = Engine(load_model(path, dtype="float32", device="cuda:0"), max_tokens=7 * 64, max_seqs=7, max_step_tokens=3)
        reqs = [Request(list(p), 6) for p in prompts]
        got = Generator(EngineBackend(engine, run_ahead=run_ahead), max_batch=7).run(reqs)
        assert [r.tokens for r in got] == want, f"run_ahead={run_ahead}"
        engine.cache.check()
