"""The engine against the plain implementation: each request alone and whole, with the
last 32 tokens one by one, and in batches of unequal lengths whose slots are used again;
in 32-bit and in bfloat16, on tiny configurations that differ in every size."""
import pytest
import torch

from tests import helpers
from tests.plain import qwen3_plain as plain

pytestmark = pytest.mark.gpu

# Largest absolute difference over the largest absolute logit.
TOL = {"float32": 2e-5, "bfloat16": 2e-2}
LENGTHS = {"A": [5, 9, 13, 100], "B": [1, 7, 16, 33, 130], "C": [3, 24, 25, 70, 97], "D": [2, 64, 65, 150],
           "E": [1, 40, 129], "F": [70, 150], "G": [12, 95, 76], "H": [7, 65, 200, 321]}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    root = tmp_path_factory.mktemp("models")
    out = {}
    for name, (cfg, seed) in helpers.TINY.items():
        path = helpers.make_model_dir(root, cfg, seed, torch.float32)
        out[name] = (path, helpers.read_config(path), helpers.read_weights(path))
    return out


def _engine(path, dtype, max_tokens=4096):
    from rocml_amd.engine import Engine
    from rocml_amd.weights import load_model
    return Engine(load_model(path, dtype=dtype, device="cuda:0"), max_tokens=max_tokens)


def _oracle_weights(weights, dtype):
    """The plain implementation sees the weights the engine computes with: matrices
    rounded to bfloat16 in the bfloat16 path, gains as stored."""
    if dtype == "float32":
        return weights
    return {k: (v if v.dim() == 1 else v.to(torch.bfloat16).to(torch.float32)) for k, v in weights.items()}


# The worst position's largest difference over that position's largest logit: 32-bit against the
# plain implementation, bfloat16 against the plain implementation rounding where the engine does.
POSITION_TOL = 1e-4
ROUNDED_TOL = 1e-2
# (configuration F sums 2,048 rounded terms where the others sum a hundred: its rounding noise was
# measured at 1.2e-2 of a position's largest logit; the bound that held for whole requests holds
# for each of its positions)
ROUNDED_TOL_BY_NAME = {"F": 2e-2}


def _rounding_oracle(cfg, weights, p, few_tokens=False):
    plain_kernel = cfg["head_dim"] not in (32, 64, 96, 128, 192, 256)
    return plain.forward(cfg, weights, p, rounded=plain.round_bfloat16,
                         rounded_probs=(lambda t: t) if plain_kernel else None,
                         ffn_norm_rounds_before_scale=few_tokens and cfg["hidden_size"] % 8 == 0)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E", "F", "G", "H"])
def test_whole_tail_and_batches(models, name, dtype):
    path, cfg, weights = models[name]
    engine = _engine(path, dtype)
    oracle_w = _oracle_weights(weights, dtype)
    prompts = [helpers.random_tokens(n, cfg["vocab_size"], 100 + i) for i, n in enumerate(LENGTHS[name])]
    refs = [plain.forward(cfg, oracle_w, p) for p in prompts]
    tol = TOL[dtype]
    # Position by position as well, so that one bad place does not hide under the largest logit of
    # a whole request: in bfloat16 against the oracle that rounds where the engine does.
    sharp_refs, sharp_tol = refs, POSITION_TOL
    if dtype == "bfloat16":
        sharp_refs = [_rounding_oracle(cfg, weights, p) for p in prompts]
        sharp_tol = ROUNDED_TOL_BY_NAME.get(name, ROUNDED_TOL)

    def check(got, i, what):
        assert helpers.rel_to_max(got, refs[i]) < tol, what
        assert helpers.per_position(got, sharp_refs[i]) < sharp_tol, what + " (position by position)"

    for i, p in enumerate(prompts):
        check(helpers.run_whole(engine, p), i, f"whole, length {len(p)}")
        check(helpers.run_tail_by_one(engine, p, 32), i, f"tail by one, length {len(p)}")
    # Two batches one after the other: the second uses the slots and pages of the first.
    for order in (list(range(len(prompts))), list(reversed(range(len(prompts))))):
        batch = [prompts[i] for i in order]
        n_prefill = [max(1, len(p) - 3 * (j + 1)) for j, p in enumerate(batch)]
        got = helpers.run_batch(engine, batch, n_prefill)
        for j, i in enumerate(order):
            check(got[j], i, f"batch order {order}, sequence {i}")
    engine.cache.check()
    assert not engine.cache.lengths


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_internal_cutting_of_long_steps_is_invisible(models, dtype):
    """A step of more tokens than the engine runs at once is cut into pieces; sequences
    straddle the cuts and wanted rows come from several pieces."""
    from rocml_amd.engine import Engine, StepEntry
    from rocml_amd.weights import load_model
    path, cfg, weights = models["D"]
    engine = Engine(load_model(path, dtype=dtype, device="cuda:0"), max_tokens=4096, max_step_tokens=37)
    oracle_w = _oracle_weights(weights, dtype)
    prompts = [helpers.random_tokens(n, cfg["vocab_size"], 200 + i) for i, n in enumerate([90, 5, 64, 131])]
    refs = [plain.forward(cfg, oracle_w, p) for p in prompts]
    slots = [engine.new_sequence() for _ in prompts]
    want = [[0, len(p) // 2, len(p) - 1] for p in prompts]
    logits = engine.step([StepEntry(s, p, w) for s, p, w in zip(slots, prompts, want)]).cpu()
    expect = torch.cat([ref[w] for ref, w in zip(refs, want)])
    assert helpers.rel_to_max(logits, expect) < TOL[dtype]
    # the group that keeps every position took its pages for the whole step at once, a page per
    # sequence and round, however the step was cut: the sequences' first pages are neighbours
    kept = [g for g in engine.cache.kv_groups if g.window is None][0]
    first_pages = sorted(kept.page_table(s)[0] for s in slots)
    assert first_pages[-1] - first_pages[0] == len(slots) - 1
    # the cache the pieces left is the one a whole step would leave: decode one more token each
    nxt = [7, 8, 9, 10]
    logits = engine.step([StepEntry(s, [t], [0]) for s, t in zip(slots, nxt)]).cpu()
    expect = torch.stack([plain.forward(cfg, oracle_w, p + [t])[-1] for p, t in zip(prompts, nxt)])
    assert helpers.rel_to_max(logits, expect) < TOL[dtype]
    for s in slots:
        engine.release(s)
    engine.cache.check()


def test_refused_steps_leave_the_engine_as_it_was(models):
    from rocml_amd.engine import Engine, StepEntry
    from rocml_amd.errors import CacheFullError, ContextOverflowError, RocmlError
    from rocml_amd.weights import load_model
    path, cfg, weights = models["A"]                       # 128 positions
    engine = Engine(load_model(path, dtype="float32", device="cuda:0"), max_tokens=64 * 2)
    a, b = engine.new_sequence(), engine.new_sequence()
    toks = helpers.random_tokens(100, cfg["vocab_size"], 9)
    ref = plain.forward(cfg, weights, toks)
    engine.step([StepEntry(a, toks[:60], [])])
    with pytest.raises(CacheFullError):                    # b would need 2 pages, 1 is free
        engine.step([StepEntry(b, toks[:], [0]), StepEntry(a, [toks[60]], [0])])
    with pytest.raises(ContextOverflowError):
        engine.step([StepEntry(a, helpers.random_tokens(69, cfg["vocab_size"], 1), [0])])
    with pytest.raises(RocmlError, match="vocabulary"):
        engine.step([StepEntry(a, [cfg["vocab_size"]], [0])])
    with pytest.raises(RocmlError, match="twice"):
        engine.step([StepEntry(a, [1], [0]), StepEntry(a, [2], [0])])
    with pytest.raises(RocmlError, match="live"):
        engine.step([StepEntry(17, [1], [0])])
    assert engine.length(a) == 60 and engine.length(b) == 0
    engine.cache.check()
    got = engine.step([StepEntry(a, toks[60:], list(range(40)))]).cpu()    # goes on as if nothing had happened
    assert helpers.rel_to_max(got, ref[60:]) < TOL["float32"]


# Against an oracle that rounds to bfloat16 exactly where the engine does (matrices, normalised
# activations, q, cached k and v, probabilities, attention output, gated activation), the engine's
# logits are the oracle's to seven digits, until one value lies so close to the middle between two
# bfloat16 numbers that 32-bit and 64-bit arithmetic round it to different sides; that one step
# of the type spreads through every later rounded tensor and the difference becomes the noise of
# the type (a few thousandths of the largest logit).  A sequence of one to four tokens has so few
# rounded values that most stay clear of it.  So:
#  * of twelve whole prompts of two to five tokens at least four must agree to 1e-5 (measured: 1e-7
#    for six to twelve of them, the more the smaller the model): a tensor rounded in another
#    place, or not rounded, or a constant that is off, fails all of them
#    (in a step of so few tokens the norm before the feed-forward is prepared by the product
#    before it, which stores x * gain and leaves the row's scale to the gated epilogue: the oracle
#    is told so; the norm before the attention is prepared that way only in decode steps);
#  * every position of every way of cutting stays within 1e-2 of its own largest logit.
# Head sizes that run the plain attention kernel (A, C, E) multiply probabilities and values in
# 32-bit, so their oracle leaves the probabilities alone, and their decode steps, which cut the
# keys as a prompt does, agree like whole prompts; the matrix-core kernels round a probability
# relative to the largest score seen so far, which in a decode step (cached keys, then the new
# one) is not the largest of all, and only the loose bound holds there.
ALIKE_TOL = 1e-5


@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E", "G", "H"])
def test_bfloat16_against_an_oracle_that_rounds_where_the_engine_does(models, name):
    path, cfg, weights = models[name]
    engine = _engine(path, "bfloat16")
    plain_kernel = cfg["head_dim"] not in (32, 64, 96, 128, 192, 256)

    def oracle(p, few_tokens=False):
        return _rounding_oracle(cfg, weights, p, few_tokens)
    short = [helpers.random_tokens(2 + i % 4, cfg["vocab_size"], 400 + i) for i in range(12)]
    whole = [helpers.per_position(helpers.run_whole(engine, p), oracle(p, True)) for p in short]
    assert max(whole) < ROUNDED_TOL
    assert sum(e < ALIKE_TOL for e in whole) >= 4, f"whole prompts: {whole}"
    if plain_kernel:
        tails = [helpers.per_position(helpers.run_tail_by_one(engine, p, 3), oracle(p, True)) for p in short]
        assert max(tails) < ROUNDED_TOL and sum(e < ALIKE_TOL for e in tails) >= 4, f"token by token: {tails}"
    prompts = [helpers.random_tokens(n, cfg["vocab_size"], 300 + i) for i, n in enumerate(LENGTHS[name])]
    refs = [oracle(p) for p in prompts]
    for p, ref in zip(prompts, refs):
        assert helpers.per_position(helpers.run_whole(engine, p), ref) < ROUNDED_TOL, f"whole, length {len(p)}"
        assert helpers.per_position(helpers.run_tail_by_one(engine, p, 32), ref) < ROUNDED_TOL, f"tail, length {len(p)}"
    got = helpers.run_batch(engine, prompts, [max(1, len(p) - 3 * (j + 1)) for j, p in enumerate(prompts)])
    for g, ref in zip(got, refs):
        assert helpers.per_position(g, ref) < ROUNDED_TOL
    engine.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,n_seqs", [("H", 33), ("H", 64), ("F", 33), ("F", 64), ("H", 130), ("F", 100)])
def test_many_sequences_in_a_step(models, name, dtype, n_seqs):
    """33 to 130 sequences of unequal lengths (beyond 64 rows every product is the tile kernel's): their prompts in one step, then decode steps in
    which the shorter requests end one after the other, so the batch shrinks through the row
    counts the few-rows kernels are built for; then the same slots again with every sequence
    decoding side by side, the steps recorded once and replayed.  H takes the decode attention
    that reads the projection itself, F is wide enough for products cut along K."""
    from rocml_amd.engine import StepEntry
    path, cfg, weights = models[name]
    engine = _engine(path, dtype, max_tokens=64 * 4 * n_seqs)
    oracle_w = _oracle_weights(weights, dtype)
    lengths = [10 + (7 * i) % 90 for i in range(n_seqs)]
    tails = [1 + i % 8 for i in range(n_seqs)]                  # tokens fed one by one after the prompt
    seqs = [helpers.random_tokens(n + t, cfg["vocab_size"], 500 + i) for i, (n, t) in enumerate(zip(lengths, tails))]
    refs = [plain.forward(cfg, oracle_w, s) for s in seqs]
    got = helpers.run_batch(engine, seqs, lengths)
    worst = max(helpers.rel_to_max(g, r) for g, r in zip(got, refs))
    assert worst < TOL[dtype], f"{n_seqs} sequences: {worst}"
    sharp_refs, sharp_tol = refs, POSITION_TOL
    if dtype == "bfloat16":
        sharp_refs = [_rounding_oracle(cfg, weights, s) for s in seqs]
        sharp_tol = ROUNDED_TOL_BY_NAME.get(name, ROUNDED_TOL)
    worst = max(helpers.per_position(g, r) for g, r in zip(got, sharp_refs))
    assert worst < sharp_tol, f"{n_seqs} sequences, position by position: {worst}"
    engine.cache.check()
    assert not engine.cache.lengths
    slots = [engine.new_sequence() for _ in seqs]
    engine.step([StepEntry(s, q[:5], []) for s, q in zip(slots, seqs)])
    for k in range(5, 10):
        logits = engine.step([StepEntry(s, [q[k]], [0]) for s, q in zip(slots, seqs)]).cpu()
        expect = torch.stack([r[k] for r in refs])
        assert helpers.rel_to_max(logits, expect) < TOL[dtype], f"decode step {k}"
        assert helpers.per_position(logits, torch.stack([r[k] for r in sharp_refs])) < sharp_tol, f"decode step {k}, row by row"
    recorded = [key for key, entry in engine._graphs.items() if entry[1] is not None]
    assert engine.use_graphs and any(key[0] == n_seqs for key in recorded)
    for s in slots:
        engine.release(s)
    engine.cache.check()


@pytest.mark.parametrize("name", ["B", "D", "G", "H"])
def test_prompt_steps_whose_attention_prepares_its_queries(models, name, monkeypatch):
    """Long prompt steps hand the attention kernel the q/k/v projection instead of prepared
    queries.  With the length from which they do so set to two tokens, the tiny configurations
    whose head sizes the kernel knows and whose projections come whole (64 with a window in every other layer, 96, 128) go that
    way: whole requests, the tail token by token behind such a prompt, and batches of unequal
    lengths, position by position against the plain implementation that rounds where the engine does."""
    from rocml_amd.parts.attention import Attention
    monkeypatch.setattr(Attention, "FUSED_PREFILL_MIN_TOKENS", 2)
    path, cfg, weights = models[name]
    engine = _engine(path, "bfloat16")
    calls = []
    from rocml_amd import ops
    real = ops.attention_prefill_fused
    monkeypatch.setattr(ops, "attention_prefill_fused", lambda *a, **k: (calls.append(1), real(*a, **k))[1])
    tol = ROUNDED_TOL_BY_NAME.get(name, ROUNDED_TOL)
    prompts = [helpers.random_tokens(n, cfg["vocab_size"], 900 + i) for i, n in enumerate(LENGTHS[name])]
    refs = [_rounding_oracle(cfg, weights, p) for p in prompts]
    for p, ref in zip(prompts, refs):
        assert helpers.per_position(helpers.run_whole(engine, p), ref) < tol, f"whole, length {len(p)}"
        if len(p) > 8:
            assert helpers.per_position(helpers.run_tail_by_one(engine, p, 4), ref) < tol, f"tail, length {len(p)}"
    got = helpers.run_batch(engine, prompts, [max(1, len(p) - 3 * (j + 1)) for j, p in enumerate(prompts)])
    for g, ref in zip(got, refs):
        assert helpers.per_position(g, ref) < tol
    assert calls, "no prompt step went through the kernel that prepares its queries"
    engine.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_short_prompt_steps_of_a_shape_seen_before_are_replayed(models, dtype):
    """A prompt step of a shape that came before (the same token counts and first positions) is
    recorded the second time and replayed from then on; only the tables differ between replays:
    other tokens, other wanted places, other slots and pages.  Every run must give what the plain
    implementation gives, and other shapes in between must not disturb the recorded one."""
    from rocml_amd.engine import StepEntry
    path, cfg, weights = models["H"]
    engine = _engine(path, dtype)
    oracle_w = _oracle_weights(weights, dtype)
    tol = TOL[dtype]

    def once(seed, lengths, firsts, want_of):
        """Sequences whose first ``firsts[i]`` tokens are already cached bring ``lengths[i]`` more."""
        seqs = [helpers.random_tokens(f + n, cfg["vocab_size"], seed + i) for i, (n, f) in enumerate(zip(lengths, firsts))]
        slots = [engine.new_sequence() for _ in seqs]
        held = [(s, q[:f]) for s, q, f in zip(slots, seqs, firsts) if f]
        if held:
            engine.step([StepEntry(s, q, []) for s, q in held])
        wants = [want_of(n) for n in lengths]
        got = engine.step([StepEntry(s, q[f:], w) for s, q, f, w in zip(slots, seqs, firsts, wants)]).cpu()
        expect = torch.cat([plain.forward(cfg, oracle_w, q)[[f + j for j in w]] for q, f, w in zip(seqs, firsts, wants)])
        assert helpers.rel_to_max(got, expect) < tol, (seed, lengths, firsts)
        for s in slots:
            engine.release(s)

    shape = ([17, 5, 40], [0, 0, 0])
    for k in range(4):
        once(700 + 10 * k, *shape, want_of=lambda n, k=k: [k % n, n - 1])
        once(800 + 10 * k, [9], [0], want_of=lambda n: [n - 1])            # another shape in between
    recorded = [key for key, entry in engine._graphs.items() if key[0] == "prompt" and entry[1] is not None]
    assert ("prompt", (17, 5, 40), (0, 0, 0), 6, 1) in recorded and ("prompt", (9,), (0,), 1, 1) in recorded
    # a continuation deep in a sequence, over a page border, is a shape of its own
    for k in range(3):
        once(900 + 10 * k, [30, 3], [50, 64], want_of=lambda n: [0, n - 1])
    assert any(key[:3] == ("prompt", (30, 3), (50, 64)) and entry[1] is not None for key, entry in engine._graphs.items())
    engine.cache.check()
    # of the prompt shapes only the last few are kept
    engine.max_prompt_graphs = 2
    once(990, [4], [0], want_of=lambda n: [0])
    assert sum(1 for key in engine._graphs if key[0] == "prompt") == 2


LONG = {"architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "vocab_size": 300,
        "hidden_size": 64, "intermediate_size": 96, "num_hidden_layers": 1,
        "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 64,
        "rope_theta": 1000000.0, "rms_norm_eps": 1e-6, "tie_word_embeddings": True,
        "max_position_embeddings": 40960, "hidden_act": "silu", "attention_bias": False}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_prompt_of_33000_tokens_and_decoding_behind_it(tmp_path, dtype):
    """A sequence as long as the long-context figures are quoted for: a prompt of 33,000 tokens
    (five pieces of the engine's cut, a block table of 516 pages and more, the most key splits in
    the decode steps), then tokens one by one across a page border, a short sequence beside it.
    The model has one layer, so keys and values of every position follow from the embeddings
    alone and the plain implementation's parts give the logits of the last places without the
    33,000 x 33,000 scores of a whole pass."""
    import math
    from rocml_amd.engine import Engine, StepEntry
    from rocml_amd.weights import load_model
    path = helpers.make_model_dir(tmp_path, LONG, 31, torch.float32)
    cfg, weights = helpers.read_config(path), helpers.read_weights(path)
    w = {k: v.double() for k, v in _oracle_weights(weights, dtype).items()}
    n_prompt, n_decode, last = 33000, 40, 6
    toks = helpers.random_tokens(n_prompt + n_decode, cfg["vocab_size"], 41)
    short = helpers.random_tokens(20 + n_decode, cfg["vocab_size"], 42)

    def last_logits(tokens, places):
        d, hq, hkv, eps = cfg["head_dim"], cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["rms_norm_eps"]
        t = len(tokens)
        p = "model.layers.0."
        x = plain.embedding(w["model.embed_tokens.weight"], tokens)
        xn = plain.rmsnorm(x, w[p + "input_layernorm.weight"], eps)
        pos = list(range(t))
        k = plain.rope_neox(plain.rmsnorm(plain.linear(xn, w[p + "self_attn.k_proj.weight"]).reshape(t, hkv, d),
                                          w[p + "self_attn.k_norm.weight"], eps), pos, cfg["rope_theta"])
        v = plain.linear(xn, w[p + "self_attn.v_proj.weight"]).reshape(t, hkv, d)
        rows = torch.tensor(places)
        q = plain.rope_neox(plain.rmsnorm(plain.linear(xn[rows], w[p + "self_attn.q_proj.weight"]).reshape(len(places), hq, d),
                                          w[p + "self_attn.q_norm.weight"], eps), places, cfg["rope_theta"])
        o = torch.zeros(len(places), hq, d, dtype=torch.float64)
        for i, place in enumerate(places):             # the attention's formula, row by row (plain.causal_attention)
            for h in range(hq):
                s = (k[:place + 1, h // (hq // hkv)] @ q[i, h]) / math.sqrt(d)
                e = torch.exp(s - s.max())
                o[i, h] = (e @ v[:place + 1, h // (hq // hkv)]) / e.sum()
        x = x[rows] + plain.linear(o.reshape(len(places), hq * d), w[p + "self_attn.o_proj.weight"])
        x = x + plain.mlp_block(plain.rmsnorm(x, w[p + "post_attention_layernorm.weight"], eps), w, p)
        return plain.linear(plain.rmsnorm(x, w["model.norm.weight"], eps), w["model.embed_tokens.weight"])

    engine = Engine(load_model(path, dtype=dtype, device="cuda:0"), max_tokens=(n_prompt + n_decode + 64) // 64 * 64 + 128,
                    max_seqs=2)
    a, b = engine.new_sequence(), engine.new_sequence()
    places = list(range(n_prompt - last, n_prompt))
    got = [engine.step([StepEntry(a, toks[:n_prompt], places), StepEntry(b, short[:20], [19])]).cpu()]
    for i in range(n_decode):
        got.append(engine.step([StepEntry(a, [toks[n_prompt + i]], [0]), StepEntry(b, [short[20 + i]], [0])]).cpu())
    assert engine.cache.table_width([a, b]) >= 516
    long_rows = torch.cat([got[0][:last]] + [g[:1] for g in got[1:]])
    short_rows = torch.cat([got[0][last:]] + [g[1:] for g in got[1:]])
    want = last_logits(toks, places + list(range(n_prompt, n_prompt + n_decode)))
    tol = TOL[dtype]
    assert helpers.rel_to_max(long_rows, want) < tol and helpers.per_position(long_rows, want) < 5 * tol
    want_short = last_logits(short, list(range(19, 20 + n_decode)))
    assert helpers.rel_to_max(short_rows, want_short) < tol
    engine.release(a)
    engine.release(b)
    engine.cache.check()
