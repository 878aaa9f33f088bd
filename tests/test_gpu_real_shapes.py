"""Real layer sizes against the plain implementation: the Qwen3-0.6B (tied output matrix, both
norms of a decode layer prepared by the products before them), Qwen3-8B and Qwen3-14B shapes of
the catalog cut to their first two layers, with the real vocabulary, in 32-bit and in bfloat16;
an unequal batch whose last tokens are fed one by one.  The tiny configurations cannot show a
fault that needs a width of 4096 or 5120, a head size of 128 with 32 or 40 heads, or a
vocabulary of 151,936 (kernel choices, tile edges and split counts all depend on them)."""
import numpy as np
import pytest
import torch

from tests import helpers
from tests.plain import qwen3_plain as plain

pytestmark = pytest.mark.gpu

TAIL = 4          # tokens fed one by one
WANT = 8          # places compared per request: the last ones


@pytest.mark.parametrize("name,lengths", [("qwen3-0.6b", [40, 200, 333]), ("qwen3-8b", [70, 333, 600]),
                                          ("qwen3-14b", [128, 257, 700])])
def test_two_layers_of_a_real_shape(tmp_path, name, lengths):
    from rocml_amd.config.catalog import resolve
    from rocml_amd.engine import Engine, StepEntry
    from rocml_amd.weights import load_model, write_model_dir
    cfg = dict(resolve(name).entry.config, num_hidden_layers=2)
    rng = np.random.default_rng(3)
    prompts = [[int(t) for t in rng.integers(0, cfg["vocab_size"], size=n)] for n in lengths]
    # stored in bfloat16, so both paths and the plain implementation compute with the same weights
    path = write_model_dir(str(tmp_path / "m"), cfg, 14, dtype=torch.bfloat16, norm_jitter=True, device="cuda:0")
    weights = {k: v.float() for k, v in helpers.read_weights(path).items()}
    refs = [plain.forward(cfg, weights, p, dtype=torch.float32, last=WANT) for p in prompts]
    for dtype, tol in (("float32", 5e-5), ("bfloat16", 2e-2)):
        engine = Engine(load_model(path, dtype=dtype, device="cuda:0"), max_tokens=64 * 16 * len(prompts))
        slots = [engine.new_sequence() for _ in prompts]
        got = [[] for _ in prompts]
        first = engine.step([StepEntry(s, p[:-TAIL], list(range(len(p) - WANT, len(p) - TAIL)))
                             for s, p in zip(slots, prompts)]).cpu()
        for i in range(len(prompts)):
            got[i].append(first[(WANT - TAIL) * i:(WANT - TAIL) * (i + 1)])
        for k in range(TAIL, 0, -1):
            out = engine.step([StepEntry(s, [p[-k]], [0]) for s, p in zip(slots, prompts)]).cpu()
            for i in range(len(prompts)):
                got[i].append(out[i:i + 1])
        for i, ref in enumerate(refs):
            g = torch.cat(got[i])
            assert helpers.rel_to_max(g, ref) < tol, f"{name} {dtype}, request of {lengths[i]} tokens"
            if dtype == "float32":
                assert torch.equal(g.argmax(-1), ref.argmax(-1))
        for s in slots:
            engine.release(s)
        engine.cache.check()
        del engine
        torch.cuda.empty_cache()


def test_sixteen_unequal_prompts_past_the_internal_cut_at_a_real_width(tmp_path):
    """Sixteen prompts of 128 to 4,096 tokens in one step at two layers of the Qwen3-8B shape:
    12,529 tokens, which the engine cuts at 8,192 (a prompt straddles the cut), two prompts
    longer than one pass of the prompt attention's 2,048 keys, then one token each.  The last
    eight places of every prompt and the decoded place against the plain implementation."""
    from rocml_amd.config.catalog import resolve
    from rocml_amd.engine import Engine, StepEntry
    from rocml_amd.weights import load_model, write_model_dir
    cfg = dict(resolve("qwen3-8b").entry.config, num_hidden_layers=2)
    lengths = [4096, 3300, 128, 257, 700, 130, 512, 1024, 150, 333, 200, 640, 129, 300, 450, 180]
    assert sum(lengths) > 8192 and len(lengths) == 16
    rng = np.random.default_rng(5)
    seqs = [[int(t) for t in rng.integers(0, cfg["vocab_size"], size=n + 1)] for n in lengths]
    path = write_model_dir(str(tmp_path / "m"), cfg, 15, dtype=torch.bfloat16, norm_jitter=True, device="cuda:0")
    weights = {k: v.float() for k, v in helpers.read_weights(path).items()}
    refs = [plain.forward(cfg, weights, s, dtype=torch.float32, last=WANT + 1) for s in seqs]
    for dtype, tol in (("float32", 5e-5), ("bfloat16", 2e-2)):
        engine = Engine(load_model(path, dtype=dtype, device="cuda:0"), max_tokens=sum(-(-(n + 1) // 64) * 64 for n in lengths),
                        max_seqs=16)
        assert engine.max_step_tokens == 8192
        slots = [engine.new_sequence() for _ in seqs]
        first = engine.step([StepEntry(s, q[:-1], list(range(len(q) - 1 - WANT, len(q) - 1)))
                             for s, q in zip(slots, seqs)]).cpu()
        last = engine.step([StepEntry(s, [q[-1]], [0]) for s, q in zip(slots, seqs)]).cpu()
        for i, ref in enumerate(refs):
            g = torch.cat([first[WANT * i:WANT * (i + 1)], last[i:i + 1]])
            assert helpers.rel_to_max(g, ref) < tol, f"{dtype}, request {i} of {lengths[i]} tokens"
            assert helpers.per_position(g, ref) < 5 * tol, f"{dtype}, request {i}, position by position"
            if dtype == "float32":
                assert torch.equal(g.argmax(-1), ref.argmax(-1))
        for s in slots:
            engine.release(s)
        engine.cache.check()
        del engine
        torch.cuda.empty_cache()
