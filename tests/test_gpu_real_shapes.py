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
