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
LENGTHS = {"A": [5, 9, 13, 100], "B": [1, 7, 16, 33, 130], "C": [3, 24, 25, 70, 97], "D": [2, 64, 65, 150]}


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


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_whole_tail_and_batches(models, name, dtype):
    path, cfg, weights = models[name]
    engine = _engine(path, dtype)
    oracle_w = _oracle_weights(weights, dtype)
    prompts = [helpers.random_tokens(n, cfg["vocab_size"], 100 + i) for i, n in enumerate(LENGTHS[name])]
    refs = [plain.forward(cfg, oracle_w, p) for p in prompts]
    tol = TOL[dtype]
    for p, ref in zip(prompts, refs):
        got = helpers.run_whole(engine, p)
        assert helpers.rel_to_max(got, ref) < tol, f"whole, length {len(p)}"
        got = helpers.run_tail_by_one(engine, p, 32)
        assert helpers.rel_to_max(got, ref) < tol, f"tail by one, length {len(p)}"
    # Two batches one after the other: the second uses the slots and pages of the first.
    for order in (list(range(len(prompts))), list(reversed(range(len(prompts))))):
        batch = [prompts[i] for i in order]
        n_prefill = [max(1, len(p) - 3 * (j + 1)) for j, p in enumerate(batch)]
        got = helpers.run_batch(engine, batch, n_prefill)
        for j, i in enumerate(order):
            assert helpers.rel_to_max(got[j], refs[i]) < tol, f"batch order {order}, sequence {i}"
    engine.cache.check()
    assert not engine.cache.lengths
