"""Weights: random model folders, loading by name, one error for everything that does not
fit (no GPU: the model is built on the CPU and no kernel runs)."""
import os

import pytest
import torch
from safetensors.torch import load_file, save_file

from rocml_amd.errors import WeightsError
from rocml_amd.weights import load_model, write_model_dir
from tests import helpers


def test_random_weights_follow_seed_and_name_only(tmp_path):
    a = load_file(os.path.join(write_model_dir(str(tmp_path / "a"), helpers.TINY_B, 1, torch.float32), "model.safetensors"))
    b = load_file(os.path.join(write_model_dir(str(tmp_path / "b"), helpers.TINY_B, 1, torch.float32), "model.safetensors"))
    c = load_file(os.path.join(write_model_dir(str(tmp_path / "c"), helpers.TINY_B, 2, torch.float32), "model.safetensors"))
    assert a.keys() == b.keys() and all(torch.equal(a[k], b[k]) for k in a)
    assert not torch.equal(a["model.embed_tokens.weight"], c["model.embed_tokens.weight"])
    # a model with fewer layers has the same tensors where names coincide
    small = load_file(os.path.join(write_model_dir(str(tmp_path / "s"), dict(helpers.TINY_B, num_hidden_layers=1), 1,
                                                   torch.float32), "model.safetensors"))
    assert all(torch.equal(small[k], a[k]) for k in small)
    assert "lm_head.weight" in a                                        # B is untied
    w = a["model.layers.0.self_attn.q_proj.weight"]
    assert w.shape == (192, 96) and abs(float(w.std()) - 0.02) < 2e-3
    g = a["model.layers.1.input_layernorm.weight"]
    assert abs(float(g.mean()) - 1.0) < 0.02 and float(g.std()) > 0.005     # gains 1 + N(0, 0.02)
    tied = load_file(os.path.join(write_model_dir(str(tmp_path / "t"), helpers.TINY_A, 0, torch.bfloat16), "model.safetensors"))
    assert "lm_head.weight" not in tied and tied["model.embed_tokens.weight"].dtype == torch.bfloat16


def test_types_after_loading(tmp_path):
    p32 = write_model_dir(str(tmp_path / "f32"), helpers.TINY_A, 0, torch.float32)
    p16 = write_model_dir(str(tmp_path / "bf16"), helpers.TINY_A, 0, torch.bfloat16)
    stored = load_file(os.path.join(p32, "model.safetensors"))
    m = load_model(p32, dtype="float32", device="cpu")
    assert m.embed.dtype == torch.float32 and torch.equal(m.embed, stored["model.embed_tokens.weight"])   # 32-bit stays so
    assert m.lm_head is m.embed                                                                    # tied: one buffer
    m = load_model(p16, dtype="bfloat16", device="cpu")
    assert m.embed.dtype == torch.bfloat16
    assert m.blocks[0].mixer_norm.gain.dtype == torch.float32                                      # gains are 32-bit
    assert m.blocks[0].mixer.w_qkv.shape == (64 + 2 * 32, 64) and m.blocks[0].ffn.w_gate_up.shape == (256, 64)
    m = load_model(p16, dtype="float32", device="cpu")                                              # widening is exact
    assert torch.equal(m.embed, load_file(os.path.join(p16, "model.safetensors"))["model.embed_tokens.weight"].float())


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    path = write_model_dir(str(tmp_path / "m"), helpers.TINY_B, 1, torch.float32)
    file = os.path.join(path, "model.safetensors")
    t = load_file(file)
    del t["model.layers.1.mlp.up_proj.weight"]
    del t["model.norm.weight"]
    t["model.layers.0.self_attn.rotary.inv_freq"] = torch.zeros(16)
    t["model.layers.2.self_attn.k_norm.weight"] = torch.ones(16)              # should be 32
    t["lm_head.weight"] = torch.zeros(96, 384)                                # transposed
    t["model.layers.0.mlp.gate_proj.weight"] = torch.zeros(224, 96, dtype=torch.int32)
    save_file(t, file)
    with pytest.raises(WeightsError) as e:
        load_model(path, dtype="float32", device="cpu")
    msg = str(e.value)
    for piece in ("missing tensors", "model.layers.1.mlp.up_proj.weight", "model.norm.weight",
                  "unexpected tensors", "model.layers.0.self_attn.rotary.inv_freq",
                  "model.layers.2.self_attn.k_norm.weight is [16], the model needs [32]",
                  "lm_head.weight is [96, 384], the model needs [384, 96]",
                  "model.layers.0.mlp.gate_proj.weight is stored as I32"):
        assert piece in msg, piece


def test_missing_file_and_sharded_folder(tmp_path):
    path = write_model_dir(str(tmp_path / "m"), helpers.TINY_A, 0, torch.float32)
    file = os.path.join(path, "model.safetensors")
    t = load_file(file)
    os.remove(file)
    with pytest.raises(WeightsError, match="model.safetensors"):
        load_model(path, dtype="float32", device="cpu")
    names = sorted(t)
    half = len(names) // 2
    save_file({k: t[k] for k in names[:half]}, os.path.join(path, "model-00001-of-00002.safetensors"))
    save_file({k: t[k] for k in names[half:]}, os.path.join(path, "model-00002-of-00002.safetensors"))
    import json
    index = {"weight_map": {k: ("model-00001-of-00002.safetensors" if i < half else "model-00002-of-00002.safetensors")
                            for i, k in enumerate(names)}}
    with open(os.path.join(path, "model.safetensors.index.json"), "w") as f:
        json.dump(index, f)
    m = load_model(path, dtype="float32", device="cpu")
    assert torch.equal(m.embed, t["model.embed_tokens.weight"])
    os.remove(os.path.join(path, "model-00002-of-00002.safetensors"))
    with pytest.raises(WeightsError, match="model-00002-of-00002"):
        load_model(path, dtype="float32", device="cpu")
