"""Pins the plain implementation by more than the reference's text: vectors its kernel
tests hold, special cases that reduce to a library routine, and invariants, each chosen so
that a plausible mistake (a wrong sign or pairing, a norm in the wrong place) fails it."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from tests import helpers
from tests.plain import qwen3_plain as plain

D64 = torch.float64


# ---- RMSNorm ---------------------------------------------------------------------------
@pytest.mark.parametrize("rows,n", [(5, 300), (1, 7)])
def test_rmsnorm_reference_vectors(rows, n):
    # inputs of rocml-kernels/tests/rmsnorm_rope.rs:27-31,70-79
    x = torch.tensor([[((r * n + i) % 29) * 0.1 - 1.4 for i in range(n)] for r in range(rows)], dtype=D64)
    w = torch.tensor([1.0 + 0.01 * i for i in range(n)], dtype=D64)
    eps = 1e-5
    got = plain.rmsnorm(x, w, eps)
    want = x.numpy() / np.sqrt((x.numpy() ** 2).mean(axis=1, keepdims=True) + eps) * w.numpy()
    assert np.abs(got.numpy() - want).max() < 1e-12


def test_rmsnorm_constant_row_and_eps_inside_root():
    c, eps = 3.0, 0.5
    got = plain.rmsnorm(torch.full((1, 8), c, dtype=D64), torch.ones(8, dtype=D64), eps)
    assert torch.allclose(got, torch.full((1, 8), c / math.sqrt(c * c + eps), dtype=D64))
    # the gain multiplies directly: a zero gain gives zero (a "1 + w" convention would not)
    assert plain.rmsnorm(torch.ones(1, 4, dtype=D64), torch.zeros(4, dtype=D64), 1e-6).abs().max() == 0


# ---- rotation --------------------------------------------------------------------------
def test_rope_identity_plane_rotation_and_pairing():
    x = torch.randn(3, 2, 8, dtype=D64)
    assert torch.equal(plain.rope_neox(x, [0, 0, 0], 1e4), x)
    v = torch.tensor([[[1.0, 0.0]]], dtype=D64)          # D = 2: f_0 = 1, a plane rotation by pos
    r = plain.rope_neox(v, [2], 1e4)
    assert torch.allclose(r, torch.tensor([[[math.cos(2.0), math.sin(2.0)]]], dtype=D64))
    # pairing is (i, i + D/2), not (2i, 2i + 1): a unit vector at 0 moves into 0 and D/2 only
    e0 = torch.zeros(1, 1, 8, dtype=D64)
    e0[0, 0, 0] = 1.0
    r = plain.rope_neox(e0, [1], 1e4)
    assert abs(float(r[0, 0, 0]) - math.cos(1.0)) < 1e-15 and abs(float(r[0, 0, 4]) - math.sin(1.0)) < 1e-15
    assert float(r[0, 0, [1, 2, 3, 5, 6, 7]].abs().max()) == 0


def test_rope_reference_shape_against_closed_form():
    # (tokens, heads, D, pos_base) = (10, 3, 16, 5), theta 1e4, x_i = (i mod 31) * 0.05 - 0.7
    # (rocml-kernels/tests/rmsnorm_rope.rs:89-148)
    t, h, d, base, theta = 10, 3, 16, 5, 1e4
    x = torch.tensor([(i % 31) * 0.05 - 0.7 for i in range(t * h * d)], dtype=D64).reshape(t, h, d)
    got = plain.rope_neox(x, list(range(base, base + t)), theta).numpy()
    half = d // 2
    pos = np.arange(base, base + t)[:, None, None]
    freq = theta ** (-2.0 * np.arange(half) / d)
    ang = pos * freq
    x0, x1 = x.numpy()[..., :half], x.numpy()[..., half:]
    want = np.concatenate([x0 * np.cos(ang) - x1 * np.sin(ang), x0 * np.sin(ang) + x1 * np.cos(ang)], axis=-1)
    assert np.abs(got - want).max() < 1e-13


def test_rope_keeps_norms_and_depends_on_distance_only():
    g = torch.Generator().manual_seed(0)
    q = torch.randn(1, 1, 32, generator=g, dtype=D64)
    k = torch.randn(1, 1, 32, generator=g, dtype=D64)
    for m, n in [(3, 1), (40, 38), (1003, 1001)]:
        qm, kn = plain.rope_neox(q, [m], 1e6), plain.rope_neox(k, [n], 1e6)
        assert abs(float(qm.norm() - q.norm())) < 1e-12
        dot = float((qm * kn).sum())
        if (m, n) == (3, 1):
            first = dot
        assert abs(dot - first) < 1e-9


# ---- attention -------------------------------------------------------------------------
def test_attention_equals_library_routine():
    g = torch.Generator().manual_seed(1)
    t, hq, hkv, d = 9, 6, 2, 8
    q = torch.randn(t, hq, d, generator=g, dtype=D64)
    k = torch.randn(t, hkv, d, generator=g, dtype=D64)
    v = torch.randn(t, hkv, d, generator=g, dtype=D64)
    scale = 0.3
    got = plain.causal_attention(q, k, v, scale)
    kk = k.repeat_interleave(hq // hkv, dim=1)      # query head h uses kv head h // group
    vv = v.repeat_interleave(hq // hkv, dim=1)
    want = F.scaled_dot_product_attention(q.transpose(0, 1), kk.transpose(0, 1), vv.transpose(0, 1),
                                          is_causal=True, scale=scale).transpose(0, 1)
    assert float((got - want).abs().max()) < 1e-12
    # one position: the output is the value row
    one = plain.causal_attention(q[:1], k[:1], v[:1], scale)
    assert torch.allclose(one[0, 4], v[0, 1])


def test_attention_window_is_a_band():
    g = torch.Generator().manual_seed(2)
    t, d, w = 12, 4, 5
    q, k, v = (torch.randn(t, 1, d, generator=g, dtype=D64) for _ in range(3))
    got = plain.causal_attention(q, k, v, 0.5, window=w)
    s = (q[:, 0] @ k[:, 0].t()) * 0.5
    i, j = torch.arange(t)[:, None], torch.arange(t)[None, :]
    s = s.masked_fill((j > i) | (j < i - w + 1), float("-inf"))
    want = torch.softmax(s, dim=-1) @ v[:, 0]
    assert float((got[:, 0] - want).abs().max()) < 1e-12
    assert torch.allclose(plain.causal_attention(q, k, v, 0.5, window=t), plain.causal_attention(q, k, v, 0.5))


# ---- feed-forward ----------------------------------------------------------------------
@pytest.mark.parametrize("n", [1000, 1])
def test_swiglu_reference_vectors(n):
    # g = (i mod 23) * 0.1 - 1.2, u = (i mod 17) * 0.2 - 1.5 (rocml-kernels/tests/activation.rs:27-33)
    gate = torch.tensor([(i % 23) * 0.1 - 1.2 for i in range(n)], dtype=D64)
    up = torch.tensor([(i % 17) * 0.2 - 1.5 for i in range(n)], dtype=D64)
    assert float((plain.swiglu(gate, up) - F.silu(gate) * up).abs().max()) < 1e-14
    assert float(plain.swiglu(torch.zeros(3, dtype=D64), torch.ones(3, dtype=D64)).abs().max()) == 0


# ---- the whole model -------------------------------------------------------------------
def _model(name, tmp_path):
    cfg, seed = helpers.TINY[name]
    path = helpers.make_model_dir(tmp_path, cfg, seed)
    return helpers.read_config(path), helpers.read_weights(path)


def test_one_layer_one_head_equals_a_direct_formula(tmp_path):
    cfg = dict(helpers.TINY_A, num_hidden_layers=1, num_attention_heads=1, num_key_value_heads=1,
               head_dim=8, tie_word_embeddings=False)
    path = helpers.make_model_dir(tmp_path, cfg, 5)
    w = {k: v.to(D64) for k, v in helpers.read_weights(path).items()}
    toks = [3, 1, 4, 1, 5, 9]
    got = plain.forward(cfg, w, toks)
    eps, d, p = cfg["rms_norm_eps"], 8, "model.layers.0."

    def norm(x, g):
        return x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps) * g

    def rot(x):                       # [T, D]
        half = d // 2
        ang = torch.arange(len(toks), dtype=D64)[:, None] * cfg["rope_theta"] ** (-2.0 * torch.arange(half, dtype=D64) / d)
        x0, x1 = x[:, :half], x[:, half:]
        return torch.cat([x0 * ang.cos() - x1 * ang.sin(), x0 * ang.sin() + x1 * ang.cos()], -1)

    x = w["model.embed_tokens.weight"][toks]
    xn = norm(x, w[p + "input_layernorm.weight"])
    q = rot(norm(xn @ w[p + "self_attn.q_proj.weight"].t(), w[p + "self_attn.q_norm.weight"]))
    k = rot(norm(xn @ w[p + "self_attn.k_proj.weight"].t(), w[p + "self_attn.k_norm.weight"]))
    v = xn @ w[p + "self_attn.v_proj.weight"].t()
    o = F.scaled_dot_product_attention(q[None], k[None], v[None], is_causal=True)[0]
    x = x + o @ w[p + "self_attn.o_proj.weight"].t()
    xn = norm(x, w[p + "post_attention_layernorm.weight"])
    x = x + (F.silu(xn @ w[p + "mlp.gate_proj.weight"].t()) * (xn @ w[p + "mlp.up_proj.weight"].t())) \
        @ w[p + "mlp.down_proj.weight"].t()
    want = norm(x, w["model.norm.weight"]) @ w["lm_head.weight"].t()
    assert float((got - want).abs().max()) < 1e-12


def test_shift_of_all_positions_changes_nothing(tmp_path):
    cfg, w = _model("B", tmp_path)
    toks = helpers.random_tokens(12, cfg["vocab_size"], 3)
    a = plain.forward(cfg, w, toks)
    b = plain.forward(cfg, w, toks, first_position=977)
    assert float((a - b).abs().max()) < 1e-9 * float(a.abs().max()) + 1e-12


def test_residual_stream_bypasses_zeroed_blocks_and_head_is_tied(tmp_path):
    cfg, w = _model("A", tmp_path)          # tied: no lm_head.weight in the file
    assert "lm_head.weight" not in w
    for name in list(w):
        if name.endswith("o_proj.weight") or name.endswith("down_proj.weight"):
            w[name] = torch.zeros_like(w[name])
    toks = [7, 8, 9]
    got = plain.forward(cfg, w, toks)
    e = w["model.embed_tokens.weight"].to(D64)
    want = plain.rmsnorm(e[toks], w["model.norm.weight"].to(D64), cfg["rms_norm_eps"]) @ e.t()
    assert float((got - want).abs().max()) < 1e-12


def test_causality_and_windows(tmp_path):
    cfg, w = _model("C", tmp_path)          # first layer slides with a window of 24
    toks = helpers.random_tokens(40, cfg["vocab_size"], 4)
    full = plain.forward(cfg, w, toks)
    assert float((plain.forward(cfg, w, toks[:17]) - full[:17]).abs().max()) < 1e-12
    assert plain.layer_windows(cfg) == [24, None]
    no_window = dict(cfg)
    del no_window["layer_types"]
    other = plain.forward(no_window, w, toks)
    assert float((other[:24] - full[:24]).abs().max()) < 1e-12      # within the window: the same
    assert float((other[30:] - full[30:]).abs().max()) > 1e-6      # beyond it: not


def test_greedy_stops_without_emitting(tmp_path):
    cfg, w = _model("A", tmp_path)
    out = plain.greedy(cfg, w, [1, 2, 3], 5)
    assert len(out) == 5
    assert plain.greedy(cfg, w, [1, 2, 3], 5, stop=[out[2]]) == out[:out.index(out[2])]
