"""Each part alone against its plain formula, and what the layer list can express: a layer
named twice, a layer that reads another layer's cache, and a toy mixer with state of its own
that is defined here, registered, built and stepped without a change to the library."""
import math
from dataclasses import dataclass

import pytest
import torch

from tests import helpers
from tests.plain import qwen3_plain as plain

pytestmark = pytest.mark.gpu

from rocml_amd.config.spec import (AttentionSpec, BlockSpec, GatedMlpSpec, ModelSpec, NormSpec, RopeSpec,  # noqa: E402
                                   ScheduleEntry)


def _tensors(model, seed, dtype_of=None):
    from rocml_amd.weights.random_init import random_tensor
    out = {}
    for name, p in model.param_specs().items():
        out[name] = random_tensor(name, p, seed, model.storage_dtype(p), True).to(model.device)
    return out


def _engine(spec, dtype, seed=0, **kw):
    from rocml_amd.engine import DecoderModel, Engine
    model = DecoderModel(spec, dtype, device="cuda:0")
    tensors = _tensors(model, seed)
    model.bind(tensors)
    return Engine(model, max_tokens=2048, **kw), {k: v.cpu().double() for k, v in tensors.items()}


def _spec(layers, schedule, hidden, vocab, tied=True):
    return ModelSpec(architecture="test", vocab=vocab, hidden=hidden, layers=tuple(layers), schedule=tuple(schedule),
                     final_norm=NormSpec(hidden, 1e-5), tie_lm_head=tied, max_positions=1024)


def _attention_spec(hidden, hq, hkv, d, window=None, norm=True, theta=1e4, rot=None):
    return AttentionSpec(hidden=hidden, n_heads=hq, n_kv_heads=hkv, head_dim=d, scale=1 / math.sqrt(d), window=window,
                         qk_norm=NormSpec(d, 1e-5) if norm else None,
                         position=RopeSpec(d, rot or d, theta) if theta else None)


def _block(hidden, mixer, inter=48):
    return BlockSpec(mixer=mixer, ffn=GatedMlpSpec(hidden, inter), mixer_norm=NormSpec(hidden, 1e-5),
                     ffn_norm=NormSpec(hidden, 1e-5))


# ---- plain versions of a block built from the parts' own parameter names --------------------
def plain_attention(xn, w, pre, s, positions, k_cache=None):
    t = xn.shape[0]
    q = (xn @ w[pre + "q_proj.weight"].t()).reshape(t, s.n_heads, s.head_dim)
    if k_cache is None:
        k = (xn @ w[pre + "k_proj.weight"].t()).reshape(t, s.n_kv_heads, s.head_dim)
        v = (xn @ w[pre + "v_proj.weight"].t()).reshape(t, s.n_kv_heads, s.head_dim)
        if s.qk_norm is not None:
            k = plain.rmsnorm(k, w[pre + "k_norm.weight"], s.qk_norm.eps)
        if s.position is not None:
            r = s.position.rot_dim
            k = torch.cat([plain.rope_neox(k[..., :r], positions, s.position.theta), k[..., r:]], -1)
    else:
        k, v = k_cache
    if s.qk_norm is not None:
        q = plain.rmsnorm(q, w[pre + "q_norm.weight"], s.qk_norm.eps)
    if s.position is not None:
        r = s.position.rot_dim
        q = torch.cat([plain.rope_neox(q[..., :r], positions, s.position.theta), q[..., r:]], -1)
    o = plain.causal_attention(q, k, v, s.scale, s.window)
    return o.reshape(t, -1) @ w[pre + "o_proj.weight"].t(), (k, v)


def plain_model(spec, w, tokens):
    x = w["embed.weight"][tokens]
    positions = list(range(len(tokens)))
    caches = {}
    for i, e in enumerate(spec.schedule):
        b = spec.layers[e.layer]
        pre = f"layers.{e.layer}."
        xn = plain.rmsnorm(x, w[pre + "mixer_norm.weight"], b.mixer_norm.eps)
        out, kv = plain_attention(xn, w, pre + "mixer.", b.mixer, positions,
                                  caches[e.reads_cache_of] if e.reads_cache_of is not None else None)
        caches[i] = kv
        x = x + out
        xn = plain.rmsnorm(x, w[pre + "ffn_norm.weight"], b.ffn_norm.eps)
        g = xn @ w[pre + "ffn.gate_proj.weight"].t()
        u = xn @ w[pre + "ffn.up_proj.weight"].t()
        x = x + plain.swiglu(g, u) @ w[pre + "ffn.down_proj.weight"].t()
    xn = plain.rmsnorm(x, w["final_norm.weight"], spec.final_norm.eps)
    return xn @ (w["embed.weight"] if spec.tie_lm_head else w["lm_head.weight"]).t()


@pytest.mark.parametrize("mixer", [
    _attention_spec(40, 5, 5, 16), _attention_spec(40, 4, 2, 32, window=9), _attention_spec(40, 6, 2, 48, norm=False),
    _attention_spec(40, 2, 1, 64, theta=None), _attention_spec(40, 4, 4, 32, rot=16, theta=5e5),
    _attention_spec(40, 8, 2, 128, window=70)])
def test_attention_part_options(mixer):
    """One block whose mixer has the option under test; whole and token by token."""
    spec = _spec([_block(40, mixer)], [ScheduleEntry(0)], 40, 97)
    for dtype, tol in (("float32", 2e-5), ("bfloat16", 2.5e-2)):
        engine, w = _engine(spec, dtype, seed=3)
        if dtype == "bfloat16":
            w = {k: (v if v.dim() == 1 else v.float().to(torch.bfloat16).double()) for k, v in w.items()}
        toks = helpers.random_tokens(90, 97, 1)
        ref = plain_model(spec, w, toks)
        assert helpers.rel_to_max(helpers.run_whole(engine, toks), ref) < tol
        assert helpers.rel_to_max(helpers.run_tail_by_one(engine, toks, 32), ref) < tol


@pytest.mark.parametrize("dtype,d,tol", [("float32", 16, 2e-5), ("bfloat16", 64, 2.5e-2)])
def test_layer_named_twice_and_shared_cache(dtype, d, tol):
    """(bfloat16 with a head size of 64: the decode steps of the layer that reads another layer's
    cache take the attention kernel that reads the projection, without appending.)"""
    a = _block(48, _attention_spec(48, 4, 2, d))
    b = _block(48, _attention_spec(48, 4, 2, d, window=20), inter=80)
    schedule = [ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(1), ScheduleEntry(0, reads_cache_of=0)]
    spec = _spec([a, b], schedule, 48, 131, tied=False)
    engine, w = _engine(spec, dtype, seed=4)
    assert len(engine.cache.kv_groups) == 2                          # full and windowed lines apart
    assert engine.cache.kv_groups[0].n_lines == 1 and engine.cache.kv_groups[1].n_lines == 2
    toks = helpers.random_tokens(70, 131, 2)
    ref = plain_model(spec, w, toks)
    assert helpers.rel_to_max(helpers.run_whole(engine, toks), ref) < tol
    assert helpers.rel_to_max(helpers.run_tail_by_one(engine, toks, 32), ref) < tol
    got = helpers.run_batch(engine, [toks, toks[:33], toks[:5]], [60, 20, 1])
    for g, n in zip(got, (70, 33, 5)):
        assert helpers.rel_to_max(g, ref[:n]) < tol


def test_norm_rope_and_mlp_parts_alone():
    from rocml_amd.engine import Workspace
    from rocml_amd.engine.batch import StepContext
    from rocml_amd.parts import BuildContext, build_feed_forward, build_norm, build_position
    ctx = BuildContext(dtype=torch.float32, device=torch.device("cuda:0"))
    g = torch.Generator().manual_seed(0)
    norm = build_norm(NormSpec(72, 3e-6), ctx)
    gain = torch.randn(72, generator=g)
    norm.bind({"weight": gain.cuda()})
    x = torch.randn(9, 72, generator=g)
    out = torch.empty(9, 72, device="cuda")
    norm.forward(x.cuda(), out)
    assert float((out.cpu().double() - plain.rmsnorm(x.double(), gain.double(), 3e-6)).abs().max()) < 1e-5
    ffn = build_feed_forward(GatedMlpSpec(72, 100), ctx)
    ws = {n: (torch.randn(p.shape, generator=g) * 0.1) for n, p in ffn.param_specs().items()}
    ffn.bind({n: t.cuda() for n, t in ws.items()})
    pos = torch.tensor([5, 6, 7, 0, 1, 2, 3, 4, 900], dtype=torch.int32).cuda()
    step = StepContext(n_tokens=9, n_seqs=1, token_ids=pos, token_seq=pos, token_pos=pos, cu_seqlens=pos, seq_lens=pos,
                       seq_slots=pos, max_new=9, max_len=9, new_counts=(9,), workspace=Workspace("cuda:0"))
    acc = x.cuda().clone()
    ffn.forward(step, x.cuda(), acc)
    step.workspace.flush_pending()                                       # a part may leave its last sum to the next norm
    xd = x.double()
    want = xd + plain.swiglu(xd @ ws["gate_proj.weight"].double().t(), xd @ ws["up_proj.weight"].double().t()) \
        @ ws["down_proj.weight"].double().t()
    assert float((acc.cpu().double() - want).abs().max()) < 1e-5
    rope = build_position(RopeSpec(32, 16, 7e4), ctx)
    cos, sin = rope.tables(step)
    assert rope.tables(step)[0] is cos                                  # one table per step, shared
    ang = pos.cpu().double()[:, None] * torch.tensor([7e4 ** (-2.0 * i / 16) for i in range(8)], dtype=torch.float64)
    assert float((cos.cpu().double() - ang.cos()).abs().max()) < 1e-7 and float((sin.cpu().double() - ang.sin()).abs().max()) < 1e-7


# ---- a toy mixer with state of its own ---------------------------------------------------
@dataclass(frozen=True)
class DecaySpec:
    hidden: int
    width: int
    decay: float
    kind: str = "toy_decay"


def _toy_parts():
    from rocml_amd.parts import Mixer, ParamSpec, StateRequest, register_mixer

    class DecayMixer(Mixer):
        """state <- decay * state + W_in x, out = W_out state: a running sum per sequence,
        kept in the cache's fixed-size state and advanced once per token, in order."""
        graph_safe = False        # loops over tokens on the host

        def __init__(self, spec, ctx):
            self.spec = spec

        def param_specs(self):
            s = self.spec
            return {"in_proj.weight": ParamSpec((s.width, s.hidden)), "out_proj.weight": ParamSpec((s.hidden, s.width))}

        def bind(self, tensors):
            self.w_in, self.w_out = tensors["in_proj.weight"].float(), tensors["out_proj.weight"].float()

        def cache_request(self):
            return StateRequest((self.spec.width,))

        def forward(self, step, xn, x_accum, cache, owns_cache):
            u = xn.float() @ self.w_in.t()                      # [T, width]
            slots = cache.slots.cpu().tolist()
            cu = step.cu_seqlens.cpu().tolist()
            for b, slot in enumerate(slots):
                state = cache.state[slot]
                for t in range(cu[b], cu[b + 1]):
                    state.mul_(self.spec.decay).add_(u[t])
                    x_accum[t] += state @ self.w_out.t()
    register_mixer("toy_decay", DecayMixer)


def test_toy_mixer_with_state_registers_builds_and_steps():
    _toy_parts()
    toy = _block(32, DecaySpec(32, 12, 0.9))
    att = _block(32, _attention_spec(32, 2, 1, 16))
    spec = _spec([toy, att, toy], [ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(2)], 32, 77)
    engine, w = _engine(spec, "float32", seed=5)
    assert not engine.use_graphs                                 # a part of the model said it cannot be recorded
    assert len(engine.cache.state_groups) == 1 and engine.cache.state_groups[0].n_lines == 2

    def reference(tokens):
        x = w["embed.weight"][tokens]
        for i, b in enumerate(spec.layers):
            pre = f"layers.{i}."
            xn = plain.rmsnorm(x, w[pre + "mixer_norm.weight"], 1e-5)
            if b.mixer.kind == "toy_decay":
                state = torch.zeros(12, dtype=torch.float64)
                out = []
                for t in range(len(tokens)):
                    state = 0.9 * state + w[pre + "mixer.in_proj.weight"] @ xn[t]
                    out.append(w[pre + "mixer.out_proj.weight"] @ state)
                x = x + torch.stack(out)
            else:
                x = x + plain_attention(xn, w, pre + "mixer.", b.mixer, list(range(len(tokens))))[0]
            xn = plain.rmsnorm(x, w[pre + "ffn_norm.weight"], 1e-5)
            x = x + plain.swiglu(xn @ w[pre + "ffn.gate_proj.weight"].t(), xn @ w[pre + "ffn.up_proj.weight"].t()) \
                @ w[pre + "ffn.down_proj.weight"].t()
        return plain.rmsnorm(x, w["final_norm.weight"], 1e-5) @ w["embed.weight"].t()

    a, b = helpers.random_tokens(40, 77, 6), helpers.random_tokens(23, 77, 7)
    ra, rb = reference(a), reference(b)
    assert helpers.rel_to_max(helpers.run_whole(engine, a), ra) < 1e-4
    # the slot is handed out again: its state must start at zero
    assert helpers.rel_to_max(helpers.run_tail_by_one(engine, b, 10), rb) < 1e-4
    got = helpers.run_batch(engine, [a, b], [30, 3])
    assert helpers.rel_to_max(got[0], ra) < 1e-4 and helpers.rel_to_max(got[1], rb) < 1e-4


# ---- a toy feed-forward with routing, and a toy position encoding ---------------------------
@dataclass(frozen=True)
class RoutedSpec:
    hidden: int
    inter: int
    n_experts: int
    top_k: int
    kind: str = "toy_routed"


@dataclass(frozen=True)
class SlowedRopeSpec:
    """Rotation whose angle grows with position / factor: the attention part only sees tables."""
    head_dim: int
    rot_dim: int
    theta: float
    factor: float
    kind: str = "toy_slowed_rope"


def _toy_routed_and_position():
    from rocml_amd.parts import FeedForward, ParamSpec, PositionEncoding, register_feed_forward, register_position

    class RoutedFfn(FeedForward):
        """Router logits in 32-bit, the best ``top_k`` experts per token weighted by a softmax over
        their logits, each expert a small SwiGLU; tokens are gathered per expert."""
        graph_safe = False        # the gathers have sizes that depend on the routing

        def __init__(self, spec, ctx):
            self.spec = spec

        def param_specs(self):
            s = self.spec
            return {"router.weight": ParamSpec((s.n_experts, s.hidden), role="gain", init="normal"),
                    "experts.gate_up.weight": ParamSpec((s.n_experts, 2 * s.inter, s.hidden)),
                    "experts.down.weight": ParamSpec((s.n_experts, s.hidden, s.inter))}

        def bind(self, tensors):
            self.router = tensors["router.weight"]
            self.gate_up = tensors["experts.gate_up.weight"].float()
            self.down = tensors["experts.down.weight"].float()

        def forward(self, step, xn, x_accum):
            s = self.spec
            x = xn.float()
            logits = x @ self.router.t()
            best, idx = torch.topk(logits, s.top_k, dim=-1)
            weight = torch.softmax(best, dim=-1)
            for e in range(s.n_experts):
                tok, slot = torch.nonzero(idx == e, as_tuple=True)
                if tok.numel() == 0:
                    continue
                gu = x[tok] @ self.gate_up[e].t()
                h = torch.nn.functional.silu(gu[:, :s.inter]) * gu[:, s.inter:]
                x_accum.index_add_(0, tok, (h @ self.down[e].t()) * weight[tok, slot][:, None])

    class SlowedRope(PositionEncoding):
        def __init__(self, spec, ctx):
            self.spec, self.rot_dim = spec, spec.rot_dim
            half = spec.rot_dim // 2
            self.inv = torch.tensor([spec.theta ** (-2.0 * i / spec.rot_dim) for i in range(half)],
                                    dtype=torch.float64, device=ctx.device)

        def tables(self, step):
            hit = step.memo.get(("toy_slowed_rope", self.spec))
            if hit is None:
                ang = step.token_pos.double()[:, None] / self.spec.factor * self.inv
                hit = (ang.cos().float().contiguous(), ang.sin().float().contiguous())
                step.memo[("toy_slowed_rope", self.spec)] = hit
            return hit

    class NeighbourRope(SlowedRope):
        """The same angles, but the values (2i, 2i + 1) of a head turn together."""
        pairing = "neighbours"

    register_feed_forward("toy_routed", RoutedFfn)
    register_position("toy_slowed_rope", SlowedRope)
    register_position("toy_neighbour_rope", NeighbourRope)


def test_toy_routed_feed_forward_and_toy_position_encoding():
    """Another feed-forward (a router and experts) and another position encoding, defined here and
    registered: layers 0 and 2 use them, layer 1 is the library's own block."""
    _toy_routed_and_position()
    hidden, d = 40, 16
    slow = SlowedRopeSpec(d, d, 1e4, 4.0)
    att_slow = AttentionSpec(hidden=hidden, n_heads=4, n_kv_heads=2, head_dim=d, scale=1 / math.sqrt(d), window=None,
                             qk_norm=NormSpec(d, 1e-5), position=slow)
    routed = RoutedSpec(hidden, 24, 5, 2)

    def block(mixer, ffn):
        return BlockSpec(mixer=mixer, ffn=ffn, mixer_norm=NormSpec(hidden, 1e-5), ffn_norm=NormSpec(hidden, 1e-5))
    layers = [block(att_slow, routed), _block(hidden, _attention_spec(hidden, 4, 2, d)), block(att_slow, routed)]
    spec = _spec(layers, [ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(2)], hidden, 83)
    engine, w = _engine(spec, "float32", seed=8)

    def rope_slow(x, positions):
        return plain.rope_neox(x, [p / slow.factor for p in positions], slow.theta)

    def reference(tokens):
        x = w["embed.weight"][tokens]
        pos = list(range(len(tokens)))
        t = len(tokens)
        for i, b in enumerate(spec.layers):
            pre = f"layers.{i}."
            xn = plain.rmsnorm(x, w[pre + "mixer_norm.weight"], 1e-5)
            if b.mixer.position.kind == "toy_slowed_rope":
                m = b.mixer
                q = plain.rmsnorm((xn @ w[pre + "mixer.q_proj.weight"].t()).reshape(t, m.n_heads, d), w[pre + "mixer.q_norm.weight"], 1e-5)
                k = plain.rmsnorm((xn @ w[pre + "mixer.k_proj.weight"].t()).reshape(t, m.n_kv_heads, d), w[pre + "mixer.k_norm.weight"], 1e-5)
                v = (xn @ w[pre + "mixer.v_proj.weight"].t()).reshape(t, m.n_kv_heads, d)
                o = plain.causal_attention(rope_slow(q, pos), rope_slow(k, pos), v, m.scale, None)
                x = x + o.reshape(t, -1) @ w[pre + "mixer.o_proj.weight"].t()
            else:
                x = x + plain_attention(xn, w, pre + "mixer.", b.mixer, pos)[0]
            xn = plain.rmsnorm(x, w[pre + "ffn_norm.weight"], 1e-5)
            if b.ffn.kind == "toy_routed":
                logits = xn @ w[pre + "ffn.router.weight"].t()
                out = torch.zeros_like(x)
                for r in range(t):
                    best, idx = torch.topk(logits[r], routed.top_k)
                    wt = torch.softmax(best, -1)
                    for j in range(routed.top_k):
                        gu = w[pre + "ffn.experts.gate_up.weight"][idx[j]] @ xn[r]
                        h = plain.swiglu(gu[:routed.inter], gu[routed.inter:])
                        out[r] += wt[j] * (w[pre + "ffn.experts.down.weight"][idx[j]] @ h)
                x = x + out
            else:
                x = x + plain.swiglu(xn @ w[pre + "ffn.gate_proj.weight"].t(), xn @ w[pre + "ffn.up_proj.weight"].t()) \
                    @ w[pre + "ffn.down_proj.weight"].t()
        return plain.rmsnorm(x, w["final_norm.weight"], 1e-5) @ w["embed.weight"].t()

    a, b = helpers.random_tokens(50, 83, 9), helpers.random_tokens(19, 83, 10)
    ra, rb = reference(a), reference(b)
    assert helpers.rel_to_max(helpers.run_whole(engine, a), ra) < 1e-4
    assert helpers.rel_to_max(helpers.run_tail_by_one(engine, b, 12), rb) < 1e-4
    got = helpers.run_batch(engine, [a, b], [35, 4])
    assert helpers.rel_to_max(got[0], ra) < 1e-4 and helpers.rel_to_max(got[1], rb) < 1e-4


@pytest.mark.parametrize("dtype,tol", [("float32", 1e-4), ("bfloat16", 2e-2)])
def test_toy_position_encoding_that_pairs_neighbours(dtype, tol):
    """A position encoding whose pairs are (2i, 2i + 1): the part only says so (``pairing``); the
    attention's kernels take the pairing as a parameter, and the decode kernel that rotates inside
    the attention, which knows halves only, is not taken (head size 64 in bfloat16 would take it)."""
    _toy_routed_and_position()
    hidden, d = 48, 64
    rope = SlowedRopeSpec(d, d, 1e4, 1.0, kind="toy_neighbour_rope")
    att = AttentionSpec(hidden=hidden, n_heads=4, n_kv_heads=2, head_dim=d, scale=1 / math.sqrt(d), window=None,
                        qk_norm=NormSpec(d, 1e-5), position=rope)
    spec = _spec([_block(hidden, att), _block(hidden, att)], [ScheduleEntry(0), ScheduleEntry(1)], hidden, 97)
    engine, w = _engine(spec, dtype, seed=12)
    assert not engine.model.blocks[0].mixer._fused_decode(type("S", (), {"max_new": 1})())
    if dtype == "bfloat16":
        w = {k: (v if v.dim() == 1 else v.to(torch.bfloat16).double()) for k, v in w.items()}

    def turn(x, positions):
        order = list(range(0, d, 2)) + list(range(1, d, 2))
        back = [order.index(i) for i in range(d)]
        return plain.rope_neox(x[..., order], positions, rope.theta)[..., back]

    def reference(tokens):
        x = w["embed.weight"][tokens]
        pos = list(range(len(tokens)))
        t = len(tokens)
        for i in range(2):
            pre = f"layers.{i}."
            xn = plain.rmsnorm(x, w[pre + "mixer_norm.weight"], 1e-5)
            q = plain.rmsnorm((xn @ w[pre + "mixer.q_proj.weight"].t()).reshape(t, 4, d), w[pre + "mixer.q_norm.weight"], 1e-5)
            k = plain.rmsnorm((xn @ w[pre + "mixer.k_proj.weight"].t()).reshape(t, 2, d), w[pre + "mixer.k_norm.weight"], 1e-5)
            v = (xn @ w[pre + "mixer.v_proj.weight"].t()).reshape(t, 2, d)
            o = plain.causal_attention(turn(q, pos), turn(k, pos), v, att.scale, None)
            x = x + o.reshape(t, -1) @ w[pre + "mixer.o_proj.weight"].t()
            xn = plain.rmsnorm(x, w[pre + "ffn_norm.weight"], 1e-5)
            x = x + plain.swiglu(xn @ w[pre + "ffn.gate_proj.weight"].t(), xn @ w[pre + "ffn.up_proj.weight"].t()) \
                @ w[pre + "ffn.down_proj.weight"].t()
        return plain.rmsnorm(x, w["final_norm.weight"], 1e-5) @ w["embed.weight"].t()

    a, b = helpers.random_tokens(70, 97, 19), helpers.random_tokens(9, 97, 20)
    ra, rb = reference(a), reference(b)
    assert helpers.rel_to_max(helpers.run_whole(engine, a), ra) < tol
    assert helpers.rel_to_max(helpers.run_tail_by_one(engine, b, 6), rb) < tol
    got = helpers.run_batch(engine, [a, b], [60, 3])
    assert helpers.rel_to_max(got[0], ra) < tol and helpers.rel_to_max(got[1], rb) < tol
    # (and the pairing does matter: with halves as pairs the logits are others)
    wrong = SlowedRopeSpec(d, d, 1e4, 1.0)
    att2 = AttentionSpec(hidden=hidden, n_heads=4, n_kv_heads=2, head_dim=d, scale=1 / math.sqrt(d), window=None,
                         qk_norm=NormSpec(d, 1e-5), position=wrong)
    other, _ = _engine(_spec([_block(hidden, att2), _block(hidden, att2)], [ScheduleEntry(0), ScheduleEntry(1)], hidden, 97), dtype, seed=12)
    assert helpers.rel_to_max(helpers.run_whole(other, a), ra) > 10 * tol


# ---- a toy embedding with learned positions and a toy head with a soft cap ------------------
@dataclass(frozen=True)
class PositionedTableSpec:
    """Token row plus a learned row for the token's position: an additive position encoding."""
    vocab: int
    hidden: int
    max_positions: int
    kind: str = "toy_positioned_table"


@dataclass(frozen=True)
class CappedHeadSpec:
    """Norm, product with a matrix of its own, then ``cap * tanh(logits / cap)``."""
    vocab: int
    hidden: int
    eps: float
    cap: float
    kind: str = "toy_capped_head"


def _toy_embedding_and_head():
    from rocml_amd import ops
    from rocml_amd.parts import Embedding, Head, ParamSpec, register_embedding, register_head

    class PositionedTable(Embedding):
        def __init__(self, spec, ctx):
            self.spec = spec

        def param_specs(self):
            s = self.spec
            return {"tokens.weight": ParamSpec((s.vocab, s.hidden)),
                    "positions.weight": ParamSpec((s.max_positions, s.hidden))}

        def bind(self, tensors):
            self.tokens, self.positions = tensors["tokens.weight"], tensors["positions.weight"]

        def forward(self, step, x):
            ops.embed_gather(self.tokens, step.token_ids, x, 1.0)
            x += self.positions.float()[step.token_pos.long()]

    class CappedHead(Head):
        def __init__(self, spec, ctx):
            self.spec, self.dtype = spec, ctx.dtype

        def param_specs(self):
            s = self.spec
            return {"out_norm.weight": ParamSpec((s.hidden,), role="gain", init="gain"),
                    "out.weight": ParamSpec((s.vocab, s.hidden))}

        def bind(self, tensors, shared=None):
            self.gain, self.matrix = tensors["out_norm.weight"], tensors["out.weight"]

        def forward(self, step, x, want_rows, n_want):
            ws = step.workspace
            xn = ws.get("toy_head.xn", (n_want, self.spec.hidden), self.dtype)
            ops.rmsnorm(x, self.gain, self.spec.eps, xn, want_rows)
            logits = ws.get("toy_head.logits", (n_want, self.spec.vocab), torch.float32)
            ops.gemm(xn, self.matrix, logits, workspace=ws.scratch())
            logits.copy_(self.spec.cap * torch.tanh(logits / self.spec.cap))
            return logits

    register_embedding("toy_positioned_table", PositionedTable)
    register_head("toy_capped_head", CappedHead)


def test_toy_embedding_with_learned_positions_and_toy_capped_head():
    """The model's two ends are parts like the others: an embedding that adds a learned row per
    position (attention then runs without rotation) and a head with a soft cap on the logits,
    defined here and registered; the head does not declare that it takes deferred sums, so the
    model completes the residual stream before it.  Decode steps are recorded and replayed."""
    _toy_embedding_and_head()
    hidden, vocab, d, cap = 40, 77, 16, 0.4
    layers = [_block(hidden, _attention_spec(hidden, 4, 2, d, theta=None)) for _ in range(2)]
    spec = ModelSpec(architecture="test", vocab=vocab, hidden=hidden, layers=tuple(layers),
                     schedule=(ScheduleEntry(0), ScheduleEntry(1)), final_norm=NormSpec(hidden, 1e-5),
                     tie_lm_head=False, max_positions=256,
                     embedding=PositionedTableSpec(vocab, hidden, 256), head=CappedHeadSpec(vocab, hidden, 1e-5, cap))
    for dtype, tol in (("float32", 1e-4), ("bfloat16", 3e-2)):
        engine, w = _engine(spec, dtype, seed=11)
        assert set(k for k in w if not k.startswith("layers.")) == \
            {"embed.tokens.weight", "embed.positions.weight", "out_norm.weight", "out.weight"}

        def reference(tokens):
            t = len(tokens)
            pos = list(range(t))
            x = w["embed.tokens.weight"][tokens] + w["embed.positions.weight"][pos]
            for i, b in enumerate(spec.layers):
                pre = f"layers.{i}."
                xn = plain.rmsnorm(x, w[pre + "mixer_norm.weight"], 1e-5)
                x = x + plain_attention(xn, w, pre + "mixer.", b.mixer, pos)[0]
                xn = plain.rmsnorm(x, w[pre + "ffn_norm.weight"], 1e-5)
                x = x + plain.swiglu(xn @ w[pre + "ffn.gate_proj.weight"].t(), xn @ w[pre + "ffn.up_proj.weight"].t()) \
                    @ w[pre + "ffn.down_proj.weight"].t()
            logits = plain.rmsnorm(x, w["out_norm.weight"], 1e-5) @ w["out.weight"].t()
            return cap * torch.tanh(logits / cap)

        a, b = helpers.random_tokens(45, vocab, 12), helpers.random_tokens(21, vocab, 13)
        ra, rb = reference(a), reference(b)
        assert ra.abs().max() > 0.5 * cap                      # the cap bends the largest logits
        assert helpers.rel_to_max(helpers.run_whole(engine, a), ra) < tol
        assert helpers.rel_to_max(helpers.run_tail_by_one(engine, b, 12), rb) < tol
        got = helpers.run_batch(engine, [a, b], [30, 5])
        assert helpers.rel_to_max(got[0], ra) < tol and helpers.rel_to_max(got[1], rb) < tol
