"""The memory-bound kernels alone against plain formulas, with the vectors of the
reference's kernel tests (rocml-kernels/tests/rmsnorm_rope.rs:19-148, activation.rs:19-71,
embedding_elementwise.rs:18-193): shapes that are no multiple of the block size and
degenerate ones."""
import pytest
import torch

pytestmark = pytest.mark.gpu

from rocml_amd import ops  # noqa: E402
from tests.plain import qwen3_plain as plain  # noqa: E402


def _bf16(x):
    return x.to(torch.bfloat16).to(torch.float64)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embedding(dtype):
    table = torch.randn(37, 50).to(dtype).cuda()
    ids = torch.tensor([0, 36, 5, 5, 17], dtype=torch.int32).cuda()
    out = torch.empty(5, 50, device="cuda")
    ops.embed_gather(table, ids, out)
    assert torch.equal(out, table[ids.long()].float())
    ops.embed_gather(table, ids, out, scale=0.5)
    assert torch.equal(out, table[ids.long()].float() * 0.5)


@pytest.mark.parametrize("rows,n", [(5, 300), (1, 7), (3, 4096), (2, 96), (1, 8192), (2, 8196)])
def test_rmsnorm(rows, n):
    x = torch.tensor([[((r * n + i) % 29) * 0.1 - 1.4 for i in range(n)] for r in range(rows)])
    w = torch.tensor([1.0 + 0.01 * (i % 50) for i in range(n)])
    eps = 1e-5
    want = plain.rmsnorm(x.double(), w.double(), eps)
    out = torch.empty(rows, n, device="cuda")
    ops.rmsnorm(x.cuda(), w.cuda(), eps, out)
    assert float((out.cpu().double() - want).abs().max()) < 1e-5
    out16 = torch.empty(rows, n, dtype=torch.bfloat16, device="cuda")
    ops.rmsnorm(x.cuda(), w.cuda(), eps, out16)
    assert float((out16.cpu().double() - want).abs().max()) < 8e-3 * float(want.abs().max())
    if rows > 1:                                   # gathered rows
        idx = torch.tensor([rows - 1, 0, rows - 1], dtype=torch.int32).cuda()
        got = torch.empty(3, n, device="cuda")
        ops.rmsnorm(x.cuda(), w.cuda(), eps, got, rows=idx)
        assert float((got.cpu().double() - want[[rows - 1, 0, rows - 1]]).abs().max()) < 1e-5


@pytest.mark.parametrize("rows,n,splits", [(3, 4096, 8), (2, 96, 3), (5, 300, 1), (1, 30, 5)])
def test_rmsnorm_adds_partial_sums(rows, n, splits):
    g = torch.Generator().manual_seed(0)
    x = torch.randn(rows, n, generator=g)
    w = 1 + 0.1 * torch.randn(n, generator=g)
    partials = torch.randn(splits, rows, n, generator=g)
    total = x.double() + partials.double().sum(0)
    want = plain.rmsnorm(total, w.double(), 1e-5)
    xd, out = x.cuda(), torch.empty(rows, n, device="cuda")
    ops.rmsnorm(xd, w.cuda(), 1e-5, out, partials=partials.cuda())
    assert float((out.cpu().double() - want).abs().max()) < 1e-5
    assert float((xd.cpu().double() - total).abs().max()) < 1e-5          # the sum went back into x
    xd = x.cuda()
    idx = torch.tensor([rows - 1, rows - 1, 0], dtype=torch.int32).cuda()
    got = torch.empty(3, n, device="cuda")
    ops.rmsnorm(xd, w.cuda(), 1e-5, got, rows=idx, partials=partials.cuda())
    assert float((got.cpu().double() - want[[rows - 1, rows - 1, 0]]).abs().max()) < 1e-5
    assert torch.equal(xd.cpu(), x)                                       # gathered rows: x is left alone


@pytest.mark.parametrize("tokens,inter", [(1, 1000), (1, 1), (7, 33)])
def test_swiglu(tokens, inter):
    n = tokens * inter
    gate = torch.tensor([(i % 23) * 0.1 - 1.2 for i in range(n)]).reshape(tokens, inter)
    up = torch.tensor([(i % 17) * 0.2 - 1.5 for i in range(n)]).reshape(tokens, inter)
    want = plain.swiglu(gate.double(), up.double())
    gu = torch.cat([gate, up], dim=1).cuda()
    out = torch.empty(tokens, inter, device="cuda")
    ops.swiglu(gu, out)
    assert float((out.cpu().double() - want).abs().max()) < 1e-6
    out16 = torch.empty(tokens, inter, dtype=torch.bfloat16, device="cuda")
    ops.swiglu(gu, out16)
    assert float((out16.cpu().double() - want).abs().max()) < 8e-3 * max(1.0, float(want.abs().max()))
    pairs = torch.stack([gate, up], dim=2).reshape(tokens, 2 * inter).cuda()
    ops.swiglu(pairs, out, interleaved=True)
    assert float((out.cpu().double() - want).abs().max()) < 1e-6


def test_add_into():
    x = torch.randn(5, 33, device="cuda")
    y = torch.randn(5, 33, device="cuda")
    want = x + y
    ops.add_into(x, y)
    assert torch.equal(x, want)
    y16 = torch.randn(5, 33, device="cuda").to(torch.bfloat16)
    want = x + y16.float()
    ops.add_into(x, y16)
    assert torch.equal(x, want)


def _rope_neighbours(x, positions, theta):
    """The rotation with neighbours as pairs: values (2i, 2i + 1) of a head turn by the angle
    pos * theta^(-2i/D).  It is the rotation over halves applied to the head with its even
    values first and its odd values behind them."""
    d = x.shape[-1]
    order = list(range(0, d, 2)) + list(range(1, d, 2))
    back = [order.index(i) for i in range(d)]
    return plain.rope_neox(x[..., order], positions, theta)[..., back]


def _qkv_case(tokens, hq, hkv, d, pos_base, theta, rot, norm, dtype, seed=0, splits=1, pairing="halves"):
    """Runs the fused kernel on one sequence whose pages are handed out backwards; returns
    (q, k rows, v rows) read back from q_out and the cache, and the plain expectation."""
    g = torch.Generator().manual_seed(seed)
    page = 64
    ld = (hq + 2 * hkv) * d
    qkv = torch.tensor([(i % 31) * 0.05 - 0.7 for i in range(tokens * ld)]).reshape(tokens, ld)
    qkv = qkv + 0.01 * torch.randn(tokens, ld, generator=g)
    qg = 1 + 0.1 * torch.randn(d, generator=g)
    kg = 1 + 0.1 * torch.randn(d, generator=g)
    eps = 1e-5
    positions = list(range(pos_base, pos_base + tokens))
    n_pages = (pos_base + tokens + page - 1) // page
    table = torch.tensor([[n_pages - 1 - i for i in range(n_pages)]], dtype=torch.int32)
    kc = torch.zeros(n_pages, hkv, page, d, dtype=dtype, device="cuda")
    vc = torch.zeros(n_pages, hkv, d, page, dtype=dtype, device="cuda")
    q_out = torch.empty(tokens, hq * d, dtype=dtype, device="cuda")
    cos = sin = None
    if rot:
        inv = torch.tensor([theta ** (-2.0 * i / rot) for i in range(rot // 2)], dtype=torch.float64).cuda()
        cos = torch.empty(tokens, rot // 2, device="cuda")
        sin = torch.empty(tokens, rot // 2, device="cuda")
        ops.rope_table(torch.tensor(positions, dtype=torch.int32).cuda(), inv, cos, sin)
    fed = qkv.cuda()
    if splits > 1:                      # the same values as a sum of parts
        parts = torch.randn(splits, tokens, ld, generator=g)
        parts[0] = qkv - parts[1:].sum(0)
        qkv = parts.sum(0)
        fed = parts.cuda()
    ops.qk_norm_rope_append(fed, hq, hkv, d, qg.cuda() if norm else None, kg.cuda() if norm else None, eps,
                            cos, sin, rot, q_out, kc, vc, table.cuda(),
                            torch.zeros(tokens, dtype=torch.int32).cuda(),
                            torch.tensor(positions, dtype=torch.int32).cuda(), n_splits=splits, pairing=pairing)
    q = qkv[:, :hq * d].reshape(tokens, hq, d).double()
    k = qkv[:, hq * d:(hq + hkv) * d].reshape(tokens, hkv, d).double()
    v = qkv[:, (hq + hkv) * d:].reshape(tokens, hkv, d).double()
    if norm:
        q, k = plain.rmsnorm(q, qg.double(), eps), plain.rmsnorm(k, kg.double(), eps)
    if rot:
        turn = plain.rope_neox if pairing == "halves" else _rope_neighbours
        q = torch.cat([turn(q[..., :rot], positions, theta), q[..., rot:]], -1)
        k = torch.cat([turn(k[..., :rot], positions, theta), k[..., rot:]], -1)
    got_k = torch.stack([kc[table[0, p // page], :, p % page].cpu() for p in positions]).double()
    got_v = torch.stack([vc[table[0, p // page], :, :, p % page].cpu() for p in positions]).double()
    return q_out.cpu().double().reshape(tokens, hq, d), got_k, got_v, q, k, v, (kc, vc, table, positions)


@pytest.mark.parametrize("tokens,hq,hkv,d,pos_base,rot,norm", [
    (10, 3, 3, 16, 5, 16, True), (1, 2, 1, 4, 0, 4, True), (70, 4, 2, 48, 100, 48, True),
    (5, 2, 2, 128, 60, 64, True), (5, 6, 2, 32, 0, 32, False), (3, 2, 1, 16, 7, 0, True), (2, 1, 1, 264, 1, 264, True),
    # whole head rotated with both values of a pair in one lane; many tokens: values through the transposing kernel
    (3, 8, 2, 128, 60, 128, True), (150, 4, 2, 128, 37, 128, True), (64, 2, 1, 256, 0, 256, True), (129, 2, 2, 80, 63, 80, False)])
def test_qk_norm_rope_append(tokens, hq, hkv, d, pos_base, rot, norm):
    gq, gk, gv, q, k, v, (kc, vc, table, positions) = _qkv_case(tokens, hq, hkv, d, pos_base, 1e4, rot, norm, torch.float32)
    assert float((gq - q).abs().max()) < 1e-5
    assert float((gk - k).abs().max()) < 1e-5
    assert float((gv - v).abs().max()) == 0.0
    # nothing else in the cache was touched
    written = torch.zeros(kc.shape[0], 64, dtype=torch.bool)
    for p in positions:
        written[table[0, p // 64], p % 64] = True
    assert float(kc.cpu()[~written.unsqueeze(1).expand(-1, kc.shape[1], -1)].abs().sum()) == 0.0
    assert float(vc.cpu().transpose(2, 3)[~written.unsqueeze(1).expand(-1, vc.shape[1], -1)].abs().sum()) == 0.0
    gq, gk, gv, *_ = _qkv_case(tokens, hq, hkv, d, pos_base, 1e4, rot, norm, torch.bfloat16)
    assert float((gq - q).abs().max()) < 8e-3 * float(q.abs().max())
    assert float((gk - k).abs().max()) < 8e-3 * float(k.abs().max())
    assert float((gv - _bf16(v)).abs().max()) == 0.0


@pytest.mark.parametrize("tokens,hq,hkv,d,pos_base,rot,norm", [
    (10, 3, 3, 16, 5, 16, True), (70, 4, 2, 48, 100, 48, True), (5, 2, 2, 128, 60, 64, True),
    (3, 8, 2, 128, 60, 128, True), (150, 4, 2, 128, 37, 128, False), (2, 1, 1, 264, 1, 264, True)])
def test_qk_norm_rope_append_with_neighbours_as_pairs(tokens, hq, hkv, d, pos_base, rot, norm):
    """The other pairing of the rotation: (2i, 2i + 1) instead of (i, i + rot/2); a wrong partner,
    a wrong angle column or a wrong sign fails it."""
    for dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 8e-3)):
        gq, gk, gv, q, k, v, _ = _qkv_case(tokens, hq, hkv, d, pos_base, 1e4, rot, norm, dtype, pairing="neighbours")
        assert float((gq - q).abs().max()) < tol * max(1.0, float(q.abs().max()))
        assert float((gk - k).abs().max()) < tol * max(1.0, float(k.abs().max()))
    *_, q_halves, k_halves, _, _ = _qkv_case(tokens, hq, hkv, d, pos_base, 1e4, rot, norm, torch.float32)
    assert float((q - q_halves).abs().max()) > 1e-2            # (the two pairings do differ on this input)
    with pytest.raises(Exception, match="pairing"):
        _qkv_case(2, 1, 1, 16, 0, 1e4, 16, True, torch.float32, pairing="thirds")


@pytest.mark.parametrize("splits", [2, 5, 8])
def test_qk_norm_rope_append_adds_partial_sums(splits):
    gq, gk, gv, q, k, v, _ = _qkv_case(9, 4, 2, 128, 60, 1e4, 128, True, torch.float32, splits=splits)
    assert float((gq - q).abs().max()) < 2e-5 and float((gk - k).abs().max()) < 2e-5 and float((gv - v).abs().max()) < 2e-6


def test_rotation_table_at_large_positions():
    pos = torch.tensor([0, 1, 4095, 40959, 1_000_000], dtype=torch.int32).cuda()
    half, theta = 64, 1e6
    inv = torch.tensor([theta ** (-2.0 * i / (2 * half)) for i in range(half)], dtype=torch.float64)
    cos = torch.empty(5, half, device="cuda")
    sin = torch.empty(5, half, device="cuda")
    ops.rope_table(pos, inv.cuda(), cos, sin)
    ang = pos.cpu().double()[:, None] * inv[None, :]
    assert float((cos.cpu().double() - ang.cos()).abs().max()) < 1e-7
    assert float((sin.cpu().double() - ang.sin()).abs().max()) < 1e-7


def test_refusals():
    from rocml_amd.errors import KernelError
    x = torch.randn(2, 8)
    with pytest.raises(KernelError, match="GPU"):
        ops.rmsnorm(x, torch.ones(8), 1e-5, torch.empty(2, 8))
    with pytest.raises(KernelError, match="eps"):
        ops.rmsnorm(x.cuda(), torch.ones(8).cuda(), 0.0, torch.empty(2, 8).cuda())
    with pytest.raises(KernelError):
        ops.rmsnorm(x.cuda(), torch.ones(9).cuda(), 1e-5, torch.empty(2, 8).cuda())
    with pytest.raises(KernelError):
        ops.swiglu(torch.randn(2, 9).cuda(), torch.empty(2, 4).cuda())
