"""The matrix product kernels alone against a plain 32-bit product of the same operands,
at sizes other than the engine's: sizes that are no multiple of a tile, single rows,
every algorithm and epilogue."""
import pytest
import torch

pytestmark = pytest.mark.gpu

from rocml_amd import ops  # noqa: E402
from rocml_amd.errors import KernelError  # noqa: E402

PLAIN, TILE, SKINNY, KPAR, TILE256, TILE192, TILE128X192, TILE256X96, TILE64X256 = 1, 2, 3, 4, 5, 6, 7, 8, 9


def _operands(m, n, k, dtype, seed):
    g = torch.Generator(device="cpu").manual_seed(seed)
    x = torch.randn(m, k, generator=g).to(dtype).cuda()
    w = (torch.randn(n, k, generator=g) * 0.05).to(dtype).cuda()
    return x, w


def _ref(x, w):
    return (x.double() @ w.double().t())


@pytest.mark.parametrize("m,n,k", [(1, 7, 5), (3, 64, 16), (65, 130, 33), (200, 96, 257), (17, 384, 96)])
def test_plain_float32(m, n, k):
    x, w = _operands(m, n, k, torch.float32, 1)
    out = torch.empty(m, n, dtype=torch.float32, device="cuda")
    ops.gemm(x, w, out, algo=PLAIN)
    ref = _ref(x, w)
    assert float((out.double() - ref).abs().max()) < 1e-5 * max(1.0, float(ref.abs().max()))
    base = torch.randn(m, n, device="cuda")
    acc = base.clone()
    ops.gemm(x, w, acc, accumulate=True, algo=PLAIN)
    assert float((acc.double() - (ref + base.double())).abs().max()) < 1e-5 * max(1.0, float(ref.abs().max()))


SHAPES = [(1, 64, 64), (5, 200, 72), (16, 130, 512), (17, 96, 264), (33, 4096, 1024), (48, 1000, 776), (64, 257, 4096),
          (8, 1000, 2056), (128, 128, 64), (129, 300, 200), (300, 515, 72), (2048, 512, 1024),
          (1409, 300, 128), (2561, 200, 64)]       # 12 and 21 tile rows of 128, 6 and 11 of 256: whole bands of eight and a rest


@pytest.mark.parametrize("algo", [PLAIN, TILE, SKINNY, KPAR, TILE256, TILE192, TILE128X192, TILE256X96, TILE64X256])
@pytest.mark.parametrize("m,n,k", SHAPES)
def test_bfloat16_algorithms(m, n, k, algo):
    if (algo == SKINNY and m > 64) or (algo == KPAR and m > 16):
        pytest.skip("the few-rows kernels take at most 64 and 16 rows")
    x, w = _operands(m, n, k, torch.bfloat16, 2)
    ref = _ref(x, w)
    scale = max(1.0, float(ref.abs().max()))
    ws = torch.empty(64 << 20, dtype=torch.uint8, device="cuda")
    out = torch.full((m, n), float("nan"), dtype=torch.float32, device="cuda")
    ops.gemm(x, w, out, algo=algo, workspace=ws)
    assert float((out.double() - ref).abs().max()) < 2e-5 * scale, "32-bit output"
    out16 = torch.empty(m, n, dtype=torch.bfloat16, device="cuda")
    ops.gemm(x, w, out16, algo=algo, workspace=ws)
    assert float((out16.double() - ref).abs().max()) < 5e-3 * scale, "bfloat16 output"
    base = torch.randn(m, n, device="cuda")
    acc = base.clone()
    ops.gemm(x, w, acc, accumulate=True, algo=algo, workspace=ws)
    assert float((acc.double() - (ref + base.double())).abs().max()) < 2e-5 * scale, "accumulating"


def test_strided_rows_and_refusals():
    from rocml_amd.errors import KernelError
    big = torch.randn(40, 200, device="cuda").to(torch.bfloat16)
    x = big[:, 8:72]                       # row stride 200, 64 columns
    w = (torch.randn(48, 64, device="cuda") * 0.1).to(torch.bfloat16)
    out = torch.empty(40, 48, dtype=torch.float32, device="cuda")
    ops.gemm(x, w, out)
    assert float((out.double() - _ref(x, w)).abs().max()) < 1e-4
    odd = torch.randn(4, 36, device="cuda").to(torch.bfloat16)   # K = 36 is no multiple of 8
    w2 = torch.randn(8, 36, device="cuda").to(torch.bfloat16)
    out2 = torch.empty(4, 8, dtype=torch.float32, device="cuda")
    ops.gemm(odd, w2, out2)                # falls back to the plain kernel
    assert float((out2.double() - _ref(odd, w2)).abs().max()) < 1e-3
    with pytest.raises(KernelError):
        ops.gemm(odd, w2, out2, algo=TILE)
    with pytest.raises(KernelError):
        ops.gemm(x.cpu(), w, out)


@pytest.mark.parametrize("algo", [PLAIN, TILE, SKINNY, KPAR, TILE256, TILE192, TILE128X192, TILE256X96, TILE64X256])
@pytest.mark.parametrize("m,n,k", [(1, 64, 64), (7, 448, 96), (25, 300, 520), (41, 130, 1032), (64, 1000, 264), (130, 256, 128), (300, 2048, 512)])
def test_gated_epilogue(m, n, k, algo):
    """Rows of the weight are (gate, up) pairs; the output is silu(gate) * up, formed from
    the 32-bit sums."""
    if (algo == SKINNY and m > 64) or (algo == KPAR and m > 16):
        pytest.skip("the few-rows kernels take at most 64 and 16 rows")
    x, w = _operands(m, n, k, torch.bfloat16, 3)
    full = _ref(x, w)
    gate, up = full[:, 0::2], full[:, 1::2]
    ref = gate / (1 + torch.exp(-gate)) * up
    ws = torch.empty(16 << 20, dtype=torch.uint8, device="cuda")
    out = torch.empty(m, n // 2, dtype=torch.bfloat16, device="cuda")
    ops.gemm(x, w, out, algo=algo, workspace=ws, epilogue="swiglu")
    assert float((out.double().cpu() - ref.cpu()).abs().max()) < 5e-3 * max(1.0, float(ref.abs().max()))
    if algo == PLAIN:
        x32, w32 = x.float(), w.float()
        out32 = torch.empty(m, n // 2, dtype=torch.float32, device="cuda")
        ops.gemm(x32, w32, out32, workspace=ws, epilogue="swiglu")
        assert float((out32.double().cpu() - ref.cpu()).abs().max()) < 2e-5 * max(1.0, float(ref.abs().max()))


def test_deferred_split_sums():
    """A product split along K may leave its partial sums to the caller; adding them in split
    order gives the product."""
    x, w = _operands(8, 256, 4096, torch.bfloat16, 4)
    ref = _ref(x, w)
    ws = torch.empty(16 << 20, dtype=torch.uint8, device="cuda")
    base = torch.randn(8, 256, device="cuda")
    out = base.clone()
    splits = ops.gemm(x, w, out, accumulate=True, workspace=ws, defer=True)
    assert splits > 1 and torch.equal(out, base)              # nothing was added yet
    partials = ws[:splits * 8 * 256 * 4].view(torch.float32).view(splits, 8, 256)
    assert float((partials.double().sum(0) - ref).abs().max()) < 2e-5 * float(ref.abs().max())
    ops.splitk_reduce(partials, out, accumulate=True)
    assert float((out.double() - (ref + base.double())).abs().max()) < 2e-5 * float(ref.abs().max())
    assert ops.gemm(x, w, out, workspace=None, defer=True) == 0   # no workspace: no split, complete result
    assert float((out.double() - ref).abs().max()) < 2e-5 * float(ref.abs().max())


@pytest.mark.parametrize("m,n,k", [(512, 768, 4096), (300, 515, 2056), (1000, 256, 2048), (100, 384, 1544)])
def test_many_rows_with_k_cut_in_pieces(m, n, k):
    """Few tiles and a long K: the tile kernel gives each piece of K to a block of its own and
    adds the pieces in order, or leaves them to the caller."""
    x, w = _operands(m, n, k, torch.bfloat16, 5)
    ref = _ref(x, w)
    scale = max(1.0, float(ref.abs().max()))
    ws = torch.empty(32 << 20, dtype=torch.uint8, device="cuda")
    out = torch.full((m, n), float("nan"), dtype=torch.float32, device="cuda")
    assert ops.gemm(x, w, out, workspace=ws) == 0
    assert float((out.double() - ref).abs().max()) < 2e-5 * scale
    base = torch.randn(m, n, device="cuda")
    acc = base.clone()
    splits = ops.gemm(x, w, acc, accumulate=True, workspace=ws, defer=True)
    assert 2 <= splits <= 8 and torch.equal(acc, base)
    partials = ws[:splits * m * n * 4].view(torch.float32).view(splits, m, n)
    ops.splitk_reduce(partials, acc, accumulate=True)
    assert float((acc.double() - (ref + base.double())).abs().max()) < 2e-5 * scale
    # without room for the pieces the product is done in one
    small = torch.empty(m * n * 4, dtype=torch.uint8, device="cuda")
    out16 = torch.empty(m, n, dtype=torch.bfloat16, device="cuda")
    assert ops.gemm(x, w, out16, workspace=small, defer=True) == 0
    assert float((out16.double() - ref).abs().max()) < 5e-3 * scale


@pytest.mark.parametrize("waves", [0, 4, 8])
@pytest.mark.parametrize("m,n,k", [(1, 64, 64), (3, 100, 72), (8, 4096, 1032), (16, 130, 4096), (7, 515, 264), (2, 88, 12288)])
def test_residual_sum_that_prepares_the_next_norm(m, n, k, waves):
    """resid += x W^T with whole sums, xg = bfloat16(resid * gain), and per 16 columns the sum of
    squares of the new residual row, from which the consumer forms the norm's scale."""
    x, w = _operands(m, n, k, torch.bfloat16, 5)
    g = torch.Generator().manual_seed(6)
    base = torch.randn(m, n, generator=g)
    gain = 1 + 0.2 * torch.randn(n, generator=g)
    resid = base.cuda()
    xg = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    tiles = (n + ops.PRESCALE_TILE - 1) // ops.PRESCALE_TILE
    ssq = torch.full((m, tiles), float("nan"), device="cuda")
    assert ops.gemm_residual_prescale_fits(x, w)
    ops.gemm_residual_prescale(x, w, resid, gain.cuda(), xg, ssq, waves=waves)
    want = base.double() + _ref(x, w).cpu()
    scale = max(1.0, float(want.abs().max()))
    assert float((resid.double().cpu() - want).abs().max()) < 2e-5 * scale
    assert float((xg.double().cpu() - want * gain.double()).abs().max()) < 5e-3 * float((want * gain.double()).abs().max())
    padded = torch.zeros(m, tiles * 16, dtype=torch.float64)
    padded[:, :n] = want ** 2
    assert float((ssq.double().cpu() - padded.view(m, tiles, 16).sum(-1)).abs().max()) < 1e-5 * float(padded.max()) * 16
    # the norm's output, put together the way a consumer does
    eps = 1e-5
    inv = 1.0 / torch.sqrt(ssq.double().cpu().sum(-1, keepdim=True) / n + eps)
    normed = want / torch.sqrt((want ** 2).mean(-1, keepdim=True) + eps) * gain.double()
    assert float((xg.double().cpu() * inv - normed).abs().max()) < 5e-3 * float(normed.abs().max())
    with pytest.raises(KernelError):
        ops.gemm_residual_prescale(torch.zeros(17, k, dtype=torch.bfloat16, device="cuda"), w,
                                   torch.zeros(17, n, device="cuda"), gain.cuda(),
                                   torch.zeros(17, n, dtype=torch.bfloat16, device="cuda"), torch.zeros(17, tiles, device="cuda"))


@pytest.mark.parametrize("algo", [0, SKINNY, KPAR])
@pytest.mark.parametrize("m,n,k,parts", [(1, 64, 64, 4), (2, 24576, 4096, 256), (8, 448, 96, 6), (16, 1000, 264, 17), (13, 300, 1032, 64)])
def test_gated_epilogue_applies_a_row_scale(m, n, k, parts, algo):
    """The operand lacks its norm's scale; the gated epilogue multiplies the sums of a row by
    1 / sqrt(sum of the row's parts / K + eps) before the activation."""
    x, w = _operands(m, n, k, torch.bfloat16, 7)
    g = torch.Generator().manual_seed(8)
    ssq = (torch.rand(m, parts, generator=g) * 3 * k / parts).cuda()
    eps = 1e-5
    inv = 1.0 / torch.sqrt(ssq.double().sum(-1, keepdim=True) / k + eps)
    full = _ref(x, w) * inv
    gate, up = full[:, 0::2], full[:, 1::2]
    ref = gate / (1 + torch.exp(-gate)) * up
    ws = torch.empty(16 << 20, dtype=torch.uint8, device="cuda")
    out = torch.empty(m, n // 2, dtype=torch.bfloat16, device="cuda")
    ops.gemm(x, w, out, algo=algo, workspace=ws, epilogue="swiglu", row_scale=ops.RowScale(ssq, eps, k))
    assert float((out.double() - ref).abs().max()) < 5e-3 * max(1.0, float(ref.abs().max()))
    with pytest.raises(KernelError):                       # not without the gated epilogue, not for more rows
        ops.gemm(x, w, torch.empty(m, n, device="cuda"), workspace=ws, row_scale=ops.RowScale(ssq, eps, k))
    with pytest.raises(KernelError):
        ops.gemm(torch.zeros(17, k, dtype=torch.bfloat16, device="cuda"), w, torch.empty(17, n // 2, dtype=torch.bfloat16, device="cuda"),
                 workspace=ws, epilogue="swiglu", row_scale=ops.RowScale(torch.ones(17, parts, device="cuda"), eps, k))


@pytest.mark.parametrize("m", [3, 16, 20, 40, 64])
@pytest.mark.parametrize("n,k", [(34816, 264), (51200, 512), (65568, 256), (90, 2056)])
def test_wide_gated_products_take_blocks_of_many_waves(m, n, k):
    """The gated product runs on blocks of as many waves as make one round over the chip: nine at
    34816 columns, thirteen (sixteen at 49 to 64 rows) at 51200, and beyond one round of sixteen
    waves the count that leaves the busiest CU the fewest columns; with and without a row scale."""
    x, w = _operands(m, n, k, torch.bfloat16, 11)
    full = _ref(x, w)
    ws = torch.empty(16 << 20, dtype=torch.uint8, device="cuda")
    out = torch.empty(m, n // 2, dtype=torch.bfloat16, device="cuda")
    for scaled in (False, True):
        if scaled and m > ops.ROW_SCALE_MAX_ROWS:
            continue
        inv = 1.0
        scale = None
        if scaled:
            ssq = (torch.rand(m, 5, generator=torch.Generator().manual_seed(12)) * k).cuda()
            inv = 1.0 / torch.sqrt(ssq.double().sum(-1, keepdim=True) / k + 1e-6)
            scale = ops.RowScale(ssq, 1e-6, k)
        gate, up = (full * inv)[:, 0::2], (full * inv)[:, 1::2]
        ref = gate / (1 + torch.exp(-gate)) * up
        out.fill_(float("nan"))
        ops.gemm(x, w, out, workspace=ws, epilogue="swiglu", row_scale=scale)
        assert float((out.double() - ref).abs().max()) < 5e-3 * max(1.0, float(ref.abs().max()))


@pytest.mark.parametrize("m", [5, 16, 24, 32])
@pytest.mark.parametrize("n,k", [(6144, 4096), (7168, 5120), (5120, 5120), (1000, 3080), (4096, 4096)])
def test_few_rows_products_with_chosen_blocks(m, n, k):
    """A product cut along K whose waves a block and K pieces are chosen for the busiest CU (six
    waves and four pieces at 6144 x 4096, seven at 7168 x 5120, five at 5120 x 5120), complete or
    with its partial sums left to the caller."""
    x, w = _operands(m, n, k, torch.bfloat16, 13)
    ref = _ref(x, w)
    tol = 2e-5 * max(1.0, float(ref.abs().max()))
    ws = torch.empty(32 << 20, dtype=torch.uint8, device="cuda")
    base = torch.randn(m, n, device="cuda")
    out = base.clone()
    ops.gemm(x, w, out, accumulate=True, workspace=ws)
    assert float((out.double() - (ref + base.double())).abs().max()) < tol
    splits = ops.gemm(x, w, out, workspace=ws, defer=True)
    if splits:
        partials = ws[:splits * m * n * 4].view(torch.float32).view(splits, m, n)
        assert float((partials.double().sum(0) - ref).abs().max()) < tol
    else:
        assert float((out.double() - ref).abs().max()) < tol
