"""The attention kernels alone against plain softmax attention written here, at other
sizes than the engine's.  Shapes follow the reference's kernel tests
(rocml-kernels/tests/attn_decode.rs:198-256, attn_prefill.rs:153-202): one cached
position, lengths that are no multiple of a tile, several splits with a remainder, group
sizes 1, 2 and 4, a head size of 256, a cache much longer than the sequence, a chunk that
starts deep in the sequence.  Pages of the cache are handed out in a scrambled order and
unused pages hold large values, so a read outside a sequence's pages or beyond its
length shows.
"""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

from rocml_amd import ops  # noqa: E402

PAGE = 64
PLAIN, MFMA = 1, 2


def _reference(q, k, v, positions, scale, window):
    """q [n, Hq, D] for the tokens at ``positions`` of one sequence; k, v [L, Hkv, D]."""
    n, hq, d = q.shape
    group = hq // k.shape[1]
    out = torch.zeros(n, hq, d, dtype=torch.float64)
    for i, p in enumerate(positions):
        lo = 0 if window is None else max(0, p - window + 1)
        for h in range(hq):
            s = (k[lo:p + 1, h // group].double() @ q[i, h].double()) * scale
            w = torch.softmax(s, dim=0)
            out[i, h] = w @ v[lo:p + 1, h // group].double()
    return out


def _build(seqs, hq, hkv, d, dtype, seed, spare_pages=3):
    """seqs: list of (context length after the step, new tokens).  Returns device tensors of a
    packed step and the per-sequence K, V, Q on the CPU."""
    g = torch.Generator().manual_seed(seed)
    n_pages = sum((length + PAGE - 1) // PAGE for length, _ in seqs) + spare_pages
    order = torch.randperm(n_pages, generator=g).tolist()
    kc = torch.full((n_pages, hkv, PAGE, d), 1e4, dtype=dtype)
    vc = torch.full((n_pages, hkv, d, PAGE), 1e4, dtype=dtype)
    width = max((length + PAGE - 1) // PAGE for length, _ in seqs)
    table = torch.full((len(seqs), width), -1, dtype=torch.int32)
    ks, vs, qs, tok_seq, tok_pos, cu = [], [], [], [], [], [0]
    for b, (length, n_new) in enumerate(seqs):
        k = torch.randn(length, hkv, d, generator=g).to(dtype)
        v = torch.randn(length, hkv, d, generator=g).to(dtype)
        q = torch.randn(n_new, hq, d, generator=g).to(dtype)
        for lp in range((length + PAGE - 1) // PAGE):
            page = order.pop()
            table[b, lp] = page
            rows = slice(lp * PAGE, min(length, (lp + 1) * PAGE))
            n = rows.stop - rows.start
            kc[page, :, :n] = k[rows].transpose(0, 1)
            vc[page, :, :, :n] = v[rows].permute(1, 2, 0)
            # the rest of the sequence's last page stays finite, as in the engine's cache
            kc[page, :, n:] = 0
            vc[page, :, :, n:] = 0
        ks.append(k), vs.append(v), qs.append(q)
        tok_seq += [b] * n_new
        tok_pos += list(range(length - n_new, length))
        cu.append(cu[-1] + n_new)
    dev = dict(q=torch.cat(qs).reshape(-1, hq * d).cuda(), kc=kc.cuda(), vc=vc.cuda(), table=table.cuda(),
               tok_seq=torch.tensor(tok_seq, dtype=torch.int32).cuda(),
               tok_pos=torch.tensor(tok_pos, dtype=torch.int32).cuda(),
               cu=torch.tensor(cu, dtype=torch.int32).cuda())
    return dev, ks, vs, qs


def _run(dev, seqs, hq, hkv, d, scale, window, algo, n_splits=0):
    out = torch.full_like(dev["q"], float("nan"))
    ws = torch.empty(32 << 20, dtype=torch.uint8, device="cuda")
    ops.attention(dev["q"], out, dev["kc"], dev["vc"], dev["table"], dev["tok_seq"], dev["tok_pos"], hq, hkv,
                  d, scale, window, algo=algo, workspace=ws, cu_seqlens=dev["cu"],
                  max_new=max(n for _, n in seqs), q_counts=[n for _, n in seqs],
                  max_len=max(length for length, _ in seqs), n_splits=n_splits)
    return out.cpu()


def _check(seqs, hq, hkv, d, dtype, algo, window=None, n_splits=0, seed=0):
    dev, ks, vs, qs = _build(seqs, hq, hkv, d, dtype, seed)
    scale = 1.0 / math.sqrt(d)
    got = _run(dev, seqs, hq, hkv, d, scale, window, algo, n_splits).double().reshape(-1, hq, d)
    at = 0
    tol = 1e-4 if dtype == torch.float32 else 1.5e-2     # bfloat16: probabilities and output are rounded
    for (length, n_new), k, v, q in zip(seqs, ks, vs, qs):
        ref = _reference(q, k, v, list(range(length - n_new, length)), scale, window)
        err = float((got[at:at + n_new] - ref).abs().max())
        assert err < tol, f"sequence of {length} with {n_new} new tokens: error {err}"
        at += n_new


# (Hq, Hkv, D, context length, splits): rocml-kernels/tests/attn_decode.rs:198-256
DECODE = [(16, 8, 128, 1, 0), (16, 8, 128, 3, 0), (16, 8, 128, 33, 0), (16, 8, 128, 257, 1), (16, 8, 128, 257, 4),
          (16, 8, 128, 2048, 1), (16, 8, 128, 2048, 8), (8, 2, 256, 400, 0), (8, 2, 256, 1024, 6),
          (8, 8, 128, 300, 0), (16, 8, 128, 100, 0), (6, 2, 32, 77, 3), (4, 1, 64, 130, 2), (16, 1, 64, 65, 0),
          (12, 4, 96, 200, 0), (12, 4, 96, 200, 3), (16, 2, 96, 9, 2), (24, 3, 192, 500, 5)]


@pytest.mark.parametrize("hq,hkv,d,length,splits", DECODE)
def test_decode_bfloat16_mfma(hq, hkv, d, length, splits):
    _check([(length, 1)], hq, hkv, d, torch.bfloat16, MFMA, n_splits=splits)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hq,hkv,d,length,splits", DECODE[:4] + [(5, 5, 48, 70, 0), (4, 2, 16, 129, 0)])
def test_decode_plain(hq, hkv, d, length, splits, dtype):
    _check([(length, 1)], hq, hkv, d, dtype, PLAIN)


def test_decode_batch_of_unequal_lengths_and_windows():
    seqs = [(1, 1), (64, 1), (65, 1), (700, 1), (129, 1), (2, 1), (1000, 1)]
    for window in (None, 1, 70, 128):
        _check(seqs, 8, 2, 128, torch.bfloat16, MFMA, window=window, seed=3)
        _check(seqs, 8, 2, 128, torch.bfloat16, MFMA, window=window, n_splits=5, seed=3)
        _check(seqs[:5], 6, 3, 48, torch.float32, PLAIN, window=window, seed=4)


# (Hq, Hkv, D, new tokens, first position): rocml-kernels/tests/attn_prefill.rs:153-202
PREFILL = [(16, 8, 128, 1, 0), (16, 8, 128, 1, 99), (16, 8, 128, 17, 0), (8, 2, 256, 64, 0), (8, 2, 256, 64, 200),
           (16, 4, 128, 33, 50), (8, 8, 128, 40, 0), (16, 8, 128, 256, 1024), (16, 4, 128, 13, 0),
           (6, 2, 32, 130, 0), (4, 1, 64, 300, 77), (12, 4, 96, 129, 3)]


@pytest.mark.parametrize("hq,hkv,d,n_new,first", PREFILL)
def test_prefill_bfloat16_mfma(hq, hkv, d, n_new, first):
    _check([(first + n_new, n_new)], hq, hkv, d, torch.bfloat16, MFMA)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hq,hkv,d,n_new,first", PREFILL[:3] + [(5, 5, 48, 70, 10), (4, 2, 16, 129, 0)])
def test_prefill_plain(hq, hkv, d, n_new, first, dtype):
    _check([(first + n_new, n_new)], hq, hkv, d, dtype, PLAIN)


def test_prefill_batch_of_unequal_lengths_and_windows():
    seqs = [(5, 5), (200, 130), (64, 64), (129, 1), (400, 257), (1, 1)]
    for window in (None, 1, 24, 70, 200):
        _check(seqs, 8, 2, 64, torch.bfloat16, MFMA, window=window, seed=5)
        _check(seqs[:4], 6, 2, 48, torch.float32, PLAIN, window=window, seed=6)


def test_a_far_key_decides():
    """One key far back among hundreds carries almost all weight: scale the query and that
    key so that its score stands out; the output must be that key's value row."""
    hq, hkv, d, length = 8, 2, 128, 900
    for algo, n_new in ((MFMA, 1), (MFMA, 40), (PLAIN, 1)):
        dev, ks, vs, qs = _build([(length, n_new)], hq, hkv, d, torch.bfloat16, 7)
        far = 37
        q = torch.zeros(n_new, hq, d)
        q[:, :, 5] = 40.0
        k_row = torch.zeros(hkv, d)
        k_row[:, 5] = 40.0
        page = int(dev["table"][0, far // PAGE])
        dev["q"] = q.reshape(n_new, hq * d).to(torch.bfloat16).cuda()
        dev["kc"][page, :, far % PAGE] = k_row.to(torch.bfloat16).cuda()
        got = _run(dev, [(length, n_new)], hq, hkv, d, 1.0, None, algo).double().reshape(n_new, hq, d)
        want = vs[0][far].double()            # [Hkv, D]
        for h in range(hq):
            assert float((got[:, h] - want[h // (hq // hkv)]).abs().max()) < 2e-2


def _fused_case(seqs, hq, hkv, d, qkv_splits, attn_splits, window, seed, norm=True, rotate=True):
    """A decode step through the fused kernel: random projection output (cut into partial sums),
    gains and rotation angles; the position of every sequence's new token holds a large value in
    the cache beforehand, so a row that is not replaced shows.  Checked against the two-kernel
    path (same cache rows, same output within rounding of q) and against plain attention over
    the keys and values computed here."""
    dev, ks, vs, _ = _build(seqs, hq, hkv, d, torch.bfloat16, seed)
    g = torch.Generator().manual_seed(seed + 1)
    n = len(seqs)
    rows = (hq + 2 * hkv) * d
    parts = torch.randn(qkv_splits, n, rows, generator=g) * (1.0 / math.sqrt(qkv_splits))
    qkv = parts.double().sum(0)
    q_gain = (1 + 0.3 * torch.randn(d, generator=g)) if norm else None
    k_gain = (1 + 0.3 * torch.randn(d, generator=g)) if norm else None
    eps = 1e-5
    angle = torch.rand(n, d // 2, generator=g).double() * 6.28
    cos, sin = (torch.cos(angle).float(), torch.sin(angle).float()) if rotate else (None, None)

    def prepare(x, gain):          # [n, heads, d] in float64
        if gain is not None:
            x = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * gain.double()
        if rotate:
            c, s_ = cos.double()[:, None], sin.double()[:, None]
            lo_, hi_ = x[..., :d // 2], x[..., d // 2:]
            x = torch.cat([lo_ * c - hi_ * s_, lo_ * s_ + hi_ * c], dim=-1)
        return x
    q = prepare(qkv[:, :hq * d].reshape(n, hq, d), q_gain)
    k_new = prepare(qkv[:, hq * d:(hq + hkv) * d].reshape(n, hkv, d), k_gain)
    v_new = qkv[:, (hq + hkv) * d:].reshape(n, hkv, d)
    scale = 1.0 / math.sqrt(d)
    table = dev["table"].cpu()
    for b, (length, _) in enumerate(seqs):      # spoil the new token's row
        page, at = int(table[b, (length - 1) // PAGE]), (length - 1) % PAGE
        dev["kc"][page, :, at] = 1e4
        dev["vc"][page, :, :, at] = 1e4
    cuda = lambda t: None if t is None else t.cuda()
    ws = torch.empty(32 << 20, dtype=torch.uint8, device="cuda")
    parts_dev = parts.cuda() if qkv_splits > 1 else parts[0].cuda()
    max_len = max(length for length, _ in seqs)
    # the two-kernel path on a copy of the cache
    kc2, vc2 = dev["kc"].clone(), dev["vc"].clone()
    q_dev = torch.empty(n, hq * d, dtype=torch.bfloat16, device="cuda")
    out2 = torch.full_like(q_dev, float("nan"))
    ops.qk_norm_rope_append(parts_dev, hq, hkv, d, cuda(q_gain), cuda(k_gain), eps, cuda(cos), cuda(sin),
                            d if rotate else 0, q_dev, kc2, vc2, dev["table"], dev["tok_seq"], dev["tok_pos"],
                            n_splits=qkv_splits)
    ops.attention(q_dev, out2, kc2, vc2, dev["table"], dev["tok_seq"], dev["tok_pos"], hq, hkv, d, scale, window,
                  algo=MFMA, workspace=ws, cu_seqlens=dev["cu"], max_new=1, q_counts=[1] * n, max_len=max_len,
                  n_splits=attn_splits)
    out = torch.full_like(q_dev, float("nan"))
    kc3, vc3 = dev["kc"].clone(), dev["vc"].clone()
    ops.attention_decode_fused(parts_dev, out, dev["kc"], dev["vc"], dev["table"], dev["tok_seq"], dev["tok_pos"],
                               hq, hkv, d, scale, cuda(q_gain), cuda(k_gain), eps, cuda(cos), cuda(sin),
                               window=window, workspace=ws, max_len=max_len, n_splits=attn_splits)
    # without the sequence table: token t is sequence t, as in this step
    out3 = torch.full_like(q_dev, float("nan"))
    ops.attention_decode_fused(parts_dev, out3, kc3, vc3, dev["table"], None, dev["tok_pos"],
                               hq, hkv, d, scale, cuda(q_gain), cuda(k_gain), eps, cuda(cos), cuda(sin),
                               window=window, workspace=ws, max_len=max_len, n_splits=attn_splits)
    torch.cuda.synchronize()
    assert torch.equal(out, out3) and torch.equal(kc3, dev["kc"]) and torch.equal(vc3, dev["vc"])
    # the cache: a 32-bit sum in another order may round a value to the neighbouring bfloat16
    for got, want in ((dev["kc"], kc2), (dev["vc"], vc2)):
        diff = (got.float() - want.float()).abs()
        assert float((diff / want.float().abs().clamp_min(1e-3)).max()) < 1e-2
    got = out.cpu().double().reshape(n, hq, d)
    assert float((got - out2.cpu().double().reshape(n, hq, d)).abs().max()) < 2e-2
    for b, ((length, _), k, v) in enumerate(zip(seqs, ks, vs)):
        k = k.double().clone()
        v = v.double().clone()
        k[length - 1], v[length - 1] = k_new[b].bfloat16().double(), v_new[b].bfloat16().double()
        ref = _reference(q[b:b + 1].bfloat16(), k, v, [length - 1], scale, window)
        err = float((got[b:b + 1] - ref).abs().max())
        assert err < 1.5e-2, f"sequence {b} of length {length}: error {err}"


# (Hq, Hkv, D, context lengths, splits of the projection, splits of the keys, window)
FUSED = [(16, 8, 128, [1], 1, 0, None), (16, 8, 128, [2, 33, 64, 65, 257], 1, 0, None),
         (32, 8, 128, [2048, 700, 1, 129], 4, 8, None), (8, 2, 256, [400, 1024, 63], 2, 6, None),
         (4, 1, 64, [130, 31, 32, 96, 97], 3, 2, None), (16, 1, 64, [65, 128], 1, 0, None),
         (24, 3, 192, [500, 9], 5, 5, None), (8, 2, 128, [1, 64, 65, 700, 129, 2, 1000], 4, 5, 70),
         (8, 2, 128, [1, 64, 65, 700, 129], 1, 3, 1), (6, 2, 64, [300, 5], 2, 0, 128)]


@pytest.mark.parametrize("hq,hkv,d,lengths,qkv_splits,attn_splits,window", FUSED)
def test_decode_fused_with_norm_rotation_and_append(hq, hkv, d, lengths, qkv_splits, attn_splits, window):
    _fused_case([(n, 1) for n in lengths], hq, hkv, d, qkv_splits, attn_splits, window, seed=11)


def test_decode_fused_applies_a_row_scale():
    """The projection's operand lacked its norm's scale: the kernel multiplies every sum of the
    projection of token t by 1 / sqrt(sum of ssq[t] / width + eps) first.  Handing it the sums divided
    by that number must give what the sums themselves give without a scale."""
    hq, hkv, d, width = 8, 2, 128, 520
    seqs = [(n, 1) for n in (1, 64, 65, 700, 129)]
    n = len(seqs)
    scale = 1.0 / math.sqrt(d)
    g = torch.Generator().manual_seed(21)
    for parts_per_row, qkv_splits in ((33, 1), (256, 3)):
        ssq = torch.rand(n, parts_per_row, generator=g) * 5.0
        eps = 1e-5
        factor = 1.0 / torch.sqrt(ssq.double().sum(-1) / width + eps)            # per token
        sums = torch.randn(qkv_splits, n, (hq + 2 * hkv) * d, generator=g) / math.sqrt(qkv_splits)
        gains = [(1 + 0.3 * torch.randn(d, generator=g)).cuda() for _ in range(2)]
        angle = torch.rand(n, d // 2, generator=g) * 6.28
        cos, sin = torch.cos(angle).cuda(), torch.sin(angle).cuda()
        ws = torch.empty(32 << 20, dtype=torch.uint8, device="cuda")
        results = []
        for lacking in (False, True):
            dev, _, _, _ = _build(seqs, hq, hkv, d, torch.bfloat16, 22)
            given = (sums.double() / factor[None, :, None]).float() if lacking else sums
            given = given.cuda() if qkv_splits > 1 else given[0].cuda()
            out = torch.full((n, hq * d), float("nan"), dtype=torch.bfloat16, device="cuda")
            ops.attention_decode_fused(given, out, dev["kc"], dev["vc"], dev["table"], None, dev["tok_pos"], hq, hkv, d, scale,
                                       gains[0], gains[1], eps, cos, sin, workspace=ws, max_len=700, n_splits=3,
                                       row_scale=ops.RowScale(ssq.cuda(), eps, width) if lacking else None)
            results.append((out.float().cpu(), dev["kc"].float().cpu(), dev["vc"].float().cpu()))
        for a, b in zip(*results):
            assert float((a - b).abs().max()) <= 1e-2 * float(a.abs().max())


def test_decode_fused_without_norm_or_rotation():
    _fused_case([(77, 1), (200, 1)], 8, 4, 128, 2, 3, None, seed=12, norm=False)
    _fused_case([(77, 1), (200, 1)], 8, 4, 128, 1, 0, None, seed=13, rotate=False)


def test_decode_fused_one_key_decides():
    """The projection is made so that one key carries almost all weight: first the step's own
    key, which never comes from the cache, then a key far back in it.  The output must be that
    key's value row."""
    hq, hkv, d, length = 8, 2, 128, 900
    for own in (True, False):
        for splits in (0, 1, 7):
            dev, ks, vs, _ = _build([(length, 1)], hq, hkv, d, torch.bfloat16, 7)
            far = 37
            qkv = torch.zeros(1, (hq + 2 * hkv) * d)
            qkv[0, :hq * d].view(hq, d)[:, 5] = 40.0
            v_new = torch.randn(hkv, d, generator=torch.Generator().manual_seed(3))
            qkv[0, (hq + hkv) * d:] = v_new.reshape(-1)
            if own:
                qkv[0, hq * d:(hq + hkv) * d].view(hkv, d)[:, 5] = 40.0
                want = v_new.bfloat16().double()
            else:
                page = int(dev["table"][0, far // PAGE])
                k_row = torch.zeros(hkv, d)
                k_row[:, 5] = 40.0
                dev["kc"][page, :, far % PAGE] = k_row.to(torch.bfloat16).cuda()
                want = vs[0][far].double()
            out = torch.full((1, hq * d), float("nan"), dtype=torch.bfloat16, device="cuda")
            ws = torch.empty(8 << 20, dtype=torch.uint8, device="cuda")
            ops.attention_decode_fused(qkv.cuda(), out, dev["kc"], dev["vc"], dev["table"], None, dev["tok_pos"],
                                       hq, hkv, d, 1.0, None, None, 1.0, None, None, workspace=ws,
                                       max_len=length, n_splits=splits)
            got = out.cpu().double().reshape(hq, d)
            for h in range(hq):
                assert float((got[h] - want[h // (hq // hkv)]).abs().max()) < 2e-2, (own, splits, h)


def test_decode_fused_refuses_other_head_sizes():
    from rocml_amd.errors import KernelError
    with pytest.raises(KernelError):
        _fused_case([(10, 1)], 4, 2, 96, 1, 0, None, seed=0)


def test_refusals():
    from rocml_amd.errors import KernelError
    dev, *_ = _build([(10, 1)], 4, 2, 48, torch.bfloat16, 0)
    with pytest.raises(KernelError):
        _run(dev, [(10, 1)], 4, 2, 48, 1.0, None, MFMA)      # head size 48 has no MFMA kernel
    dev, *_ = _build([(10, 1)], 4, 3, 32, torch.bfloat16, 0)
    with pytest.raises(KernelError):
        _run(dev, [(10, 1)], 4, 3, 32, 1.0, None, PLAIN)     # 4 heads over 3 kv heads


# ---- contexts of tens of thousands of tokens ---------------------------------------------------
def _reference_rows(q, k, v, positions, scale, window):
    """The same as ``_reference`` without loops over positions: q [n, Hq, D] at ``positions``,
    k, v [L, Hkv, D], everything in float64, a head at a time."""
    n, hq, d = q.shape
    group = hq // k.shape[1]
    pos = torch.tensor(positions)
    keys = torch.arange(k.shape[0])
    seen = keys[None, :] <= pos[:, None]
    if window is not None:
        seen &= keys[None, :] > pos[:, None] - window
    out = torch.zeros(n, hq, d, dtype=torch.float64)
    for h in range(hq):
        s = (q[:, h].double() @ k[:, h // group].double().T) * scale
        s = s.masked_fill(~seen, float("-inf"))
        out[:, h] = torch.softmax(s, dim=-1) @ v[:, h // group].double()
    return out


def _needles(length, n_new):
    """Places whose keys are made to carry the weight: the ends of the sequence, both sides of
    page borders near and far, the middle."""
    first_new = length - n_new
    places = {0, 63, 64, 4095, 4096, length // 2 + 17, first_new - 65, first_new - 64, first_new - 1, first_new - 4000}
    return sorted(p for p in places if 0 <= p < first_new)


def _long_case(length, n_new, hq, hkv, d, window, n_splits, seed):
    """A sequence of ``length`` positions whose last ``n_new`` are the step's: among the random
    keys a handful point along the first query of their kv head, four times as long, so that
    those few share nearly all weight and each of them missing, doubled or taken from a wrong
    page moves the output by a tenth and more."""
    seqs = [(length, n_new)]
    dev, ks, vs, qs = _build(seqs, hq, hkv, d, torch.bfloat16, seed, spare_pages=5)
    group = hq // hkv
    k, table = ks[0], dev["table"].cpu()
    for j in range(hkv):
        lead = qs[0][0, j * group].float()
        for p in _needles(length, n_new):
            k[p, j] = (4.0 * lead).to(torch.bfloat16)
            dev["kc"][int(table[0, p // PAGE]), j, p % PAGE] = k[p, j].cuda()
    scale = 1.0 / math.sqrt(d)
    got = _run(dev, seqs, hq, hkv, d, scale, window, MFMA, n_splits).double().reshape(-1, hq, d)
    ref = _reference_rows(qs[0], k, vs[0], list(range(length - n_new, length)), scale, window)
    err = float((got - ref).abs().max())
    assert err < 1.5e-2, f"length {length}, {n_new} new, window {window}, {n_splits} splits: error {err}"
    # (the needles do decide: without them the first head's output is another one)
    assert float((ref[0, 0] - vs[0][:length - n_new, 0].double().mean(0)).abs().max()) > 0.1


# (Hq, Hkv, D, (context length after the step, new tokens) per sequence, window, norm, rotation)
PREFILL_FUSED = [(16, 8, 128, [(300, 300)], None, True, True), (8, 2, 128, [(5, 5), (200, 130), (64, 64), (129, 1), (400, 257)], None, True, True),
                 (8, 2, 128, [(900, 600), (70, 3)], 70, True, True), (4, 1, 64, [(130, 130), (31, 31)], None, True, False),
                 (6, 2, 32, [(77, 50)], None, False, True), (12, 4, 96, [(200, 129), (10, 10)], 24, True, True),
                 (6, 3, 192, [(150, 100)], None, True, True), (4, 2, 256, [(100, 64), (65, 65)], None, False, False)]


@pytest.mark.parametrize("hq,hkv,d,seqs,window,norm,rotate", PREFILL_FUSED)
def test_prefill_fused_prepares_its_queries(hq, hkv, d, seqs, window, norm, rotate):
    """The prompt kernel that takes its queries from the q/k/v projection (norm, rotation and
    rounding inside) against the two kernels it replaces, on the same projection, and against the
    64-bit attention over the queries those prepared.  The caches must come out bit for bit the
    same: keys and values go through the same kernel either way."""
    dev, ks, vs, qs = _build(seqs, hq, hkv, d, torch.bfloat16, 21)
    n = sum(m for _, m in seqs)
    g = torch.Generator().manual_seed(22)
    rows = hq + 2 * hkv
    # (queries as large as the other tests': the norm brings them there, without it the projection does)
    proj = (torch.randn(n, rows * d, generator=g) * (1.5 if norm else 1.0)).cuda()
    q_gain = (1 + 0.3 * torch.randn(d, generator=g)).cuda() if norm else None
    k_gain = (1 + 0.3 * torch.randn(d, generator=g)).cuda() if norm else None
    eps = 3e-5
    cos = sin = None
    if rotate:
        angle = dev["tok_pos"].float()[:, None] * (10000.0 ** (-torch.arange(d // 2, device="cuda").float() / (d // 2)))[None, :]
        cos, sin = torch.cos(angle).contiguous(), torch.sin(angle).contiguous()
    scale = 1.0 / math.sqrt(d)
    ws = torch.empty(32 << 20, dtype=torch.uint8, device="cuda")
    counts = [m for _, m in seqs]
    # the two kernels
    kc2, vc2 = dev["kc"].clone(), dev["vc"].clone()
    q_dev = torch.empty(n, hq * d, dtype=torch.bfloat16, device="cuda")
    ops.qk_norm_rope_append(proj, hq, hkv, d, q_gain, k_gain, eps, cos, sin, d if rotate else 0, q_dev, kc2, vc2,
                            dev["table"], dev["tok_seq"], dev["tok_pos"])
    out2 = torch.full_like(q_dev, float("nan"))
    ops.attention(q_dev, out2, kc2, vc2, dev["table"], dev["tok_seq"], dev["tok_pos"], hq, hkv, d, scale, window,
                  algo=MFMA, workspace=ws, cu_seqlens=dev["cu"], max_new=max(counts), q_counts=counts,
                  max_len=max(length for length, _ in seqs))
    # the append without queries, then the kernel that prepares them
    ops.qk_norm_rope_append(proj, hq, hkv, d, q_gain, k_gain, eps, cos, sin, d if rotate else 0, None, dev["kc"], dev["vc"],
                            dev["table"], dev["tok_seq"], dev["tok_pos"])
    out = torch.full_like(q_dev, float("nan"))
    ops.attention_prefill_fused(proj, out, dev["kc"], dev["vc"], dev["table"], dev["tok_pos"], hq, hkv, d, scale,
                                q_gain, eps, cos, sin, window, dev["cu"], counts)
    torch.cuda.synchronize()
    assert torch.equal(dev["kc"], kc2) and torch.equal(dev["vc"], vc2)
    got = out.cpu().double().reshape(n, hq, d)
    assert float((got - out2.cpu().double().reshape(n, hq, d)).abs().max()) < 2e-2
    # the 64-bit attention over the prepared queries and the cache's keys and values
    table, at = dev["table"].cpu(), 0
    kc_cpu, vc_cpu = kc2.cpu(), vc2.cpu()
    for b, (length, m) in enumerate(seqs):
        k = torch.stack([kc_cpu[int(table[b, p_ // PAGE]), :, p_ % PAGE] for p_ in range(length)])
        v = torch.stack([vc_cpu[int(table[b, p_ // PAGE]), :, :, p_ % PAGE] for p_ in range(length)])
        ref = _reference_rows(q_dev[at:at + m].cpu().reshape(m, hq, d), k, v, list(range(length - m, length)), scale, window)
        err = float((got[at:at + m] - ref).abs().max())
        assert err < 1.5e-2, f"sequence {b} of length {length} with {m} new tokens: error {err}"
        at += m


@pytest.mark.parametrize("climb", [30.0, 4.0, -30.0])
def test_prompt_whose_scores_climb_slowly(climb):
    """The prefill kernel moves the reference of a row's exponents only when the row's maximum has
    run ahead of it by more than 2^8.  Keys that lie along the queries of a kv head's first query
    head, a little longer from one position to the next: the maximum grows by less than that per
    piece for many pieces (probabilities far above one in between) and by several times that over
    the sequence; with ``climb`` = 4 it never moves again after the first piece; falling scores
    never move it at all.  Every row against the 64-bit softmax."""
    hq, hkv, d, length, n_new = 4, 2, 128, 1500, 300
    seqs = [(length, n_new)]
    dev, ks, vs, qs = _build(seqs, hq, hkv, d, torch.bfloat16, 41)
    group = hq // hkv
    k, q, table = ks[0], qs[0], dev["table"].cpu()
    scale = 1.0 / math.sqrt(d)
    for j in range(hkv):
        lead = torch.randn(d, generator=torch.Generator().manual_seed(50 + j))
        lead = lead / lead.norm()
        q[:, j * group] = (lead * math.sqrt(d)).to(torch.bfloat16)          # score of key p: its length along lead
        ramp = torch.arange(length, dtype=torch.float32) / length * climb
        k[:, j] = (ramp[:, None] * lead[None, :] + 0.05 * k[:, j].float()).to(torch.bfloat16)
    dev["q"] = q.reshape(-1, hq * d).cuda()
    for p_ in range(length):
        dev["kc"][int(table[0, p_ // PAGE]), :, p_ % PAGE] = k[p_].cuda()
    got = _run(dev, seqs, hq, hkv, d, scale, None, MFMA).double().reshape(-1, hq, d)
    ref = _reference_rows(q, k, vs[0], list(range(length - n_new, length)), scale, None)
    err = float((got - ref).abs().max())
    assert err < 1.5e-2, f"climb {climb}: error {err}"


@pytest.mark.parametrize("length", [32768, 40960])
@pytest.mark.parametrize("window,n_splits", [(None, 1), (None, 8), (None, 64), (None, 0), (4096, 8), (4096, 64), (70, 0)])
def test_decode_over_tens_of_thousands_of_keys(length, window, n_splits):
    _long_case(length, 1, 8, 2, 128, window, n_splits, seed=31)


@pytest.mark.parametrize("length,window", [(32768, None), (32768, 5000), (40960, None)])
def test_a_chunk_deep_in_a_long_sequence(length, window):
    _long_case(length, 256, 4, 2, 128, window, 0, seed=32)
