"""Typed launch helpers over the compiled HIP libraries.

The counterpart of the reference's ``Kernels`` struct, which loads each code object
once and offers one typed method per kernel that fixes grid, block and LDS
(rocml/src/forward/kernels.rs:97-229,232-720).  Here the grid is chosen inside the
library; these helpers check devices, types and shapes, pass raw pointers and the
current stream, and turn a nonzero status into ``KernelError`` with the library's
message.  There is no fallback: a missing library is compiled, and if that fails the
call raises.
"""
from __future__ import annotations

import ctypes
from typing import Dict, Optional, Sequence

import torch

from ..csrc import build as _build
from ..errors import KernelError

_P = ctypes.c_void_p
_I = ctypes.c_int
_F = ctypes.c_float
_LL = ctypes.c_longlong

_DTYPE_CODE = {torch.float32: 0, torch.bfloat16: 1}

_SIGNATURES = {
    "elementwise": {
        "rocml_embed_gather": [_P, _I, _P, _P, _I, _I, _I, _F, _P],
        "rocml_rmsnorm": [_P, _P, _P, _I, _P, _I, _I, _F, _P, _I, _LL, _P],
        "rocml_swiglu": [_P, _I, _P, _I, _I, _I, _I, _P],
        "rocml_rope_table": [_P, _P, _P, _P, _I, _I, _P],
        "rocml_qk_norm_rope_append": [_P, _I, _I, _I, _I, _I, _I, _P, _P, _F, _P, _P, _I, _I, _P, _P, _P,
                                      _I, _P, _I, _P, _P, _I, _I, _I, _LL, _P],
        "rocml_add_into": [_P, _P, _I, _LL, _P],
    },
    "gemm": {
        "rocml_gemm": [_P, _I, _I, _P, _I, _I, _P, _I, _I, _I, _I, _I, _I, _I, _I, _I, _P, _P, _LL, _P, _I, _F, _I, _P],
        "rocml_splitk_reduce": [_P, _P, _I, _I, _I, _I, _I, _I, _P],
        "rocml_gemm_residual_prescale_pays": [_I, _I, _I],
        "rocml_gemm_residual_prescale": [_P, _I, _P, _I, _P, _I, _P, _P, _I, _P, _I, _I, _I, _I, _P],
    },
    "attention": {
        "rocml_attention": [_P, _P, _P, _P, _I, _P, _I, _P, _P, _I, _I, _I, _I, _I, _F, _I, _I,
                            _P, _I, _I, _P, _I, _I, _P, _LL, _P],
        "rocml_attention_decode_fused": [_P, _I, _I, _LL, _P, _P, _F, _P, _P, _I, _P, _P, _P, _P, _I, _P, _P,
                                         _I, _I, _I, _I, _I, _F, _I, _I, _I, _P, _LL, _P, _I, _F, _I, _P],
        "rocml_attention_prefill_fused": [_P, _I, _P, _F, _P, _P, _P, _P, _P, _P, _I, _P, _I, _I, _I, _I, _I, _F, _I,
                                          _P, _I, _P, _P],
    },
    "sampling": {
        "rocml_sample": [_P, _P, _I, _I, _P, _P, _P, _P, _P, _P, _I, _P, _I, _P, _P],
        "rocml_argmax": [_P, _I, _I, _P, _P, _P],
    },
}

_libs: Dict[str, ctypes.CDLL] = {}


def library(family: str) -> ctypes.CDLL:
    """The family's shared library, compiled on first use if it is not there."""
    lib = _libs.get(family)
    if lib is None:
        lib = ctypes.CDLL(_build.ensure(family))
        for name, argtypes in _SIGNATURES[family].items():
            fn = getattr(lib, name)
            fn.argtypes = argtypes
            fn.restype = _I
        err = getattr(lib, f"{family}_last_error")
        err.restype = ctypes.c_char_p
        err.argtypes = []
        _libs[family] = lib
    return lib


MODEL_FAMILIES = ("elementwise", "gemm", "attention")   # what a model's step needs; sampling comes with generation


def prepare(families=tuple(_SIGNATURES)) -> None:
    """Loads the named families; those that are not built yet are compiled together first."""
    _build.build([f for f in families], force=False)
    for family in families:
        library(family)


def load_all() -> None:
    prepare()


def _check(family: str, status: int) -> None:
    if status != 0:
        msg = getattr(library(family), f"{family}_last_error")().decode("utf-8", "replace")
        raise KernelError(msg)


_cus = {}


def cu_count(device) -> int:
    """Compute units of ``device`` (256 on an MI355X, which is also the answer for a device that is
    not a GPU, where parts are built only to be counted); launch sizes are phrased in it."""
    device = torch.device(device)
    if device.type != "cuda":
        return 256
    if device not in _cus:
        _cus[device] = int(torch.cuda.get_device_properties(device).multi_processor_count)
    return _cus[device]


# The raw handle of the current device's current stream.  torch's public call builds a Stream
# object and checks the device on the way (8 us a call, a quarter of a prompt step's host time);
# the same answer comes from the two calls below in a fraction of a microsecond where torch has
# them.
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream() -> int:
    if _raw_stream is not None and _raw_device is not None:
        return _raw_stream(_raw_device())
    return torch.cuda.current_stream().cuda_stream


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _dev(*tensors: Optional[torch.Tensor]) -> None:
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise KernelError("kernel arguments must be GPU tensors; this library has no CPU path")
        if not t.is_contiguous():
            raise KernelError(f"kernel arguments must be contiguous, got strides {t.stride()} for shape {tuple(t.shape)}")


def _code(t: torch.Tensor) -> int:
    try:
        return _DTYPE_CODE[t.dtype]
    except KeyError:
        raise KernelError(f"unsupported element type {t.dtype}") from None


def _want(t: torch.Tensor, dtype: torch.dtype, what: str) -> None:
    if t.dtype != dtype:
        raise KernelError(f"{what} must be {dtype}, got {t.dtype}")


# ---- elementwise ---------------------------------------------------------------------
def embed_gather(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor, scale: float = 1.0) -> None:
    _dev(table, ids, out)
    _want(ids, torch.int32, "token ids")
    _want(out, torch.float32, "embedding output")
    vocab, hidden = table.shape
    n = ids.numel()
    if out.shape != (n, hidden):
        raise KernelError(f"embedding output is {tuple(out.shape)}, expected {(n, hidden)}")
    _check("elementwise", library("elementwise").rocml_embed_gather(
        _ptr(table), _code(table), _ptr(ids), _ptr(out), n, hidden, vocab, scale, _stream()))


def rmsnorm(x: torch.Tensor, gain: torch.Tensor, eps: float, out: torch.Tensor,
            rows: Optional[torch.Tensor] = None, partials: Optional[torch.Tensor] = None) -> None:
    """``partials`` ([splits, rows of x, n] float32) are split-K partial sums that belong to
    ``x``: the kernel adds them to ``x`` first (and stores the sum back unless rows are
    gathered)."""
    _dev(x, gain, out, rows, partials)
    _want(x, torch.float32, "norm input")
    _want(gain, torch.float32, "norm gain")
    n = x.shape[-1]
    if gain.numel() != n or out.shape[-1] != n:
        raise KernelError(f"norm sizes differ: input {n}, gain {gain.numel()}, output {out.shape[-1]}")
    n_rows = out.numel() // n
    if rows is not None:
        _want(rows, torch.int32, "row indices")
        if rows.numel() != n_rows:
            raise KernelError("one row index per output row is needed")
    elif x.numel() != out.numel():
        raise KernelError("norm input and output differ in size")
    n_splits, stride = 0, 0
    if partials is not None:
        _want(partials, torch.float32, "partial sums")
        if partials.dim() != 3 or partials.shape[1] * partials.shape[2] != x.numel():
            raise KernelError(f"partial sums {tuple(partials.shape)} do not fit the norm input {tuple(x.shape)}")
        n_splits, stride = partials.shape[0], x.numel()
    _check("elementwise", library("elementwise").rocml_rmsnorm(
        _ptr(x), _ptr(gain), _ptr(out), _code(out), _ptr(rows), n_rows, n, eps, _ptr(partials), n_splits,
        stride, _stream()))


def swiglu(gate_up: torch.Tensor, out: torch.Tensor, interleaved: bool = False) -> None:
    """``gate_up`` rows hold the gate half then the up half, or (gate, up) pairs when
    ``interleaved``."""
    _dev(gate_up, out)
    n_tokens, inter = out.shape
    if gate_up.shape != (n_tokens, 2 * inter):
        raise KernelError(f"gate/up is {tuple(gate_up.shape)}, expected {(n_tokens, 2 * inter)}")
    _check("elementwise", library("elementwise").rocml_swiglu(
        _ptr(gate_up), _code(gate_up), _ptr(out), _code(out), n_tokens, inter, 1 if interleaved else 0, _stream()))


def rope_table(positions: torch.Tensor, inv_freq: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> None:
    _dev(positions, inv_freq, cos, sin)
    _want(positions, torch.int32, "positions")
    _want(inv_freq, torch.float64, "inverse frequencies")
    _want(cos, torch.float32, "cos table")
    _want(sin, torch.float32, "sin table")
    n, half = positions.numel(), inv_freq.numel()
    if cos.shape != (n, half) or sin.shape != (n, half):
        raise KernelError(f"rotation tables must be {(n, half)}")
    _check("elementwise", library("elementwise").rocml_rope_table(
        _ptr(positions), _ptr(inv_freq), _ptr(cos), _ptr(sin), n, half, _stream()))


ROPE_PAIRINGS = {"halves": 0, "neighbours": 1}


def qk_norm_rope_append(qkv: torch.Tensor, n_heads: int, n_kv_heads: int, head_dim: int,
                        q_gain: Optional[torch.Tensor], k_gain: Optional[torch.Tensor], eps: float,
                        cos: Optional[torch.Tensor], sin: Optional[torch.Tensor], rot_dim: int,
                        q_out: Optional[torch.Tensor], k_cache: Optional[torch.Tensor],
                        v_cache: Optional[torch.Tensor], block_table: Optional[torch.Tensor],
                        token_seq: torch.Tensor, token_pos: torch.Tensor, write_kv: bool = True,
                        n_splits: int = 1, pairing: str = "halves") -> None:
    """``qkv`` is ``[T, ld]`` with q, k, v side by side (k and v may be absent when
    ``write_kv`` is false).  Keys are ``[pages, Hkv, page_size, D]``, values
    ``[pages, Hkv, D, page_size]``.  ``pairing``: which two values of the rotated width turn
    together by the angle in column ``i`` of the tables: ``"halves"``, ``(i, i + rot_dim / 2)``,
    or ``"neighbours"``, ``(2 i, 2 i + 1)``.  ``q_out`` None: only keys and values are prepared
    and appended (the caller's attention kernel prepares its queries itself)."""
    if pairing not in ROPE_PAIRINGS:
        raise KernelError(f"unknown rotation pairing {pairing!r}; known: {sorted(ROPE_PAIRINGS)}")
    _dev(qkv, q_gain, k_gain, cos, sin, q_out, k_cache, v_cache, block_table, token_seq, token_pos)
    split_stride = 0
    if n_splits > 1:                      # [splits, T, ld] split-K partial sums, added in the kernel
        if qkv.dim() != 3 or qkv.shape[0] != n_splits:
            raise KernelError("partial sums of the projection must be [splits, tokens, width]")
        split_stride = qkv.shape[1] * qkv.shape[2]
        qkv = qkv[0]
    n_tokens, ld = qkv.shape
    for g in (q_gain, k_gain):
        if g is not None:
            _want(g, torch.float32, "head norm gain")
            if g.numel() != head_dim:
                raise KernelError(f"head norm gain has {g.numel()} values for head size {head_dim}")
    if cos is not None:
        if cos.shape != (n_tokens, rot_dim // 2) or sin is None or sin.shape != cos.shape:
            raise KernelError(f"rotation tables must be {(n_tokens, rot_dim // 2)}")
    if q_out is None and not write_kv:
        raise KernelError("nothing to do: no q output and no append to the cache")
    if (q_out is not None and q_out.shape != (n_tokens, n_heads * head_dim)) or token_seq.numel() != n_tokens \
            or token_pos.numel() != n_tokens:
        raise KernelError("q output or token tables do not match the number of tokens")
    page_size = bt_width = 0
    if write_kv:
        if k_cache is None or v_cache is None or block_table is None:
            raise KernelError("appending to the cache needs the cache and the block table")
        if k_cache.shape[1:] != (n_kv_heads, k_cache.shape[2], head_dim) \
                or v_cache.shape != (k_cache.shape[0], n_kv_heads, head_dim, k_cache.shape[2]):
            raise KernelError(f"cache shape {tuple(k_cache.shape)} does not fit {n_kv_heads} heads of {head_dim}")
        if q_out is not None and k_cache.dtype != q_out.dtype:
            raise KernelError("cache and q output must share their type")
        _want(block_table, torch.int32, "block table")
        page_size, bt_width = k_cache.shape[2], block_table.shape[1]
    _check("elementwise", library("elementwise").rocml_qk_norm_rope_append(
        _ptr(qkv), _code(qkv), ld, n_tokens, n_heads, n_kv_heads, head_dim, _ptr(q_gain), _ptr(k_gain),
        eps, _ptr(cos), _ptr(sin), rot_dim if cos is not None else 0, ROPE_PAIRINGS[pairing], _ptr(q_out), _ptr(k_cache),
        _ptr(v_cache), _code(q_out if q_out is not None else k_cache), _ptr(block_table), bt_width, _ptr(token_seq),
        _ptr(token_pos), page_size, 1 if write_kv else 0, n_splits, split_stride, _stream()))


def add_into(x: torch.Tensor, y: torch.Tensor) -> None:
    _dev(x, y)
    _want(x, torch.float32, "residual")
    if x.numel() != y.numel():
        raise KernelError("residual add of different sizes")
    _check("elementwise", library("elementwise").rocml_add_into(_ptr(x), _ptr(y), _code(y), x.numel(), _stream()))


# ---- matrix product ------------------------------------------------------------------
GEMM_AUTO, GEMM_PLAIN = 0, 1
ROW_SCALE_MAX_ROWS = 16     # most rows of a product whose consumer applies a row scale


class RowScale:
    """What is left of a norm whose operand ``bfloat16(x * gain)`` was prepared by the product that
    completed ``x`` (``gemm_residual_prescale``): ``ssq [rows, parts]`` float32 sums of squares
    whose total over a row, divided by ``width`` and with ``eps`` added, is the square of what the
    row still has to be divided by.  The consumer of the next product applies it to its sums."""

    def __init__(self, ssq: torch.Tensor, eps: float, width: int):
        _dev(ssq)
        _want(ssq, torch.float32, "sums of squares")
        if ssq.dim() != 2:
            raise KernelError("sums of squares must be [rows, parts]")
        self.ssq, self.eps, self.width = ssq, float(eps), int(width)


def gemm(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, accumulate: bool = False,
         algo: int = GEMM_AUTO, workspace: Optional[torch.Tensor] = None, epilogue: Optional[str] = None,
         defer: bool = False, row_scale: Optional["RowScale"] = None, max_splits: int = 0) -> int:
    """``out (+)= x @ w.T`` for ``x [M, K]``, ``w [N, K]``, ``out [M, N]`` (rows may be
    strided views with unit inner stride).  ``epilogue="swiglu"``: ``w``'s rows are (gate, up)
    pairs and ``out`` is ``[M, N/2] = silu(gate) * up``.  With ``defer`` a product that was
    split along K leaves its partial sums ``[splits, M, N]`` at the start of ``workspace`` and
    returns their number for the caller's next kernel to add; it returns 0 when ``out`` is
    complete.  ``row_scale``: ``x`` lacks its norm's scale (see ``RowScale``), which the gated
    epilogue applies; at most ``ROW_SCALE_MAX_ROWS`` rows.  ``max_splits``: the most pieces K may
    be cut into (0: as the kernels see fit)."""
    for t in (x, w, out):
        if not t.is_cuda:
            raise KernelError("kernel arguments must be GPU tensors; this library has no CPU path")
        if t.dim() != 2 or t.stride(1) != 1:
            raise KernelError("matrix product operands must be 2-D with unit inner stride")
    if epilogue not in (None, "swiglu"):
        raise KernelError(f"unknown epilogue {epilogue!r}")
    m, k = x.shape
    n = w.shape[0]
    cols = n // 2 if epilogue else n
    if w.shape[1] != k or out.shape != (m, cols):
        raise KernelError(f"matrix product shapes do not fit: x {tuple(x.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)}")
    ws_ptr, ws_bytes = (None, 0) if workspace is None else (workspace.data_ptr(), workspace.numel() * workspace.element_size())
    deferred = ctypes.c_int(0)
    ssq_ptr, parts, eps = None, 0, 0.0
    if row_scale is not None:
        if epilogue != "swiglu" or m > ROW_SCALE_MAX_ROWS or row_scale.width != k or row_scale.ssq.shape[0] < m:
            raise KernelError("a row scale goes with the gated epilogue of at most 16 rows whose K is the norm's width")
        ssq_ptr, parts, eps = row_scale.ssq.data_ptr(), row_scale.ssq.shape[1], row_scale.eps
    _check("gemm", library("gemm").rocml_gemm(
        _ptr(x), _code(x), x.stride(0) if m > 1 else max(x.stride(0), k), _ptr(w), _code(w), w.stride(0),
        _ptr(out), _code(out), out.stride(0) if m > 1 else max(out.stride(0), cols), m, n, k,
        1 if accumulate else 0, algo, 1 if epilogue else 0, 1 if defer else 0, ctypes.byref(deferred), ws_ptr,
        ws_bytes, ssq_ptr, parts, eps, int(max_splits), _stream()))
    return deferred.value


PRESCALE_MAX_ROWS = 16      # most rows gemm_residual_prescale takes
PRESCALE_TILE = 16          # columns whose squares one entry of its sums of squares covers


def gemm_residual_prescale_fits(x: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether ``gemm_residual_prescale`` takes this product."""
    return (x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and 1 <= x.shape[0] <= PRESCALE_MAX_ROWS
            and x.shape[1] % 8 == 0 and x.stride(0) % 8 == 0 and w.stride(0) % 8 == 0)


def gemm_residual_prescale_pays(x: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether it takes the product and is the faster way (the library's own rule)."""
    return gemm_residual_prescale_fits(x, w) and \
        library("gemm").rocml_gemm_residual_prescale_pays(x.shape[0], w.shape[0], x.shape[1]) != 0


def gemm_residual_prescale(x: torch.Tensor, w: torch.Tensor, resid: torch.Tensor, gain: torch.Tensor,
                           xg: torch.Tensor, ssq: torch.Tensor, waves: int = 0) -> None:
    """``resid += x @ w.T`` (whole sums, at most 16 rows of bfloat16 operands) and, for the norm
    with ``gain`` that reads ``resid`` next: ``xg = bfloat16(resid * gain)`` and ``ssq[row][j]`` =
    the sum of squares of columns ``16 j .. 16 j + 15`` of the row.  The norm's output is
    ``xg * (1 / sqrt(ssq[row].sum() / N + eps))``; the scale commutes with the next product."""
    _dev(gain, ssq)
    for t in (x, w, resid, xg):
        if not t.is_cuda:
            raise KernelError("kernel arguments must be GPU tensors; this library has no CPU path")
        if t.dim() != 2 or t.stride(1) != 1:
            raise KernelError("matrix product operands must be 2-D with unit inner stride")
    m, k = x.shape
    n = w.shape[0]
    if not gemm_residual_prescale_fits(x, w):
        raise KernelError(f"gemm_residual_prescale does not take x {tuple(x.shape)} {x.dtype}, w {tuple(w.shape)} {w.dtype}")
    _want(resid, torch.float32, "residual stream")
    _want(gain, torch.float32, "norm gain")
    _want(xg, torch.bfloat16, "prepared operand")
    _want(ssq, torch.float32, "sums of squares")
    tiles = (n + PRESCALE_TILE - 1) // PRESCALE_TILE
    if w.shape[1] != k or resid.shape != (m, n) or xg.shape != (m, n) or gain.numel() != n or ssq.shape != (m, tiles):
        raise KernelError(f"shapes do not fit: x {tuple(x.shape)}, w {tuple(w.shape)}, residual {tuple(resid.shape)}, "
                          f"prepared {tuple(xg.shape)}, gain {gain.numel()}, sums {tuple(ssq.shape)} (need {(m, tiles)})")
    _check("gemm", library("gemm").rocml_gemm_residual_prescale(
        _ptr(x), max(x.stride(0), k), _ptr(w), w.stride(0), _ptr(resid), max(resid.stride(0), n), _ptr(gain), _ptr(xg),
        max(xg.stride(0), n), _ptr(ssq), m, n, k, waves, _stream()))


def splitk_reduce(partials: torch.Tensor, out: torch.Tensor, accumulate: bool = False) -> None:
    """``out (+)= partials.sum(0)`` in split order, for ``partials [splits, M, N]`` float32."""
    _dev(partials, out)
    _want(partials, torch.float32, "partial sums")
    splits, m, n = partials.shape
    if out.shape != (m, n):
        raise KernelError("partial sums and output differ in shape")
    _check("gemm", library("gemm").rocml_splitk_reduce(_ptr(partials), _ptr(out), _code(out), out.stride(0), m, n,
                                                       splits, 1 if accumulate else 0, _stream()))


# ---- attention -----------------------------------------------------------------------
ATTN_AUTO, ATTN_PLAIN, ATTN_MFMA = 0, 1, 2


def attention(q: torch.Tensor, out: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
              block_table: torch.Tensor, token_seq: torch.Tensor, token_pos: torch.Tensor,
              n_heads: int, n_kv_heads: int, head_dim: int, scale: float, window: Optional[int] = None,
              algo: int = ATTN_AUTO, workspace: Optional[torch.Tensor] = None,
              cu_seqlens: Optional[torch.Tensor] = None, max_new: int = 0,
              q_counts: Optional[Sequence[int]] = None, max_len: int = 0, n_splits: int = 0) -> None:
    """Attention of the step's query tokens over the cache.  Keys are ``[pages, Hkv, page, D]``,
    values ``[pages, Hkv, D, page]``.  ``cu_seqlens`` (device), ``q_counts`` (the same knowledge on
    the host: query tokens of each sequence), ``max_new`` (the most of them) and ``max_len``
    (longest context) describe the step to the fast kernels; without them the plain kernel runs."""
    _dev(q, out, k_cache, v_cache, block_table, token_seq, token_pos, cu_seqlens)
    n_tokens = q.shape[0]
    if q.shape != (n_tokens, n_heads * head_dim) or out.shape != q.shape or out.dtype != q.dtype:
        raise KernelError("attention input and output must both be [tokens, heads * head_dim] of one type")
    page = k_cache.shape[2]
    if k_cache.dtype != q.dtype or v_cache.dtype != q.dtype \
            or k_cache.shape[1:] != (n_kv_heads, page, head_dim) \
            or v_cache.shape != (k_cache.shape[0], n_kv_heads, head_dim, page):
        raise KernelError(f"cache {tuple(k_cache.shape)} / {tuple(v_cache.shape)} {k_cache.dtype} does not fit the queries")
    _want(block_table, torch.int32, "block table")
    _want(token_seq, torch.int32, "token sequence table")
    _want(token_pos, torch.int32, "token position table")
    if token_seq.numel() != n_tokens or token_pos.numel() != n_tokens:
        raise KernelError("one sequence index and one position per token are needed")
    n_seqs = 0
    counts = None
    if cu_seqlens is not None:
        _want(cu_seqlens, torch.int32, "sequence offsets")
        n_seqs = cu_seqlens.numel() - 1
        if q_counts is not None:
            if len(q_counts) != n_seqs:
                raise KernelError(f"{len(q_counts)} query counts for {n_seqs} sequences")
            counts = (ctypes.c_int * n_seqs)(*[int(c) for c in q_counts])
    ws_ptr, ws_bytes = (None, 0) if workspace is None else (workspace.data_ptr(), workspace.numel() * workspace.element_size())
    _check("attention", library("attention").rocml_attention(
        _ptr(q), _ptr(out), _ptr(k_cache), _ptr(v_cache), _code(q), _ptr(block_table),
        block_table.shape[1], _ptr(token_seq), _ptr(token_pos), n_tokens, n_heads, n_kv_heads, head_dim,
        page, scale, 0 if window is None else int(window), algo, _ptr(cu_seqlens), n_seqs, max_new,
        counts, max_len, n_splits, ws_ptr, ws_bytes, _stream()))


FUSED_DECODE_HEAD_DIMS = (64, 128, 192, 256)
FUSED_DECODE_PAGE = 64
# The most partial sums of the projection the fused decode attention should be handed: it adds four in
# one trip to memory and each further one in a trip of its own.  Measured at 64 sequences (8B shape,
# decoded tokens a second): at most 4 pieces 8,022, 5 8,073, 6 8,003, 8 7,932, no limit 7,960; at 16
# to 48 sequences the limit makes no difference.
FUSED_DECODE_SPLITS = 5


def decode_splits(pairs: int, n_cus: int, most: int) -> int:
    """Splits of the key range for ``pairs`` (token, kv head) pairs of a decode step, at most
    ``most``.  A CU works at its full rate with two blocks on it, or with one whose waves keep two
    pieces on their way (which the kernel does when the chip holds at most a block a CU); every
    block costs about three pages' time beside its own pages, a merge of splits as much again and
    a little per split.  The choice is the count with the least work on the busiest CU by that
    account, for a nominal 32 pages a sequence: it must not follow the lengths, so that a recorded
    step can be replayed as the sequences grow.  Measured at the Qwen3-8B shape, 2,048-token
    contexts (decoded tokens a second): 14 sequences 3,040 with 2 or 4 splits, 2,850 with 9;
    18 sequences 3,555 with 3, 3,375 with 5; 24 sequences 4,480 with none, 4,310 with 4;
    32 sequences 5,620 with none, 5,375 with 2; 40 sequences 5,990 with 3, 5,720 with none;
    56 sequences 7,330 with none, 7,000 with 2.  Below 8 sequences' worth of pairs (64) the
    rule is about a block a CU."""
    if pairs * 4 < n_cus:
        # a few sequences: about a block a CU (two pieces of each wave are then on their way); measured,
        # one block a CU against two: one sequence 277.5 against 274.8 tokens a second, two 542 against
        # 532, four 1,050 against 1,029, six 1,518 against 1,501
        return max(1, min(n_cus // pairs, most))
    pages, per_block, merge, per_split = 32.0, 3.0, 3.0, 0.3
    best, best_cost = 1, float("inf")
    for s in range(1, max(1, min(most, 16)) + 1):
        blocks = pairs * s
        cost = -(-blocks // n_cus) * (pages / s + per_block) + (merge + per_split * s if s > 1 else 0.0)
        if cost < best_cost - 1e-9:
            best, best_cost = s, cost
    return best


def attention_decode_fusable(dtype: torch.dtype, n_heads: int, n_kv_heads: int, head_dim: int, page: int,
                             rot_dim: Optional[int], pairing: str = "halves") -> bool:
    """Whether ``attention_decode_fused`` takes this layer: bfloat16 cache in pages of 64, a head
    size it has a kernel for, at most 16 query heads per kv head, and a rotation (if any) of the
    whole head in pairs ``(i, i + head_dim / 2)``."""
    return (dtype == torch.bfloat16 and page == 64 and head_dim in FUSED_DECODE_HEAD_DIMS
            and n_heads // n_kv_heads <= 16 and (rot_dim is None or (rot_dim == head_dim and pairing == "halves")))


PREFILL_FUSED_PAGE = 64
PREFILL_FUSED_HEAD_DIMS = (32, 64, 96, 128, 192, 256)


def attention_prefill_fusable(dtype: torch.dtype, head_dim: int, page_size: int, rot_dim: Optional[int],
                              pairing: str = "halves") -> bool:
    """Whether ``attention_prefill_fused`` takes a layer: a bfloat16 cache with pages of 64 positions,
    a head size the MFMA kernels know, and a rotation of the whole head with halves as pairs (or none)."""
    return (dtype == torch.bfloat16 and page_size == PREFILL_FUSED_PAGE and head_dim in PREFILL_FUSED_HEAD_DIMS
            and (rot_dim is None or (rot_dim == head_dim and pairing == "halves")))


def attention_prefill_fused(qkv: torch.Tensor, out: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                            block_table: torch.Tensor, token_pos: torch.Tensor, n_heads: int, n_kv_heads: int,
                            head_dim: int, scale: float, q_gain: Optional[torch.Tensor], eps: float,
                            cos: Optional[torch.Tensor], sin: Optional[torch.Tensor], window: Optional[int],
                            cu_seqlens: torch.Tensor, q_counts: Sequence[int], max_len: int = 0) -> None:
    """A prompt step's attention with the queries taken from the q/k/v projection ``qkv`` (float32
    ``[tokens, ld]``, complete sums, a token's q heads first): per-head norm, rotation and rounding
    of the queries happen in the attention kernel.  The new tokens' keys and values are in the
    cache already (``qk_norm_rope_append`` without a q output puts them there).  ``max_len``
    (the longest context) is what ``--profile`` prices the call with; the kernel does not need it."""
    _dev(qkv, out, k_cache, v_cache, block_table, token_pos, q_gain, cos, sin, cu_seqlens)
    _want(qkv, torch.float32, "projection output")
    if qkv.dim() != 2:
        raise KernelError("the projection must be [tokens, width] (complete sums)")
    n_tokens, ld = qkv.shape
    page = k_cache.shape[2]
    if not attention_prefill_fusable(k_cache.dtype, head_dim, page, None if cos is None else 2 * cos.shape[-1]):
        raise KernelError(f"fused prefill attention does not take this layer (cache {k_cache.dtype}, pages of {page}, "
                          f"head size {head_dim})")
    if out.shape != (n_tokens, n_heads * head_dim) or out.dtype != k_cache.dtype:
        raise KernelError("attention output must be [tokens, heads * head_dim] of the cache's type")
    if v_cache.dtype != k_cache.dtype or k_cache.shape[1:] != (n_kv_heads, page, head_dim) \
            or v_cache.shape != (k_cache.shape[0], n_kv_heads, head_dim, page):
        raise KernelError(f"cache {tuple(k_cache.shape)} / {tuple(v_cache.shape)} does not fit {n_kv_heads} heads of {head_dim}")
    if q_gain is not None:
        _want(q_gain, torch.float32, "head norm gain")
        if q_gain.numel() != head_dim:
            raise KernelError(f"head norm gain has {q_gain.numel()} values for head size {head_dim}")
    if cos is not None:
        _want(cos, torch.float32, "rotation table")
        if cos.shape != (n_tokens, head_dim // 2) or sin is None or sin.shape != cos.shape or sin.dtype != cos.dtype:
            raise KernelError(f"rotation tables must be float32 {(n_tokens, head_dim // 2)}")
    _want(block_table, torch.int32, "block table")
    _want(token_pos, torch.int32, "token position table")
    _want(cu_seqlens, torch.int32, "sequence offsets")
    n_seqs = cu_seqlens.numel() - 1
    if token_pos.numel() != n_tokens or len(q_counts) != n_seqs or block_table.shape[0] < n_seqs:
        raise KernelError("one position per token, one query count and one block table row per sequence are needed")
    counts = (ctypes.c_int * n_seqs)(*[int(c) for c in q_counts])
    _check("attention", library("attention").rocml_attention_prefill_fused(
        _ptr(qkv), ld, _ptr(q_gain), eps, _ptr(cos), _ptr(sin), _ptr(out), _ptr(k_cache), _ptr(v_cache),
        _ptr(block_table), block_table.shape[1], _ptr(token_pos), n_tokens, n_heads, n_kv_heads, head_dim, page,
        scale, 0 if window is None else int(window), _ptr(cu_seqlens), n_seqs, counts, _stream()))


def attention_decode_fused(qkv: torch.Tensor, out: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                           block_table: torch.Tensor, token_seq: Optional[torch.Tensor], token_pos: torch.Tensor,
                           n_heads: int, n_kv_heads: int, head_dim: int, scale: float,
                           q_gain: Optional[torch.Tensor], k_gain: Optional[torch.Tensor], eps: float,
                           cos: Optional[torch.Tensor], sin: Optional[torch.Tensor], write_kv: bool = True,
                           window: Optional[int] = None, workspace: Optional[torch.Tensor] = None,
                           max_len: int = 0, n_splits: int = 0, row_scale: Optional[RowScale] = None) -> None:
    """A decode step's attention straight from the q/k/v projection ``qkv`` (float32
    ``[tokens, ld]``, or its split-K partial sums ``[splits, tokens, ld]``): per-head norm,
    rotation, append of the new key and value to the cache and attention over the cache in one
    launch.  ``token_seq`` None: token ``t`` is the one token of the step's sequence ``t`` (row
    ``t`` of the block table).  ``workspace`` must not overlap ``qkv``.  ``row_scale``: the
    projection's operand lacked its norm's scale, which is applied to the projection's sums here."""
    _dev(qkv, out, k_cache, v_cache, block_table, token_seq, token_pos, q_gain, k_gain, cos, sin)
    _want(qkv, torch.float32, "projection output")
    qkv_splits, split_stride = 1, 0
    if qkv.dim() == 3:
        qkv_splits, split_stride = qkv.shape[0], qkv.shape[1] * qkv.shape[2]
        qkv = qkv[0]
    n_tokens, ld = qkv.shape
    page = k_cache.shape[2]
    if not attention_decode_fusable(k_cache.dtype, n_heads, n_kv_heads, head_dim, page,
                                    None if cos is None else 2 * cos.shape[-1]):
        raise KernelError(f"fused decode attention does not take this layer (cache {k_cache.dtype}, pages of {page}, "
                          f"head size {head_dim}, {n_heads} heads over {n_kv_heads})")
    if out.shape != (n_tokens, n_heads * head_dim) or out.dtype != k_cache.dtype:
        raise KernelError("attention output must be [tokens, heads * head_dim] of the cache's type")
    if v_cache.dtype != k_cache.dtype or k_cache.shape[1:] != (n_kv_heads, page, head_dim) \
            or v_cache.shape != (k_cache.shape[0], n_kv_heads, head_dim, page):
        raise KernelError(f"cache {tuple(k_cache.shape)} / {tuple(v_cache.shape)} does not fit {n_kv_heads} heads of {head_dim}")
    for g in (q_gain, k_gain):
        if g is not None:
            _want(g, torch.float32, "head norm gain")
            if g.numel() != head_dim:
                raise KernelError(f"head norm gain has {g.numel()} values for head size {head_dim}")
    if cos is not None:
        _want(cos, torch.float32, "rotation table")
        if cos.shape != (n_tokens, head_dim // 2) or sin is None or sin.shape != cos.shape or sin.dtype != cos.dtype:
            raise KernelError(f"rotation tables must be float32 {(n_tokens, head_dim // 2)}")
    _want(block_table, torch.int32, "block table")
    _want(token_pos, torch.int32, "token position table")
    if token_seq is not None:
        _want(token_seq, torch.int32, "token sequence table")
    elif block_table.shape[0] < n_tokens:
        raise KernelError(f"the block table has {block_table.shape[0]} rows for {n_tokens} sequences")
    if (token_seq is not None and token_seq.numel() != n_tokens) or token_pos.numel() != n_tokens:
        raise KernelError("one sequence index and one position per token are needed")
    ws_ptr, ws_bytes = (None, 0) if workspace is None else (workspace.data_ptr(), workspace.numel() * workspace.element_size())
    ssq_ptr, parts, row_eps, width = None, 0, 0.0, 0
    if row_scale is not None:
        if row_scale.ssq.shape[0] < n_tokens:
            raise KernelError("the row scale has fewer rows than the step has tokens")
        ssq_ptr, parts, row_eps, width = row_scale.ssq.data_ptr(), row_scale.ssq.shape[1], row_scale.eps, row_scale.width
    _check("attention", library("attention").rocml_attention_decode_fused(
        _ptr(qkv), ld, qkv_splits, split_stride, _ptr(q_gain), _ptr(k_gain), eps, _ptr(cos), _ptr(sin),
        1 if write_kv else 0, _ptr(out), _ptr(k_cache), _ptr(v_cache), _ptr(block_table), block_table.shape[1],
        _ptr(token_seq), _ptr(token_pos), n_tokens, n_heads, n_kv_heads, head_dim, page, scale,
        0 if window is None else int(window), max_len, n_splits, ws_ptr, ws_bytes, ssq_ptr, parts, row_eps, width,
        _stream()))


# ---- sampling ------------------------------------------------------------------------
ARGMAX_WORK_WORDS = 64      # 32-bit words of workspace per row for the two-stage argmax
SAMPLE_SMALL_K = 64         # the largest top-k that the slice kernels of the sampler take


def argmax(logits: torch.Tensor, out: torch.Tensor, work: Optional[torch.Tensor] = None) -> None:
    """First index of each row's maximum.  With ``work`` (``ARGMAX_WORK_WORDS`` 32-bit words
    per row) long rows are searched by several blocks."""
    _dev(logits, out, work)
    _want(logits, torch.float32, "logits")
    _want(out, torch.int32, "token output")
    batch, vocab = logits.shape
    if work is not None and work.numel() * work.element_size() < batch * ARGMAX_WORK_WORDS * 4:
        raise KernelError("argmax workspace is too small")
    _check("sampling", library("sampling").rocml_argmax(_ptr(logits), batch, vocab, _ptr(out), _ptr(work), _stream()))


def sample(logits: torch.Tensor, work: torch.Tensor, temperature: torch.Tensor, uniform: torch.Tensor,
           out: torch.Tensor, top_k: Optional[torch.Tensor] = None, top_p: Optional[torch.Tensor] = None,
           penalty: Optional[torch.Tensor] = None, history: Optional[torch.Tensor] = None,
           history_len: Optional[torch.Tensor] = None, small_k: int = 0) -> None:
    """``small_k``: 0, or a bound of at most 64 such that every sequence with a positive
    temperature has its top_k in ``[1, small_k]``: the caller's promise, which lets the selection
    run on slices of the vocabulary instead of whole rows."""
    _dev(logits, work, temperature, uniform, out, top_k, top_p, penalty, history, history_len)
    _want(logits, torch.float32, "logits")
    _want(work, torch.float32, "sampling workspace")
    batch, vocab = logits.shape
    if work.numel() < logits.numel():
        raise KernelError("sampling workspace is smaller than the logits")
    for t, dt, name in ((temperature, torch.float32, "temperature"), (uniform, torch.float32, "uniform"),
                        (top_p, torch.float32, "top_p"), (penalty, torch.float32, "penalty"),
                        (top_k, torch.int32, "top_k"), (history, torch.int32, "history"),
                        (history_len, torch.int32, "history lengths"), (out, torch.int32, "token output")):
        if t is not None:
            _want(t, dt, name)
            if name != "history" and t.numel() != batch:
                raise KernelError(f"{name} needs one value per sequence")
    if penalty is not None and (history is None or history_len is None or history.shape[0] != batch):
        raise KernelError("a repeat penalty needs the history and its lengths")
    _check("sampling", library("sampling").rocml_sample(
        _ptr(logits), _ptr(work), batch, vocab, _ptr(temperature), _ptr(top_k), _ptr(top_p), _ptr(uniform),
        _ptr(penalty), _ptr(history), 0 if history is None else history.shape[1], _ptr(history_len),
        int(small_k), _ptr(out), _stream()))
