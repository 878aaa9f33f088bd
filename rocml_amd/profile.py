"""Per-operation timing of a generation with a roofline report.

The reference's ``--profile`` brackets every operation of a forward pass with HIP events,
tags it with its phase (prefill or decode), its bytes and its flops, and reports per
operation kind: time share, achieved GB/s and GFLOP/s, percent of the two rooflines, the
analytical minimum ``t_min = max(bytes / bandwidth, flops / peak)``, ``efficiency = t_min /
t_actual`` and ``wasted = t_actual - t_min``, the column its worklist is sorted on
(rocml/src/profile/report.rs:1-75, rocml/src/profile/mod.rs:187-191).  Here the launch
helpers of ``rocml_amd.ops`` are wrapped while a profiler is active; the engine then runs
every step launch by launch (no recorded graphs), so the figures are those of single
launches with the gaps between them left out, not the step time of a replayed graph.

Bytes are what a launch must move once: its operand and result tensors, and for attention
the keys and values of the longest sequence times the number of sequences (an upper bound;
the launch helper does not know every length).  Peaks are MI355X's published ones.
"""
from __future__ import annotations

import json
from dataclasses import asdict, dataclass, field
from typing import Callable, Dict, List, Optional, Tuple

import torch

HBM_BYTES_PER_S = 8.0e12
PEAK_FLOPS = {torch.bfloat16: 2.5e15, torch.float32: 157.3e12}

_active: Optional["OpProfiler"] = None


def active() -> Optional["OpProfiler"]:
    """The profiler that is recording, if any (the engine asks before it replays a graph)."""
    return _active


def set_phase(phase: str) -> None:
    if _active is not None:
        _active.phase = phase


def _nbytes(*tensors) -> int:
    return sum(t.numel() * t.element_size() for t in tensors if isinstance(t, torch.Tensor))


def _gemm_cost(x, w, out, *a, **kw) -> Tuple[int, int]:
    m, k = x.shape
    return _nbytes(x, w, out), 2 * m * w.shape[0] * k


def _attention_cost(q, out, k_cache, v_cache, block_table, token_seq, token_pos, n_heads, n_kv_heads, head_dim,
                    *a, **kw) -> Tuple[int, int]:
    n_tokens, max_new, max_len = q.shape[0], kw.get("max_new", 0), kw.get("max_len", 0)
    n_seqs = block_table.shape[0]
    kv = 2 * n_seqs * max_len * n_kv_heads * head_dim * k_cache.element_size()
    keys_per_query = max_len if max_new <= 1 else max(1, max_len - max_new // 2)     # causal: half of the new part
    return _nbytes(q, out) + kv, 4 * n_heads * head_dim * n_tokens * keys_per_query


def _fused_attention_cost(qkv, out, k_cache, v_cache, block_table, token_seq, token_pos, n_heads, n_kv_heads, head_dim,
                          *a, **kw) -> Tuple[int, int]:
    max_len = kw.get("max_len", 0)
    n_seqs = out.shape[0]
    kv = 2 * n_seqs * max_len * n_kv_heads * head_dim * k_cache.element_size()
    return _nbytes(qkv, out) + kv, 4 * n_heads * head_dim * n_seqs * max_len


def _prefill_fused_cost(qkv, out, k_cache, v_cache, block_table, token_pos, n_heads, n_kv_heads, head_dim,
                        scale, q_gain, eps, cos, sin, window, cu_seqlens, q_counts, max_len=0) -> Tuple[int, int]:
    n_tokens, n_seqs, max_new = qkv.shape[0], len(q_counts), max(q_counts)
    kv = 2 * n_seqs * max_len * n_kv_heads * head_dim * k_cache.element_size()
    keys_per_query = max(1, max_len - max_new // 2)                                   # causal: half of the new part
    read_q = n_tokens * n_heads * head_dim * qkv.element_size()                       # the q columns of the projection
    return read_q + _nbytes(out, cos, sin) + kv, 4 * n_heads * head_dim * n_tokens * keys_per_query


def _tensor_args_cost(skip: Tuple[int, ...] = (), flops_per_byte: float = 0.0) -> Callable:
    def cost(*a, **kw) -> Tuple[int, int]:
        tensors = [t for i, t in enumerate(a) if i not in skip] + list(kw.values())
        b = _nbytes(*tensors)
        return b, int(b * flops_per_byte)
    return cost


# launch helper -> (label of the report row, bytes and flops of a call)
_COSTS: Dict[str, Tuple[str, Callable]] = {
    "gemm": ("product", _gemm_cost),
    "gemm_residual_prescale": ("product", lambda x, w, resid, gain, xg, ssq, *a, **kw: (
        _nbytes(x, w, resid, resid, gain, xg, ssq), 2 * x.shape[0] * w.shape[0] * x.shape[1])),
    "attention": ("attention", _attention_cost),
    "attention_decode_fused": ("attention (norm, rotation, append)", _fused_attention_cost),
    "attention_prefill_fused": ("attention (query norm, rotation)", _prefill_fused_cost),
    "qk_norm_rope_append": ("q/k norm, rotation, append", _tensor_args_cost(skip=(11, 12))),   # not the whole cache
    "rmsnorm": ("rmsnorm", _tensor_args_cost(flops_per_byte=0.5)),
    "swiglu": ("swiglu", _tensor_args_cost(flops_per_byte=0.5)),
    "embed_gather": ("embedding", lambda table, ids, out, *a, **kw: (2 * _nbytes(out) + _nbytes(ids), 0)),
    "rope_table": ("rotation table", _tensor_args_cost()),
    "add_into": ("residual add", _tensor_args_cost()),
    "splitk_reduce": ("sum of K pieces", _tensor_args_cost()),
    "argmax": ("argmax", _tensor_args_cost()),
    "sample": ("sampling", lambda logits, *a, **kw: (_nbytes(logits), 0)),
}


@dataclass
class Row:
    label: str
    count: int = 0
    bytes: int = 0
    flops: int = 0
    elapsed_ms: float = 0.0
    gb_per_sec: float = 0.0
    gflop_per_sec: float = 0.0
    pct_of_bandwidth_roofline: float = 0.0
    pct_of_flop_roofline: float = 0.0
    pct_of_phase_time: float = 0.0
    t_min_ms: float = 0.0
    efficiency: float = 0.0
    wasted_ms: float = 0.0


@dataclass
class PhaseReport:
    phase: str
    total_elapsed_ms: float
    total_bytes: int
    total_flops: int
    by_op: List[Row] = field(default_factory=list)


@dataclass
class Report:
    phases: List[PhaseReport]
    worklist: List[str]

    def to_dict(self) -> Dict:
        return asdict(self)

    def to_json(self) -> str:
        return json.dumps({"report": self.to_dict()})

    def to_human(self) -> str:
        lines = []
        for ph in self.phases:
            lines.append(f"{ph.phase}: {ph.total_elapsed_ms:.3f} ms in launches, {ph.total_bytes / 1e9:.3f} GB, "
                         f"{ph.total_flops / 1e12:.3f} TFLOP")
            lines.append(f"  {'operation':<36} {'calls':>6} {'ms':>9} {'%':>6} {'GB/s':>8} {'%bw':>6} {'TFLOP/s':>8} "
                         f"{'%peak':>6} {'t_min ms':>9} {'eff':>5} {'wasted ms':>10}")
            for r in ph.by_op:
                lines.append(f"  {r.label:<36} {r.count:>6} {r.elapsed_ms:>9.3f} {r.pct_of_phase_time:>6.1f} "
                             f"{r.gb_per_sec:>8.0f} {r.pct_of_bandwidth_roofline:>6.1f} {r.gflop_per_sec / 1e3:>8.1f} "
                             f"{r.pct_of_flop_roofline:>6.1f} {r.t_min_ms:>9.3f} {r.efficiency:>5.2f} {r.wasted_ms:>10.3f}")
        if self.worklist:
            lines.append("most time above the analytical minimum:")
            lines.extend("  " + w for w in self.worklist)
        return "\n".join(lines)


class OpProfiler:
    """``with OpProfiler(dtype) as p: model.generate(...)``, then ``p.finish()``."""

    def __init__(self, dtype: torch.dtype = torch.bfloat16):
        self.peak_flops = PEAK_FLOPS.get(dtype, PEAK_FLOPS[torch.bfloat16])
        self.phase = "prefill"
        self._records: List[Tuple[str, str, int, int, torch.cuda.Event, torch.cuda.Event]] = []
        self._saved: Dict[str, Callable] = {}

    def __enter__(self) -> "OpProfiler":
        global _active
        from . import ops
        if _active is not None:
            raise RuntimeError("a profiler is already recording")
        for name, (label, cost) in _COSTS.items():
            fn = getattr(ops, name)
            self._saved[name] = fn
            setattr(ops, name, self._wrap(fn, label, cost))
        _active = self
        return self

    def __exit__(self, *exc) -> None:
        global _active
        from . import ops
        for name, fn in self._saved.items():
            setattr(ops, name, fn)
        self._saved.clear()
        _active = None

    def _wrap(self, fn: Callable, label: str, cost: Callable) -> Callable:
        def timed(*a, **kw):
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            result = fn(*a, **kw)
            end.record()
            b, f = cost(*a, **kw)
            self._records.append((self.phase, label, int(b), int(f), start, end))
            return result
        return timed

    def finish(self) -> Report:
        torch.cuda.synchronize()
        return build_report([(ph, label, b, f, s.elapsed_time(e)) for ph, label, b, f, s, e in self._records],
                            self.peak_flops)


def build_report(records: List[Tuple[str, str, int, int, float]], peak_flops: float) -> Report:
    """Rows per phase and operation from ``(phase, label, bytes, flops, elapsed ms)`` records
    (rocml/src/profile/report.rs:91-160)."""
    phases: List[PhaseReport] = []
    worklist: List[Tuple[float, str]] = []
    for phase in ("prefill", "decode"):
        mine = [r for r in records if r[0] == phase]
        if not mine:
            continue
        total_ms = sum(r[4] for r in mine)
        rows: Dict[str, Row] = {}
        for _, label, b, f, ms in mine:
            row = rows.setdefault(label, Row(label))
            row.count += 1
            row.bytes += b
            row.flops += f
            row.elapsed_ms += ms
        for row in rows.values():
            secs = row.elapsed_ms / 1e3
            if secs > 0:
                row.gb_per_sec = row.bytes / secs / 1e9
                row.gflop_per_sec = row.flops / secs / 1e9
            row.pct_of_bandwidth_roofline = 100.0 * row.gb_per_sec * 1e9 / HBM_BYTES_PER_S
            row.pct_of_flop_roofline = 100.0 * row.gflop_per_sec * 1e9 / peak_flops
            row.pct_of_phase_time = 100.0 * row.elapsed_ms / total_ms if total_ms > 0 else 0.0
            row.t_min_ms = 1e3 * max(row.bytes / HBM_BYTES_PER_S, row.flops / peak_flops)
            row.efficiency = row.t_min_ms / row.elapsed_ms if row.elapsed_ms > 0 else 0.0
            row.wasted_ms = row.elapsed_ms - row.t_min_ms
            worklist.append((row.wasted_ms, f"{phase} {row.label}: {row.wasted_ms:.3f} ms above its minimum "
                                            f"({row.pct_of_phase_time:.1f}% of {phase} time, efficiency {row.efficiency:.2f})"))
        ordered = sorted(rows.values(), key=lambda r: -r.elapsed_ms)
        phases.append(PhaseReport(phase, total_ms, sum(r.bytes for r in ordered), sum(r.flops for r in ordered), ordered))
    worklist.sort(key=lambda w: -w[0])
    return Report(phases, [text for _, text in worklist[:5]])
