#!/usr/bin/env python3
"""Decode and prefill speed of the Qwen3 shapes with random bfloat16 weights on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--model qwen3-8b|qwen3-14b|qwen3-32b]

The default run is the Qwen3-8B shape.  A step is one decode step of a batch of 8 sequences,
each with a 2,048-token random prompt in the cache (context length 4,096): the engine's step
over the cache, greedy sampling on the device and the copy of the drawn ids to the host,
exactly as the library's generation loop runs it (the loop is the one that is timed, through
its per-step hook).  Prints one JSON line: ``value`` is decoded tokens per second; ``prefill``
is one 2,048-token prompt; ``roofline`` relates the decode step to the bytes it must read
(every weight once and the live cache) at 8 TB/s; ``points`` holds batch 1 and 64, batch 8
over 32,768-token prompts (``decode_b8_ctx32k``, the cache filled by running the prompts) and
the wall time of prompt steps of 17, 64 and 256 tokens (``prefill_short_*_ms``);
``point_fracs`` are the decode points' fractions of their rooflines.

``--model qwen3-14b`` runs the unequal batch of 16 prompts of 128 to 4,096 tokens with 128
decode steps, ``--model qwen3-32b`` 32 prompts of 8,192 tokens with 256 decode steps: ``value``
is then decoded tokens per second over all decode steps of that workload, ``prefill`` the
prompt step of the whole batch, and ``--steps`` / ``--warmup`` only bound the decode steps.

The workloads follow the reference's bench (rocml-cli/src/cmd_bench.rs:79-243): synthetic
prompts, greedy, no stop token, warm-up first; times are taken around synchronised steps.
"""
import argparse
import json
import sys
import time

HBM_PEAK_GBS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}
PROMPT_LEN = 2048
CONTEXT = 4096
LONG_PROMPT = 32768
# model -> (sequences, shortest prompt, longest prompt, decode steps): the workloads quoted with
# the larger shapes
WORKLOADS = {"qwen3-14b": (16, 128, 4096, 128), "qwen3-32b": (32, 8192, 8192, 256)}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=None, help="sequences of the timed batch (8; the workload's own for the larger shapes)")
    ap.add_argument("--model", default="qwen3-8b", help="catalog name")
    ap.add_argument("--layers", type=int, default=None, help="run fewer layers than the model has")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--no-points", action="store_true", help="skip the further points")
    ap.add_argument("--prefill-runs", type=int, default=3)
    ap.add_argument("--skip-prompts", action="store_true",
                    help="profiling aid: give the sequences their 2,048 positions without running the "
                         "prompts (the cache holds zeros); the timed decode steps are the same")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported by this library")
        return 2

    import numpy as np
    import torch
    from rocml_amd import ops
    from rocml_amd.config.catalog import resolve
    from rocml_amd.engine import Engine, EngineBackend, Generator, Request, StepEntry
    from rocml_amd.sampling import SamplingParams
    from rocml_amd.weights import random_model

    ops.load_all()
    raw = resolve(args.model).entry.config              # config.json's keys
    model = random_model(raw, seed=0, dtype=args.dtype, device="cuda:0", n_layers=args.layers)
    spec = model.spec
    n_layers = len(spec.schedule)
    workload = WORKLOADS.get(args.model)
    rng = np.random.default_rng(0)
    peak = PEAK_FLOPS["bf16" if args.dtype == "bfloat16" else "fp32"]
    dtype_name = "bf16" if args.dtype == "bfloat16" else "fp32"

    def tokens(n: int):
        return [int(t) for t in rng.integers(0, spec.vocab, size=n)]

    def sync():
        torch.cuda.synchronize()

    def key(name, default=None):
        return raw.get(name, default)

    def model_config():
        return {"model": args.model, "layers": n_layers, "layers_of_model": key("num_hidden_layers"),
                "hidden": spec.hidden, "q_heads": key("num_attention_heads"),
                "kv_heads": key("num_key_value_heads"), "head_dim": key("head_dim"),
                "intermediate": key("intermediate_size"), "vocab": spec.vocab,
                "rope_theta": key("rope_theta"), "rms_norm_eps": key("rms_norm_eps"),
                "tied_lm_head": spec.tie_lm_head, "parallelism": "single GPU"}

    weight_bytes = model.step_weight_bytes()

    class SkippingBackend(EngineBackend):
        """Hands the sequences their prompt's positions without running it."""

        def step(self, slots, toks):
            if all(len(t) == 1 for t in toks):
                return super().step(slots, toks)
            cache = self.engine.cache
            new_lens = [cache.length(s) + len(t) for s, t in zip(slots, toks)]
            cache.reserve(list(slots), new_lens)
            cache.commit(list(slots), new_lens)
            return torch.zeros((len(slots), spec.vocab), dtype=torch.float32, device=model.device)

    def decode(engine, prompts, steps: int, warmup: int):
        """Seconds of ``steps`` decode steps of the generation loop after ``warmup`` of them, the
        mean number of cached positions over the timed steps, and the seconds the prompts took."""
        backend = (SkippingBackend if args.skip_prompts else EngineBackend)(engine)
        gen = Generator(backend, max_batch=len(prompts))
        marks = {}

        def on_step(k: int) -> None:
            if k == warmup or k == warmup + steps:
                sync()
                marks[k] = time.perf_counter()
        gen.on_step = on_step
        greedy = SamplingParams.greedy()
        # one token more than the steps: the last token of a sequence is drawn, not run
        requests = [Request(p, warmup + steps + 1, greedy) for p in prompts]
        results = gen.run(requests)
        assert all(len(r.tokens) == warmup + steps + 1 for r in results) and gen.stats.batches == 1
        live = sum(len(p) for p in prompts) + len(prompts) * (warmup + (steps + 1) / 2.0)
        return marks[warmup + steps] - marks[warmup], live, gen.stats.prompt_seconds

    def achieved_gbs(engine, dt_step: float, live_positions: float):
        return (weight_bytes + live_positions * engine.cache.bytes_per_token()) / dt_step / 1e9

    if workload is not None:
        return run_workload(args, workload, model, Engine, decode, achieved_gbs, tokens, model_config, peak, dtype_name)

    batch = args.batch or 8
    batches = [batch] if args.no_points else sorted({1, batch, 64})
    max_batch = max(batches)
    max_tokens = max_batch * CONTEXT
    if not args.no_points:
        max_tokens = max(max_tokens, 8 * (LONG_PROMPT + 64))
    engine = Engine(model, max_tokens=max_tokens, max_seqs=max_batch, max_step_tokens=8192)

    # ---- prefill: one 2,048-token prompt, logits of its last token -------------------
    def prompt_step(n: int) -> float:
        slot = engine.new_sequence()
        toks = tokens(n)
        sync()
        t0 = time.perf_counter()
        engine.step([StepEntry(slot, toks, [n - 1])])
        sync()
        dt = time.perf_counter() - t0
        engine.release(slot)
        return dt

    def median_prompt_step(n: int, runs: int) -> float:
        if runs <= 0:
            return float("nan")
        prompt_step(n)
        times = sorted(prompt_step(n) for _ in range(runs))
        return times[len(times) // 2]

    prefill_s = median_prompt_step(PROMPT_LEN, args.prefill_runs)
    prefill_flops = model.step_flops([PROMPT_LEN], [0], 1)

    # ---- decode ----------------------------------------------------------------------
    steps = max(1, min(args.steps, CONTEXT - PROMPT_LEN - args.warmup - 2))
    dt, live, _ = decode(engine, [tokens(PROMPT_LEN) for _ in range(batch)], steps, args.warmup)
    ms_per_step = dt / steps * 1e3
    value = batch * steps / dt
    achieved = achieved_gbs(engine, dt / steps, live)
    points, fracs = {}, {}
    if not args.no_points:
        for b in (1, 64):
            if b == batch:
                points[f"decode_b{b}"] = round(value, 2)
                fracs[f"decode_b{b}"] = round(achieved / HBM_PEAK_GBS, 4)
                continue
            p_steps = max(1, min(steps, 64))
            p_warm = min(args.warmup, 4)
            p_dt, p_live, _ = decode(engine, [tokens(PROMPT_LEN) for _ in range(b)], p_steps, p_warm)
            points[f"decode_b{b}"] = round(b * p_steps / p_dt, 2)
            fracs[f"decode_b{b}"] = round(achieved_gbs(engine, p_dt / p_steps, p_live) / HBM_PEAK_GBS, 4)
        # batch 8 over prompts of 32,768 tokens, which are run, not skipped
        if spec.max_positions >= LONG_PROMPT + 64:
            p_steps, p_warm = max(1, min(steps, 16)), min(args.warmup, 3)
            p_dt, p_live, p_prompt = decode(engine, [tokens(LONG_PROMPT) for _ in range(8)], p_steps, p_warm)
            points["decode_b8_ctx32k"] = round(8 * p_steps / p_dt, 2)
            fracs["decode_b8_ctx32k"] = round(achieved_gbs(engine, p_dt / p_steps, p_live) / HBM_PEAK_GBS, 4)
            if not args.skip_prompts:
                points["prefill_8x32k_tok_s"] = round(8 * LONG_PROMPT / p_prompt, 1)
        # short prompts: the wall time of one prompt step (host and GPU), median of five
        for n in (17, 64, 256):
            points[f"prefill_short_{n}_ms"] = round(median_prompt_step(n, 5) * 1e3, 3)

    out = {
        "metric": f"decode tok/s ({args.model} shape, {dtype_name}, batch {batch}, {PROMPT_LEN}-token prompts)",
        "value": round(value, 2), "unit": "tok/s", "n_gpus": 1, "steps": steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": dtype_name,
        "data": "synthetic: uniform random token ids, random N(0, 0.02) weights, unit norm gains",
        "config": dict(model_config(), global_batch=batch, prompt_len=PROMPT_LEN, seq_len=CONTEXT),
        "prefill": {"value": round(PROMPT_LEN / prefill_s, 1), "tokens": PROMPT_LEN,
                    "ms": round(prefill_s * 1e3, 3), "frac": round(prefill_flops / prefill_s / peak, 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
        "points": points,
        "point_fracs": fracs,
    }
    print(json.dumps(out))
    return 0


def run_workload(args, workload, model, Engine, decode, achieved_gbs, tokens, model_config, peak, dtype_name) -> int:
    """The batch quoted with a larger shape: its prompts in one step of the generation loop, then
    its decode steps, all of them timed but the warm-up."""
    import numpy as np
    n_seqs, lo, hi, n_decode = workload
    n_seqs = args.batch or n_seqs
    lengths = [int(n) for n in np.random.default_rng(1).integers(lo, hi + 1, size=n_seqs)]
    warmup = min(args.warmup, 4)
    steps = max(1, min(args.steps, n_decode) - warmup)
    room = sum(-(-(n + warmup + steps + 2) // 64) * 64 for n in lengths)
    engine = Engine(model, max_tokens=room, max_seqs=n_seqs, max_step_tokens=8192)
    # a first, short pass so that buffers reach their size and kernels are set up
    decode(engine, [tokens(min(n, 256)) for n in lengths], 2, 1)
    dt, live, prompt_s = decode(engine, [tokens(n) for n in lengths], steps, warmup)
    value = n_seqs * steps / dt
    achieved = achieved_gbs(engine, dt / steps, live)
    prompt_tokens = sum(lengths)
    prefill_flops = model.step_flops(lengths, [0] * n_seqs, n_seqs)
    shown = f"{lo}-token" if lo == hi else f"{lo} to {hi}-token"
    out = {
        "metric": f"decode tok/s ({args.model} shape, {dtype_name}, batch {n_seqs}, {shown} prompts)",
        "value": round(value, 2), "unit": "tok/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": round(dt / steps * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": dtype_name,
        "data": "synthetic: uniform random token ids, random N(0, 0.02) weights, unit norm gains",
        "config": dict(model_config(), global_batch=n_seqs, prompt_len_min=min(lengths), prompt_len_max=max(lengths),
                       prompt_tokens=prompt_tokens, decode_steps=warmup + steps),
        "prefill": {"value": round(prompt_tokens / prompt_s, 1), "tokens": prompt_tokens,
                    "ms": round(prompt_s * 1e3, 3), "frac": round(prefill_flops / prompt_s / peak, 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
        "points": {}, "point_fracs": {},
    }
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
