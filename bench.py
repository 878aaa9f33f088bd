#!/usr/bin/env python3
"""Decode and prefill speed of the Qwen3-8B shape with random bfloat16 weights on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one decode step of a batch of 8 sequences, each with a 2,048-token random
prompt in the cache (context length 4,096): the engine's step over the cache, greedy
sampling on the device and the copy of the drawn ids to the host, exactly as the library's
generation loop runs it (the loop is the one that is timed, through its per-step hook).
Prints one JSON line: ``value`` is decoded tokens per second; ``prefill`` is one
2,048-token prompt; ``roofline`` relates the decode step to the bytes it must read
(every weight once and the live cache) at 8 TB/s; ``points`` holds batch 1 and 64 and
``point_fracs`` their fractions of that roofline.
The workload follows the reference's bench (rocml-cli/src/cmd_bench.rs:79-243): synthetic
prompt, greedy, no stop token, warm-up first; times are taken around synchronised steps.
"""
import argparse
import json
import sys
import time

HBM_PEAK_GBS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}
PROMPT_LEN = 2048
CONTEXT = 4096


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--model", default="qwen3-8b", help="catalog name")
    ap.add_argument("--layers", type=int, default=None, help="run fewer layers than the model has")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 and 64 points")
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
    batches = [args.batch] if args.no_points else sorted({1, args.batch, 64})
    max_batch = max(batches)
    engine = Engine(model, max_tokens=max_batch * CONTEXT, max_seqs=max_batch, max_step_tokens=8192)
    rng = np.random.default_rng(0)

    def prompt():
        return [int(t) for t in rng.integers(0, spec.vocab, size=PROMPT_LEN)]

    def sync():
        torch.cuda.synchronize()

    # ---- prefill: one 2,048-token prompt, logits of its last token -------------------
    def prefill_once():
        slot = engine.new_sequence()
        engine.step([StepEntry(slot, prompt(), [PROMPT_LEN - 1])])
        sync()
        engine.release(slot)

    if args.prefill_runs > 0:
        prefill_once()
    times = [float("nan")] if args.prefill_runs <= 0 else []
    for _ in range(args.prefill_runs):
        sync()
        t0 = time.perf_counter()
        prefill_once()
        times.append(time.perf_counter() - t0)
    prefill_s = sorted(times)[len(times) // 2]
    prefill_flops = model.step_flops([PROMPT_LEN], [0], 1)
    peak = PEAK_FLOPS["bf16" if args.dtype == "bfloat16" else "fp32"]

    # ---- decode ----------------------------------------------------------------------
    weight_bytes = model.step_weight_bytes()
    kv_bytes_per_token = engine.cache.bytes_per_token()

    class SkippingBackend(EngineBackend):
        """Hands the sequences their prompt's positions without running it."""

        def step(self, slots, tokens):
            if all(len(t) == 1 for t in tokens):
                return super().step(slots, tokens)
            cache = self.engine.cache
            new_lens = [cache.length(s) + len(t) for s, t in zip(slots, tokens)]
            cache.reserve(list(slots), new_lens)
            cache.commit(list(slots), new_lens)
            return torch.zeros((len(slots), spec.vocab), dtype=torch.float32, device=model.device)

    def decode(batch: int, steps: int, warmup: int):
        """Seconds of ``steps`` decode steps of the generation loop after ``warmup`` of them, and
        the mean sequence length over the timed steps."""
        backend = (SkippingBackend if args.skip_prompts else EngineBackend)(engine)
        gen = Generator(backend, max_batch=batch)
        marks = {}

        def on_step(k: int) -> None:
            if k == warmup or k == warmup + steps:
                sync()
                marks[k] = time.perf_counter()
        gen.on_step = on_step
        greedy = SamplingParams.greedy()
        # one token more than the steps: the last token of a sequence is drawn, not run
        requests = [Request(prompt(), warmup + steps + 1, greedy) for _ in range(batch)]
        results = gen.run(requests)
        assert all(len(r.tokens) == warmup + steps + 1 for r in results) and gen.stats.batches == 1
        mean_len = PROMPT_LEN + warmup + (steps + 1) / 2.0
        return marks[warmup + steps] - marks[warmup], mean_len

    def roofline(batch: int, dt_step: float, mean_len: float):
        step_bytes = weight_bytes + batch * mean_len * kv_bytes_per_token
        return step_bytes / dt_step / 1e9

    steps = max(1, min(args.steps, CONTEXT - PROMPT_LEN - args.warmup - 2))
    dt, mean_len = decode(args.batch, steps, args.warmup)
    ms_per_step = dt / steps * 1e3
    value = args.batch * steps / dt
    achieved = roofline(args.batch, dt / steps, mean_len)
    points, fracs = {}, {}
    if not args.no_points:
        for b in (1, 64):
            if b == args.batch:
                points[f"decode_b{b}"] = round(value, 2)
                fracs[f"decode_b{b}"] = round(achieved / HBM_PEAK_GBS, 4)
                continue
            p_steps = max(1, min(steps, 64))
            p_warm = min(args.warmup, 4)
            p_dt, p_len = decode(b, p_steps, p_warm)
            points[f"decode_b{b}"] = round(b * p_steps / p_dt, 2)
            fracs[f"decode_b{b}"] = round(roofline(b, p_dt / p_steps, p_len) / HBM_PEAK_GBS, 4)

    def key(name, default=None):
        return raw.get(name, default)

    out = {
        "metric": f"decode tok/s ({args.model} shape, {'bf16' if args.dtype == 'bfloat16' else 'fp32'}, "
                  f"batch {args.batch}, {PROMPT_LEN}-token prompts)",
        "value": round(value, 2), "unit": "tok/s", "n_gpus": 1, "steps": steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic: uniform random token ids, random N(0, 0.02) weights, unit norm gains",
        "config": {"model": args.model, "layers": n_layers, "layers_of_model": key("num_hidden_layers"),
                   "hidden": spec.hidden, "q_heads": key("num_attention_heads"),
                   "kv_heads": key("num_key_value_heads"), "head_dim": key("head_dim"),
                   "intermediate": key("intermediate_size"), "vocab": spec.vocab,
                   "rope_theta": key("rope_theta"), "rms_norm_eps": key("rms_norm_eps"),
                   "tied_lm_head": spec.tie_lm_head, "global_batch": args.batch,
                   "prompt_len": PROMPT_LEN, "seq_len": CONTEXT, "parallelism": "single GPU"},
        "prefill": {"value": round(PROMPT_LEN / prefill_s, 1), "tokens": PROMPT_LEN,
                    "ms": round(prefill_s * 1e3, 3), "frac": round(prefill_flops / prefill_s / peak, 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
        "points": points,
        "point_fracs": fracs,
    }
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
