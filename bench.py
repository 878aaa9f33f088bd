#!/usr/bin/env python3
"""Decode and prefill speed of the Qwen3-8B shape with random bfloat16 weights on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one decode step of a batch of 8 sequences, each with a 2,048-token random
prompt in the cache (context length 4,096): the engine's step over the cache, greedy
sampling on the device and the copy of the drawn ids to the host, as generation does it.
Prints one JSON line: ``value`` is decoded tokens per second; ``prefill`` is one
2,048-token prompt; ``roofline`` relates the decode step to the bytes it must read
(every weight once and the live cache) at 8 TB/s; ``points`` holds batch 1 and 64.
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
    from rocml_amd.engine import Engine, StepEntry
    from rocml_amd.sampling import DeviceSampler, SamplingParams, SequenceSampling
    from rocml_amd.weights import random_model

    ops.load_all()
    entry = resolve(args.model).entry
    cfg_full = entry.config
    model = random_model(cfg_full, seed=0, dtype=args.dtype, device="cuda:0", n_layers=args.layers)
    cfg = model.config
    spec = model.spec
    n_layers = cfg.num_hidden_layers
    batches = [args.batch] if args.no_points else sorted({1, args.batch, 64})
    max_batch = max(batches)
    engine = Engine(model, max_tokens=max_batch * CONTEXT, max_seqs=max_batch, max_step_tokens=8192)
    sampler = DeviceSampler(model.device)
    rng = np.random.default_rng(0)

    def prompt():
        return [int(t) for t in rng.integers(0, cfg.vocab_size, size=PROMPT_LEN)]

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
    lin = (cfg.q_dim + 2 * cfg.kv_dim) * cfg.hidden_size + cfg.hidden_size * cfg.q_dim \
        + 3 * cfg.intermediate_size * cfg.hidden_size
    prefill_flops = n_layers * (2 * PROMPT_LEN * lin
                                + 4 * cfg.num_attention_heads * cfg.head_dim * PROMPT_LEN * (PROMPT_LEN + 1) // 2) \
        + 2 * cfg.vocab_size * cfg.hidden_size
    peak = PEAK_FLOPS["bf16" if args.dtype == "bfloat16" else "fp32"]

    # ---- decode ----------------------------------------------------------------------
    elem = 2 if args.dtype == "bfloat16" else 4
    weight_bytes = (n_layers * lin + cfg.vocab_size * cfg.hidden_size) * elem
    kv_bytes_per_token = engine.cache.bytes_per_token()

    def decode(batch: int, steps: int, warmup: int):
        slots = [engine.new_sequence() for _ in range(batch)]
        greedy = [SequenceSampling.start(SamplingParams.greedy(), i, []) for i in range(batch)]
        # All prompts in one step, as the generation loop sends them (the engine cuts the step
        # into pieces of its own; the prefill is not what is timed here).
        if args.skip_prompts:
            engine.cache.reserve(slots, [PROMPT_LEN] * batch)
            engine.cache.commit(slots, [PROMPT_LEN] * batch)
            tokens = [1] * batch
        else:
            logits = engine.step([StepEntry(s, prompt(), [PROMPT_LEN - 1]) for s in slots])
            tokens = sampler.sample(logits, greedy)

        def one_step(toks):
            logits = engine.step([StepEntry(s, [t], [0]) for s, t in zip(slots, toks)])
            return sampler.sample(logits, greedy)

        for _ in range(warmup):
            tokens = one_step(tokens)
        sync()
        len0 = engine.length(slots[0])
        t0 = time.perf_counter()
        for _ in range(steps):
            tokens = one_step(tokens)
        sync()
        dt = time.perf_counter() - t0
        mean_len = len0 + (steps + 1) / 2.0
        for s in slots:
            engine.release(s)
        return dt, mean_len

    steps = max(1, min(args.steps, CONTEXT - PROMPT_LEN - args.warmup - 1))
    dt, mean_len = decode(args.batch, steps, args.warmup)
    ms_per_step = dt / steps * 1e3
    value = args.batch * steps / dt
    step_bytes = weight_bytes + args.batch * mean_len * kv_bytes_per_token
    achieved = step_bytes / (dt / steps) / 1e9
    points = {}
    if not args.no_points:
        for b in (1, 64):
            if b == args.batch:
                points[f"decode_b{b}"] = round(value, 2)
                continue
            p_steps = max(1, min(steps, 64))
            p_dt, _ = decode(b, p_steps, min(args.warmup, 4))
            points[f"decode_b{b}"] = round(b * p_steps / p_dt, 2)

    out = {
        "metric": f"decode tok/s ({args.model} shape, {'bf16' if args.dtype == 'bfloat16' else 'fp32'}, "
                  f"batch {args.batch}, {PROMPT_LEN}-token prompts)",
        "value": round(value, 2), "unit": "tok/s", "n_gpus": 1, "steps": steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic: uniform random token ids, random N(0, 0.02) weights, unit norm gains",
        "config": {"model": args.model, "layers": n_layers, "layers_of_model": cfg_full["num_hidden_layers"],
                   "hidden": cfg.hidden_size, "q_heads": cfg.num_attention_heads,
                   "kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
                   "intermediate": cfg.intermediate_size, "vocab": cfg.vocab_size,
                   "rope_theta": cfg.rope_theta, "rms_norm_eps": cfg.rms_norm_eps,
                   "tied_lm_head": cfg.tie_word_embeddings, "global_batch": args.batch,
                   "prompt_len": PROMPT_LEN, "seq_len": CONTEXT, "parallelism": "single GPU"},
        "prefill": {"value": round(PROMPT_LEN / prefill_s, 1), "tokens": PROMPT_LEN,
                    "ms": round(prefill_s * 1e3, 3), "frac": round(prefill_flops / prefill_s / peak, 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
        "points": points,
    }
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
