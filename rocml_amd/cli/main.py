"""Command line in the manner of the reference's ``rocml-cli`` (rocml-cli/src/main.rs:25-48):
the subcommands ``generate``, ``bench`` and ``models`` with its option names where it has
them, plus ``init``, which writes a model folder with random weights, (rocml-cli/src/common.rs:38-57,146-177; cmd_generate.rs:19-49; cmd_bench.rs:15-77).
Prompts are token ids (``--prompt-ids``); ``--prompt`` takes text when the model folder has a
``tokenizer.json``.  There is no chat template, so ``--raw`` is accepted and changes nothing.
"""
from __future__ import annotations

import argparse
import json
import statistics
import sys
from typing import List, Optional

from ..errors import RocmlError


def _add_model_args(p: argparse.ArgumentParser) -> None:
    p.add_argument("--model", required=True, help="catalog name or a folder with config.json and model.safetensors")
    p.add_argument("--no-download", action="store_true", help="accepted for compatibility; nothing is ever downloaded")
    p.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"],
                   help="compute and cache type (the reference's --kv-cache picks its cache type)")
    p.add_argument("--batch", type=int, default=8, help="most sequences that run together")


def _add_sampling_args(p: argparse.ArgumentParser) -> None:
    # Unset flags fall back to the model's catalog preset, then to greedy
    # (rocml-cli/src/common.rs:167-176).
    p.add_argument("-t", "--temperature", type=float, default=None)
    p.add_argument("--top-p", type=float, default=None)
    p.add_argument("--top-k", type=int, default=None)
    p.add_argument("--seed", type=int, default=None)
    p.add_argument("--repeat-penalty", type=float, default=None)


def sampling_from_args(args, preset):
    from ..sampling import SamplingParams
    base = preset or SamplingParams()
    return SamplingParams(
        temperature=base.temperature if args.temperature is None else args.temperature,
        top_k=base.top_k if args.top_k is None else args.top_k,
        top_p=base.top_p if args.top_p is None else args.top_p,
        seed=base.seed if args.seed is None else args.seed,
        repeat_penalty=base.repeat_penalty if args.repeat_penalty is None else args.repeat_penalty,
        repeat_penalty_window=base.repeat_penalty_window)


def _parse_ids(text: str) -> List[int]:
    return [int(t) for t in text.replace(",", " ").split()]


def _load(args, ctx: Optional[int]):
    from ..api import LoadOptions, Model
    return Model.load(args.model, LoadOptions(dtype=args.dtype, ctx=ctx, max_batch=args.batch,
                                              seed=getattr(args, "weights_seed", 0)))


def _tokenizer(model_path: str):
    import os
    path = os.path.join(model_path, "tokenizer.json")
    if not os.path.isfile(path):
        raise RocmlError(f"--prompt needs {path}; give token ids with --prompt-ids instead")
    from tokenizers import Tokenizer
    return Tokenizer.from_file(path)


def cmd_generate(args) -> int:
    prompts: List[List[int]] = [_parse_ids(p) for p in (args.prompt_ids or [])]
    tok = None
    if args.prompt is not None:
        tok = _tokenizer(args.model)
        prompts.append(tok.encode(args.prompt).ids)
    if not prompts:
        raise RocmlError("give --prompt-ids (token ids) or --prompt (text, with a tokenizer.json)")
    model = _load(args, args.ctx)
    params = sampling_from_args(args, model.entry.sampling if model.entry else None)
    profiler = _profiler(args.dtype) if args.profile else None
    kwargs = dict(max_new_tokens=args.n, stop_tokens=_parse_ids(args.stop_ids or ""), ignore_eos=args.ignore_eos)
    # One prompt is written out as it is generated, token by token
    # (rocml-cli/src/cmd_generate.rs:113-127); several are written when all are done.
    streamed = len(prompts) == 1
    if streamed:
        shown = []

        def on_token(_index: int, token: int) -> None:
            if tok is not None:
                shown.append(token)
                text = tok.decode(shown)
                if not text.endswith("\ufffd"):            # (a piece may end inside a character)
                    sys.stdout.write(text[on_token.written:])
                    on_token.written = len(text)
            else:
                sys.stdout.write(("" if on_token.written == 0 else " ") + str(token))
                on_token.written += 1
            sys.stdout.flush()
        on_token.written = 0
        kwargs["on_token"] = on_token
    if profiler is not None:
        with profiler:
            results = model.generate(prompts, params, **kwargs)
    else:
        results = model.generate(prompts, params, **kwargs)
    if streamed:
        if tok is not None:
            sys.stdout.write(tok.decode(results[0].tokens)[on_token.written:])    # what a held-back piece left
        print()
    else:
        for i, r in enumerate(results):
            if tok is not None and i == len(results) - 1 and args.prompt is not None:
                print(tok.decode(r.tokens))
            else:
                print(" ".join(str(t) for t in r.tokens))
    s = model.last_stats
    print(f"prompt: {s.prompt_tokens} tokens in {s.prompt_seconds:.3f} s ({s.prompt_tok_s():.1f} tok/s); "
          f"generated: {s.generated_tokens} tokens in {s.decode_seconds:.3f} s ({s.decode_tok_s():.1f} tok/s)",
          file=sys.stderr)
    if profiler is not None:
        print(profiler.finish().to_human())
    return 0


def _profiler(dtype: str):
    """Per-operation timing with a roofline report (rocml-cli/src/cmd_generate.rs:46-48,140-141)."""
    import torch
    from ..profile import OpProfiler
    return OpProfiler(torch.bfloat16 if dtype == "bfloat16" else torch.float32)


def cmd_bench(args) -> int:
    """Synthetic prompt, greedy, no stop token, medians over runs
    (rocml-cli/src/cmd_bench.rs:79-243)."""
    import numpy as np
    prompt_tokens = args.depth if args.depth is not None else args.prompt_tokens
    if args.prompt_range is not None:
        if not 1 <= args.prompt_range[0] <= args.prompt_range[1]:
            raise RocmlError("--prompt-range needs 1 <= LO <= HI")
        prompt_tokens = args.prompt_range[1]
    ctx = args.ctx or max(4096, prompt_tokens + args.decode_tokens)
    model = _load(args, ctx)
    rng = np.random.default_rng(args.prompt_seed)
    prefill, decode = [], []
    # Only the last run is profiled; it still counts for the medians, as in the reference
    # (rocml-cli/src/cmd_bench.rs:129-141), though its steps run launch by launch.
    want_profile = args.profile or args.profile_json is not None
    report = None
    for run in range(args.runs):
        if args.prompt_range is not None:
            # unequal prompts, lengths uniform in [LO, HI], the same in every run of a seed
            lo, hi = args.prompt_range
            lengths = [int(n) for n in rng.integers(lo, hi + 1, size=args.batch)]
        else:
            lengths = [prompt_tokens] * args.batch
        prompts = [[int(t) for t in rng.integers(0, model.vocab_size, size=n)] for n in lengths]
        if want_profile and run + 1 == args.runs:
            with _profiler(args.dtype) as profiler:
                model.generate(prompts, max_new_tokens=args.decode_tokens, ignore_eos=True)
            report = profiler.finish()
        else:
            model.generate(prompts, max_new_tokens=args.decode_tokens, ignore_eos=True)
        s = model.last_stats
        prefill.append(s.prompt_tok_s())
        decode.append(s.decode_tok_s())
    out = {"model": args.model, "dtype": args.dtype, "batch": args.batch,
           "prompt_tokens": prompt_tokens if args.prompt_range is None else sorted(lengths),
           "decode_tokens": args.decode_tokens, "runs": args.runs,
           "prefill_tok_s": statistics.median(prefill), "decode_tok_s": statistics.median(decode)}
    if args.json:
        print(json.dumps(out))
    else:
        shown = f"{prompt_tokens} tokens" if args.prompt_range is None else f"{min(lengths)} to {max(lengths)} tokens"
        print(f"{args.model} {args.dtype} batch {args.batch}: prefill {out['prefill_tok_s']:.1f} tok/s "
              f"({shown}), decode {out['decode_tok_s']:.1f} tok/s ({args.decode_tokens} tokens), "
              f"median of {args.runs}")
    if report is not None and args.profile:
        print(report.to_human())
    if report is not None and args.profile_json is not None:
        with open(args.profile_json, "w", encoding="utf-8") as f:
            json.dump({"bench": out, "report": report.to_dict()}, f, indent=1)
    return 0


def _describe(spec) -> str:
    """A part's spec in a few words: its kind and its sizes (the width it shares with the model
    left out)."""
    import dataclasses
    if not dataclasses.is_dataclass(spec):
        return getattr(spec, "kind", type(spec).__name__)
    fields = [f"{f.name}={getattr(spec, f.name)}" for f in dataclasses.fields(spec)
              if f.name not in ("kind", "hidden") and isinstance(getattr(spec, f.name), (int, str)) and not isinstance(getattr(spec, f.name), bool)]
    return f"{spec.kind}({', '.join(fields)})"


def cmd_models(args) -> int:
    """Lists the catalog (rocml-cli/src/cmd_models.rs:13-38 prints name, family, presence); every
    figure comes from the model that the entry's architecture builds, without weights."""
    import torch
    from ..config import architecture_of
    from ..config.catalog import CATALOG
    from ..engine.model import DecoderModel
    print(f"{'name':<12} {'architecture':<18} {'layers':>6} {'hidden':>6} {'vocab':>7} {'params':>9} {'bf16 GB':>8}  first layer")
    for e in CATALOG:
        arch = architecture_of(e.config)
        spec = arch.to_spec(arch.read_config(e.config))
        model = DecoderModel(spec, torch.bfloat16, device="meta")
        first = spec.layers[spec.schedule[0].layer]
        print(f"{e.name:<12} {spec.architecture:<18} {len(spec.schedule):>6} {spec.hidden:>6} {spec.vocab:>7} "
              f"{model.n_params() / 1e9:>8.3f}B {model.weight_bytes() / 1e9:>8.2f}  {_describe(first.mixer)}, {_describe(first.ffn)}")
    return 0


def cmd_init(args) -> int:
    """Writes a model folder (config.json, model.safetensors) with random weights for a catalog
    entry or a config.json; the reference has no counterpart (it only reads checkpoints)."""
    import torch
    from ..config import read_config_json
    from ..config.catalog import resolve
    from ..weights import write_model_dir
    found = resolve(args.model)
    config = found.entry.config if found.entry is not None else read_config_json(found.path)
    jitter = found.entry.init_norm_jitter if found.entry is not None else True
    dtype = torch.bfloat16 if args.dtype == "bfloat16" else torch.float32
    path = write_model_dir(args.out, config, args.weights_seed, dtype=dtype, norm_jitter=jitter, device=args.device)
    print(path)
    return 0


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(prog="rocml_amd", description="Qwen3 generation on one MI355X")
    sub = ap.add_subparsers(dest="command", required=True)
    g = sub.add_parser("generate", help="continue prompts")
    _add_model_args(g)
    g.add_argument("--prompt", default=None, help="prompt text (needs tokenizer.json in the model folder)")
    g.add_argument("--prompt-ids", action="append", help="prompt as token ids, e.g. '1 2 3'; repeat for a batch")
    g.add_argument("--raw", action="store_true", help="accepted for compatibility: prompts are always raw")
    g.add_argument("-n", "--max-tokens", dest="n", type=int, default=64)
    g.add_argument("--ctx", type=int, default=None, help="longest sequence the cache is sized for")
    g.add_argument("--stop-ids", default=None, help="token ids that end a sequence")
    g.add_argument("--ignore-eos", action="store_true",
                   help="do not stop at the model's end-of-sequence id (eos_token_id of config.json or generation_config.json)")
    g.add_argument("--weights-seed", type=int, default=0, help="seed of the random weights of a catalog model")
    g.add_argument("--profile", action="store_true", help="time every operation and print a roofline report")
    _add_sampling_args(g)
    g.set_defaults(fn=cmd_generate)
    b = sub.add_parser("bench", help="measure prefill and decode speed")
    _add_model_args(b)
    b.add_argument("--prompt-tokens", type=int, default=64)
    b.add_argument("--decode-tokens", type=int, default=128)
    b.add_argument("--runs", type=int, default=3)
    b.add_argument("--depth", type=int, default=None, help="prompt of this many tokens, then decode")
    b.add_argument("--ctx", type=int, default=None)
    b.add_argument("--prompt-range", type=int, nargs=2, default=None, metavar=("LO", "HI"),
                   help="unequal prompts: every sequence's length drawn uniformly from LO..HI")
    b.add_argument("--prompt-seed", type=int, default=0, help="seed of the synthetic prompts")
    b.add_argument("--weights-seed", type=int, default=0, help="seed of the random weights of a catalog model")
    b.add_argument("--json", action="store_true")
    b.add_argument("--profile", action="store_true", help="time every operation of the last run and print a roofline report")
    b.add_argument("--profile-json", default=None, metavar="PATH", help="write that report as JSON (implies profiling)")
    b.set_defaults(fn=cmd_bench)
    m = sub.add_parser("models", help="list the catalog")
    m.set_defaults(fn=cmd_models)
    i = sub.add_parser("init", help="write a model folder with random weights")
    i.add_argument("--model", required=True, help="catalog name, or a folder whose config.json to use")
    i.add_argument("--out", required=True, help="folder to write config.json and model.safetensors to")
    i.add_argument("--weights-seed", type=int, default=0)
    i.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"], help="storage type of the tensors")
    i.add_argument("--device", default="cpu", help="where the values are drawn (the same on any device); cuda:0 is faster for large models")
    i.set_defaults(fn=cmd_init)
    return ap


def main(argv=None) -> int:
    args = build_parser().parse_args(argv)
    try:
        return args.fn(args)
    except RocmlError as e:
        print(f"error: {e}", file=sys.stderr)
        return 1


if __name__ == "__main__":
    sys.exit(main())
