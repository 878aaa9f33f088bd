"""The Python entry point: load a model, step it, generate with it.

It follows the reference's library surface (rocml/src/lib.rs:25-38): ``resolve`` a name or
a path, ``Model.load(path, options)``, the forward calls, ``reset`` and the ``generate``
family, with ``SamplingParams`` and ``Rng`` beside them.  Differences come from batching:
the forward call is ``step`` over several sequences, and ``generate`` takes a list of
prompts (token ids) and returns one result per prompt.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Iterable, List, Optional, Sequence, Union

from .config.catalog import DEFAULT_CTX, ModelEntry, Resolved, resolve
from .engine import Engine, EngineBackend, GenerateStats, Generator, Request, Result, StepEntry
from .errors import RocmlError
from .sampling import SamplingParams


@dataclass(frozen=True)
class LoadOptions:
    """Knobs fixed when a model is loaded (rocml/src/load_opts.rs:61-165 has ``ctx`` and the
    cache type; a quantized cache is not offered here).  ``ctx`` is the longest sequence the
    cache is sized for, ``max_batch`` the most sequences that run together; the cache holds
    ``ctx * max_batch`` positions unless ``max_tokens`` says otherwise."""
    dtype: str = "bfloat16"
    ctx: Optional[int] = None
    max_batch: int = 8
    max_tokens: Optional[int] = None
    device: str = "cuda:0"
    seed: int = 0                 # for models without a file (random weights)
    use_graphs: bool = True


def _generation_config_eos(path: str, vocab: int) -> frozenset:
    import json
    import os
    file = os.path.join(path, "generation_config.json")
    if not os.path.isfile(file):
        return frozenset()
    try:
        with open(file, "r", encoding="utf-8") as f:
            eos = json.load(f).get("eos_token_id")
    except (OSError, ValueError) as e:
        raise RocmlError(f"{file} cannot be read: {e}") from e
    if eos is None:
        return frozenset()
    ids = eos if isinstance(eos, (list, tuple)) else [eos]
    for t in ids:
        if isinstance(t, bool) or not isinstance(t, int) or not 0 <= t < vocab:
            raise RocmlError(f"{file}: eos_token_id must name token ids below {vocab}, found {eos!r}")
    return frozenset(ids)


class Model:
    """A loaded model with its engine."""

    def __init__(self, engine: Engine, options: LoadOptions, entry: Optional[ModelEntry]):
        self.engine = engine
        self.options = options
        self.entry = entry
        self.last_stats: Optional[GenerateStats] = None
        # ids that end a sequence by default: config.json's, and generation_config.json's if the
        # folder has one (the reference takes the id from its checkpoint and stops there unless
        # told not to, rocml/src/generate/resumed.rs:170,217-219)
        self.eos_token_ids = frozenset(engine.model.spec.eos_token_ids)

    @staticmethod
    def load(name_or_path: str, options: Optional[LoadOptions] = None, **kwargs) -> "Model":
        """``name_or_path`` is a folder with config.json and model.safetensors, or a catalog
        name; a catalog model has no file and gets random weights from ``options.seed``."""
        from .weights import load_model, random_model
        options = options or LoadOptions(**kwargs)
        found: Resolved = resolve(name_or_path)
        if found.path is not None:
            model = load_model(found.path, dtype=options.dtype, device=options.device)
        else:
            model = random_model(found.entry.config, seed=options.seed, dtype=options.dtype,
                                 device=options.device, norm_jitter=found.entry.init_norm_jitter)
        ctx = options.ctx or (found.entry.default_ctx if found.entry else DEFAULT_CTX)
        ctx = min(ctx, model.spec.max_positions)
        max_tokens = options.max_tokens or ctx * options.max_batch
        engine = Engine(model, max_tokens=max_tokens, max_seqs=max(options.max_batch, 1),
                        use_graphs=options.use_graphs)
        loaded = Model(engine, options, found.entry)
        if found.path is not None:
            loaded.eos_token_ids |= _generation_config_eos(found.path, model.spec.vocab)
        return loaded

    @property
    def config(self):
        return self.engine.model.config

    @property
    def vocab_size(self) -> int:
        return self.engine.model.spec.vocab

    def default_sampling(self) -> SamplingParams:
        """The catalog's preset for this model, else greedy (flag > preset > greedy is the
        command line's rule, rocml-cli/src/common.rs:167-176)."""
        if self.entry is not None and self.entry.sampling is not None:
            return self.entry.sampling
        return SamplingParams.greedy()

    # -- stepping ------------------------------------------------------------------------
    def new_sequence(self) -> int:
        return self.engine.new_sequence()

    def release(self, slot: int) -> None:
        self.engine.release(slot)

    def step(self, entries: Sequence[StepEntry]):
        return self.engine.step(entries)

    def position(self, slot: int) -> int:
        """Tokens the sequence holds so far (the reference's ``position()``,
        rocml/src/model.rs:112-130, per sequence here)."""
        return self.engine.length(slot)

    def reset(self) -> None:
        """Ends every live sequence; their slots and pages are given back and nothing is
        cleared, as rows beyond a length are never read (the reference's ``reset()`` sets
        its one position to zero, rocml/src/forward/mod.rs:224-232)."""
        for slot in sorted(self.engine.cache.slots.live):
            self.engine.release(slot)

    # -- generation ----------------------------------------------------------------------
    def generate(self, prompts: Sequence[Sequence[int]],
                 sampling: Union[SamplingParams, Sequence[SamplingParams], None] = None,
                 max_new_tokens: int = 64, stop_tokens: Iterable[int] = (), ignore_eos: bool = False,
                 on_step=None, on_token=None) -> List[Result]:
        """Continues every prompt (lists of token ids).  ``sampling`` is one set of parameters
        for all prompts or one per prompt; ``None`` means greedy.  A stop token ends its
        sequence and is not part of the result; the model's end-of-sequence ids are stop tokens
        unless ``ignore_eos``.  ``on_step`` is called after every decode step with their number,
        ``on_token(prompt index, token id)`` for every token as it is drawn."""
        if sampling is None:
            sampling = SamplingParams.greedy()
        if isinstance(sampling, SamplingParams):
            sampling = [sampling] * len(prompts)
        if len(sampling) != len(prompts):
            raise RocmlError("one SamplingParams for all prompts, or one per prompt")
        stop = frozenset(int(t) for t in stop_tokens)
        if not ignore_eos:
            stop |= self.eos_token_ids
        requests = [Request(list(p), max_new_tokens, s, stop) for p, s in zip(prompts, sampling)]
        gen = Generator(EngineBackend(self.engine), max_batch=self.options.max_batch)
        gen.on_step = on_step
        gen.on_token = on_token
        results = gen.run(requests)
        self.last_stats = gen.stats
        return results
