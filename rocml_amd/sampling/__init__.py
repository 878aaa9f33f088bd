from .params import Rng, SamplingParams, sequence_seed
from .sampler import DeviceSampler, SequenceSampling

__all__ = ["DeviceSampler", "Rng", "SamplingParams", "SequenceSampling", "sequence_seed"]
