"""Dense Qwen3 generation on one MI355X: configuration, weights, parts, cache, step,
generation, sampling, hand-written HIP kernels."""
from .errors import (CacheFullError, ConfigError, ContextOverflowError, ExtensionMissingError,
                     KernelError, RocmlError, UnknownModelError, UnsupportedArchitectureError,
                     WeightsError)

__version__ = "0.1.0"
