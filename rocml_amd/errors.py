"""Error types of the library; every failure a caller can cause is one of these.

Mirrors the reference's single error enum (rocml/src/error.rs:8-99): unknown
model, unsupported architecture, bad configuration, bad weights, context
overflow, and failures of the GPU layer with code and message
(rocml-hip/src/error.rs:32-48).
"""


class RocmlError(Exception):
    """Base class of every error this library raises on purpose."""


class ConfigError(RocmlError):
    """config.json lacks a key, or a value breaks a rule the kernels rely on."""


class UnknownModelError(RocmlError):
    """A model name that is neither in the catalog nor a model folder."""


class UnsupportedArchitectureError(RocmlError):
    """config.json names an architecture that is not registered."""


class WeightsError(RocmlError):
    """Tensors of a checkpoint do not fit the model: lists every problem at once."""


class CacheFullError(RocmlError):
    """The cache cannot hold the tokens or sequences a step asks for."""


class MemoryBudgetError(RocmlError):
    """The cache that was asked for does not fit the free memory of the GPU."""


class ContextOverflowError(RocmlError):
    """A sequence would grow beyond the positions the model was built for."""


class KernelError(RocmlError):
    """A HIP kernel refused its arguments, or the GPU runtime reported a failure."""


class ExtensionMissingError(RocmlError):
    """The compiled HIP library is missing and could not be built."""
