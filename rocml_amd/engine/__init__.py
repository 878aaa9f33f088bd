from .batch import StepContext, StepEntry
from .engine import Engine
from .model import DecoderModel
from .workspace import Workspace

__all__ = ["DecoderModel", "Engine", "StepContext", "StepEntry", "Workspace"]
