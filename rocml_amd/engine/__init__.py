from .batch import StepContext, StepEntry
from .engine import Engine
from .generate import EngineBackend, GenerateStats, Generator, Request, Result
from .model import DecoderModel
from .workspace import Workspace

__all__ = ["DecoderModel", "Engine", "EngineBackend", "GenerateStats", "Generator", "Request", "Result", "StepContext", "StepEntry", "Workspace"]
