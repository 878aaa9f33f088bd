from .spec import (AttentionSpec, BlockSpec, GatedMlpSpec, ModelSpec, NormSpec, RopeSpec,
                   ScheduleEntry, default_schedule)
from .qwen3 import Qwen3Config
from .registry import (Architecture, architecture, architecture_of, known_architectures,
                       read_config_json, register_architecture)

__all__ = ["AttentionSpec", "BlockSpec", "GatedMlpSpec", "ModelSpec", "NormSpec", "RopeSpec",
           "ScheduleEntry", "default_schedule", "Qwen3Config", "Architecture", "architecture",
           "architecture_of", "known_architectures", "read_config_json", "register_architecture"]
