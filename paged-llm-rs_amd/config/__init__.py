from .dimalix import DimalixConfig
from .generation import GenerationConfig
from .lefavik import LefavikConfig
from .mukenex import MukenexConfig
from .papivik import PapivikConfig
from .qwen3 import Qwen3Config, read_json
from .registry import architectures, config_class_for, load_config, register_architecture
from .specs import (AttentionSpec, GatedMlpSpec, LayerSpec, ModelSpec, NormSpec, PositionSpec,
                    ScheduleEntry)

__all__ = [
    "GenerationConfig", "Qwen3Config", "PapivikConfig", "LefavikConfig", "MukenexConfig", "DimalixConfig", "read_json", "architectures", "config_class_for",
    "load_config", "register_architecture", "AttentionSpec", "GatedMlpSpec", "LayerSpec",
    "ModelSpec", "NormSpec", "PositionSpec", "ScheduleEntry",
]
