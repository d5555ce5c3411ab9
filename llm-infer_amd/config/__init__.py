from .spec import PartSpec, LayerSpec, ScheduleEntry, ModelSpec, ConfigError
from .llama import LlamaConfig

__all__ = ["PartSpec", "LayerSpec", "ScheduleEntry", "ModelSpec", "ConfigError", "LlamaConfig"]
