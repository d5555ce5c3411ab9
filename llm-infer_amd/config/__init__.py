from .spec import PartSpec, SubLayerSpec, LayerSpec, ScheduleEntry, ModelSpec, ConfigError
from .llama import LlamaConfig

__all__ = ["PartSpec", "SubLayerSpec", "LayerSpec", "ScheduleEntry", "ModelSpec", "ConfigError", "LlamaConfig"]
