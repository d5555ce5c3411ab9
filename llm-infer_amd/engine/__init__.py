from .model import DecoderModel
from .step import StepContext
from .engine import Engine, as_dtype

__all__ = ["DecoderModel", "StepContext", "Engine", "as_dtype"]
