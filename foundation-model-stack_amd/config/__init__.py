from .base import ModelConfig
from .llama import LLaMAConfig
from .zodolorn import ZodolornConfig

__all__ = ["ModelConfig", "LLaMAConfig", "ZodolornConfig"]
