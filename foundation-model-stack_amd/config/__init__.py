from .base import ModelConfig
from .defapel import DefapelConfig
from .llama import LLaMAConfig
from .zodolorn import ZodolornConfig

__all__ = ["ModelConfig", "LLaMAConfig", "ZodolornConfig", "DefapelConfig"]
