from .base import ModelConfig
from .defapel import DefapelConfig
from .llama import LLaMAConfig
from .sidalorn import SidalornConfig
from .zodolorn import ZodolornConfig

__all__ = ["ModelConfig", "LLaMAConfig", "ZodolornConfig", "DefapelConfig", "SidalornConfig"]
