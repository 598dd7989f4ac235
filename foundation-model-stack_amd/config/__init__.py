from .base import ModelConfig
from .basopel import BasopelConfig
from .defapel import DefapelConfig
from .llama import LLaMAConfig
from .sidalorn import SidalornConfig
from .zodolorn import ZodolornConfig

__all__ = ["ModelConfig", "LLaMAConfig", "ZodolornConfig", "DefapelConfig", "SidalornConfig", "BasopelConfig"]
