from .base import ModelConfig
from .llama import LLaMAConfig

__all__ = ["ModelConfig", "LLaMAConfig"]
