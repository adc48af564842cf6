"""Architectures this engine knows. Importing the package registers them."""
from ..config.registry import register_architecture
from .qwen2 import Qwen2Config

register_architecture(Qwen2Config.architecture, Qwen2Config)

__all__ = ["Qwen2Config"]
