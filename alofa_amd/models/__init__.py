"""Architectures this engine knows. Importing the package registers them."""
from ..config.registry import register_architecture
from .qwen2 import Qwen2Config
from .tugalix import TugalixConfig

register_architecture(Qwen2Config.architecture, Qwen2Config)
register_architecture(TugalixConfig.architecture, TugalixConfig)

__all__ = ["Qwen2Config", "TugalixConfig"]
