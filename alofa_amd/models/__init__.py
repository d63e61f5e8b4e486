"""Architectures this engine knows. Importing the package registers them."""
from ..config.registry import register_architecture
from .ludelorn import LudelornConfig
from .qwen2 import Qwen2Config
from .rerupel import RerupelConfig
from .retotar import RetotarConfig
from .tugalix import TugalixConfig

register_architecture(Qwen2Config.architecture, Qwen2Config)
register_architecture(TugalixConfig.architecture, TugalixConfig)
register_architecture(RerupelConfig.architecture, RerupelConfig)
register_architecture(RetotarConfig.architecture, RetotarConfig)
register_architecture(LudelornConfig.architecture, LudelornConfig)

__all__ = ["LudelornConfig", "Qwen2Config", "RerupelConfig", "RetotarConfig", "TugalixConfig"]
