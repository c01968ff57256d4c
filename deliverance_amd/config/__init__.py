from .specs import (AttentionSpec, ConfigError, DenseFeedForwardSpec, LayerCall, LayerSpec,
                    ModelConfig, NormSpec, PositionSpec)
from .gpt2 import Gpt2Config
from .virudra import VirudraConfig
from .pedatar import PedatarConfig
from .pafolorn import PafolornConfig
from .salivik import SalivikConfig
from .engine_config import EngineConfig

__all__ = ["AttentionSpec", "ConfigError", "DenseFeedForwardSpec", "LayerCall", "LayerSpec",
           "ModelConfig", "NormSpec", "PositionSpec", "Gpt2Config", "VirudraConfig", "PedatarConfig", "PafolornConfig", "SalivikConfig", "EngineConfig"]
