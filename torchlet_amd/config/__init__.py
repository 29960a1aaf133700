from .base import (AttentionSpec, BlockSpec, ConfigError, ModelConfig, ModelSpec, PartSpec, RMSNormSpec, RotarySpec,
                   RunEntry, SwiGLUSpec)
from .qwen2 import Qwen2Config

__all__ = ["AttentionSpec", "BlockSpec", "ConfigError", "ModelConfig", "ModelSpec", "PartSpec", "RMSNormSpec",
           "RotarySpec", "RunEntry", "SwiGLUSpec", "Qwen2Config"]
