from .specs import (AttentionSpec, ConfigError, EmbeddingSpec, GatedMlpSpec, HeadSpec, LayerSpec, ModelSpec,
                    NormSpec, RotarySpec, YarnSpec)
from .registry import architectures, architecture_of, config_from_dict, load_config, register_architecture
from .qwen2 import ARCHITECTURE as QWEN2_ARCHITECTURE, Qwen2Config

register_architecture(QWEN2_ARCHITECTURE, Qwen2Config, model_type="qwen2")

__all__ = ["AttentionSpec", "ConfigError", "EmbeddingSpec", "GatedMlpSpec", "HeadSpec", "LayerSpec", "ModelSpec",
           "NormSpec", "RotarySpec", "YarnSpec", "architectures", "architecture_of", "config_from_dict", "load_config",
           "register_architecture", "Qwen2Config", "QWEN2_ARCHITECTURE"]
