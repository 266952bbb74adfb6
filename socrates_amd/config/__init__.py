from .qwen3 import ConfigError, Qwen3Config
from .registry import (config_class_for, known_architectures, known_presets, load_config,
                       load_preset, preset_path, register_architecture)
from .specs import (AttentionSpec, BlockSpec, ModelPlan, RMSNormSpec, RopeSpec,
                    RunStep, SwiGLUSpec, default_order)

__all__ = ["ConfigError", "Qwen3Config", "config_class_for", "known_architectures", "known_presets", "load_config", "load_preset", "preset_path",
           "register_architecture", "AttentionSpec", "BlockSpec", "ModelPlan", "RMSNormSpec",
           "RopeSpec", "RunStep", "SwiGLUSpec", "default_order"]
