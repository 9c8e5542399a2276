from .qwen3 import ConfigError, Qwen3Config
from .mitisun import MitisunConfig
from .registry import (config_class_for, known_architectures, known_presets, load_config,
                       load_preset, preset_path, register_architecture)
from .specs import (AttentionSpec, BlockSpec, ClampedGLUSpec, LatentAttentionSpec, Mamba2Spec, ModelPlan,
                    PairRopeSpec, RMSNormSpec, RopeSpec, RunStep, ScalarRMSNormSpec, SigmoidGateSpec,
                    SwiGLUSpec, WkvSpec, default_order)

__all__ = ["ConfigError", "Qwen3Config", "MitisunConfig", "config_class_for", "known_architectures", "known_presets",
           "load_config", "load_preset", "preset_path",
           "register_architecture", "AttentionSpec", "BlockSpec", "ModelPlan", "RMSNormSpec",
           "RopeSpec", "RunStep", "SwiGLUSpec", "default_order", "ClampedGLUSpec", "LatentAttentionSpec",
           "Mamba2Spec", "PairRopeSpec", "ScalarRMSNormSpec", "SigmoidGateSpec", "WkvSpec"]
