from .spec import (AttentionSpec, ConfigError, LayerSpec, Mamba2Spec, MixerSlot, ModelSpec,
                   NoPositionSpec, RmsNormSpec, RopeSpec, ScheduleEntry, SwiGLUSpec)
from .registry import (config_from_dict, load_config, register_architecture,
                       registered_architectures)
from .falcon_h1 import FalconH1Config

register_architecture(FalconH1Config)

__all__ = ["AttentionSpec", "ConfigError", "FalconH1Config", "LayerSpec", "Mamba2Spec", "MixerSlot",
           "ModelSpec", "NoPositionSpec", "RmsNormSpec", "RopeSpec", "ScheduleEntry", "SwiGLUSpec",
           "config_from_dict", "load_config", "register_architecture", "registered_architectures"]
