from .spec import (AttentionSpec, ConfigError, GeneralDeltaSpec, LayerSpec, LogDistanceBiasSpec, Mamba2Spec, MixerSlot,
                   ModelSpec, NoPositionSpec, PolyNormFFNSpec, RetentionSpec, RmsNormSpec, RopeSpec, ScheduleEntry,
                   SwiGLUSpec)
from .registry import (config_from_dict, load_config, register_architecture,
                       registered_architectures)
from .falcon_h1 import FalconH1Config
from .mukutar import MukutarConfig

register_architecture(FalconH1Config)
register_architecture(MukutarConfig)

__all__ = ["AttentionSpec", "ConfigError", "FalconH1Config", "GeneralDeltaSpec", "LayerSpec", "LogDistanceBiasSpec",
           "Mamba2Spec", "MixerSlot", "ModelSpec", "MukutarConfig", "NoPositionSpec", "PolyNormFFNSpec", "RetentionSpec",
           "RmsNormSpec", "RopeSpec", "ScheduleEntry", "SwiGLUSpec",
           "config_from_dict", "load_config", "register_architecture", "registered_architectures"]
