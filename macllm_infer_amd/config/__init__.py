from .spec import (AttentionSpec, ClampedGLUSpec, ConfigError, GeneralDeltaSpec, HashedBigramSpec, InterleavedRopeSpec,
                   LatentAttentionSpec, LayerNormSpec, LayerSpec, LogDistanceBiasSpec, Mamba2Spec, MixerSlot,
                   ModelSpec, NoPositionSpec, PolyNormFFNSpec, RetentionSpec, RmsNormSpec, RopeSpec,
                   RoutedExpertsSpec, ScheduleEntry, StreamInjection, SwiGLUSpec)
from .registry import (config_from_dict, load_config, register_architecture,
                       registered_architectures)
from .falcon_h1 import FalconH1Config
from .mukutar import MukutarConfig
from .lutosun import LutosunConfig

register_architecture(FalconH1Config)
register_architecture(MukutarConfig)
register_architecture(LutosunConfig)

__all__ = ["AttentionSpec", "ClampedGLUSpec", "ConfigError", "FalconH1Config", "GeneralDeltaSpec", "HashedBigramSpec",
           "InterleavedRopeSpec", "LatentAttentionSpec", "LayerNormSpec", "LayerSpec", "LogDistanceBiasSpec", "LutosunConfig",
           "Mamba2Spec", "MixerSlot", "ModelSpec", "MukutarConfig", "NoPositionSpec", "PolyNormFFNSpec", "RetentionSpec",
           "RmsNormSpec", "RopeSpec", "RoutedExpertsSpec", "ScheduleEntry", "StreamInjection", "SwiGLUSpec",
           "config_from_dict", "load_config", "register_architecture", "registered_architectures"]
