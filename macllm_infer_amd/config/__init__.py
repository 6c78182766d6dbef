from .spec import (AttentionSpec, ClampedGLUSpec, ConfigError, GatedLinearAttentionSpec, GeneralDeltaSpec, HashedBigramSpec,
                   InterleavedRopeSpec,
                   LatentAttentionSpec, LayerNormSpec, LayerSpec, LogDistanceBiasSpec, Mamba2Spec, MixerSlot,
                   ModelSpec, NoPositionSpec, PolyNormFFNSpec, PowerReluSpec, RampScalingSpec, RetentionSpec, RmsNormSpec, RopeSpec,
                   RoutedExpertsSpec, ScheduleEntry, StreamInjection, SwiGLUSpec, WavelengthScalingSpec)
from .registry import (config_from_dict, load_config, register_architecture,
                       registered_architectures)
from .falcon_h1 import FalconH1Config
from .mukutar import MukutarConfig
from .lutosun import LutosunConfig
from .motolix import MotolixConfig
from .pemarax import PemaraxConfig

register_architecture(FalconH1Config)
register_architecture(MukutarConfig)
register_architecture(LutosunConfig)
register_architecture(MotolixConfig)
register_architecture(PemaraxConfig)

__all__ = ["AttentionSpec", "ClampedGLUSpec", "ConfigError", "FalconH1Config", "GatedLinearAttentionSpec", "GeneralDeltaSpec", "HashedBigramSpec",
           "InterleavedRopeSpec", "LatentAttentionSpec", "LayerNormSpec", "LayerSpec", "LogDistanceBiasSpec", "LutosunConfig",
           "Mamba2Spec", "MixerSlot", "ModelSpec", "MotolixConfig", "MukutarConfig", "NoPositionSpec", "PemaraxConfig", "PolyNormFFNSpec", "PowerReluSpec", "RampScalingSpec", "RetentionSpec",
           "RmsNormSpec", "RopeSpec", "RoutedExpertsSpec", "ScheduleEntry", "StreamInjection", "SwiGLUSpec", "WavelengthScalingSpec",
           "config_from_dict", "load_config", "register_architecture", "registered_architectures"]
