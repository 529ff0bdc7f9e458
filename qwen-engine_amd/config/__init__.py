from .spec import (AttentionSpec, BareRMSNormSpec, BiasedMoESpec, ConvAttentionSpec, ParallelLayerSpec, RopeHalfAnglesSpec,
                   StreamScaleSpec, GroupedMoESpec, LatentAttentionSpec, LayerSpec, ModelSpec, PolyNormMLPSpec,
                   PostNormLayerSpec, RMSNormSpec, RopePairsSpec, RopeSpec, ScalarRMSNormSpec,
                   ScheduleEntry, ShortConvSpec, SwiGLUSpec)
from .qwen3 import ConfigError, Qwen3Config
from .zarorax import ZaroraxConfig
from .nufavik import NufavikConfig
from .registry import (config_from_dict, config_from_folder, known_architectures,
                       register_architecture, unregister_architecture)
from .engine_config import EngineConfig
