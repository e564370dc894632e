from .specs import (AttentionSpec, DenseMLPSpec, FrequencyScaling, GatedDeltaSpec, GatedMLPSpec,
                    LatentAttentionSpec, LayerSpec, LinearAttentionSpec, LoopSpec, MatrixMemorySpec,
                    ModelSpec, NormSpec, ParallelSpec, PositionSpec, RoutedMLPSpec, ScheduleEntry, StateSpaceSpec, default_schedule,
                    looped_schedule)
from .qwen3 import ConfigError, Qwen3Config
from .tirurax import TiruraxConfig
from .zadenex import ZadenexConfig
from .vafepel import VafepelConfig
from .gopuzen import GopuzenConfig
from .registry import (Architecture, known_architectures, read_config, register_architecture,
                       resolve_architecture, unregister_architecture)

register_architecture(Qwen3Config.architecture, Qwen3Config, model_types=("qwen3",))
register_architecture(TiruraxConfig.architecture, TiruraxConfig, model_types=("tirurax",))
register_architecture(ZadenexConfig.architecture, ZadenexConfig, model_types=("zadenex",))
register_architecture(VafepelConfig.architecture, VafepelConfig, model_types=("vafepel",))
register_architecture(GopuzenConfig.architecture, GopuzenConfig, model_types=("gopuzen",))

__all__ = [
    "AttentionSpec", "DenseMLPSpec", "GatedDeltaSpec", "GatedMLPSpec", "LayerSpec", "ModelSpec", "NormSpec", "PositionSpec",
    "ScheduleEntry", "default_schedule", "ConfigError", "Qwen3Config", "TiruraxConfig", "ZadenexConfig",
    "VafepelConfig", "GopuzenConfig", "LinearAttentionSpec", "ParallelSpec", "FrequencyScaling", "RoutedMLPSpec", "StateSpaceSpec",
    "LatentAttentionSpec", "LoopSpec", "MatrixMemorySpec", "looped_schedule", "Architecture",
    "known_architectures", "read_config", "register_architecture", "resolve_architecture",
    "unregister_architecture",
]
