from .registry import (ConfigError, config_class, config_from_dict, known_architectures,
                       load_config, register_architecture)
from .specs import (AttentionSpec, ClampedGluSpec, DiffAttentionSpec, GlaSpec, LayerRun, LayerSpec, Mamba2Spec, MlpSpec,
                    ModelSpec, NormSpec, PositionSpec, QueryTemperature)
from .qwen3 import Qwen3Config
from .taletar import TaletarConfig
from .pamunex import PamunexConfig
from .tigelorn import TigelornConfig
from .budorax import BudoraxConfig

__all__ = ["ConfigError", "config_class", "config_from_dict", "known_architectures", "load_config",
           "register_architecture", "AttentionSpec", "LayerRun", "LayerSpec", "MlpSpec",
           "ModelSpec", "NormSpec", "PositionSpec", "Qwen3Config", "ClampedGluSpec", "DiffAttentionSpec", "GlaSpec",
           "Mamba2Spec", "QueryTemperature", "TaletarConfig", "PamunexConfig", "TigelornConfig", "BudoraxConfig"]
