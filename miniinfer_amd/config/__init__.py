from .engine import EngineConfig, normalize_dtype
from .qwen3 import ConfigError, Qwen3Config
from .registry import (known_architectures, load_model_config, model_spec_of, read_config_json,
                       register_architecture, resolve_architecture)
from .spec import (AttentionSpec, GatedMLPSpec, LayerSpec, ModelSpec, NoPositionSpec, NormSpec, RotarySpec)

register_architecture(Qwen3Config.architecture, Qwen3Config, model_type=Qwen3Config.model_type)
