from .model_config import ConfigError, LlamaConfig, RopeScaling, read_config_json
from .engine_config import EngineConfig, parse_dtype
from .registry import (MODEL_REGISTRY, Architecture, architecture_of, build_model,
                       config_from_dict, config_from_folder, register_model)
