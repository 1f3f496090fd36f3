"""A small, whole Llama inference engine for one MI355X (gfx950)."""
from . import models as _models  # registers the architectures
from .config import EngineConfig, LlamaConfig, build_model, config_from_folder
