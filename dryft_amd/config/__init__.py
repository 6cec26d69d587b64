from .base import ConfigError, KeyReader, read_config_json
from .plan import LayerSpec, ModelPlan, PartSpec, Run
from .qwen3 import Qwen3Config

__all__ = ["ConfigError", "KeyReader", "read_config_json", "LayerSpec", "ModelPlan", "PartSpec", "Run",
           "Qwen3Config"]
