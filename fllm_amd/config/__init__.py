from .spec import ConfigError, LayerSpec, ModelSpec, PartSpec, RunEntry, default_run_order
from .files import read_config_json
from .llama import LlamaConfig, RopeScaling

__all__ = ["ConfigError", "LayerSpec", "ModelSpec", "PartSpec", "RunEntry", "default_run_order",
           "LlamaConfig", "RopeScaling", "read_config_json"]
