from .spec import ConfigError, LayerSpec, ModelSpec, PartSpec, RunEntry, default_run_order
from .llama import LlamaConfig, RopeScaling, read_config_json

__all__ = ["ConfigError", "LayerSpec", "ModelSpec", "PartSpec", "RunEntry", "default_run_order",
           "LlamaConfig", "RopeScaling", "read_config_json"]
