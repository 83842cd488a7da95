from .spec import ConfigError, LayerSpec, ModelSpec, PartSpec, RunEntry, default_run_order
from .files import read_config_json
from .dumizen import DumizenConfig
from .llama import LlamaConfig, RopeScaling
from .menitar import MenitarConfig
from .purivik import PurivikConfig

__all__ = ["ConfigError", "LayerSpec", "ModelSpec", "PartSpec", "RunEntry", "default_run_order",
           "DumizenConfig", "LlamaConfig", "MenitarConfig", "PurivikConfig", "RopeScaling", "read_config_json"]
