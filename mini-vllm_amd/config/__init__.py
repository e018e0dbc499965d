from .model_config import (ConfigError, ModelConfig, Qwen3Config, read_config_json,
                           architecture_name)
from .engine_config import EngineConfig, compute_dtype_name
from .sampling_params import SamplingParams

__all__ = ["ConfigError", "ModelConfig", "Qwen3Config", "read_config_json", "architecture_name",
           "EngineConfig", "SamplingParams", "compute_dtype_name"]
