from .model_config import (ConfigError, ModelConfig, Qwen3Config, read_config_json,
                           architecture_name)
from .engine_config import EngineConfig, compute_dtype_name
from .sampling_params import SamplingParams
from .shapes import QWEN3_SHAPES, named_shape, named_shapes, qwen3_shape

__all__ = ["ConfigError", "ModelConfig", "Qwen3Config", "read_config_json", "architecture_name",
           "EngineConfig", "SamplingParams", "compute_dtype_name", "QWEN3_SHAPES", "qwen3_shape", "named_shape",
           "named_shapes"]
