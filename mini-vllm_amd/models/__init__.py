from .registry import (Architecture, config_from_dict, get_architecture, load_config, register_architecture,
                       registered_architectures, unregister_architecture)
from . import qwen3  # registers "Qwen3ForCausalLM"
from .causal_lm import CausalLM, expected_tensors
