"""Configuration: typed parsing of config.json keys, validation, the architecture registry."""
import json

import pytest

from helpers import TINY_A, TINY_B
from minivllm_amd.config import ConfigError, EngineConfig, Qwen3Config, SamplingParams, compute_dtype_name
from minivllm_amd.models import config_from_dict, get_architecture, load_config, registered_architectures


def test_qwen3_keys_are_read():
    arch, cfg = config_from_dict(dict(TINY_B))
    assert arch.name == "Qwen3ForCausalLM" and isinstance(cfg, Qwen3Config)
    assert (cfg.num_hidden_layers, cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads) == (3, 96, 8, 2)
    assert (cfg.head_dim, cfg.intermediate_size, cfg.vocab_size) == (32, 168, 391)
    assert cfg.rope_theta == 1e6 and cfg.rms_norm_eps == 1e-5
    assert cfg.attention_bias is True and cfg.tie_word_embeddings is False
    assert cfg.eos_token_ids == (3, 5)
    assert cfg.q_dim == 256 and cfg.kv_dim == 64
    # sliding_window 21 = 21 keys with the query's own: 20 to its left
    assert [cfg.layer_window(i) for i in range(3)] == [None, 20, 20]
    assert cfg.dtype == "bfloat16"


def test_defaults_and_head_dim_fallback():
    d = {k: v for k, v in TINY_A.items() if k not in ("head_dim", "rms_norm_eps", "rope_theta", "attention_bias",
                                                      "tie_word_embeddings", "torch_dtype", "use_sliding_window",
                                                      "sliding_window", "max_window_layers")}
    _, cfg = config_from_dict(d)
    assert cfg.head_dim == 64 // 4              # the reference's fallback (executor.py:41)
    assert cfg.rms_norm_eps == 1e-6 and cfg.rope_theta == 10000.0
    assert cfg.attention_bias is False and cfg.tie_word_embeddings is False and cfg.dtype == "bfloat16"
    assert all(cfg.layer_window(i) is None for i in range(cfg.num_hidden_layers))
    assert cfg.eos_token_ids == (7,)


def test_round_trip_through_config_json(tmp_path):
    for raw in (TINY_A, TINY_B):
        _, cfg = config_from_dict(dict(raw))
        (tmp_path / "config.json").write_text(json.dumps(cfg.to_dict()))
        arch, again = load_config(str(tmp_path))
        assert again == cfg


@pytest.mark.parametrize("key", ["vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads",
                                 "intermediate_size", "max_position_embeddings"])
def test_missing_size_is_an_error(key):
    d = dict(TINY_A)
    del d[key]
    with pytest.raises(ConfigError, match=key):
        config_from_dict(d)


@pytest.mark.parametrize("patch,needle", [
    ({"hidden_act": "gelu"}, "hidden_act"),
    ({"rope_scaling": {"rope_type": "yarn", "factor": 4.0}}, "rope_scaling"),
    ({"num_key_value_heads": 3}, "multiple"),
    ({"head_dim": 15}, "even"),
    ({"vocab_size": "256"}, "integer"),
    ({"rms_norm_eps": 0.0}, "rms_norm_eps"),
    ({"use_sliding_window": True, "sliding_window": None}, "sliding_window"),
    ({"use_sliding_window": True, "sliding_window": 0}, "sliding_window"),
    ({"torch_dtype": "int8"}, "dtype"),
])
def test_unsupported_values_are_refused(patch, needle):
    with pytest.raises(ConfigError, match=needle):
        config_from_dict({**TINY_A, **patch})


def test_unknown_architecture():
    with pytest.raises(ConfigError, match="Model architecture LlamaForCausalLM is not supported"):
        config_from_dict({**TINY_A, "architectures": ["LlamaForCausalLM"]})
    with pytest.raises(ConfigError, match="architectures"):
        config_from_dict({k: v for k, v in TINY_A.items() if k != "architectures"})
    assert "Qwen3ForCausalLM" in registered_architectures()


def test_unknown_keys_are_ignored():
    _, cfg = config_from_dict({**TINY_A, "some_future_key": 1, "transformers_version": "x"})
    assert cfg.hidden_size == 64


def test_plan_is_data():
    arch, cfg = config_from_dict(dict(TINY_B))
    plan = arch.plan(cfg)
    assert len(plan.layers) == 3 and [c.layer for c in plan.calls] == [0, 1, 2]
    assert plan.layers[0].mixer.window is None and plan.layers[2].mixer.window == 20
    assert plan.layers[1].mixer.num_heads == 8 and plan.layers[1].mixer.scale == 32 ** -0.5
    assert plan.layers[1].ffn.intermediate_size == 168
    assert plan.head.tied is False and plan.final_norm.eps == 1e-5


def test_engine_config_and_sampling_params():
    ec = EngineConfig(model="x")
    # the reference's names (minivllm/config/config.py:11-46)
    for name in ("model", "max_model_len", "max_num_batched_tokens", "max_num_batched_seqs", "eos_token_ids",
                 "kv_cache_num_blocks", "kv_cache_block_size", "gpu_memory_utilization", "use_cuda_graph"):
        assert hasattr(ec, name)
    assert ec.max_model_len == 4096 and ec.max_num_batched_tokens == 16384 and ec.max_num_batched_seqs == 512
    assert ec.gpu_memory_utilization == 0.5 and ec.use_cuda_graph is True
    with pytest.raises(ValueError):
        EngineConfig(model="x", dtype="float16")
    with pytest.raises(ValueError):
        EngineConfig(model="x", gpu_memory_utilization=0.0)
    # ours: decode-only steps may run several times in a row on the device
    assert ec.num_scheduler_steps >= 1 and EngineConfig(model="x", num_scheduler_steps=1).num_scheduler_steps == 1
    assert ec.launch_ahead is True and EngineConfig(model="x", launch_ahead=False).launch_ahead is False
    with pytest.raises(ValueError):
        EngineConfig(model="x", num_scheduler_steps=0)
    sp = SamplingParams()
    # minivllm/config/sampling.py:4-10
    assert (sp.temperature, sp.max_tokens, sp.ignore_eos, sp.top_k, sp.top_p) == (1.0, 512, False, 0, 1.0)
    for bad in (dict(temperature=-1.0), dict(max_tokens=0), dict(top_k=-1), dict(top_p=0.0), dict(top_p=1.5)):
        with pytest.raises(ValueError):
            SamplingParams(**bad)


def test_float16_models_need_a_stated_dtype():
    """config.json may name float16; the engine computes in bfloat16 or float32 and picks neither
    silently (the reference computes in whatever config.json names, executor.py:17)."""
    _, cfg = config_from_dict({**TINY_A, "torch_dtype": "float16"})
    assert cfg.dtype == "float16"
    with pytest.raises(ConfigError, match="float16.*state dtype"):
        compute_dtype_name(None, cfg.dtype, "m/config.json")
    assert compute_dtype_name("float32", cfg.dtype) == "float32"
    assert compute_dtype_name("bfloat16", cfg.dtype) == "bfloat16"
    assert compute_dtype_name(None, "float32") == "float32" and compute_dtype_name(None, None) == "bfloat16"
