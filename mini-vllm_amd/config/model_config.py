"""Typed model configurations read from a model folder's ``config.json``.

Every size and constant of a model comes from here; no part of the engine carries a
default of its own for something ``config.json`` states.

Reference: the reference hands the raw ``transformers`` config object to the model
(minivllm/config/config.py:50, minivllm/models/loader.py:14) and the model reads
``head_dim``, ``num_attention_heads``, ``num_key_value_heads``, ``hidden_size``,
``intermediate_size``, ``rms_norm_eps``, ``rope_theta``, ``max_position_embeddings``,
``attention_bias``, ``tie_word_embeddings``, ``vocab_size``, ``num_hidden_layers``
(minivllm/models/models/qwen3.py:28-65,160-204). Here the same keys are parsed with
plain ``json`` into a frozen dataclass and validated.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Any, ClassVar, Dict, Optional, Tuple


class ConfigError(ValueError):
    """A ``config.json`` that the engine cannot serve correctly."""


_DTYPE_NAMES = {
    "bfloat16": "bfloat16", "bf16": "bfloat16", "torch.bfloat16": "bfloat16",
    "float32": "float32", "fp32": "float32", "float": "float32", "torch.float32": "float32",
    "float16": "float16", "fp16": "float16", "half": "float16", "torch.float16": "float16",
}


def _require(d: Dict[str, Any], key: str, typ, where: str):
    if key not in d or d[key] is None:
        raise ConfigError(f"{where}: required key '{key}' is missing")
    return _typed(d[key], key, typ, where)


def _typed(v, key: str, typ, where: str):
    if typ is int:
        if isinstance(v, bool) or not isinstance(v, int):
            raise ConfigError(f"{where}: key '{key}' must be an integer, got {v!r}")
        return v
    if typ is float:
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            raise ConfigError(f"{where}: key '{key}' must be a number, got {v!r}")
        return float(v)
    if typ is bool:
        if not isinstance(v, bool):
            raise ConfigError(f"{where}: key '{key}' must be true or false, got {v!r}")
        return v
    raise TypeError(typ)


@dataclass(frozen=True)
class ModelConfig:
    """Base of all architecture configurations.

    A subclass names the ``architectures[0]`` string it serves in ``architecture`` and
    parses its own keys in ``from_dict``; ``to_dict`` writes them back under the same
    names so that a configuration can be stored as a ``config.json`` again.
    """

    architecture: ClassVar[str] = ""

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str = "config.json") -> "ModelConfig":
        raise NotImplementedError

    def to_dict(self) -> Dict[str, Any]:
        raise NotImplementedError


@dataclass(frozen=True)
class Qwen3Config(ModelConfig):
    """Qwen3 dense decoder (reference: minivllm/models/models/qwen3.py).

    The reference's Qwen3 never passes a window to its attention layer (qwen3.py:66-71), so
    there every layer sees all keys whatever ``use_sliding_window`` says. Here the key is
    honoured with the meaning it has where it comes from: with ``use_sliding_window`` the
    layers with index >= ``max_window_layers`` see ``sliding_window`` keys, the query's own
    among them (key position > query position - sliding_window); the other layers see all.
    No file of the reference pins this: parity unpinned. The attention part counts a window as
    tokens to the left of the query besides itself (the reference's attention layer,
    minivllm/models/layers/attention.py:56-60), which is ``sliding_window - 1``.
    """

    architecture: ClassVar[str] = "Qwen3ForCausalLM"

    vocab_size: int = 0
    hidden_size: int = 0
    num_hidden_layers: int = 0
    num_attention_heads: int = 0
    num_key_value_heads: int = 0
    head_dim: int = 0
    intermediate_size: int = 0
    max_position_embeddings: int = 0
    rms_norm_eps: float = 1e-6
    rope_theta: float = 10000.0
    attention_bias: bool = False
    tie_word_embeddings: bool = False
    use_sliding_window: bool = False
    sliding_window: Optional[int] = None
    max_window_layers: int = 0
    dtype: str = "bfloat16"
    eos_token_ids: Tuple[int, ...] = ()
    bos_token_id: Optional[int] = None

    @property
    def q_dim(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_dim(self) -> int:
        return self.num_key_value_heads * self.head_dim

    def layer_window(self, layer: int) -> Optional[int]:
        """How many tokens to the left of a query ``layer`` sees besides the query itself
        (``sliding_window`` keys in all, the query's own included), or None for all."""
        if self.use_sliding_window and layer >= self.max_window_layers:
            return self.sliding_window - 1
        return None

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str = "config.json") -> "Qwen3Config":
        hidden = _require(d, "hidden_size", int, where)
        heads = _require(d, "num_attention_heads", int, where)
        kv_heads = d.get("num_key_value_heads")
        kv_heads = heads if kv_heads is None else _typed(kv_heads, "num_key_value_heads", int, where)
        head_dim = d.get("head_dim")
        if head_dim is None:
            # the reference's cache sizing falls back the same way (minivllm/executor/executor.py:41)
            if hidden % heads:
                raise ConfigError(f"{where}: no 'head_dim' and hidden_size {hidden} is not divisible by "
                                  f"num_attention_heads {heads}")
            head_dim = hidden // heads
        else:
            head_dim = _typed(head_dim, "head_dim", int, where)

        act = d.get("hidden_act", "silu")
        if act != "silu":
            # the reference applies SiLU whatever the key says (minivllm/models/models/qwen3.py:119)
            raise ConfigError(f"{where}: hidden_act '{act}' is not supported; Qwen3's feed-forward uses 'silu'")
        scaling = d.get("rope_scaling")
        if scaling not in (None, {}):
            rtype = scaling.get("rope_type", scaling.get("type")) if isinstance(scaling, dict) else scaling
            if rtype not in (None, "default"):
                raise ConfigError(f"{where}: rope_scaling {scaling!r} is not supported (plain rotary "
                                  f"embedding with rope_theta only)")
        if "rope_parameters" in d and isinstance(d["rope_parameters"], dict):
            rp = d["rope_parameters"]
            if rp.get("rope_type", "default") != "default":
                raise ConfigError(f"{where}: rope_parameters {rp!r} is not supported")
            if "rope_theta" not in d and "rope_theta" in rp:
                d = dict(d, rope_theta=rp["rope_theta"])

        use_window = d.get("use_sliding_window", False)
        use_window = False if use_window is None else _typed(use_window, "use_sliding_window", bool, where)
        window = d.get("sliding_window")
        layers = _require(d, "num_hidden_layers", int, where)
        max_window_layers = d.get("max_window_layers")
        if use_window:
            if window is None:
                raise ConfigError(f"{where}: use_sliding_window is true but 'sliding_window' is missing")
            window = _typed(window, "sliding_window", int, where)
            if window < 1:
                raise ConfigError(f"{where}: sliding_window counts the keys a query sees, its own included, "
                                  f"and must be >= 1, got {window}")
            max_window_layers = layers if max_window_layers is None else _typed(
                max_window_layers, "max_window_layers", int, where)
        else:
            window = None if window is None else _typed(window, "sliding_window", int, where)
            max_window_layers = layers if max_window_layers is None else _typed(
                max_window_layers, "max_window_layers", int, where)

        dtype = d.get("dtype", d.get("torch_dtype", "bfloat16"))
        if dtype is None:
            dtype = "bfloat16"
        if str(dtype) not in _DTYPE_NAMES:
            raise ConfigError(f"{where}: unknown dtype {dtype!r}")
        dtype = _DTYPE_NAMES[str(dtype)]

        eos = d.get("eos_token_id")
        if eos is None:
            eos_ids: Tuple[int, ...] = ()
        elif isinstance(eos, int) and not isinstance(eos, bool):
            eos_ids = (eos,)
        elif isinstance(eos, (list, tuple)) and all(isinstance(e, int) for e in eos):
            eos_ids = tuple(eos)
        else:
            raise ConfigError(f"{where}: eos_token_id must be an integer or a list of integers, got {eos!r}")
        bos = d.get("bos_token_id")

        cfg = cls(
            vocab_size=_require(d, "vocab_size", int, where),
            hidden_size=hidden,
            num_hidden_layers=layers,
            num_attention_heads=heads,
            num_key_value_heads=kv_heads,
            head_dim=head_dim,
            intermediate_size=_require(d, "intermediate_size", int, where),
            max_position_embeddings=_require(d, "max_position_embeddings", int, where),
            rms_norm_eps=_typed(d.get("rms_norm_eps", 1e-6), "rms_norm_eps", float, where),
            rope_theta=_typed(d.get("rope_theta", 10000.0), "rope_theta", float, where),
            attention_bias=_typed(d.get("attention_bias", False) or False, "attention_bias", bool, where),
            tie_word_embeddings=_typed(d.get("tie_word_embeddings", False) or False,
                                       "tie_word_embeddings", bool, where),
            use_sliding_window=use_window,
            sliding_window=window,
            max_window_layers=max_window_layers,
            dtype=dtype,
            eos_token_ids=eos_ids,
            bos_token_id=bos if isinstance(bos, int) else None,
        )
        cfg.validate(where)
        return cfg

    def validate(self, where: str = "config") -> None:
        for name in ("vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads",
                     "num_key_value_heads", "head_dim", "intermediate_size", "max_position_embeddings"):
            if getattr(self, name) <= 0:
                raise ConfigError(f"{where}: {name} must be positive, got {getattr(self, name)}")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(f"{where}: num_attention_heads {self.num_attention_heads} is not a multiple of "
                              f"num_key_value_heads {self.num_key_value_heads}")
        if self.head_dim % 2:
            raise ConfigError(f"{where}: head_dim {self.head_dim} must be even for the rotary embedding")
        if self.rms_norm_eps <= 0:
            raise ConfigError(f"{where}: rms_norm_eps must be positive, got {self.rms_norm_eps}")
        if self.rope_theta <= 0:
            raise ConfigError(f"{where}: rope_theta must be positive, got {self.rope_theta}")

    def to_dict(self) -> Dict[str, Any]:
        eos: Any
        if len(self.eos_token_ids) == 0:
            eos = None
        elif len(self.eos_token_ids) == 1:
            eos = self.eos_token_ids[0]
        else:
            eos = list(self.eos_token_ids)
        return {
            "architectures": [self.architecture],
            "model_type": "qwen3",
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "intermediate_size": self.intermediate_size,
            "max_position_embeddings": self.max_position_embeddings,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "rope_scaling": None,
            "hidden_act": "silu",
            "attention_bias": self.attention_bias,
            "tie_word_embeddings": self.tie_word_embeddings,
            "use_sliding_window": self.use_sliding_window,
            "sliding_window": self.sliding_window,
            "max_window_layers": self.max_window_layers,
            "torch_dtype": self.dtype,
            "eos_token_id": eos,
            "bos_token_id": self.bos_token_id,
        }


def read_config_json(model_dir: str) -> Dict[str, Any]:
    path = os.path.join(model_dir, "config.json")
    if not os.path.isdir(model_dir):
        raise ConfigError(f"model path {model_dir!r} is not a directory")
    if not os.path.isfile(path):
        raise ConfigError(f"{model_dir!r} holds no config.json")
    with open(path, "r", encoding="utf-8") as f:
        d = json.load(f)
    if not isinstance(d, dict):
        raise ConfigError(f"{path}: top level is not an object")
    return d


def architecture_name(d: Dict[str, Any], where: str = "config.json") -> str:
    """``architectures[0]``, the key the reference selects the model class by
    (minivllm/models/loader.py:10)."""
    archs = d.get("architectures")
    if not isinstance(archs, (list, tuple)) or not archs or not isinstance(archs[0], str):
        raise ConfigError(f"{where}: 'architectures' must be a non-empty list of names")
    return archs[0]
