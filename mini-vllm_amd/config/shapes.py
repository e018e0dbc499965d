"""Named Qwen3 shapes for random-weights models: the sizes of the published Qwen3 dense models
(what their config.json files state) and a tiny one. Used by ``run.py --random-model`` and by the
benchmark; a shape is a dictionary of config.json keys that ``Qwen3Config.from_dict`` reads."""
from __future__ import annotations

from typing import Any, Dict

QWEN3_SHAPES: Dict[str, Dict[str, Any]] = {
    "tiny": dict(num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
                 intermediate_size=128, vocab_size=256, rope_theta=10000.0, rms_norm_eps=1e-6,
                 tie_word_embeddings=True),
    "0.6b": dict(num_hidden_layers=28, hidden_size=1024, num_attention_heads=16, num_key_value_heads=8, head_dim=128,
                 intermediate_size=3072, vocab_size=151936, rope_theta=1e6, rms_norm_eps=1e-6,
                 tie_word_embeddings=True),
    "8b": dict(num_hidden_layers=36, hidden_size=4096, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
               intermediate_size=12288, vocab_size=151936, rope_theta=1e6, rms_norm_eps=1e-6,
               tie_word_embeddings=False),
    "32b": dict(num_hidden_layers=64, hidden_size=5120, num_attention_heads=64, num_key_value_heads=8, head_dim=128,
                intermediate_size=25600, vocab_size=151936, rope_theta=1e6, rms_norm_eps=1e-6,
                tie_word_embeddings=False),
}


def named_shapes() -> Dict[str, Dict[str, Any]]:
    """Every named shape as a raw config.json dictionary, ``architectures`` included: the registry
    picks the architecture from it, as it does for a model folder. Another architecture's shapes are
    added here."""
    return {name: qwen3_shape(name) for name in QWEN3_SHAPES}


def named_shape(name: str, **overrides) -> Dict[str, Any]:
    shapes = named_shapes()
    if name not in shapes:
        raise KeyError(f"unknown shape {name!r} (known: {sorted(shapes)})")
    return dict(shapes[name], **overrides)


def qwen3_shape(name: str, **overrides) -> Dict[str, Any]:
    """The raw config dictionary of a named shape (``architectures`` and a position limit included)."""
    if name not in QWEN3_SHAPES:
        raise KeyError(f"unknown shape {name!r} (known: {sorted(QWEN3_SHAPES)})")
    raw = dict(QWEN3_SHAPES[name], architectures=["Qwen3ForCausalLM"], max_position_embeddings=40960)
    raw.update(overrides)
    return raw
