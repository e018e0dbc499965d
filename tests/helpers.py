"""Shared by the tests: tiny Qwen3 configurations, random weights by on-disk name (made here,
not by the engine), model folders in temporary places, and comparisons."""
from __future__ import annotations

import copy
import json
import os
from typing import Dict, List, Optional

import numpy as np
import torch

from plain import qwen3_plain as plain

# Three tiny configurations that differ in every size and option.
TINY_A = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3",
    "num_hidden_layers": 2, "hidden_size": 64, "num_attention_heads": 4, "num_key_value_heads": 2,
    "head_dim": 16, "intermediate_size": 128, "vocab_size": 256, "max_position_embeddings": 1024,
    "rope_theta": 10000.0, "rms_norm_eps": 1e-6, "tie_word_embeddings": True, "attention_bias": False,
    "use_sliding_window": False, "sliding_window": None, "max_window_layers": 2,
    "hidden_act": "silu", "torch_dtype": "float32", "eos_token_id": 7,
}
TINY_B = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3",
    "num_hidden_layers": 3, "hidden_size": 96, "num_attention_heads": 8, "num_key_value_heads": 2,
    "head_dim": 32, "intermediate_size": 168, "vocab_size": 391, "max_position_embeddings": 2048,
    "rope_theta": 1000000.0, "rms_norm_eps": 1e-5, "tie_word_embeddings": False, "attention_bias": True,
    "use_sliding_window": True, "sliding_window": 21, "max_window_layers": 1,
    "hidden_act": "silu", "torch_dtype": "bfloat16", "eos_token_id": [3, 5],
}
TINY_C = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3",
    "num_hidden_layers": 1, "hidden_size": 80, "num_attention_heads": 6, "num_key_value_heads": 3,
    "head_dim": 48, "intermediate_size": 112, "vocab_size": 300, "max_position_embeddings": 512,
    "rope_theta": 50000.0, "rms_norm_eps": 3e-6, "tie_word_embeddings": False, "attention_bias": False,
    "hidden_act": "silu", "torch_dtype": "bfloat16", "eos_token_id": 1,
}
# The second tiny configuration exactly as the benchmark description states it: no bias and no
# window, so every layer keeps all keys and prefix reuse can be on (cache pages of 8, portions of 7).
TINY_B0 = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3",
    "num_hidden_layers": 3, "hidden_size": 96, "num_attention_heads": 8, "num_key_value_heads": 2,
    "head_dim": 32, "intermediate_size": 160, "vocab_size": 384, "max_position_embeddings": 2048,
    "rope_theta": 1000000.0, "rms_norm_eps": 1e-5, "tie_word_embeddings": False, "attention_bias": False,
    "hidden_act": "silu", "torch_dtype": "float32", "eos_token_id": 2,
}
# Head sizes the MFMA attention kernels serve (128 and 64), widths the MFMA products serve.
TINY_D128 = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3",
    "num_hidden_layers": 2, "hidden_size": 256, "num_attention_heads": 4, "num_key_value_heads": 2,
    "head_dim": 128, "intermediate_size": 512, "vocab_size": 1000, "max_position_embeddings": 4096,
    "rope_theta": 1000000.0, "rms_norm_eps": 1e-6, "tie_word_embeddings": True, "attention_bias": False,
    "hidden_act": "silu", "torch_dtype": "bfloat16", "eos_token_id": 0,
}
TINY_D64 = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3",
    "num_hidden_layers": 3, "hidden_size": 192, "num_attention_heads": 6, "num_key_value_heads": 1,
    "head_dim": 64, "intermediate_size": 320, "vocab_size": 777, "max_position_embeddings": 4096,
    "rope_theta": 50000.0, "rms_norm_eps": 2e-6, "tie_word_embeddings": False, "attention_bias": True,
    "hidden_act": "silu", "torch_dtype": "bfloat16", "eos_token_id": 0,
}
# Head size 64 with a window shorter than the longest request, on the layers from the second on: in
# bfloat16 the MFMA attention kernels meet a window, pages that the window has given back and, in
# decode steps, the fused kernel with key splits under a window.
TINY_W64 = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3",
    "num_hidden_layers": 3, "hidden_size": 192, "num_attention_heads": 4, "num_key_value_heads": 2,
    "head_dim": 64, "intermediate_size": 256, "vocab_size": 515, "max_position_embeddings": 4096,
    "rope_theta": 200000.0, "rms_norm_eps": 4e-6, "tie_word_embeddings": True, "attention_bias": False,
    "use_sliding_window": True, "sliding_window": 38, "max_window_layers": 1,
    "hidden_act": "silu", "torch_dtype": "bfloat16", "eos_token_id": 0,
}
TINY = {"A": TINY_A, "B": TINY_B, "C": TINY_C, "B0": TINY_B0, "D128": TINY_D128, "D64": TINY_D64, "W64": TINY_W64}


def tensor_shapes(cfg: Dict) -> Dict[str, tuple]:
    """On-disk names and shapes of a Qwen3 checkpoint (reference parameter names,
    minivllm/models/models/qwen3.py:53-65,111-113,129-139,165,176,201)."""
    h, I, V = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    H, Hkv = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    d = cfg["head_dim"]
    shapes = {"model.embed_tokens.weight": (V, h), "model.norm.weight": (h,)}
    if not cfg["tie_word_embeddings"]:
        shapes["lm_head.weight"] = (V, h)
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        shapes[p + "input_layernorm.weight"] = (h,)
        shapes[p + "post_attention_layernorm.weight"] = (h,)
        shapes[p + "self_attn.q_proj.weight"] = (H * d, h)
        shapes[p + "self_attn.k_proj.weight"] = (Hkv * d, h)
        shapes[p + "self_attn.v_proj.weight"] = (Hkv * d, h)
        shapes[p + "self_attn.o_proj.weight"] = (h, H * d)
        if cfg.get("attention_bias"):
            shapes[p + "self_attn.q_proj.bias"] = (H * d,)
            shapes[p + "self_attn.k_proj.bias"] = (Hkv * d,)
            shapes[p + "self_attn.v_proj.bias"] = (Hkv * d,)
            shapes[p + "self_attn.o_proj.bias"] = (h,)
        shapes[p + "self_attn.q_norm.weight"] = (d,)
        shapes[p + "self_attn.k_norm.weight"] = (d,)
        shapes[p + "mlp.gate_proj.weight"] = (I, h)
        shapes[p + "mlp.up_proj.weight"] = (I, h)
        shapes[p + "mlp.down_proj.weight"] = (h, I)
    return shapes


def make_weights(cfg: Dict, seed: int, stored: torch.dtype = torch.float32, std: float = 0.05,
                 qk_gain: float = 1.0) -> Dict[str, torch.Tensor]:
    """Random weights: matrices N(0, std), norm weights 1 + N(0, std), biases N(0, std).
    ``qk_gain`` multiplies the q/k norm weights, which sharpens the attention so that a wrong
    key shows in the logits. Values are rounded to ``stored`` (what the file will hold)."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        t = torch.randn(shape, generator=g, dtype=torch.float32) * std
        if name.endswith("norm.weight") or name.endswith("layernorm.weight"):
            t = t + 1.0
        if name.endswith("q_norm.weight") or name.endswith("k_norm.weight"):
            t = t * qk_gain
        out[name] = t.to(stored)
    return out


def write_model_dir(path: str, cfg: Dict, weights: Dict[str, torch.Tensor]) -> str:
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in weights.items()}, os.path.join(path, "model.safetensors"))
    return path


def plain_logits(cfg: Dict, weights: Dict[str, torch.Tensor], tokens: List[int], device=None) -> np.ndarray:
    return plain.forward(cfg, weights, tokens, dtype=torch.float64, device=device).numpy()


def random_tokens(cfg: Dict, n: int, seed: int) -> List[int]:
    rng = np.random.default_rng(seed)
    return [int(t) for t in rng.integers(0, cfg["vocab_size"], size=n)]


# error of `got` against `want`, relative to the largest wanted magnitude
def rel_err(got: np.ndarray, want: np.ndarray) -> float:
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, (got.shape, want.shape)
    assert np.isfinite(got).all(), "non-finite values in the result"
    return float(np.abs(got - want).max() / max(np.abs(want).max(), 1e-30))


def plain_logits_bf16(cfg: Dict, weights: Dict[str, torch.Tensor], tokens: List[int], device=None) -> np.ndarray:
    """The plain model with every stored activation rounded to bfloat16."""
    return plain.forward(cfg, weights, tokens, dtype=torch.float64, rnd=plain.round_to_bfloat16, device=device).numpy()


# Tolerance on rel_err of float32 logits against the float64 plain model.
TOL_F32 = 3e-5
# bfloat16: how far rounding moves the logits depends on the model and the input (sharp attention
# amplifies it). The bound is therefore taken from the case itself: the error that bfloat16
# storage alone causes in the plain model (plain_logits_bf16 against plain_logits), with a
# factor for the different order of roundings, plus a floor.
BF16_FACTOR = 1.5
BF16_FLOOR = 5e-3


def bf16_tolerance(emulation_error: float) -> float:
    return BF16_FACTOR * emulation_error + BF16_FLOOR


def plain_logits_f32(cfg: Dict, weights: Dict[str, torch.Tensor], tokens: List[int], device=None) -> np.ndarray:
    """The plain model evaluated in float32: how far 32-bit arithmetic alone moves the logits."""
    return plain.forward(cfg, weights, tokens, dtype=torch.float32, device=device).numpy()


def f32_tolerance(emulation_error: float) -> float:
    """For cases whose rows are ill-conditioned in 32-bit already (very sharp attention over thousands of
    keys: a score of 70 carries an absolute rounding error of 1e-5 into the exponent): the usual bound,
    or the plain model's own float32 error with the factor that bfloat16 gets, whichever is larger."""
    return max(TOL_F32, BF16_FACTOR * emulation_error)
