"""Qwen3 dense decoder as a plan of parts.

Reference: minivllm/models/models/qwen3.py. Per layer: RMSNorm -> attention (packed q/k/v
projection, per-head q and k RMSNorm with one weight of head_dim shared by all heads, rotary
embedding over the whole head, grouped key/value heads, scale head_dim^-0.5, causal) ->
residual; RMSNorm -> SwiGLU feed-forward -> residual (qwen3.py:26-156). Then the final
RMSNorm and the output head, which shares the embedding table when ``tie_word_embeddings``
is set (qwen3.py:176,201-204).

Tensor names on disk are the reference's parameter names before packing (qwen3.py:223-245):
``model.embed_tokens.weight``, ``model.layers.{i}.input_layernorm.weight``,
``model.layers.{i}.self_attn.{q,k,v,o}_proj.{weight,bias}``,
``model.layers.{i}.self_attn.{q,k}_norm.weight``,
``model.layers.{i}.post_attention_layernorm.weight``,
``model.layers.{i}.mlp.{gate,up,down}_proj.weight``, ``model.norm.weight``, ``lm_head.weight``.
"""
from __future__ import annotations

from typing import FrozenSet

from ..config.model_config import Qwen3Config
from ..parts.attention import AttentionSpec
from ..parts.block import PreNormBlockSpec
from ..parts.mlp import SwiGLUSpec
from ..parts.norm import RMSNormSpec
from ..parts.plan import Call, EmbeddingSpec, HeadSpec, LayerPlan, ModelPlan, TensorLocation
from ..parts.rope import RotarySpec
from .registry import Architecture, register_architecture


def qwen3_plan(config: Qwen3Config) -> ModelPlan:
    rope = RotarySpec(rotary_dim=config.head_dim, theta=config.rope_theta, interleaved=False)
    block_norm = RMSNormSpec(size=config.hidden_size, eps=config.rms_norm_eps)
    layers = []
    for i in range(config.num_hidden_layers):
        attention = AttentionSpec(
            hidden_size=config.hidden_size,
            num_heads=config.num_attention_heads,
            num_kv_heads=config.num_key_value_heads,
            head_dim=config.head_dim,
            scale=config.head_dim ** -0.5,
            qk_norm=True,
            qk_norm_eps=config.rms_norm_eps,
            bias=config.attention_bias,
            window=config.layer_window(i),
            position=rope,
        )
        ffn = SwiGLUSpec(hidden_size=config.hidden_size, intermediate_size=config.intermediate_size)
        layers.append(LayerPlan(block=PreNormBlockSpec(), mixer=attention, ffn=ffn,
                                norms=(("mixer", block_norm), ("ffn", block_norm))))
    plan = ModelPlan(
        hidden_size=config.hidden_size,
        vocab_size=config.vocab_size,
        max_positions=config.max_position_embeddings,
        embedding=EmbeddingSpec(vocab_size=config.vocab_size, hidden_size=config.hidden_size, scale=1.0),
        layers=tuple(layers),
        calls=tuple(Call(layer=i) for i in range(config.num_hidden_layers)),
        final_norm=block_norm,
        head=HeadSpec(vocab_size=config.vocab_size, hidden_size=config.hidden_size,
                      tied=config.tie_word_embeddings),
    )
    plan.validate()
    return plan


_ATTENTION_NAMES = {
    "q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "o": "o_proj.weight",
    "q_bias": "q_proj.bias", "k_bias": "k_proj.bias", "v_bias": "v_proj.bias", "o_bias": "o_proj.bias",
    "q_norm": "q_norm.weight", "k_norm": "k_norm.weight",
}
_MLP_NAMES = {"gate": "gate_proj.weight", "up": "up_proj.weight", "down": "down_proj.weight"}
_NORM_NAMES = {"norm.mixer": "input_layernorm", "norm.ffn": "post_attention_layernorm"}


def qwen3_tensor_name(config: Qwen3Config, loc: TensorLocation) -> str:
    if loc.layer is None:
        if loc.role == "embedding":
            return "model.embed_tokens.weight"
        if loc.role == "final_norm":
            return "model.norm.weight"
        if loc.role == "head":
            return "model.embed_tokens.weight" if config.tie_word_embeddings else "lm_head.weight"
        raise KeyError(loc)
    prefix = f"model.layers.{loc.layer}."
    if loc.role == "mixer":
        return prefix + "self_attn." + _ATTENTION_NAMES[loc.name]
    if loc.role == "ffn":
        return prefix + "mlp." + _MLP_NAMES[loc.name]
    if loc.role in _NORM_NAMES:
        return prefix + _NORM_NAMES[loc.role] + "." + loc.name
    raise KeyError(loc)


def qwen3_ignorable(config: Qwen3Config) -> FrozenSet[str]:
    # a tied model may still store its head; the reference skips it (qwen3.py:231-232)
    return frozenset({"lm_head.weight"}) if config.tie_word_embeddings else frozenset()


QWEN3 = register_architecture(Architecture(
    name=Qwen3Config.architecture,
    config_class=Qwen3Config,
    plan=qwen3_plan,
    tensor_name=qwen3_tensor_name,
    ignorable=qwen3_ignorable,
))
