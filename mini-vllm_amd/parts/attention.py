"""Softmax attention over the paged cache, with grouped key/value heads.

Reference: minivllm/models/models/qwen3.py:26-101 (projection, per-head q/k norm before the
rotary embedding, output projection) and minivllm/models/layers/attention.py:46-92 (cache
write, then causal attention over the request's keys). ``scale`` is head_dim^-0.5
(qwen3.py:32). ``window`` is the number of tokens to the left of a query that it sees besides
itself (attention.py:56-60); None sees all.

Every size is a parameter of the spec. q, k and v are packed into one matrix product; the
per-head norms, the rotary embedding and the cache write are one kernel.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Optional

import torch

from .base import CacheNeed, KeepAll, KeepWindow, KeyValueNeed, Mixer, PartSpec, Runtime, TensorDecl, register_mixer


@dataclass(frozen=True)
class AttentionSpec(PartSpec):
    kind = "attention"
    hidden_size: int = 0
    num_heads: int = 0
    num_kv_heads: int = 0
    head_dim: int = 0
    scale: float = 1.0
    qk_norm: bool = False
    qk_norm_eps: float = 1e-6
    bias: bool = False
    window: Optional[int] = None
    position: Optional[PartSpec] = None
    shares_kv: bool = False        # no k/v of its own: reads the cache of the call named by the plan

    @property
    def q_dim(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def kv_dim(self) -> int:
        return self.num_kv_heads * self.head_dim


@register_mixer(AttentionSpec.kind)
class Attention(Mixer):
    spec_class = AttentionSpec
    accepts_pending_norm = True      # the input is used by one packed product only
    accepts_fold = True              # the output comes from one product

    @classmethod
    def tensors(cls, spec: AttentionSpec) -> Dict[str, TensorDecl]:
        t = {"q": TensorDecl((spec.q_dim, spec.hidden_size)), "o": TensorDecl((spec.hidden_size, spec.q_dim))}
        if not spec.shares_kv:
            t["k"] = TensorDecl((spec.kv_dim, spec.hidden_size))
            t["v"] = TensorDecl((spec.kv_dim, spec.hidden_size))
        if spec.bias:
            t["q_bias"] = TensorDecl((spec.q_dim,), init="zeros_normal")
            t["o_bias"] = TensorDecl((spec.hidden_size,), init="zeros_normal")
            if not spec.shares_kv:
                t["k_bias"] = TensorDecl((spec.kv_dim,), init="zeros_normal")
                t["v_bias"] = TensorDecl((spec.kv_dim,), init="zeros_normal")
        if spec.qk_norm:
            t["q_norm"] = TensorDecl((spec.head_dim,), init="ones_normal")
            if not spec.shares_kv:
                t["k_norm"] = TensorDecl((spec.head_dim,), init="ones_normal")
        return t

    @classmethod
    def cache_need(cls, spec: AttentionSpec) -> Optional[CacheNeed]:
        if spec.shares_kv:
            return None
        return KeyValueNeed(retention=KeepAll() if spec.window is None else KeepWindow(spec.window),
                            num_kv_heads=spec.num_kv_heads, head_dim=spec.head_dim)

    def __init__(self, spec: AttentionSpec, tensors: Dict[str, torch.Tensor], rt: Runtime,
                 position: Optional[object] = None):
        if spec.num_heads % spec.num_kv_heads:
            raise ValueError(f"{spec.num_heads} query heads are not a multiple of {spec.num_kv_heads} kv heads")
        self.spec = spec
        self.rt = rt
        parts = ["q"] if spec.shares_kv else ["q", "k", "v"]
        dtypes = {tensors[p].dtype for p in parts}
        if len(dtypes) != 1:
            raise ValueError(f"q, k and v projections are stored in different dtypes {dtypes}; cannot pack them")
        self.w_qkv = tensors["q"] if spec.shares_kv else torch.cat([tensors[p] for p in parts], dim=0).contiguous()
        self.b_qkv = None
        self.b_o = None
        if spec.bias:
            self.b_qkv = tensors["q_bias"] if spec.shares_kv else torch.cat(
                [tensors[p + "_bias"] for p in parts], dim=0).contiguous()
            self.b_o = tensors["o_bias"]
        self.w_o = tensors["o"]
        self.q_norm = tensors.get("q_norm")
        self.k_norm = tensors.get("k_norm")
        self.position = position
        self.rotary = position.rotary() if position is not None else None
        if position is not None and self.rotary is None and not hasattr(position, "apply"):
            raise ValueError("a position encoding must offer rotary() or apply()")
        self.width = spec.q_dim + (0 if spec.shares_kv else 2 * spec.kv_dim)

    def first_product(self):
        return self.w_qkv.shape[0], self.w_qkv.shape[1], False

    def forward(self, x: torch.Tensor, ctx, call: int, fold=None) -> torch.Tensor:
        spec, rt, ops = self.spec, self.rt, self.rt.ops
        n = x.shape[0]
        ws = rt.workspace
        qkv = ws.get("attn.qkv", (n, self.width), rt.dtype)
        ops.gemm(x, self.w_qkv, qkv, self.b_qkv)
        kv = ctx.kv(call)
        table, interleaved = (self.rotary if self.rotary is not None else (None, False))
        if self.position is not None and self.rotary is None:
            q3 = qkv[:, :spec.q_dim].unflatten(1, (spec.num_heads, spec.head_dim))
            k3 = None if spec.shares_kv else qkv[:, spec.q_dim:spec.q_dim + spec.kv_dim].unflatten(
                1, (spec.num_kv_heads, spec.head_dim))
            if spec.qk_norm:
                raise NotImplementedError("a position encoding without a rotary table cannot follow the fused "
                                          "q/k norm; give it a table or leave qk_norm off")
            self.position.apply(q3, k3, ctx)
        attn = ws.get("attn.out", (n, spec.q_dim), rt.dtype)
        plan = ctx.attention_plan
        if plan is not None and plan.decode_only:
            # a decode step: norm, rotation, cache write and attention in one kernel where it is taken
            if ops.attention_decode_fused(qkv, attn, kv.k_pages, kv.v_pages, kv.block_table, kv.page_size,
                                          ctx.positions, ctx.token_seq, spec.num_heads, spec.num_kv_heads,
                                          spec.head_dim, spec.scale, spec.window, plan, self.q_norm, self.k_norm,
                                          spec.qk_norm_eps, table, interleaved, not spec.shares_kv,
                                          rope_rows=ctx.position_rows.get(self.position)):
                y = ws.get("mixer.out", (n, spec.hidden_size), rt.dtype)
                return ops.gemm(attn, self.w_o, y, self.b_o, defer_sum=True, fold=fold) or y
        ops.qk_norm_rope_store(
            qkv, spec.num_heads, spec.num_kv_heads, spec.head_dim, ctx.positions, ctx.token_seq,
            self.q_norm, self.k_norm, spec.qk_norm_eps, table, interleaved,
            None if spec.shares_kv else kv.k_pages, None if spec.shares_kv else kv.v_pages,
            None if spec.shares_kv else kv.block_table, kv.page_size)
        ops.attention(qkv[:, :spec.q_dim] if self.width != spec.q_dim else qkv, attn, kv.k_pages, kv.v_pages,
                      kv.block_table, kv.page_size, ctx.positions, ctx.token_seq, spec.num_heads,
                      spec.num_kv_heads, spec.head_dim, spec.scale, spec.window, plan=ctx.attention_plan)
        y = ws.get("mixer.out", (n, spec.hidden_size), rt.dtype)
        # (the sums of a product whose K was split may be left to the next norm)
        return ops.gemm(attn, self.w_o, y, self.b_o, defer_sum=True, fold=fold) or y
