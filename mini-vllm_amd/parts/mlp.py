"""Gated feed-forward: y = (silu(x Wg^T) * (x Wu^T)) Wd^T.

Reference: minivllm/models/models/qwen3.py:104-121 — three bias-free projections, SiLU on the
gate. Gate and up are packed into one matrix product here; the activation and the product
are computed in float32.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict

import torch

from .base import FeedForward, PartSpec, Runtime, TensorDecl, register_feed_forward


@dataclass(frozen=True)
class SwiGLUSpec(PartSpec):
    kind = "swiglu"
    hidden_size: int = 0
    intermediate_size: int = 0


@register_feed_forward(SwiGLUSpec.kind)
class SwiGLU(FeedForward):
    spec_class = SwiGLUSpec
    accepts_pending_norm = True      # the input is used by one packed product only
    accepts_fold = True              # the output comes from one product

    @classmethod
    def tensors(cls, spec: SwiGLUSpec) -> Dict[str, TensorDecl]:
        return {"gate": TensorDecl((spec.intermediate_size, spec.hidden_size)),
                "up": TensorDecl((spec.intermediate_size, spec.hidden_size)),
                "down": TensorDecl((spec.hidden_size, spec.intermediate_size))}

    def __init__(self, spec: SwiGLUSpec, tensors: Dict[str, torch.Tensor], rt: Runtime):
        self.spec = spec
        self.rt = rt
        if tensors["gate"].dtype != tensors["up"].dtype:
            raise ValueError("gate and up projections are stored in different dtypes; cannot pack them")
        self.w_gate_up = torch.cat([tensors["gate"], tensors["up"]], dim=0).contiguous()
        self.w_down = tensors["down"]

    def first_product(self):
        return self.w_gate_up.shape[0], self.w_gate_up.shape[1], True

    def forward(self, x: torch.Tensor, ctx, fold=None) -> torch.Tensor:
        spec, rt, ops = self.spec, self.rt, self.rt.ops
        n = x.shape[0]
        act = rt.workspace.get("ffn.act", (n, spec.intermediate_size), rt.dtype)
        if not ops.gemm_swiglu(x, self.w_gate_up, act):      # one pass over the weight for few rows
            gu = rt.workspace.get("ffn.gate_up", (n, 2 * spec.intermediate_size), rt.dtype)
            if not isinstance(x, torch.Tensor):
                x = x.materialize()
            ops.gemm(x, self.w_gate_up, gu)
            ops.swiglu(gu, act)
        y = rt.workspace.get("ffn.out", (n, spec.hidden_size), rt.dtype)
        # (the sums of a product whose K was split may be left to the next norm, or the residual add and
        # that norm folded into the product)
        return ops.gemm(act, self.w_down, y, defer_sum=True, fold=fold) or y
