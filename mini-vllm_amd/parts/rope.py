"""Rotary position embedding.

Reference: minivllm/models/layers/rotary.py. The table is ``cat(cos, sin)`` of
``position * inv_freq`` with ``inv_freq_i = 1 / theta^(2i / rotary_dim)``, all float32
(rotary.py:35-46); the rotation pairs element i with i + rotary_dim/2 (rotary.py:11-14) and
is computed in float32. ``inv_freq`` is evaluated here by the same float32 expression, the
angles and their cosines and sines by a kernel; the rotation itself is fused into the
attention's q/k kernel, which takes the table from ``rotary()``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Optional, Tuple

import torch

from .base import PartSpec, PositionEncoding, Runtime, register_position_encoding


@dataclass(frozen=True)
class RotarySpec(PartSpec):
    kind = "rotary"
    rotary_dim: int = 0
    theta: float = 10000.0
    interleaved: bool = False      # pairs (2i, 2i+1) instead of (i, i + rotary_dim/2)


def inverse_frequencies(rotary_dim: int, theta: float) -> torch.Tensor:
    """float32 [rotary_dim / 2], evaluated as the reference does (rotary.py:35)."""
    return 1.0 / (theta ** (torch.arange(0, rotary_dim, 2, dtype=torch.float) / rotary_dim))


@register_position_encoding(RotarySpec.kind)
class RotaryEmbedding(PositionEncoding):
    spec_class = RotarySpec

    def __init__(self, spec: RotarySpec, tensors: Dict[str, torch.Tensor], rt: Runtime):
        if spec.rotary_dim <= 0 or spec.rotary_dim % 2:
            raise ValueError(f"rotary_dim must be positive and even, got {spec.rotary_dim}")
        self.spec = spec
        self.rt = rt
        inv_freq = inverse_frequencies(spec.rotary_dim, spec.theta).to(rt.device)
        self.table = rt.ops.rope_table(inv_freq, rt.max_positions)

    def rotary(self) -> Optional[Tuple[torch.Tensor, bool]]:
        return self.table, self.spec.interleaved

    def step_gather(self, ctx):
        """In a step of single decoded tokens every layer needs the table's rows at the same few
        positions: they are gathered once, in front of the layers, so that no layer has to wait for a
        position before it can ask for its angles."""
        plan = ctx.attention_plan
        if plan is None or not plan.decode_only or self.spec.interleaved or not self.rt.ops.use_fast_kernels:
            return None
        rows = self.rt.workspace.get(f"rotary.rows.{self.spec.rotary_dim}.{self.spec.theta}",
                                     (ctx.n_tokens, self.spec.rotary_dim), torch.float32)
        ctx.position_rows[self] = rows
        return ctx.positions, self.table, rows
