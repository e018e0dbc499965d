"""RMS normalisation.

Reference: the block norms, the per-head q/k norms and the final norm are ``nn.RMSNorm`` with
``eps = rms_norm_eps`` (minivllm/models/models/qwen3.py:64-65,134-139,176); the intended
numerics are spelled out in the file's own class (qwen3.py:18-23): mean of squares and the
scaling in float32, the weight multiplies. Here the sum, the scaling and the weight product
are float32 and the result is rounded once.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Optional

import torch

from .base import HiddenStream, Norm, PartSpec, PendingNorm, Runtime, TensorDecl, register_norm


@dataclass(frozen=True)
class RMSNormSpec(PartSpec):
    kind = "rmsnorm"
    size: int = 0
    eps: float = 1e-6
    unit_offset: bool = False      # weight is (1 + w) instead of w


@register_norm(RMSNormSpec.kind)
class RMSNorm(Norm):
    spec_class = RMSNormSpec

    @classmethod
    def tensors(cls, spec: RMSNormSpec) -> Dict[str, TensorDecl]:
        return {"weight": TensorDecl((spec.size,), init="zeros_normal" if spec.unit_offset else "ones_normal")}

    def __init__(self, spec: RMSNormSpec, tensors: Dict[str, torch.Tensor], rt: Runtime):
        self.spec = spec
        self.rt = rt
        self.weight = tensors["weight"]

    def forward(self, stream: HiddenStream, ctx, rows: Optional[torch.Tensor] = None,
                tag: str = "normed") -> torch.Tensor:
        n = stream.resid.shape[0] if rows is None else rows.numel()
        out = self.rt.workspace.get(tag, (n, self.spec.size), self.rt.dtype)
        self.rt.ops.add_rmsnorm(stream.resid, stream.delta, self.weight, self.spec.eps, out, rows=rows,
                                unit_offset=self.spec.unit_offset)
        if rows is None:
            stream.delta = None
        return out

    def pending(self, stream: HiddenStream, ctx):
        """Deferred when the step is small enough for the fused add + norm + product kernel."""
        if stream.spare is not None and self.rt.ops.can_fuse_norm(stream.resid.shape[0], self.spec.size):
            return PendingNorm(self, stream, ctx)
        return self.forward(stream, ctx)

    def as_scaled_rms(self):
        return self.weight, self.spec.eps, self.spec.unit_offset

    def apply(self, x: torch.Tensor, out: torch.Tensor) -> None:
        self.rt.ops.rmsnorm(x, self.weight, self.spec.eps, out, unit_offset=self.spec.unit_offset)
