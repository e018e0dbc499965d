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

from .base import HiddenStream, Norm, NormFold, PartSpec, PendingNorm, Runtime, TensorDecl, register_norm


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
        taken = self._take_weighted(stream)
        if taken is not None:
            if rows is not None:
                raise RuntimeError("rows left half normalised for a norm that wants only some of them")
            return taken.materialize()
        n = stream.resid.shape[0] if rows is None else rows.numel()
        out = self.rt.workspace.get(tag, (n, self.spec.size), self.rt.dtype)
        self.rt.ops.add_rmsnorm(stream.resid, stream.delta, self.weight, self.spec.eps, out, rows=rows,
                                unit_offset=self.spec.unit_offset)
        if rows is None:
            stream.delta = None
        return out

    def _take_weighted(self, stream: HiddenStream):
        """The rows the product in front left half normalised for this norm (``fold``), if any."""
        taken = stream.weighted
        if taken is None:
            return None
        stream.weighted = None
        if taken.norm is not self or stream.delta is not None:
            raise RuntimeError("the stream holds rows that were prepared for another norm")
        return taken

    def fold(self, stream: HiddenStream, ctx, consumer=None) -> Optional[NormFold]:
        """The residual add and this norm, offered to the product in front of them, for steps of more
        rows than the fused add + norm + product kernel takes. ``consumer``: the product that comes
        behind the norm, (weight rows, weight columns, gated); without it, or when the kernels would
        not take that product from half-normalised rows, nothing is offered."""
        n, size = stream.resid.shape[0], self.spec.size
        if consumer is None or consumer[1] != size or not self.rt.ops.can_fold_norm(n, size, consumer):
            return None
        ws = self.rt.workspace
        return NormFold(self, stream, self.weight, self.spec.eps, self.spec.unit_offset,
                        ws.get("fold.weighted", (n, size), self.rt.dtype),
                        ws.get("fold.partial", (n * ((size + 3) // 4),), torch.float32),
                        ws.get("normed", (n, size), self.rt.dtype))

    def pending(self, stream: HiddenStream, ctx):
        """Deferred when the step is small enough for the fused add + norm + product kernel; rows that
        the product in front left half normalised go on as they are."""
        taken = self._take_weighted(stream)
        if taken is not None:
            return taken
        if stream.spare is not None and self.rt.ops.can_fuse_norm(stream.resid.shape[0], self.spec.size):
            return PendingNorm(self, stream, ctx)
        return self.forward(stream, ctx)

    def as_scaled_rms(self):
        return self.weight, self.spec.eps, self.spec.unit_offset

    def apply(self, x: torch.Tensor, out: torch.Tensor) -> None:
        self.rt.ops.rmsnorm(x, self.weight, self.spec.eps, out, unit_offset=self.spec.unit_offset)
