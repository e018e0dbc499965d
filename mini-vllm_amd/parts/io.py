"""The two ends of the model: token embedding and output head.

Reference: minivllm/models/models/qwen3.py:165,184 (``nn.Embedding``, no scaling) and
qwen3.py:201-204,219 (``lm_head``: a bias-free linear map over the rows whose logits are wanted,
sharing the embedding's table when ``tie_word_embeddings``). Logits are float32 here (the
reference keeps them in the model's dtype).

Both are parts like the others: a spec with the sizes and constants, a class registered under the
spec's kind. A head that scales or caps its logits, or an embedding with a learned offset, is
another registered class; the model code does not change.
"""
from __future__ import annotations

from typing import Dict

import torch

from .base import Embedding, Head, Runtime, TensorDecl, register_embedding, register_head
from .plan import EmbeddingSpec, HeadSpec


@register_embedding(EmbeddingSpec.kind)
class TokenEmbedding(Embedding):
    spec_class = EmbeddingSpec
    carries_gather = True

    @classmethod
    def tensors(cls, spec: EmbeddingSpec) -> Dict[str, TensorDecl]:
        return {"weight": TensorDecl((spec.vocab_size, spec.hidden_size))}

    def __init__(self, spec: EmbeddingSpec, tensors: Dict[str, torch.Tensor], rt: Runtime):
        self.spec, self.rt = spec, rt
        self.table = tensors["weight"]

    def forward(self, ctx, resid: torch.Tensor, gather=None) -> None:
        self.rt.ops.embedding(ctx.token_ids, self.table, resid, self.spec.scale, gather=gather)


@register_head(HeadSpec.kind)
class LinearHead(Head):
    spec_class = HeadSpec

    @classmethod
    def tensors(cls, spec: HeadSpec) -> Dict[str, TensorDecl]:
        return {"weight": TensorDecl((spec.vocab_size, spec.hidden_size))}

    def __init__(self, spec: HeadSpec, tensors: Dict[str, torch.Tensor], rt: Runtime):
        self.spec, self.rt = spec, rt
        self.weight = tensors["weight"]

    def forward(self, h: torch.Tensor, ctx) -> torch.Tensor:
        logits = self.rt.workspace.get("logits", (h.shape[0], self.spec.vocab_size), torch.float32)
        self.rt.ops.gemm(h, self.weight, logits)
        return logits
