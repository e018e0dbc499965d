"""Block arrangements: how a layer's norms, mixer and feed-forward are wired.

Reference: minivllm/models/models/qwen3.py:141-156 — norm before the mixer, residual add,
norm before the feed-forward, residual add; nothing after either.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Tuple

from .base import Block, FeedForward, HiddenStream, Mixer, Norm, PartSpec, register_block


@dataclass(frozen=True)
class PreNormBlockSpec(PartSpec):
    kind = "pre_norm"


@register_block(PreNormBlockSpec.kind)
class PreNormBlock(Block):
    """x = x + mixer(norm_mixer(x)); x = x + ffn(norm_ffn(x)). Each residual add is deferred
    into the next norm's kernel through the stream's pending delta."""
    norm_slots: Tuple[str, ...] = ("mixer", "ffn")

    def __init__(self, spec: PreNormBlockSpec, norms: Dict[str, Norm], mixer: Mixer, ffn: FeedForward):
        self.norm_mixer = norms["mixer"]
        self.norm_ffn = norms["ffn"]
        self.mixer = mixer
        self.ffn = ffn

    def forward(self, stream: HiddenStream, ctx, call: int) -> None:
        # a part that starts with one matrix product over its input may get the norm unrun, to
        # fuse it into that product
        defer = getattr(self.mixer, "accepts_pending_norm", False)
        h = self.norm_mixer.pending(stream, ctx) if defer else self.norm_mixer.forward(stream, ctx)
        stream.delta = self.mixer.forward(h, ctx, call)
        defer = getattr(self.ffn, "accepts_pending_norm", False)
        h = self.norm_ffn.pending(stream, ctx) if defer else self.norm_ffn.forward(stream, ctx)
        stream.delta = self.ffn.forward(h, ctx)
