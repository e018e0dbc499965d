"""Block arrangements: how a layer's norms, mixer and feed-forward are wired.

Reference: minivllm/models/models/qwen3.py:141-156 — norm before the mixer, residual add,
norm before the feed-forward, residual add; nothing after either.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Optional, Tuple

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

    accepts_next_norm = True

    def entry_norm(self) -> Norm:
        return self.norm_mixer

    def entry_part(self):
        return self.mixer

    def forward(self, stream: HiddenStream, ctx, call: int, next_norm: Optional[Norm] = None, next_part=None) -> None:
        # a part that starts with one matrix product over its input may get the norm unrun, to
        # fuse it into that product; a part that ends with one may be offered the add and the norm
        # that follow it, to fold them into that product, when the part behind that norm can go on
        # from rows that are not yet divided by their root mean square
        self._run(stream, ctx, self.norm_mixer, self.mixer, self.norm_ffn, self.ffn, (call,))
        self._run(stream, ctx, self.norm_ffn, self.ffn, next_norm, next_part, ())

    @staticmethod
    def _run(stream: HiddenStream, ctx, norm: Norm, part, norm_after: Optional[Norm], part_after, extra: tuple) -> None:
        defer = getattr(part, "accepts_pending_norm", False)
        h = norm.pending(stream, ctx) if defer else norm.forward(stream, ctx)
        fold = None
        if norm_after is not None and getattr(part, "accepts_fold", False) \
                and getattr(part_after, "accepts_pending_norm", False):
            make = getattr(norm_after, "fold", None)
            first = getattr(part_after, "first_product", None)
            if make is not None and first is not None:
                fold = make(stream, ctx, first())
        out = part.forward(h, ctx, *extra, fold=fold) if fold is not None else part.forward(h, ctx, *extra)
        if getattr(out, "is_weighted_rows", False):
            stream.delta, stream.weighted = None, out      # already added to the residual
        else:
            stream.delta = out
