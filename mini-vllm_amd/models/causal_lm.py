"""A causal language model built from a ``ModelPlan``: embedding, the plan's calls in order,
final norm on the rows whose logits are wanted, output head.

Reference: minivllm/models/models/qwen3.py:159-220 — embed, layers, norm, select rows, head.
The reference norms every row and then selects (qwen3.py:189,215-217); here only the wanted
rows are normalised and projected. Logits are float32.

This class knows no architecture: which mixers, feed-forwards, norms and arrangement a layer
has, in which order layers run and whose cache a call reads are all read from the plan.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Tuple

import torch

from ..parts.base import (BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS, POSITION_ENCODINGS, CacheNeed,
                          HiddenStream, Runtime, TensorDecl)
from ..parts.plan import ModelPlan, TensorLocation
from .registry import Architecture


def _model_level_decls(plan: ModelPlan) -> List[Tuple[TensorLocation, TensorDecl]]:
    out = []
    for name, decl in EMBEDDINGS.get(plan.embedding.kind).tensors(plan.embedding).items():
        out.append((TensorLocation(None, "embedding", name), decl))
    for name, decl in NORMS.get(plan.final_norm.kind).tensors(plan.final_norm).items():
        out.append((TensorLocation(None, "final_norm", name), decl))
    for name, decl in HEADS.get(plan.head.kind).tensors(plan.head).items():
        out.append((TensorLocation(None, "head", name), decl))
    return out


def plan_tensors(plan: ModelPlan) -> List[Tuple[TensorLocation, TensorDecl]]:
    """Every (location, declaration) the plan's parts ask for."""
    out = _model_level_decls(plan)
    for i, layer in enumerate(plan.layers):
        block_cls = BLOCKS.get(layer.block.kind)
        slots = dict(layer.norms)
        for slot in getattr(block_cls, "norm_slots", tuple(slots)):
            if slot not in slots:
                raise ValueError(f"layer {i}: block arrangement {layer.block.kind!r} needs a norm for slot {slot!r}")
        for slot, nspec in layer.norms:
            for name, decl in NORMS.get(nspec.kind).tensors(nspec).items():
                out.append((TensorLocation(i, f"norm.{slot}", name), decl))
        if layer.mixer is not None:
            for name, decl in MIXERS.get(layer.mixer.kind).tensors(layer.mixer).items():
                out.append((TensorLocation(i, "mixer", name), decl))
        if layer.ffn is not None:
            for name, decl in FEED_FORWARDS.get(layer.ffn.kind).tensors(layer.ffn).items():
                out.append((TensorLocation(i, "ffn", name), decl))
    # a position encoding is shared by every mixer that names the same spec: its tensors (a learned
    # table, say) belong to the model, under the role "position.<kind>"
    seen = set()
    for layer in plan.layers:
        pspec = getattr(layer.mixer, "position", None)
        if pspec is not None and pspec not in seen:
            seen.add(pspec)
            for name, decl in POSITION_ENCODINGS.get(pspec.kind).tensors(pspec).items():
                out.append((TensorLocation(None, f"position.{pspec.kind}", name), decl))
    return out


def expected_tensors(arch: Architecture, config, plan: Optional[ModelPlan] = None) -> Dict[str, TensorDecl]:
    """Name on disk -> declaration, for everything the model reads. Two locations may share a
    name (a tied head); their shapes must then agree."""
    plan = plan or arch.plan(config)
    out: Dict[str, TensorDecl] = {}
    for loc, decl in plan_tensors(plan):
        name = arch.tensor_name(config, loc)
        if name in out and out[name].shape != decl.shape:
            raise ValueError(f"tensor {name!r} is asked for with shapes {out[name].shape} and {decl.shape}")
        out.setdefault(name, decl)
    return out


class CausalLM:
    def __init__(self, arch: Architecture, config, plan: ModelPlan, source, rt: Runtime):
        """``source.get(name)`` returns the named tensor on the device (the same object for the
        same name while it is alive, so tied tensors share memory)."""
        plan.validate()
        self.arch, self.config, self.plan, self.rt = arch, config, plan, rt

        def fetch(layer: Optional[int], role: str, decls: Dict[str, TensorDecl]) -> Dict[str, torch.Tensor]:
            return {name: source.get(arch.tensor_name(config, TensorLocation(layer, role, name))) for name in decls}

        emb_cls = EMBEDDINGS.get(plan.embedding.kind)
        self.embedding = emb_cls(plan.embedding, fetch(None, "embedding", emb_cls.tensors(plan.embedding)), rt)
        norm_cls = NORMS.get(plan.final_norm.kind)
        self.final_norm = norm_cls(plan.final_norm, fetch(None, "final_norm", norm_cls.tensors(plan.final_norm)), rt)
        head_cls = HEADS.get(plan.head.kind)
        self.head = head_cls(plan.head, fetch(None, "head", head_cls.tensors(plan.head)), rt)

        position_parts: Dict[object, object] = {}
        self.position_parts = position_parts
        self.graph_safe = True          # every part allows its forward to be captured in a graph
        self.blocks = []
        self.mixers = []
        for i, layer in enumerate(plan.layers):
            norms = {}
            for slot, nspec in layer.norms:
                cls = NORMS.get(nspec.kind)
                norms[slot] = cls(nspec, fetch(i, f"norm.{slot}", cls.tensors(nspec)), rt)
            kwargs = {}
            pspec = getattr(layer.mixer, "position", None)
            if pspec is not None:
                if pspec not in position_parts:
                    pcls = POSITION_ENCODINGS.get(pspec.kind)
                    position_parts[pspec] = pcls(pspec, fetch(None, f"position.{pspec.kind}", pcls.tensors(pspec)), rt)
                kwargs["position"] = position_parts[pspec]
            mixer = ffn = None
            if layer.mixer is not None:
                mixer_cls = MIXERS.get(layer.mixer.kind)
                mixer = mixer_cls(layer.mixer, fetch(i, "mixer", mixer_cls.tensors(layer.mixer)), rt, **kwargs)
            if layer.ffn is not None:
                ffn_cls = FEED_FORWARDS.get(layer.ffn.kind)
                ffn = ffn_cls(layer.ffn, fetch(i, "ffn", ffn_cls.tensors(layer.ffn)), rt)
            self.mixers.append(mixer)
            self.blocks.append(BLOCKS.get(layer.block.kind)(layer.block, norms, mixer, ffn))
            parts = [mixer, ffn, kwargs.get("position")] + list(norms.values())
            self.graph_safe = self.graph_safe and all(getattr(p, "graph_safe", True) for p in parts if p is not None)
        self.graph_safe = self.graph_safe and all(getattr(p, "graph_safe", True)
                                                  for p in (self.embedding, self.final_norm, self.head))

    # ------------------------------------------------------------------------------------
    def cache_needs(self) -> List[Optional[CacheNeed]]:
        """Per call: the paged memory its mixer needs, None if it keeps none (it has no cache
        or reads another call's)."""
        needs: List[Optional[CacheNeed]] = []
        for call in self.plan.calls:
            spec = self.plan.layers[call.layer].mixer
            need = None if spec is None else MIXERS.get(spec.kind).cache_need(spec)
            if call.cache_from is not None:
                if need is not None:
                    raise ValueError(f"a call reads the cache of call {call.cache_from} but its mixer "
                                     f"({spec.kind}) asks for a cache of its own")
                need = None
            needs.append(need)
        return needs

    def state_shapes(self) -> List[Optional[Tuple[Tuple[int, ...], torch.dtype]]]:
        out = []
        for call in self.plan.calls:
            spec = self.plan.layers[call.layer].mixer
            out.append(None if spec is None else MIXERS.get(spec.kind).state_shape(spec))
        return out

    # ------------------------------------------------------------------------------------
    def forward(self, ctx) -> torch.Tensor:
        """Runs the step described by ``ctx`` and returns float32 logits [len(logit_rows), vocab]."""
        rt, plan = self.rt, self.plan
        rt.ops.bind_stream()
        try:
            return self._forward(ctx)
        finally:
            rt.ops.unbind_stream()

    def _forward(self, ctx) -> torch.Tensor:
        rt, plan = self.rt, self.plan
        n = ctx.n_tokens
        resid = rt.workspace.get("resid", (n, plan.hidden_size), torch.float32)
        # what position encodings want gathered for the whole step rides on the first kernel
        ctx.position_rows = {}
        gathers = [job for job in (part.step_gather(ctx) for part in self.position_parts.values()
                                   if hasattr(part, "step_gather")) if job is not None]
        if gathers and getattr(self.embedding, "carries_gather", False):
            self.embedding.forward(ctx, resid, gather=gathers.pop(0))
        else:
            self.embedding.forward(ctx, resid)
        for index, table, out in gathers:
            rt.ops.gather_rows(index, table, out)
        stream = HiddenStream(resid, rt.workspace.get("resid.spare", (n, plan.hidden_size), torch.float32))
        for call_index, call in enumerate(plan.calls):
            block = self.blocks[call.layer]
            after = None
            if getattr(block, "accepts_next_norm", False) and call_index + 1 < len(plan.calls):
                # the norm the next block starts with may be folded into this block's last product
                after = self.blocks[plan.calls[call_index + 1].layer]
            if after is not None and hasattr(after, "entry_norm") and hasattr(after, "entry_part"):
                block.forward(stream, ctx, call_index, next_norm=after.entry_norm(), next_part=after.entry_part())
            else:
                block.forward(stream, ctx, call_index)
        m = ctx.n_logit_rows
        if m == 0:
            discard = getattr(stream.delta, "discard", None)
            if discard is not None:
                discard()
            return rt.workspace.get("logits", (0, plan.vocab_size), torch.float32)
        h = self.final_norm.forward(stream, ctx, rows=ctx.logit_rows, tag="final_normed")
        # the stream ends here: a last delta that was left as partial sums is not needed again
        discard = getattr(stream.delta, "discard", None)
        if discard is not None:
            discard()
        return self.head.forward(h, ctx)
