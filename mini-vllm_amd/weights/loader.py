"""Checks a model folder against what the architecture's plan asks for, then builds the model.

Reference: minivllm/models/loader.py:24-29 and qwen3.py:223-245. The reference raises a bare
``KeyError`` for an unknown tensor name, does not notice missing tensors and leaves a wrong
shape to ``copy_``. Here every problem of a folder is found before any data is read and is
reported in one ``WeightError`` that lists missing tensors, unexpected tensors, wrong
shapes, wrong kinds (integer against floating) and stored types the engine does not keep
(float16, 8-bit floats: it converts nothing silently).
"""
from __future__ import annotations

from typing import Dict, List, Optional, Tuple


from ..parts.base import TensorDecl
from .source import KEPT_FLOAT_TYPES, SafetensorsSource, TensorSource


class WeightError(ValueError):
    def __init__(self, where: str, missing: List[str], unexpected: List[str],
                 wrong_shape: List[Tuple[str, Tuple[int, ...], Tuple[int, ...]]],
                 wrong_type: List[Tuple[str, str]], unsupported_dtype: Optional[List[Tuple[str, str]]] = None):
        self.missing, self.unexpected, self.wrong_shape, self.wrong_type = missing, unexpected, wrong_shape, wrong_type
        self.unsupported_dtype = unsupported_dtype = list(unsupported_dtype or [])
        lines = [f"the weights in {where} do not fit the model:"]
        if missing:
            lines.append(f"  missing tensors ({len(missing)}):")
            lines += [f"    {n}" for n in missing]
        if unexpected:
            lines.append(f"  unexpected tensors ({len(unexpected)}):")
            lines += [f"    {n}" for n in unexpected]
        if wrong_shape:
            lines.append(f"  wrong shapes ({len(wrong_shape)}):")
            lines += [f"    {n}: found {list(got)}, expected {list(want)}" for n, got, want in wrong_shape]
        if wrong_type:
            lines.append(f"  wrong kinds ({len(wrong_type)}):")
            lines += [f"    {n}: {why}" for n, why in wrong_type]
        if unsupported_dtype:
            kinds = sorted({t for _, t in unsupported_dtype})
            lines.append(f"  unsupported dtype {', '.join(kinds)} ({len(unsupported_dtype)} tensors; the engine keeps "
                         f"bfloat16 and float32 as stored and converts nothing else: save the checkpoint again in "
                         f"bfloat16 or float32 to serve it):")
            lines += [f"    {n}: {t}" for n, t in unsupported_dtype]
        super().__init__("\n".join(lines))


def check_tensors(source: TensorSource, expected: Dict[str, TensorDecl], ignorable=frozenset(),
                  where: str = "the model folder") -> None:
    have = set(source.names())
    missing = sorted(n for n in expected if n not in have)
    unexpected = sorted(n for n in have if n not in expected and n not in ignorable)
    wrong_shape, wrong_type, unsupported = [], [], []
    for name, decl in expected.items():
        if name not in have:
            continue
        got = tuple(source.shape(name))
        if got != tuple(decl.shape):
            wrong_shape.append((name, got, tuple(decl.shape)))
        if source.is_integer(name) != decl.integer:
            wrong_type.append((name, "integer tensor where a floating one is expected" if not decl.integer
                               else "floating tensor where an integer table is expected"))
        elif not decl.integer and source.stored_type(name) not in KEPT_FLOAT_TYPES:
            unsupported.append((name, source.stored_type(name)))
    if missing or unexpected or wrong_shape or wrong_type or unsupported:
        raise WeightError(where, missing, unexpected, sorted(wrong_shape), sorted(wrong_type), sorted(unsupported))


def open_model_folder(model_dir: str) -> TensorSource:
    return SafetensorsSource(model_dir)
