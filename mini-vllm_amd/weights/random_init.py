"""Random weights for an architecture, from a configuration and a seed.

Every matrix, embedding and bias is drawn from N(0, std); every norm weight from
1 + N(0, std) (N(0, std) for norms that add one to their weight). A tensor's values depend only
on (seed, its name on disk), not on the order in which tensors are made. ``write_model_folder``
stores them as ``config.json`` + ``model.safetensors``, so that a random model goes through
the same loading path as a real one. The reference has no such mode.
"""
from __future__ import annotations

import hashlib
import json
import os
from typing import Dict, Optional

import torch

from ..parts.base import TensorDecl

DEFAULT_STD = 0.02


def _tensor_seed(seed: int, name: str) -> int:
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(digest[:8], "little") & 0x7FFFFFFFFFFFFFFF


def random_tensor(name: str, decl: TensorDecl, seed: int, dtype: torch.dtype, std: float = DEFAULT_STD,
                  device: str = "cpu") -> torch.Tensor:
    gen = torch.Generator(device=device)
    gen.manual_seed(_tensor_seed(seed, name))
    if decl.integer:
        return torch.randint(0, 2 ** 15, decl.shape, generator=gen, dtype=torch.int32, device=device)
    t = torch.randn(decl.shape, generator=gen, dtype=torch.float32, device=device) * std
    if decl.init == "ones_normal":
        t += 1.0
    elif decl.init not in ("normal", "zeros_normal"):
        raise ValueError(f"unknown init law {decl.init!r} for {name}")
    return t.to(dtype)


def random_tensors(expected: Dict[str, TensorDecl], seed: int, dtype: torch.dtype,
                   std: float = DEFAULT_STD, device: str = "cpu") -> Dict[str, torch.Tensor]:
    return {name: random_tensor(name, decl, seed, dtype, std, device) for name, decl in expected.items()}


def write_model_folder(out_dir: str, config, seed: int, dtype: Optional[str] = None,
                       std: float = DEFAULT_STD) -> str:
    """Writes ``config.json`` and ``model.safetensors`` for ``config`` (a typed model
    configuration of a registered architecture) and returns ``out_dir``. ``dtype`` is the stored
    type ("bfloat16" or "float32"); None takes the configuration's own."""
    from safetensors.torch import save_file
    from ..models.registry import get_architecture
    from ..models.causal_lm import expected_tensors

    arch = get_architecture(config.architecture)
    stored = dtype or getattr(config, "dtype", "bfloat16")
    torch_dtype = {"bfloat16": torch.bfloat16, "float32": torch.float32, "float16": torch.float16}[stored]
    expected = expected_tensors(arch, config)
    tensors = random_tensors(expected, seed, torch_dtype, std)
    os.makedirs(out_dir, exist_ok=True)
    cfg = config.to_dict()
    cfg["torch_dtype"] = stored
    with open(os.path.join(out_dir, "config.json"), "w", encoding="utf-8") as f:
        json.dump(cfg, f, indent=2)
    save_file({k: v.contiguous() for k, v in tensors.items()}, os.path.join(out_dir, "model.safetensors"))
    return out_dir
