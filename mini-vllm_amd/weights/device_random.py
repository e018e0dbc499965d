"""Random weights generated on the device, for benchmarks of shapes whose model folder would
take long to write: the same laws as ``random_init`` (N(0, std), norms 1 + N(0, std)), one
seeded generator per tensor name, drawn by the device's generator (so the values differ from
the folder mode's, which draws on the CPU)."""
from __future__ import annotations

from typing import Dict, List, Tuple

import torch

from ..parts.base import TensorDecl
from .random_init import DEFAULT_STD, _tensor_seed
from .source import TensorSource


class DeviceRandomSource(TensorSource):
    def __init__(self, expected: Dict[str, TensorDecl], seed: int, dtype: torch.dtype, device: torch.device,
                 std: float = DEFAULT_STD):
        self.expected, self.seed, self.dtype, self.device, self.std = expected, seed, dtype, device, std

    def names(self) -> List[str]:
        return list(self.expected)

    def shape(self, name: str) -> Tuple[int, ...]:
        return tuple(self.expected[name].shape)

    def is_integer(self, name: str) -> bool:
        return self.expected[name].integer

    def stored_type(self, name: str) -> str:
        if self.expected[name].integer:
            return "I32"
        return {torch.bfloat16: "BF16", torch.float32: "F32"}.get(self.dtype, str(self.dtype))

    def read(self, name: str) -> torch.Tensor:
        decl = self.expected[name]
        gen = torch.Generator(device=self.device)
        gen.manual_seed(_tensor_seed(self.seed, name))
        if decl.integer:
            return torch.randint(0, 2 ** 15, decl.shape, generator=gen, dtype=torch.int32, device=self.device)
        t = torch.randn(decl.shape, generator=gen, dtype=torch.float32, device=self.device) * self.std
        if decl.init == "ones_normal":
            t += 1.0
        return t.to(self.dtype)
