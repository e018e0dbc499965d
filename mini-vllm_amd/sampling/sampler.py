"""Draws one token per request from the step's logits with the HIP sampling kernel.

Reference: minivllm/models/layers/sampler.py:15-31 and the tensors built in
minivllm/executor/executor.py:165-191. The reference divides by the temperature only when some
request has one other than 1, samples only when top-k or top-p is set and takes the arg-max
otherwise; its caller passes top_k and top_p in swapped order (executor.py:195 against
sampler.py:9-13). Here temperature 0 is the arg-max and any positive temperature draws;
top_k and top_p filter as their names say. Every request has a random stream of its own, keyed
by (seed, index of the token being drawn), so what it draws does not depend on the batch.
"""
from __future__ import annotations

from typing import List, Sequence

import numpy as np
import torch

from ..config.sampling_params import SamplingParams

_MASK63 = (1 << 63) - 1


def request_seed(engine_seed: int, request_id: int, params: SamplingParams) -> int:
    """The seed of a request's random stream: its own if given, else derived from the engine's
    seed and the request's id."""
    if params.seed is not None:
        return int(params.seed) & _MASK63
    x = (engine_seed * 0x9E3779B97F4A7C15 + request_id * 0xD1B54A32D192ED03 + 0x632BE59BD9B4E019) & ((1 << 64) - 1)
    x ^= x >> 29
    return x & _MASK63


class Sampler:
    def __init__(self, ops, device: torch.device):
        self.ops = ops
        self.device = device
        self._out = torch.empty(1024, dtype=torch.int32, device=device)

    @staticmethod
    def arrays(params: Sequence[SamplingParams], seeds: Sequence[int], counters: Sequence[int]):
        """The per-request arrays the kernel reads: temperature, top_k, top_p, seed, counter."""
        return (np.array([p.temperature for p in params], dtype=np.float32),
                np.array([p.top_k for p in params], dtype=np.int32),
                np.array([p.top_p for p in params], dtype=np.float32),
                np.array(seeds, dtype=np.int64), np.array(counters, dtype=np.int64))

    def sample(self, logits: torch.Tensor, params: Sequence[SamplingParams], seeds: Sequence[int],
               counters: Sequence[int]) -> List[int]:
        """``logits`` float32 [M, V] on the device; ``params``, ``seeds`` and ``counters`` (index of
        the token each request is about to draw) have M entries. Returns M token ids."""
        M = logits.shape[0]
        if M == 0:
            return []
        if self._out.numel() < M:
            self._out = torch.empty(M, dtype=torch.int32, device=self.device)
        out = self._out[:M]
        if all(p.temperature == 0.0 for p in params):
            self.ops.sample(logits, out)
            return out.tolist()
        temps = torch.tensor([p.temperature for p in params], dtype=torch.float32).to(self.device, non_blocking=True)
        need_k = any(p.top_k > 0 for p in params)
        need_p = any(p.top_p < 1.0 for p in params)
        top_k = torch.tensor([p.top_k for p in params], dtype=torch.int32).to(self.device) if need_k else None
        top_p = torch.tensor([p.top_p for p in params], dtype=torch.float32).to(self.device) if need_p else None
        rng = torch.tensor(np.array([[s, c] for s, c in zip(seeds, counters)], dtype=np.int64)).to(self.device)
        self.ops.sample(logits, out, temps, top_k, top_p, rng)
        return out.tolist()
