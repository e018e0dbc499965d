"""The step function's input and the context every part sees during a step.

A step is a batch of (request, its next tokens): portions of prompts beside single decoded
tokens, cut anywhere. Reference: the reference builds either a prefill input (whole uncached
prompts; minivllm/executor/executor.py:81-127) or a decode input (one token per request;
executor.py:130-153) and hands the layers a ``Context`` with cu_seqlens / slot_mapping /
cache_seqlens / block_table (minivllm/executor/context.py). Here one layout serves both and
any mix: flat token ids and positions, the sequence each token belongs to, per sequence the
range of its tokens and its context length, one block table per cache group; cache slots are
computed by the kernels from position and block table.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence

import torch


@dataclass
class SeqStep:
    """One request's share of a step.

    tokens        the next tokens of the request (>= 1)
    start         position of tokens[0] = number of the request's tokens already in the cache
    block_tables  per cache group, the request's page ids by page index (-1: given back)
    state_slot    row of the state tensors that belongs to the request
    want          indices into ``tokens`` whose logits are returned, in this order
    """
    tokens: Sequence[int]
    start: int
    block_tables: Sequence[Sequence[int]]
    state_slot: int = 0
    want: Sequence[int] = ()


@dataclass
class KVView:
    """Cache of one call as its mixer sees it: the page tensors its ``CacheNeed`` named
    (``[pages, *page shape]`` each), the block table of its group and the page size."""
    pages: Dict[str, torch.Tensor]
    block_table: torch.Tensor      # int32 [sequences, width] of the call's group
    page_size: int

    @property
    def k_pages(self) -> torch.Tensor:      # softmax attention: [pages, kv_heads, page_size, head_dim]
        return self.pages["k"]

    @property
    def v_pages(self) -> torch.Tensor:      # [pages, kv_heads, head_dim, page_size]
        return self.pages["v"]


@dataclass
class AttentionPlan:
    """Host-side facts about the step that let the attention pick a kernel."""
    decode_only: bool              # every sequence brings exactly one token
    max_q_len: int
    max_context_len: int           # longest context the step (or the graph it is captured in) must serve
    n_seqs: int                    # rows of cu_seqlens - 1, padding sequences included
    q_lens: Sequence[int] = ()     # tokens per sequence, on the host
    cu_seqlens: Optional[torch.Tensor] = None   # int32 [n_seqs + 1] on the device
    workspace: Optional[object] = None          # where kernels take scratch memory from
    # decode steps: over how many workgroups a sequence's keys are dealt out; None lets the launch
    # rule choose (tests force counts)
    decode_splits: Optional[int] = None
    # prompt steps: (column tiles per wave, key groups per workgroup) of the MFMA kernel; None lets the
    # launch rule choose (tests force variants)
    prefill_variant: Optional[tuple] = None
    # steps recorded into a graph that serves any cut of up to (tokens, sequences): the kernels' grids
    # are then sized for the worst cut, not for ``q_lens`` (workgroups without work end at once)
    bound: Optional[tuple] = None
    # for measurement: keys in the cache of the step's sequences after the step (summed), and the
    # number of (query, visible key) pairs without windows
    kv_tokens: int = 0
    attention_pairs: int = 0

    def units(self, unit_tokens: int) -> int:
        """Runs of up to ``unit_tokens`` consecutive tokens of one sequence in the step: counted from
        the host's lengths, or the most that any cut within ``bound`` can have."""
        if self.bound is not None:
            tokens, seqs = self.bound
            return tokens // unit_tokens + seqs
        return sum(-(-ql // unit_tokens) for ql in self.q_lens)

    def busy_units(self, unit_tokens: int) -> int:
        """The units that hold tokens, for rules that weigh the work against the device: the count
        itself, or, of a bound, the units its tokens fill (the rest of ``units`` are spares that end
        at once)."""
        if self.bound is not None:
            return max(1, self.bound[0] // unit_tokens)
        return self.units(unit_tokens)


class StepContext:
    """Device tensors (int32) and host facts describing the step, handed to every part.

    token_ids [n]      positions [n]        token_seq [n] (sequence index, -1 = padding row)
    cu_seqlens [s+1]   context_lens [s]     state_slots [s]      logit_rows [m]
    """

    def __init__(self):
        self.n_tokens = 0
        self.n_seqs = 0
        self.n_logit_rows = 0
        self.token_ids: torch.Tensor = None
        self.positions: torch.Tensor = None
        self.token_seq: torch.Tensor = None
        self.cu_seqlens: torch.Tensor = None
        self.context_lens: torch.Tensor = None
        self.state_slots: torch.Tensor = None
        self.logit_rows: torch.Tensor = None
        self.block_tables: List[torch.Tensor] = []
        # host copies
        self.q_lens: List[int] = []
        self.starts: List[int] = []
        self.host_state_slots: List[int] = []
        self.attention_plan: Optional[AttentionPlan] = None
        # filled by the executor
        self._kv: Dict[int, "KVView"] = {}
        self._state: Dict[int, torch.Tensor] = {}
        self.page_size = 0
        # rows that a position encoding had gathered for this step (PositionEncoding.step_gather), by part
        self.position_rows: Dict[object, torch.Tensor] = {}

    def kv(self, call: int) -> KVView:
        try:
            return self._kv[call]
        except KeyError:
            raise KeyError(f"call {call} has no cache: its mixer declared no cache need") from None

    def state(self, call: int) -> torch.Tensor:
        try:
            return self._state[call]
        except KeyError:
            raise KeyError(f"call {call} has no state: its mixer declared no state shape") from None
