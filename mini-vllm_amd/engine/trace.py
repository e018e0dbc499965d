"""Trace replay: feeds given token ids through the model step by step and writes logits.

It samples nothing and has no forward pass, cache or loader of its own: it drives the
``Executor``'s step function and a ``CacheManager``, the ones generation uses. Steps come as
one JSON object per line:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

All entries of a step run as one batch. For a step in which logits are wanted the file
``<out>/<step>.f32`` receives them as little-endian float32 [wanted, vocab], in the order of
the entries and of each ``want``. After every step ``done <step>`` is printed and flushed.

With prefix caching on, the first entry of a request is looked up in the cache: leading full
pages whose tokens some earlier request already computed are shared instead of run again, up
to the first wanted position (a wanted row has to be computed) and never the entry's last
token. The step then runs only what is left of the entry; the logits are the same either way.
"""
from __future__ import annotations

import json
import os
from typing import IO, Dict, List, Optional

import numpy as np

from ..config.engine_config import EngineConfig
from ..config.model_config import read_config_json
from .executor import Executor
from .step import SeqStep

TOKEN_ROUNDING = 64       # a request's share of --max-tokens is rounded up to this


class TraceError(RuntimeError):
    pass


class TraceRunner:
    def __init__(self, model: str, dtype: str, max_tokens: int, page_size: int = 16, use_graph: bool = True,
                 max_live: int = 16, enable_prefix_caching: bool = False, poison_pages: bool = False):
        if TOKEN_ROUNDING % page_size:
            raise ValueError(f"the page size {page_size} must divide {TOKEN_ROUNDING}")
        max_tokens = max(TOKEN_ROUNDING, -(-max_tokens // TOKEN_ROUNDING) * TOKEN_ROUNDING)
        raw = read_config_json(model)
        max_pos = int(raw.get("max_position_embeddings", max_tokens))
        config = EngineConfig(
            model=model, dtype=dtype, max_model_len=min(max_pos, max_tokens),
            max_num_batched_tokens=max_tokens, max_num_batched_seqs=max_live,
            kv_cache_block_size=page_size, kv_cache_num_blocks=max_tokens // page_size,
            use_cuda_graph=use_graph, enable_prefix_caching=enable_prefix_caching,
            debug_poison_pages=poison_pages)
        self.executor = Executor(config)
        self.manager = self.executor.new_cache_manager()
        # with prefix caching: every token a live request has brought so far (full pages are
        # published under the hash of their tokens)
        self.tokens: Dict[str, List[int]] = {}
        self.num_reused_tokens = 0

    def run_step(self, step: Dict) -> Optional[np.ndarray]:
        """Runs one step object; returns the wanted logits [wanted, vocab] or None."""
        entries = step.get("entries", [])
        seqs: List[SeqStep] = []
        ids = []
        for e in entries:
            rid = e["id"]
            tokens = [int(t) for t in e["tokens"]]
            if not tokens:
                raise TraceError(f"step {step.get('step')}: entry {rid!r} brings no tokens")
            if rid in ids:
                raise TraceError(f"step {step.get('step')}: request {rid!r} appears twice")
            want = [int(w) for w in e.get("want", [])]
            if any(not (0 <= w < len(tokens)) for w in want):
                raise TraceError(f"step {step.get('step')}: entry {rid!r} wants a place outside its {len(tokens)} tokens")
            if rid not in self.manager:
                if self.manager.prefix_caching:
                    # pages up to the first wanted place may come from the cache
                    first = min(want) if want else len(tokens) - 1
                    reused = self.manager.admit(rid, tokens[:first + 1]).num_computed
                    self.num_reused_tokens += reused
                    self.tokens[rid] = list(tokens)
                    tokens, want = tokens[reused:], [w - reused for w in want]
                else:
                    self.manager.admit(rid)
            elif self.manager.prefix_caching:
                self.tokens[rid].extend(tokens)
            self.manager.reserve(rid, len(tokens))
            seq = self.manager.sequence(rid)
            seqs.append(SeqStep(tokens=tokens, start=seq.num_computed,
                                block_tables=[self.manager.block_table(rid, g)
                                              for g in range(len(self.manager.groups))],
                                state_slot=seq.state_slot, want=want))
            ids.append(rid)
        out = None
        if seqs:
            logits = self.executor.step(seqs)
            if logits.shape[0] > 0:
                out = logits.detach().cpu().numpy().astype("<f4", copy=False)
        for rid, s in zip(ids, seqs):
            self.manager.commit(rid, len(s.tokens), self.tokens.get(rid))
        for rid in step.get("end", []):
            if rid in self.manager:
                self.manager.release(rid)
            self.tokens.pop(rid, None)
        return out


def run(model: str, dtype: str, out_dir: str, max_tokens: int, stdin: IO[str], stdout: IO[str],
        page_size: int = 16, use_graph: bool = True, enable_prefix_caching: bool = False) -> int:
    os.makedirs(out_dir, exist_ok=True)
    runner = TraceRunner(model, dtype, max_tokens, page_size=page_size, use_graph=use_graph,
                         enable_prefix_caching=enable_prefix_caching)
    for line in stdin:
        line = line.strip()
        if not line:
            continue
        step = json.loads(line)
        logits = runner.run_step(step)
        if logits is not None:
            logits.tofile(os.path.join(out_dir, f"{step['step']}.f32"))
        stdout.write(f"done {step['step']}\n")
        stdout.flush()
    return 0
