"""The executor: owns the model, the device memory of the cache and the one step function.

Reference: minivllm/executor/executor.py (model load :18, warm-up :62-78, cache sizing and
allocation :31-60, input building :81-163, forward :197-214) and minivllm/executor/graph.py
(decode graphs for batch-size buckets with static inputs and inert padding rows). Differences:

* ``step`` takes any mix of prompt portions and decoded tokens and returns float32 logits at
  the wanted positions; sampling is a separate call (the reference returns token ids only);
* step inputs are packed into one pinned buffer and copied with one transfer;
* the cache is a set of page tensors per call, with the shapes the call's mixer asks for (softmax
  attention: K as [page][kv_head][slot][d] and V as [page][kv_head][d][slot]), grouped by
  retention; the reference holds one [2, layers, blocks, block_size, kv_heads, head_dim] tensor
  (executor.py:51);
* decode-only steps are replayed from a HIP graph captured per batch-size bucket on first use;
  the block-table width of a graph is ceil(max_model_len / page_size), not the pool size
  (graph.py:20);
* nothing here writes into the configuration object (the reference's does, executor.py:49).
"""
from __future__ import annotations

import logging
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..cache.manager import CacheManager, GroupSpec, groups_from_needs
from ..config.engine_config import EngineConfig, compute_dtype_name
from ..kernels.ops import Ops, dtype_from_name
from ..models.causal_lm import CausalLM, expected_tensors
from ..models.registry import Architecture, load_config
from ..parts.base import Runtime, Workspace
from ..weights.loader import check_tensors, open_model_folder
from ..weights.source import DeviceTensors, TensorSource
from .step import AttentionPlan, KVView, SeqStep, StepContext

logger = logging.getLogger(__name__)

GRAPH_BUCKETS = [1, 2, 4, 8] + list(range(16, 257, 16))     # as the reference's (graph.py:11-12)
# token counts that steps with prompt portions are padded to when they are replayed from a graph:
# at most an eighth more than the step holds
TOKEN_BUCKETS = (list(range(16, 129, 16)) + list(range(160, 257, 32)) + list(range(320, 513, 64))
                 + list(range(640, 1025, 128)) + list(range(1280, 2049, 256)) + list(range(2560, 4097, 512))
                 + list(range(5120, 8193, 1024)))
# graphs of such steps kept at a time (the one used longest ago goes first)
MIXED_GRAPHS_KEPT = 64


def _cdiv(a: int, b: int) -> int:
    return -(-a // b)


class _Staging:
    """Pinned host buffers for the step's integers, used in turn so that a buffer is never
    rewritten while its copy to the device may still be running."""

    def __init__(self, count: int = 4):
        self.buffers: List[Optional[torch.Tensor]] = [None] * count
        self.events: List[Optional[torch.cuda.Event]] = [None] * count
        self.next = 0

    def take(self, n: int) -> Tuple[torch.Tensor, int]:
        i = self.next
        self.next = (self.next + 1) % len(self.buffers)
        if self.events[i] is not None:
            self.events[i].synchronize()
        buf = self.buffers[i]
        if buf is None or buf.numel() < n:
            buf = torch.empty(max(n, 4096), dtype=torch.int32, pin_memory=True)
            self.buffers[i] = buf
        return buf, i

    def sent(self, i: int) -> None:
        ev = self.events[i]
        if ev is None:
            ev = self.events[i] = torch.cuda.Event()
        ev.record()


class RepeatedRun:
    """Decode steps in a row that were launched and may still be running."""

    def __init__(self, host: torch.Tensor, done: torch.cuda.Event, device_tokens: torch.Tensor, repeat: int,
                 bucket: int, count: int):
        self.host, self.done, self.device_tokens = host, done, device_tokens
        self.repeat, self.bucket, self.count = repeat, bucket, count

    def tokens(self) -> np.ndarray:
        """Waits for the launch; the drawn tokens, int32 [repeat, sequences]."""
        self.done.synchronize()
        n = self.repeat * self.bucket
        return self.host[:n].numpy().reshape(self.repeat, self.bucket)[:, :self.count].copy()


class Executor:
    def __init__(self, config: EngineConfig, model: Optional[Tuple[Architecture, object, TensorSource]] = None,
                 device: str = "cuda:0"):
        """``model`` = (architecture, typed model config, tensor source) serves a model that is not
        in a folder; otherwise ``config.model`` is read."""
        if not torch.cuda.is_available():
            raise RuntimeError("no GPU is visible; the engine has no CPU path")
        self.config = config
        self.device = torch.device(device)
        torch.cuda.set_device(self.device)
        if model is None:
            arch, model_config = load_config(config.model)
            source = open_model_folder(config.model)
            where = config.model
        else:
            arch, model_config, source = model
            where = "the given tensors"
        self.arch, self.model_config = arch, model_config
        self.dtype = dtype_from_name(compute_dtype_name(config.dtype, getattr(model_config, "dtype", None), where))
        self.page_size = config.kv_cache_block_size

        plan = arch.plan(model_config)
        if config.max_model_len > plan.max_positions:
            raise ValueError(f"max_model_len {config.max_model_len} exceeds the model's "
                             f"max_position_embeddings {plan.max_positions}")
        check_tensors(source, expected_tensors(arch, model_config, plan), arch.ignorable(model_config), where)

        if self.dtype == torch.bfloat16:
            wide = [n for n, d in expected_tensors(arch, model_config, plan).items()
                    if len(d.shape) == 2 and not d.integer and source.stored_type(n) != "BF16"]
            if wide:
                logger.warning("%d matrices of %s are stored in 32-bit and stay so: products with them run on the "
                               "exact kernel, not on the MFMA kernels (first: %s); store the model in bfloat16 for "
                               "serving speed", len(wide), where, wide[0])
        # an engine has its kernels' front end to itself: what it keeps between launches (scratch areas,
        # the counters of the decode attention's key splits, the state of a recording) is then never
        # shared with another engine of the process
        self.ops = Ops(self.dtype)
        self.rt = Runtime(device=self.device, dtype=self.dtype, ops=self.ops, workspace=Workspace(self.device),
                          max_positions=config.max_model_len)
        tensors = DeviceTensors(source, self.device)
        self.model = CausalLM(arch, model_config, plan, tensors, self.rt)
        self.plan = plan
        self.vocab_size = plan.vocab_size

        self.needs = self.model.cache_needs()
        self.groups: List[GroupSpec] = groups_from_needs(self.needs)
        self.group_of_call: Dict[int, int] = {c: g for g, spec in enumerate(self.groups) for c in spec.calls}
        for i, call in enumerate(plan.calls):
            if call.cache_from is not None:
                if call.cache_from not in self.group_of_call:
                    raise ValueError(f"call {i} reads the cache of call {call.cache_from}, which keeps none")
                self.group_of_call[i] = self.group_of_call[call.cache_from]
        self.state_shapes = self.model.state_shapes()
        self.has_state = any(s is not None for s in self.state_shapes)
        self.num_state_slots = config.max_num_batched_seqs
        self.max_pages_per_seq = _cdiv(config.max_model_len, self.page_size)

        self._staging = _Staging()
        self._meta_device: Optional[torch.Tensor] = None
        self._graphs: Dict[Tuple[int, int], Tuple[torch.cuda.CUDAGraph, StepContext, torch.Tensor, torch.Tensor]] = {}
        self._graph_pool = None
        self._repeat_graphs: Dict[Tuple[int, int, int], Tuple[torch.cuda.CUDAGraph, torch.Tensor, torch.Tensor]] = {}
        # steps with prompt portions: (token bucket, sequence bucket, logit rows, context cap) -> graph
        self._mixed_graphs: Dict[Tuple[int, int, int, int], Tuple] = {}
        self._graph_workspace: Optional[Workspace] = None
        # what each recorded graph holds, by kind of node (see _record)
        self.graph_census: Dict[Tuple, Dict[str, int]] = {}
        # what each recorded graph launches, in order: (entry point, bytes, operations, ...) per launch
        self.graph_ledger: Dict[tuple, list] = {}
        # pinned buffers for the tokens of launches in flight, used in turn (two launches at most are)
        self._token_buffers: List[Optional[torch.Tensor]] = [None] * 4
        self._next_token_buffer = 0
        self.kv_pages: Dict[int, Dict[str, torch.Tensor]] = {}     # per call with a cache need: its page tensors by name
        self._poison: Dict[int, List[int]] = {}                    # debug_poison_pages: pages to fill, per group
        self.state_tensors: Dict[int, torch.Tensor] = {}
        self.num_pages = 0                                         # of the largest pool
        self.group_pages: List[int] = [0] * len(self.groups)       # pages of each group's pool
        self._allocate_memory()

    # ------------------------------------------------------------------------------------
    # memory
    # ------------------------------------------------------------------------------------
    def bytes_per_page(self, group: Optional[int] = None) -> int:
        """Bytes one page index takes over all calls (of one group, or of all groups together)."""
        calls = range(len(self.needs)) if group is None else self.groups[group].calls
        return sum(self.needs[c].bytes_per_token(self.dtype) for c in calls if self.needs[c] is not None) * self.page_size

    def _pages_a_request_holds(self, group: int) -> int:
        """Most pages one request can hold in a group at a time (see Retention.most_pages_held)."""
        portion = min(self.config.max_num_batched_tokens, self.config.max_model_len)
        held = self.groups[group].retention.most_pages_held(self.config.max_model_len, self.page_size, portion)
        return self.max_pages_per_seq if held is None else max(1, min(int(held), self.max_pages_per_seq))

    def _pool_sizes(self, budget_bytes: int) -> List[int]:
        """Pages per group within ``budget_bytes``: every pool as large as the largest, except that a
        group never gets more pages than all live requests together can hold in it (a group that
        gives pages back early is bounded by that long before the memory is)."""
        n_groups = len(self.groups)
        caps = [self.config.max_num_batched_seqs * self._pages_a_request_holds(g) for g in range(n_groups)]
        per = [max(1, self.bytes_per_page(g)) for g in range(n_groups)]
        sizes: List[Optional[int]] = [None] * n_groups
        left = budget_bytes
        while True:
            open_groups = [g for g in range(n_groups) if sizes[g] is None]
            if not open_groups:
                break
            common = left // sum(per[g] for g in open_groups)
            capped = [g for g in open_groups if caps[g] <= common]
            if not capped:
                for g in open_groups:
                    sizes[g] = int(common)
                break
            for g in capped:
                sizes[g] = caps[g]
                left -= caps[g] * per[g]
        return [int(n) for n in sizes]

    def _allocate_memory(self) -> None:
        cfg = self.config
        for call, shape in enumerate(self.state_shapes):
            if shape is not None:
                dims, dt = shape
                self.state_tensors[call] = torch.zeros((self.num_state_slots,) + tuple(dims), dtype=dt,
                                                       device=self.device)
        if cfg.kv_cache_num_blocks is not None:
            given = cfg.kv_cache_num_blocks
            sizes = [int(given)] * len(self.groups) if isinstance(given, int) else [int(n) for n in given]
            if len(sizes) != len(self.groups):
                raise ValueError(f"kv_cache_num_blocks names {len(sizes)} pools, the model has {len(self.groups)} cache groups")
        else:
            self._warmup(cfg.max_num_batched_tokens)
            torch.cuda.synchronize()
            free, total = torch.cuda.mem_get_info(self.device)
            used = total - free
            budget = int(total * cfg.gpu_memory_utilization) - used
            sizes = self._pool_sizes(budget) if self.groups else []
            if sizes and min(sizes) < 1:
                raise RuntimeError(f"no memory left for the cache: {used / 2**30:.1f} GiB are in use, "
                                   f"gpu_memory_utilization {cfg.gpu_memory_utilization} of "
                                   f"{total / 2**30:.1f} GiB allows {budget / 2**30:.2f} GiB more")
        self._allocate_pages(sizes)
        logger.info("allocated cache pools of %s pages of %d tokens (%.2f GiB)", sizes, self.page_size,
                    sum(n * self.bytes_per_page(g) for g, n in enumerate(sizes)) / 2 ** 30)
        if cfg.capture_graphs_at_start and cfg.use_cuda_graph and self.model.graph_safe:
            self.capture_graphs()

    def _allocate_pages(self, sizes) -> None:
        """Page tensors ``[pages, *shape]`` for every call with a cache need, in the element types the
        need names, as many pages as the call's group has (``sizes``: one count, or one per group)."""
        if isinstance(sizes, int):
            sizes = [sizes] * len(self.groups)
        self.kv_pages.clear()
        self.group_pages = [int(n) for n in sizes]
        self.num_pages = max(self.group_pages, default=0)
        for g, spec in enumerate(self.groups):
            for call in spec.calls:
                need = self.needs[call]
                dtypes = need.page_dtypes(self.dtype)
                self.kv_pages[call] = {name: torch.zeros((self.group_pages[g],) + tuple(shape), dtype=dtypes[name],
                                                         device=self.device)
                                       for name, shape in need.page_shapes(self.page_size).items()}
        self._graphs.clear()
        self._repeat_graphs.clear()
        self._mixed_graphs.clear()

    def _warmup(self, num_tokens: int) -> None:
        """One dry step of ``num_tokens`` tokens against a throw-away cache, so that every scratch
        buffer reaches its final size before the cache is sized from what is left."""
        ps = self.page_size
        n_seqs = max(1, min(self.config.max_num_batched_seqs, _cdiv(num_tokens, ps)))
        # (no step holds more tokens of a request than max_model_len)
        per_seq = max(1, min(num_tokens // n_seqs, self.config.max_model_len))
        pages_per_seq = _cdiv(per_seq, ps)
        self._allocate_pages(n_seqs * pages_per_seq)
        seqs = []
        for s in range(n_seqs):
            table = list(range(s * pages_per_seq, (s + 1) * pages_per_seq))
            seqs.append(SeqStep(tokens=[0] * per_seq, start=0, block_tables=[table] * len(self.groups),
                                state_slot=s % self.num_state_slots, want=[per_seq - 1]))
        self.step(seqs)
        if self.config.use_cuda_graph and self.model.graph_safe:
            # the scratch area that all decode graphs share, at the size of the largest batch they serve
            self._prepare_graph_workspace()
        torch.cuda.synchronize()
        self.kv_pages.clear()
        torch.cuda.empty_cache()

    def new_cache_manager(self, enable_prefix_caching: Optional[bool] = None) -> CacheManager:
        """A manager for this executor's pages and state slots."""
        if enable_prefix_caching is None:
            enable_prefix_caching = self.config.enable_prefix_caching
        manager = CacheManager(self.groups, list(self.group_pages), self.page_size, self.num_state_slots,
                               enable_prefix_caching=enable_prefix_caching, has_state=self.has_state)
        if self.config.debug_poison_pages:
            self._poison = {g: [] for g in range(len(self.groups))}
            for g, pool in enumerate(manager.pools):
                # a page that prefix reuse may revive keeps its content until it is handed out anew
                pool.on_recycle = (lambda page, why, g=g, keep=manager.prefix_caching:
                                   None if (keep and why == "release") else self._poison[g].append(page))
        return manager

    def _flush_poison(self) -> None:
        """debug_poison_pages: NaN into every page that changed hands since the last step, enqueued
        before this step's kernels and behind those of every earlier step."""
        for g, pages in self._poison.items():
            if not pages:
                continue
            index = torch.tensor(sorted(set(pages)), dtype=torch.int64, device=self.device)
            pages.clear()
            for call in self.groups[g].calls:
                for t in self.kv_pages.get(call, {}).values():
                    if t.is_floating_point():
                        t.index_fill_(0, index, float("nan"))

    # ------------------------------------------------------------------------------------
    # building a step
    # ------------------------------------------------------------------------------------
    def _validate(self, seqs: Sequence[SeqStep], lookahead: int = 0) -> None:
        """``lookahead``: positions beyond the step's own that later runs of a repeated step write."""
        ps = self.page_size
        for i, s in enumerate(seqs):
            n = len(s.tokens) + lookahead
            if n < 1:
                raise ValueError(f"sequence {i} of the step brings no token")
            if s.start < 0 or s.start + n > self.config.max_model_len:
                raise ValueError(f"sequence {i}: positions {s.start}..{s.start + n - 1} exceed max_model_len "
                                 f"{self.config.max_model_len}")
            if len(s.block_tables) != len(self.groups):
                raise ValueError(f"sequence {i} brings {len(s.block_tables)} block tables, the model has "
                                 f"{len(self.groups)} cache groups")
            if not (0 <= s.state_slot < self.num_state_slots):
                raise ValueError(f"sequence {i}: state slot {s.state_slot} out of range")
            for w in s.want:
                if not (0 <= w < len(s.tokens)):
                    raise ValueError(f"sequence {i}: wanted index {w} outside its {n} tokens")
            last_page = (s.start + n - 1) // ps
            for g in range(len(self.groups)):
                if len(s.block_tables[g]) <= last_page:
                    raise ValueError(f"sequence {i}: group {g} has {len(s.block_tables[g])} pages, position "
                                     f"{s.start + n - 1} needs {last_page + 1}")

    def _fill(self, seqs: Sequence[SeqStep], pad_to: Optional[int] = None, bt_widths: Optional[List[int]] = None,
              lookahead: int = 0, extra_words: int = 0, check_pages: bool = True, pad_tokens: Optional[int] = None,
              pad_rows: Optional[int] = None):
        """Packs the step's integers into one int32 array. Returns (array, offsets dict, facts).
        ``pad_to`` pads sequences (and, unless ``pad_tokens`` / ``pad_rows`` say otherwise, tokens and
        logit rows) to a graph's size with inert rows. ``lookahead`` extends the check of the block
        tables to positions that later runs of a repeated step touch; ``extra_words`` leaves room at
        the end (offset "extra", 8-byte aligned)."""
        S = len(seqs)
        q_lens = [len(s.tokens) for s in seqs]
        N = sum(q_lens)
        Sp = pad_to if pad_to is not None else S
        Np = pad_tokens if pad_tokens is not None else (pad_to if pad_to is not None else N)
        want_rows: List[int] = []
        base = 0
        for s, n in zip(seqs, q_lens):
            want_rows.extend(base + w for w in s.want)
            base += n
        M = len(want_rows)
        Mp = pad_rows if pad_rows is not None else (pad_to if pad_to is not None else M)
        widths = bt_widths or [max(1, max(len(s.block_tables[g]) for s in seqs)) for g in range(len(self.groups))]
        off = {}
        cur = 0
        for name, size in (("token_ids", Np), ("positions", Np), ("token_seq", Np), ("cu_seqlens", Sp + 1),
                           ("context_lens", Sp), ("state_slots", Sp), ("logit_rows", Mp)):
            off[name] = (cur, size)
            cur += size
        for g, w in enumerate(widths):
            off[f"bt{g}"] = (cur, Sp * w)
            cur += Sp * w
        if extra_words:
            cur += cur & 1
            off["extra"] = (cur, extra_words)
            cur += extra_words
        arr = np.zeros(cur, dtype=np.int32)
        tok = arr[off["token_ids"][0]:off["token_ids"][0] + Np]
        pos = arr[off["positions"][0]:off["positions"][0] + Np]
        tsq = arr[off["token_seq"][0]:off["token_seq"][0] + Np]
        tsq[:] = -1
        cu = arr[off["cu_seqlens"][0]:off["cu_seqlens"][0] + Sp + 1]
        cl = arr[off["context_lens"][0]:off["context_lens"][0] + Sp]
        sl = arr[off["state_slots"][0]:off["state_slots"][0] + Sp]
        lr = arr[off["logit_rows"][0]:off["logit_rows"][0] + Mp]
        lr[:] = -1
        lr[:M] = want_rows
        starts = np.fromiter((s.start for s in seqs), dtype=np.int64, count=S)
        if N == S:                                  # one token each: no loop over the sequences
            tok[:S] = np.fromiter((s.tokens[0] for s in seqs), dtype=np.int64, count=S)
            pos[:S] = starts
            tsq[:S] = np.arange(S, dtype=np.int32)
            cu[:S + 1] = np.arange(S + 1, dtype=np.int32)
            cl[:S] = starts + 1
            sl[:S] = np.fromiter((s.state_slot for s in seqs), dtype=np.int64, count=S)
            base = S
        else:
            base = 0
            for i, (s, n) in enumerate(zip(seqs, q_lens)):
                tok[base:base + n] = s.tokens
                pos[base:base + n] = np.arange(s.start, s.start + n, dtype=np.int32)
                tsq[base:base + n] = i
                cu[i + 1] = base + n
                cl[i] = s.start + n
                sl[i] = s.state_slot
                base += n
        cu[S + 1:] = base
        last_page = (cl[:S].astype(np.int64) - 1 + lookahead) // self.page_size
        for g, w in enumerate(widths):
            o, size = off[f"bt{g}"]
            bt = arr[o:o + size].reshape(Sp, w)
            bt[:] = -1
            for i, s in enumerate(seqs):
                t = s.block_tables[g]
                if len(t) > w:
                    raise ValueError(f"sequence {i}: {len(t)} pages exceed the block table width {w}")
                bt[i, :len(t)] = t
            # every page a kernel may touch must be a page of the pool
            spec = self.groups[g]
            first_page = spec.retention.first_kept_pages(starts, self.page_size)
            idx = np.arange(w, dtype=np.int64)[None, :]
            touched = (idx >= first_page[:, None]) & (idx <= last_page[:, None])
            ids = bt[:S][touched]
            if check_pages and ids.size and (ids.min() < 0 or ids.max() >= self.group_pages[g]):
                raise ValueError(f"cache group {g}: a block table names a page outside the pool of "
                                 f"{self.group_pages[g]} (or one that was given back) where the step reads or writes")
        if N and (tok[:N].min() < 0 or tok[:N].max() >= self.vocab_size):
            raise ValueError(f"token ids must lie in [0, {self.vocab_size})")
        facts = dict(S=S, N=N, M=M, Sp=Sp, Np=Np, Mp=Mp, q_lens=q_lens, widths=widths)
        return arr, off, facts

    def _context(self, meta: torch.Tensor, off, facts, seqs: Sequence[SeqStep]) -> StepContext:
        ctx = StepContext()
        def view(name):
            o, size = off[name]
            return meta[o:o + size]
        ctx.n_tokens, ctx.n_seqs, ctx.n_logit_rows = facts["Np"], facts["Sp"], facts["Mp"]
        ctx.token_ids = view("token_ids")
        ctx.positions = view("positions")
        ctx.token_seq = view("token_seq")
        ctx.cu_seqlens = view("cu_seqlens")
        ctx.context_lens = view("context_lens")
        ctx.state_slots = view("state_slots")
        ctx.logit_rows = view("logit_rows")
        ctx.block_tables = [view(f"bt{g}").view(facts["Sp"], w) for g, w in enumerate(facts["widths"])]
        ctx.q_lens = facts["q_lens"]
        ctx.starts = [s.start for s in seqs]
        ctx.host_state_slots = [s.state_slot for s in seqs]
        ctx.page_size = self.page_size
        ctx.attention_plan = AttentionPlan(
            decode_only=all(q == 1 for q in facts["q_lens"]),
            max_q_len=max(facts["q_lens"]) if facts["q_lens"] else 0,
            max_context_len=max((s.start + len(s.tokens) for s in seqs), default=0),
            n_seqs=facts["Sp"], q_lens=list(facts["q_lens"]) + [0] * (facts["Sp"] - facts["S"]),
            cu_seqlens=ctx.cu_seqlens, workspace=self.rt.workspace,
            kv_tokens=sum(s.start + len(s.tokens) for s in seqs),
            attention_pairs=sum(len(s.tokens) * s.start + len(s.tokens) * (len(s.tokens) + 1) // 2 for s in seqs))
        for call in range(len(self.plan.calls)):
            g = self.group_of_call.get(call)
            if g is not None:
                owner = self.plan.calls[call].cache_from
                ctx._kv[call] = KVView(self.kv_pages[call if owner is None else owner], ctx.block_tables[g],
                                       self.page_size)
            if call in self.state_tensors:
                ctx._state[call] = self.state_tensors[call]
        return ctx

    def _upload(self, arr: np.ndarray, dst: Optional[torch.Tensor] = None) -> torch.Tensor:
        n = arr.size
        host, idx = self._staging.take(n)
        host[:n].numpy()[:] = arr
        if dst is None:
            if self._meta_device is None or self._meta_device.numel() < n:
                self._meta_device = torch.empty(max(n, 1 << 16), dtype=torch.int32, device=self.device)
            dst = self._meta_device
        dst[:n].copy_(host[:n], non_blocking=True)
        self._staging.sent(idx)
        return dst

    # ------------------------------------------------------------------------------------
    # the step function
    # ------------------------------------------------------------------------------------
    @torch.inference_mode()
    def step(self, seqs: Sequence[SeqStep]) -> torch.Tensor:
        """Runs exactly the given tokens, as one batch, against the cache that earlier steps left,
        writes their keys and values into it and returns float32 logits [wanted, vocab] in the
        order of ``seqs`` and of each ``want``. The result lives in a buffer that the next step
        overwrites."""
        if not seqs:
            return torch.empty((0, self.vocab_size), dtype=torch.float32, device=self.device)
        self._validate(seqs)
        self._zero_new_states(seqs)
        if self._poison:
            self._flush_poison()
        S = len(seqs)
        decode_only = all(len(s.tokens) == 1 for s in seqs)
        if self.config.use_cuda_graph and self.model.graph_safe and S <= GRAPH_BUCKETS[-1]:
            if decode_only and all(len(s.want) == 1 for s in seqs):
                return self._step_graph(seqs)
            # prompt portions, alone or beside decoded tokens: short ones are bound by the host's
            # launches, so they are replayed from a graph of their size class too
            n_tokens = sum(len(s.tokens) for s in seqs)
            if (n_tokens <= min(self.config.prompt_graph_max_tokens, TOKEN_BUCKETS[-1])
                    and all(len(s.want) <= 1 for s in seqs)):
                return self._step_mixed_graph(seqs, n_tokens)
        arr, off, facts = self._fill(seqs)
        meta = self._upload(arr)
        ctx = self._context(meta, off, facts, seqs)
        return self.model.forward(ctx)

    def _zero_new_states(self, seqs: Sequence[SeqStep]) -> None:
        """A request that starts at position 0 starts from a cleared state: one indexed fill per
        state tensor, whatever the number of such requests."""
        if not self.has_state:
            return
        fresh = [s.state_slot for s in seqs if s.start == 0]
        if fresh:
            index = torch.tensor(fresh, dtype=torch.int64, device=self.device)
            for t in self.state_tensors.values():
                t.index_fill_(0, index, 0)

    def _context_cap(self, seqs: Sequence[SeqStep]) -> int:
        """The context length a decode graph is planned for: the next power of two (at least
        1024) above the longest context of the step. Kernels that split the keys choose their
        split for this length, so short contexts do not pay for the longest one."""
        longest = max(s.start + 1 for s in seqs)
        cap = 1024
        while cap < longest:
            cap *= 2
        return min(cap, max(self.config.max_model_len, 1))

    def _step_graph(self, seqs: Sequence[SeqStep]) -> torch.Tensor:
        S = len(seqs)
        bucket = next(b for b in GRAPH_BUCKETS if b >= S)
        cap = self._context_cap(seqs)
        widths = [self.max_pages_per_seq] * len(self.groups)
        arr, off, facts = self._fill(seqs, pad_to=bucket, bt_widths=widths)
        entry = self._graphs.get((bucket, cap))
        if entry is None:
            entry = self._capture(bucket, cap, arr, off, facts, seqs)
        graph, ctx, meta, logits = entry
        self._upload(arr, dst=meta)
        graph.replay()
        return logits[:S]

    def _step_mixed_graph(self, seqs: Sequence[SeqStep], n_tokens: int) -> torch.Tensor:
        """A step with prompt portions from the graph of its size class: tokens and sequences are
        padded with inert rows up to the class's sizes, the kernels' grids are those of the worst
        cut the class holds. A class is recorded at its first use."""
        S = len(seqs)
        Sp = next(b for b in GRAPH_BUCKETS if b >= S)
        Np = next(b for b in TOKEN_BUCKETS if b >= n_tokens)
        M = sum(len(s.want) for s in seqs)
        Mp = Sp if M else 0                      # no wanted row: the graph ends in front of the head
        longest = max(s.start + len(s.tokens) for s in seqs)
        cap = 1024
        while cap < longest:
            cap *= 2
        cap = min(cap, max(self.config.max_model_len, 1))
        widths = [self.max_pages_per_seq] * len(self.groups)
        arr, off, facts = self._fill(seqs, pad_to=Sp, pad_tokens=Np, pad_rows=Mp, bt_widths=widths)
        key = (Np, Sp, Mp, cap)
        entry = self._mixed_graphs.pop(key, None)
        if entry is None:
            entry = self._capture(Sp, cap, arr, off, facts, seqs, mixed_key=key)
            while len(self._mixed_graphs) >= MIXED_GRAPHS_KEPT:
                self._mixed_graphs.pop(next(iter(self._mixed_graphs)))
        self._mixed_graphs[key] = entry              # (the newest at the end)
        graph, ctx, meta, logits = entry
        self._upload(arr, dst=meta)
        graph.replay()
        return logits[:M]

    # ------------------------------------------------------------------------------------
    # a decode step run several times in a row on the device
    # ------------------------------------------------------------------------------------
    def can_repeat(self, num_seqs: int) -> bool:
        return bool(self.config.use_cuda_graph) and self.model.graph_safe and num_seqs <= GRAPH_BUCKETS[-1]

    def step_repeated(self, seqs: Sequence[SeqStep], repeat: int, temperature: np.ndarray, top_k: np.ndarray,
                      top_p: np.ndarray, seeds: np.ndarray, counters: np.ndarray) -> np.ndarray:
        """``launch_repeated`` and the wait for its tokens, int32 [repeat, len(seqs)]."""
        return self.launch_repeated(seqs, repeat, temperature, top_k, top_p, seeds, counters).tokens()

    def repeat_ready(self, seqs: Sequence[SeqStep], repeat: int, lookahead: int = 0) -> bool:
        """Whether the graph that ``launch_repeated`` would replay for these sequences, ``lookahead``
        positions further on, exists already (its first use captures it, which waits for the device)."""
        S = len(seqs)
        if not self.can_repeat(S):
            return False
        bucket = next(b for b in GRAPH_BUCKETS if b >= S)
        return (bucket, self._repeat_cap(seqs, repeat + lookahead), repeat) in self._repeat_graphs

    def _repeat_cap(self, seqs: Sequence[SeqStep], span: int) -> int:
        longest = max(s.start + span for s in seqs)
        cap = 1024
        while cap < longest:
            cap *= 2
        return min(cap, max(self.config.max_model_len, 1))

    @torch.inference_mode()
    def launch_repeated(self, seqs: Sequence[SeqStep], repeat: int, temperature: np.ndarray, top_k: np.ndarray,
                        top_p: np.ndarray, seeds: np.ndarray, counters: np.ndarray,
                        after: Optional["RepeatedRun"] = None) -> "RepeatedRun":
        """Runs a step of single decoded tokens ``repeat`` times in a row, as one graph: every run
        draws a token per sequence (per-sequence sampling arrays of length len(seqs); ``counters``
        is the index of the first token each sequence draws) and the next run takes it as its
        input at the next position. The sequences must hold pages for all ``repeat`` positions.
        Returns at once; the handle's ``tokens()`` waits for the drawn tokens.

        With ``after`` (the launch before, of the same sequences in the same order, possibly still
        running) the input tokens are not the ones in ``seqs`` but the last ones that launch drew,
        taken on the device: the host has not seen them yet. ``seqs`` then says where they go
        (``start`` = the position after that launch's last)."""
        S = len(seqs)
        if not self.can_repeat(S) or repeat < 1 or any(len(s.tokens) != 1 or list(s.want) != [0] for s in seqs):
            raise ValueError("a repeated step takes graph-sized batches of single tokens, each wanted")
        self._validate(seqs, lookahead=repeat - 1)
        self._zero_new_states(seqs)
        if self._poison:
            self._flush_poison()
        bucket = next(b for b in GRAPH_BUCKETS if b >= S)
        cap = self._repeat_cap(seqs, repeat)
        if after is not None and (after.bucket != bucket or after.count != S):
            raise ValueError("a launch that follows another takes the same sequences")
        widths = [self.max_pages_per_seq] * len(self.groups)
        # sampling arrays behind the step's integers: temperature, top_k, top_p, (seed, counter) pairs
        arr, off, facts = self._fill(seqs, pad_to=bucket, bt_widths=widths, lookahead=repeat - 1,
                                     extra_words=7 * bucket)
        o = off["extra"][0]                              # even: the 64-bit pairs come first
        rng = np.zeros((bucket, 2), dtype=np.int64)
        rng[:S, 0] = np.asarray(seeds, dtype=np.int64)
        rng[:S, 1] = np.asarray(counters, dtype=np.int64)
        arr[o:o + 4 * bucket] = rng.reshape(-1).view(np.int32)
        arr[o + 4 * bucket:o + 4 * bucket + S] = np.asarray(temperature, dtype=np.float32).view(np.int32)
        arr[o + 5 * bucket:o + 5 * bucket + S] = np.asarray(top_k, dtype=np.int32)
        tp = np.ones(bucket, dtype=np.float32)
        tp[:S] = np.asarray(top_p, dtype=np.float32)
        arr[o + 6 * bucket:o + 7 * bucket] = tp.view(np.int32)
        key = (bucket, cap, repeat)
        entry = self._repeat_graphs.get(key)
        if entry is None:
            entry = self._capture_repeated(key, arr, off, facts, seqs)
        graph, meta, tokens = entry
        self._upload(arr, dst=meta)
        if after is not None:
            o_tok = off["token_ids"][0]
            meta[o_tok:o_tok + bucket].copy_(after.device_tokens[after.repeat - 1])
        graph.replay()
        # the tokens go to pinned memory at once, before a later launch of the same graph overwrites them
        host = self._token_buffers[self._next_token_buffer]
        if host is None or host.numel() < tokens.numel():
            host = torch.empty(max(tokens.numel(), 4096), dtype=torch.int32, pin_memory=True)
            self._token_buffers[self._next_token_buffer] = host
        self._next_token_buffer = (self._next_token_buffer + 1) % len(self._token_buffers)
        host[:tokens.numel()].copy_(tokens.view(-1), non_blocking=True)
        done = torch.cuda.Event()
        done.record()
        return RepeatedRun(host, done, tokens, repeat, bucket, S)

    def _capture_repeated(self, key, arr: np.ndarray, off, facts, seqs: Sequence[SeqStep]):
        bucket, cap, repeat = key
        logger.info("capturing %d decode steps in a row for %d sequences, contexts up to %d", repeat, bucket, cap)
        if (bucket, cap) not in self._graphs:
            # the single-step capture sizes the shared scratch area and loads every kernel
            a1, o1, f1 = self._fill(seqs, pad_to=bucket, bt_widths=[self.max_pages_per_seq] * len(self.groups))
            self._capture(bucket, cap, a1, o1, f1, seqs)
        eager_workspace = self.rt.workspace
        self.ops.for_graph = True
        try:
            self.rt.workspace = self._graph_workspace
            meta = torch.empty(arr.size, dtype=torch.int32, device=self.device)
            self._upload(arr, dst=meta)
            ctx = self._context(meta, off, facts, seqs)
            ctx.attention_plan.max_context_len = cap
            o = off["extra"][0]
            rng = meta[o:o + 4 * bucket].view(torch.int64).view(bucket, 2)
            temps = meta[o + 4 * bucket:o + 5 * bucket].view(torch.float32)
            top_k = meta[o + 5 * bucket:o + 6 * bucket]
            top_p = meta[o + 6 * bucket:o + 7 * bucket].view(torch.float32)
            tokens = torch.zeros((repeat, bucket), dtype=torch.int32, device=self.device)
            logits = self.model.forward(ctx)       # an eager run: it draws into row 0 and changes nothing else
            self.ops.sample(logits[:bucket], tokens[0], temps, top_k, top_p, rng)
            torch.cuda.synchronize()
            self._graph_workspace.frozen = True
            advance = (ctx.token_ids, ctx.positions, ctx.context_lens)

            def body():
                for j in range(repeat):
                    logits = self.model.forward(ctx)
                    # the sampler feeds the next run itself: the drawn tokens, one position on
                    self.ops.sample(logits[:bucket], tokens[j], temps, top_k, top_p, rng,
                                    advance=advance if j + 1 < repeat else None)

            graph = self._record(body, key)
        finally:
            self._graph_workspace.frozen = False
            self.rt.workspace = eager_workspace
            self.ops.for_graph = False
        torch.cuda.synchronize()
        entry = (graph, meta, tokens)
        self._repeat_graphs[key] = entry
        return entry

    def _padding_step(self, bucket: int, tokens: Optional[int] = None) -> StepContext:
        """A context of ``bucket`` padding sequences and ``tokens`` padding rows (``bucket`` if not
        given): every kernel runs, none touches the cache."""
        widths = [self.max_pages_per_seq] * len(self.groups)
        dummy = [SeqStep(tokens=[0], start=0, block_tables=[[0]] * len(self.groups), state_slot=0, want=[0])]
        arr, off, facts = self._fill(dummy, pad_to=bucket, pad_tokens=tokens, bt_widths=widths)
        o, size = off["token_seq"]
        arr[o:o + size] = -1
        o, size = off["logit_rows"]
        arr[o:o + size] = -1
        o, size = off["cu_seqlens"]
        arr[o:o + size] = 0                        # no sequence has a token
        meta = torch.empty(arr.size, dtype=torch.int32, device=self.device)
        self._upload(arr, dst=meta)
        return self._context(meta, off, facts, dummy)

    def _prepare_graph_workspace(self) -> None:
        """One scratch area for all graphs, sized by steps of padding rows at the largest sizes the
        graphs serve (a decode step of the largest batch, a step with prompt portions of the largest
        size class); should a later graph need a larger buffer, the old one stays alive for the
        graphs that hold it."""
        if self._graph_workspace is not None:
            return
        eager_workspace, was_for_graph = self.rt.workspace, self.ops.for_graph
        self.ops.for_graph = True
        try:
            self._graph_workspace = Workspace(self.device, retain=True)
            self.rt.workspace = self._graph_workspace
            largest = next(b for b in GRAPH_BUCKETS if b >= min(self.config.max_num_batched_seqs, GRAPH_BUCKETS[-1]))
            pad_ctx = self._padding_step(largest)
            pad_ctx.attention_plan.max_context_len = self.config.max_model_len
            self.model.forward(pad_ctx)
            most = min(self.config.prompt_graph_max_tokens, self.config.max_num_batched_tokens, TOKEN_BUCKETS[-1])
            if most > largest:
                tokens = next(b for b in TOKEN_BUCKETS if b >= most)
                pad_ctx = self._padding_step(largest, tokens=tokens)
                plan = pad_ctx.attention_plan
                plan.decode_only, plan.max_q_len, plan.q_lens, plan.bound = False, tokens, (), (tokens, largest)
                plan.max_context_len = self.config.max_model_len
                self.model.forward(pad_ctx)
            torch.cuda.synchronize()
        finally:
            self.rt.workspace = eager_workspace
            self.ops.for_graph = was_for_graph

    def _record(self, body, key) -> torch.cuda.CUDAGraph:
        """Records ``body`` into a graph and looks at what was recorded: a graph with a memset node
        is not kept (such nodes have replayed wrongly on this platform; the engine's own kernels
        record none, a library product might). It is recorded again with the engine's own products
        only, and must be clean then."""
        for library in (True, False):
            self.ops.library_in_graphs = library
            if not library:
                # the engine's own products take over shapes the library had so far: run them once
                # outside a capture, where their kernels are loaded and their scratch may still grow
                was_frozen, self._graph_workspace.frozen = self._graph_workspace.frozen, False
                try:
                    body()
                    torch.cuda.synchronize()
                finally:
                    self._graph_workspace.frozen = was_frozen
            self.ops.ledger = []
            try:
                graph = torch.cuda.CUDAGraph(keep_graph=True)
                with torch.cuda.graph(graph, pool=self._graph_pool):
                    body()
            finally:
                self.ops.library_in_graphs = True
                self.graph_ledger[key], self.ops.ledger = self.ops.ledger, None
            census = self.ops.graph_census(graph.raw_cuda_graph())
            self.graph_census[key] = census
            if census["memset"] == 0:
                graph.instantiate()
                self._graph_pool = graph.pool()
                return graph
            logger.warning("the decode graph %s holds %d memset nodes%s", key, census["memset"],
                           "; recording it again without library products" if library else "")
            del graph
        raise RuntimeError(f"the decode graph {key} holds memset nodes although only the engine's kernels ran")

    def capture_graphs(self) -> int:
        """Records, ahead of serving, every decode graph the configuration can ask for: batch-size
        buckets up to ``max_num_batched_seqs``, context caps up to ``max_model_len``, single steps
        and rows of ``num_scheduler_steps`` (the reference records its buckets when the engine
        starts, minivllm/executor/graph.py:24-58). Otherwise a graph is recorded at its first use,
        which makes that step wait. Returns the number of graphs recorded."""
        caps, cap = [], 1024
        while True:
            caps.append(min(cap, max(self.config.max_model_len, 1)))
            if cap >= self.config.max_model_len:
                break
            cap *= 2
        limit = min(self.config.max_num_batched_seqs, GRAPH_BUCKETS[-1], self.num_state_slots)
        buckets = [b for b in GRAPH_BUCKETS if b <= limit]
        if limit not in buckets:
            buckets.append(next(b for b in GRAPH_BUCKETS if b >= limit))
        k = self.config.num_scheduler_steps
        made = 0
        tables = [[0]] * len(self.groups)
        for bucket in sorted(set(buckets), reverse=True):       # the largest first: it sizes the scratch area
            n = min(bucket, limit)
            for cap in sorted(set(caps)):
                # stand-in sequences whose context reaches the cap; the recorded launches depend on the
                # sizes only, never on these values
                start = max(0, min(cap, self.config.max_model_len) - max(k, 1))
                seqs = [SeqStep(tokens=[0], start=start, block_tables=tables, state_slot=i % self.num_state_slots,
                                want=[0]) for i in range(n)]
                widths = [self.max_pages_per_seq] * len(self.groups)
                if (bucket, cap) not in self._graphs:
                    arr, off, facts = self._fill(seqs, pad_to=bucket, bt_widths=widths, check_pages=False)
                    self._as_padding(arr, off)
                    self._capture(bucket, cap, arr, off, facts, seqs)
                    made += 1
                for repeat in ([k] if k > 1 else []):   # rows have the full length or the step runs once
                    if (bucket, cap, repeat) in self._repeat_graphs:
                        continue
                    arr, off, facts = self._fill(seqs, pad_to=bucket, bt_widths=widths, extra_words=7 * bucket,
                                                 check_pages=False)
                    self._as_padding(arr, off)
                    self._capture_repeated((bucket, cap, repeat), arr, off, facts, seqs)
                    made += 1
        logger.info("recorded %d decode graphs ahead of serving", made)
        return made

    @staticmethod
    def _as_padding(arr: np.ndarray, off) -> None:
        """Turns the rows of a packed step into padding rows: every kernel runs, none touches the cache."""
        for name, value in (("token_seq", -1), ("logit_rows", -1), ("cu_seqlens", 0), ("context_lens", 0)):
            o, size = off[name]
            arr[o:o + size] = value
        o, size = off["positions"]
        arr[o:o + size] = 0

    def _capture(self, bucket: int, cap: int, arr: np.ndarray, off, facts, seqs: Sequence[SeqStep],
                 mixed_key: Optional[Tuple[int, int, int, int]] = None):
        """Records the graph of a decode step of ``bucket`` sequences, or (``mixed_key`` = (tokens,
        sequences, logit rows, cap)) of a step with prompt portions of that size class."""
        if mixed_key is None:
            logger.info("capturing the decode graph for %d sequences, contexts up to %d", bucket, cap)
        else:
            logger.info("capturing the graph of steps of up to %d tokens of %d sequences, contexts up to %d",
                        mixed_key[0], mixed_key[1], cap)
        eager_workspace = self.rt.workspace
        self.ops.for_graph = True
        try:
            self._prepare_graph_workspace()
            self.rt.workspace = self._graph_workspace
            meta = torch.empty(arr.size, dtype=torch.int32, device=self.device)
            self._upload(arr, dst=meta)
            ctx = self._context(meta, off, facts, seqs)
            # the graph serves every context length up to its cap
            plan = ctx.attention_plan
            plan.max_context_len = cap
            if mixed_key is not None:
                # ... and every cut of its size class: nothing recorded may follow this step's own lengths
                plan.decode_only, plan.max_q_len, plan.q_lens = False, mixed_key[0], ()
                plan.bound = (mixed_key[0], mixed_key[1])
                ctx.q_lens = ctx.starts = ctx.host_state_slots = None
            self.model.forward(ctx)                # loads every kernel before the capture
            torch.cuda.synchronize()
            self._graph_workspace.frozen = True    # the eager run above sized everything: nothing is allocated now
            result = []
            graph = self._record(lambda: result.append(self.model.forward(ctx)),
                                 (bucket, cap) if mixed_key is None else ("mixed",) + mixed_key)
            logits = result[-1]
        finally:
            self._graph_workspace.frozen = False
            self.rt.workspace = eager_workspace
            self.ops.for_graph = False
        torch.cuda.synchronize()
        entry = (graph, ctx, meta, logits)
        if mixed_key is None:
            self._graphs[(bucket, cap)] = entry
        return entry
