"""The scheduler: admits requests, cuts prompts into portions under a token budget, lets
running requests decode beside them, finishes and frees.

Reference: minivllm/scheduler/scheduler.py. Kept: ``waiting`` and ``running`` queues, first
come first served with head-of-line blocking at admission (scheduler.py:41-56), the limits
``max_num_batched_seqs`` and ``max_num_batched_tokens``, preemption by recomputation of the
newest running request when a decoding request cannot get a page, or of the request itself if
it is the last (scheduler.py:66-72,91-98), finishing on ``max_tokens`` or an end-of-sequence
token unless ``ignore_eos`` (scheduler.py:101-110, the end token stays in the output).

Changed: a step is one mixed batch. Every running request whose prompt is in the cache brings
one token; what is left of the token budget goes to prompt portions, first of requests in the
middle of their prompt, then of newly admitted ones (the reference runs whole prompts only,
in steps of their own, scheduler.py:83-89, and never schedules a prompt above the budget).
Pages are reserved per portion.

When pages run out:
  * a decoding request that cannot get its next page preempts the newest running request
    (its pages are given back, it returns to the front of the waiting queue and is later
    recomputed from its prompt plus what it had generated); if it is the only one, itself;
  * a prompt portion shrinks to what the free pages hold, or waits for a later step;
  * if a step would be empty although requests are running, the newest running one is
    preempted so that the others can go on;
  * a request that could never fit the pool, or exceeds ``max_model_len``, is refused at submit.

A step that holds only decoded tokens may be marked to run several times in a row
(``ScheduledStep.repeat``, at most ``max_decode_repeat``): the device feeds each run the tokens
the run before drew, and the host schedules, uploads and reads back once for all of them. It is
used only while nobody waits, and never past a request's ``max_tokens``; tokens run past an
end-of-sequence token are dropped. The reference schedules one token per step.
"""
from __future__ import annotations

import time
from collections import deque
from dataclasses import dataclass, field
from typing import Deque, List, Optional, Sequence

from ..cache.manager import CacheManager
from .request import Request, RequestState


@dataclass
class ScheduledSeq:
    request: Request
    start: int            # position of the first token run in this step
    num_tokens: int       # how many of the request's tokens run
    sample: bool          # the portion reaches the request's last token: a new token is drawn

    @property
    def is_decode(self) -> bool:
        return self.num_tokens == 1 and self.start >= self.request.prompt_token_count


@dataclass
class ScheduledStep:
    seqs: List[ScheduledSeq]
    create_time: float = field(default_factory=time.perf_counter)
    # A step of decoded tokens only may be run ``repeat`` times in a row on the device, each run
    # taking the tokens the run before drew: the host then works once per ``repeat`` tokens.
    repeat: int = 1

    @property
    def num_tokens(self) -> int:
        return sum(s.num_tokens for s in self.seqs) * self.repeat

    @property
    def requests(self) -> List[Request]:
        return [s.request for s in self.seqs]


class Scheduler:
    def __init__(self, manager: CacheManager, max_num_batched_tokens: int, max_num_batched_seqs: int,
                 max_model_len: int, eos_token_ids: Sequence[int] = (), prefill_chunk: Optional[int] = None,
                 max_decode_repeat: int = 1):
        self.manager = manager
        self.max_decode_repeat = max(1, int(max_decode_repeat))
        self.max_num_batched_tokens = max_num_batched_tokens
        self.max_num_batched_seqs = max_num_batched_seqs
        self.max_model_len = max_model_len
        self.eos_token_ids = frozenset(eos_token_ids)
        self.prefill_chunk = prefill_chunk
        self.waiting: Deque[Request] = deque()
        self.running: Deque[Request] = deque()
        self.num_preemptions = 0

    # ------------------------------------------------------------------------------------
    @property
    def finished(self) -> bool:
        return not self.waiting and not self.running

    def submit(self, req: Request) -> None:
        total = req.prompt_token_count + req.sampling_params.max_tokens
        if req.prompt_token_count >= self.max_model_len:
            raise ValueError(f"the prompt has {req.prompt_token_count} tokens; max_model_len "
                             f"{self.max_model_len} leaves no room to generate")
        longest = min(total, self.max_model_len)
        for g, spec in enumerate(self.manager.groups):
            pages = spec.retention.most_pages(longest, self.manager.page_size)
            if pages is not None and pages > self.manager.pools[g].num_pages:
                raise ValueError(f"the request may reach {longest} tokens = {pages} cache pages, the pool "
                                 f"has {self.manager.pools[g].num_pages}")
        self.waiting.append(req)

    def _computed(self, req: Request) -> int:
        return self.manager.sequence(req.id).num_computed

    def preempt(self, req: Request) -> None:
        """Back to the front of the waiting queue; everything it holds is given back and will
        be recomputed (scheduler.py:91-98)."""
        req.state = RequestState.WAITING
        req.num_preemptions += 1
        self.num_preemptions += 1
        self.manager.release(req.id)
        self.running.remove(req)
        self.waiting.appendleft(req)

    # ------------------------------------------------------------------------------------
    def _try_schedule(self) -> List[ScheduledSeq]:
        budget = self.max_num_batched_tokens
        seqs: List[ScheduledSeq] = []
        scheduled_ids = set()

        # 1. running requests that are decoding bring one token each
        for req in list(self.running):
            if req.state != RequestState.RUNNING:
                continue                                    # preempted while serving an earlier one
            if len(seqs) >= self.max_num_batched_seqs or budget <= 0:
                break
            start = self._computed(req)
            if len(req.tokens) - start != 1:
                continue
            while not (self.manager.fits(req.id, 1) or self.manager.can_reserve(req.id, 1)):
                victim = self.running[-1]
                if victim is req or victim.id in scheduled_ids:
                    # nothing newer to take pages from (those already in this step keep theirs)
                    victim = next((r for r in reversed(self.running)
                                   if r is not req and r.id not in scheduled_ids), req)
                self.preempt(victim)
                if victim is req:
                    break
            if req.state != RequestState.RUNNING:
                continue
            if not self.manager.fits(req.id, 1):
                self.manager.reserve(req.id, 1)
            seqs.append(ScheduledSeq(req, start, 1, sample=True))
            scheduled_ids.add(req.id)
            budget -= 1

        # 2. running requests in the middle of their prompt (or of a recomputation)
        for req in list(self.running):
            if len(seqs) >= self.max_num_batched_seqs or budget <= 0:
                break
            if req.id in scheduled_ids or req.state != RequestState.RUNNING:
                continue
            n = self._portion(req, budget)
            if n <= 0:
                continue
            start = self._computed(req)
            self.manager.reserve(req.id, n)
            seqs.append(ScheduledSeq(req, start, n, sample=(start + n == len(req.tokens))))
            scheduled_ids.add(req.id)
            budget -= n

        # 3. new requests, first come first served; the first that does not fit blocks the rest
        while self.waiting and len(seqs) < self.max_num_batched_seqs and budget > 0 \
                and len(self.running) < self.max_num_batched_seqs:
            req = self.waiting[0]
            if not self.manager.can_admit():
                break
            self.manager.admit(req.id, req.tokens)
            n = self._portion(req, budget)
            if n <= 0:
                self.manager.release(req.id)
                break
            start = self._computed(req)
            self.manager.reserve(req.id, n)
            self.waiting.popleft()
            req.state = RequestState.RUNNING
            self.running.append(req)
            seqs.append(ScheduledSeq(req, start, n, sample=(start + n == len(req.tokens))))
            scheduled_ids.add(req.id)
            budget -= n
        return seqs

    def _portion(self, req: Request, budget: int) -> int:
        remaining = len(req.tokens) - self._computed(req)
        n = min(remaining, budget, self.manager.reservable_tokens(req.id))
        if self.prefill_chunk is not None:
            n = min(n, self.prefill_chunk)
        return n

    def _decode_repeat(self, seqs: List[ScheduledSeq]) -> int:
        """How many times in a row the step may run: more than once only when it holds nothing
        but decoded tokens, nobody waits to be admitted or to go on with a prompt, and every
        request has that many tokens to go and the pages for them (they are reserved here). A row has
        the full length or the step runs once: the executor then needs two graphs per batch size and
        context cap, not one for every length in between (the last few tokens of a request go step by step)."""
        k = self.max_decode_repeat
        if k <= 1 or self.waiting or len(seqs) != len(self.running) or not all(s.is_decode for s in seqs):
            return 1
        for s in seqs:
            r = s.request
            k = min(k, r.sampling_params.max_tokens - r.num_completion_tokens, self.max_model_len - len(r.tokens))
        while k > 1:
            # one position each is reserved already; the others must fit together
            extra = [self.manager.pages_needed(s.request.id, k) for s in seqs]
            if all(sum(e[g] for e in extra) <= self.manager.pools[g].num_free for g in range(len(self.manager.groups))):
                break
            k -= 1
        if k < self.max_decode_repeat:
            return 1
        for s in seqs:
            self.manager.reserve(s.request.id, k)
        return k

    def schedule_ahead(self, prev: ScheduledStep) -> Optional[ScheduledStep]:
        """The step after ``prev`` while ``prev`` is still running and its tokens are unknown: the
        same requests, ``prev.repeat`` positions further on, again ``prev.repeat`` runs in a row.
        Only when that is what ``schedule`` would decide whatever the tokens turn out to be, short of
        a request ending on an end-of-sequence token: nobody waits, ``prev`` holds every running
        request as a decoded token, every request has the tokens of both steps to go, and the pages
        for them are free (they are reserved here). None otherwise; nothing is changed then.
        What such a step computes for a request that ``prev`` ends is dropped by ``update``."""
        k = prev.repeat
        if k <= 1 or k != self.max_decode_repeat or self.waiting or len(prev.seqs) != len(self.running):
            return None
        for s in prev.seqs:
            r = s.request
            if r.state != RequestState.RUNNING or not s.is_decode or not s.sample:
                return None
            if min(r.sampling_params.max_tokens - r.num_completion_tokens, self.max_model_len - len(r.tokens)) < 2 * k:
                return None
        extra = [self.manager.pages_needed(s.request.id, 2 * k) for s in prev.seqs]
        for g in range(len(self.manager.groups)):
            if sum(e[g] for e in extra) > self.manager.pools[g].num_free:
                return None
        for s in prev.seqs:
            self.manager.reserve(s.request.id, 2 * k)
        return ScheduledStep([ScheduledSeq(s.request, s.start + k, 1, sample=True) for s in prev.seqs], repeat=k)

    def schedule(self) -> Optional[ScheduledStep]:
        """The next step, or None when nothing is left to do."""
        while True:
            seqs = self._try_schedule()
            if seqs:
                if all(s.is_decode for s in seqs):
                    # longest context first: a decode step's attention starts its workgroups in this
                    # order, and the ones with most keys to read should not be the last to start
                    # (256 requests with contexts of 400 to 2,300 tokens: 3 % more tokens a second)
                    seqs.sort(key=lambda s: -s.start)
                return ScheduledStep(seqs, repeat=self._decode_repeat(seqs))
            if self.running:
                # everyone is stuck waiting for pages: the newest gives way
                self.preempt(self.running[-1])
                continue
            if self.waiting:
                raise RuntimeError("the first waiting request fits neither the free pages nor the token budget "
                                   "although nothing is running")
            return None

    # ------------------------------------------------------------------------------------
    def update(self, step: ScheduledStep, sampled: Sequence[Optional[int]]) -> List[Request]:
        """Records the step: progress of every sequence, the drawn token of those that sampled
        (``sampled`` has one entry per sequence, None where nothing was drawn). Returns the
        requests that finished."""
        done: List[Request] = []
        now = time.perf_counter()
        for seq, drawn in zip(step.seqs, sampled):
            req = seq.request
            if req.state == RequestState.FINISHED:
                continue          # a step scheduled ahead ran on for a request that the step before ended
            if not seq.sample:
                self.manager.commit(req.id, seq.num_tokens, req.tokens)
                continue
            if drawn is None:
                raise ValueError(f"request {req.id} reached its last token but no token was drawn")
            tokens = [drawn] if isinstance(drawn, int) else [int(t) for t in drawn]
            if len(tokens) != step.repeat:
                raise ValueError(f"request {req.id}: the step ran {step.repeat} times but {len(tokens)} tokens came back")
            # how many of the drawn tokens the request keeps: up to the one that ends it (what the
            # device ran past a request's end is dropped with its pages)
            sp = req.sampling_params
            keep, reason = len(tokens), None
            for j, token in enumerate(tokens):
                if token in self.eos_token_ids and not sp.ignore_eos:
                    reason = "stop"
                elif req.num_completion_tokens + j + 1 >= sp.max_tokens:
                    reason = "length"
                elif len(req.tokens) + j + 1 >= self.max_model_len:
                    reason = "length"
                if reason is not None:
                    keep = j + 1
                    break
            for token in tokens[:keep]:
                req.append_output_token(token)
            if req.first_token_time is None:
                req.first_token_time = now
            # the run that drew token j wrote the position(s) before it
            self.manager.commit(req.id, seq.num_tokens + keep - 1, req.tokens)
            if reason is not None:
                req.state = RequestState.FINISHED
                req.finish_reason = reason
                req.finish_time = now
                self.manager.release(req.id)
                self.running.remove(req)
                done.append(req)
        return done
