"""The Python entry point: ``LLM(model=...).generate(prompts, sampling_params)``.

Reference: minivllm/engine/engine.py — ``Engine(config)`` with ``submit`` / ``step`` /
``finished`` / ``generate``; ``generate`` takes prompts as lists of token ids and one
``SamplingParams`` or a list, steps until everything finished and returns, in order of
submission, one record per request with the keys ``prompt``, ``completion`` and ``tokens``
(engine.py:40-90). Those names are kept (``RequestOutput`` also answers to them); prompts may
also be strings when the model folder holds a tokenizer. ``step`` runs one mixed batch:
schedule, execute, sample, update. A batch of decoded tokens only may run several times in a row
on the device, and the row after it may be launched while it runs (``EngineConfig.launch_ahead``);
``step`` still returns one finished step per call, in order.
"""
from __future__ import annotations

import logging
import time
from typing import Dict, List, Optional, Sequence, Tuple, Union


from ..config.engine_config import EngineConfig
from ..config.sampling_params import SamplingParams
from ..sampling.sampler import Sampler, request_seed
from .executor import Executor
from .metrics import Metrics
from .request import Request, RequestOutput, RequestState
from .scheduler import ScheduledStep, Scheduler
from .step import SeqStep

logger = logging.getLogger(__name__)


def _load_tokenizer(model_dir: str):
    """The tokenizer stored in the model folder, or None (random-weight models have none)."""
    import os
    if not model_dir or not any(os.path.isfile(os.path.join(model_dir, f))
                                for f in ("tokenizer.json", "tokenizer_config.json", "vocab.json")):
        return None
    try:
        from transformers import AutoTokenizer
        return AutoTokenizer.from_pretrained(model_dir, use_fast=True)
    except Exception as e:  # a tokenizer is optional
        logger.warning("could not load a tokenizer from %s: %s", model_dir, e)
        return None


class LLM:
    def __init__(self, model: Optional[str] = None, config: Optional[EngineConfig] = None,
                 model_source: Optional[Tuple] = None, **options):
        """``LLM(model="/path", max_num_batched_tokens=2048, ...)`` or ``LLM(config=EngineConfig(...))``.
        ``model_source`` = (architecture, model config, tensor source) serves tensors that are not
        in a folder."""
        if config is None:
            config = EngineConfig(model=model or "", **options)
        elif model is not None or options:
            raise ValueError("give either a config or a model path with options")
        self.config = config
        self.tokenizer = _load_tokenizer(config.model)
        self.executor = Executor(config, model=model_source)
        self.manager = self.executor.new_cache_manager()
        eos = config.eos_token_ids
        if eos is None:
            eos = tuple(getattr(self.executor.model_config, "eos_token_ids", ()))
        self.scheduler = Scheduler(self.manager, config.max_num_batched_tokens, config.max_num_batched_seqs,
                                   config.max_model_len, eos, config.prefill_chunk,
                                   max_decode_repeat=config.num_scheduler_steps)
        self.sampler = Sampler(self.executor.ops, self.executor.device)
        self.metrics = Metrics()
        self._seeds: Dict[int, int] = {}
        # a row of decode steps that was launched ahead and is waited for by the next step():
        # (scheduled step, the executor's handle, the seeds of its requests)
        self._in_flight = None

    # ---- the reference's streaming interface ---------------------------------------------
    def submit(self, tokens: Sequence[int], sampling_params: Optional[SamplingParams] = None) -> Request:
        req = Request(list(tokens), sampling_params)
        vocab = self.executor.vocab_size
        if any((t < 0 or t >= vocab) for t in req.tokens):
            raise ValueError(f"prompt token ids must lie in [0, {vocab})")
        self.scheduler.submit(req)
        self._seeds[req.id] = request_seed(self.config.seed, req.id, req.sampling_params)
        return req

    add_request = submit

    @property
    def finished(self) -> bool:
        return self.scheduler.finished

    def has_unfinished(self) -> bool:
        return not self.scheduler.finished

    def step(self) -> Optional[ScheduledStep]:
        """One step of the engine: schedule, run the batch, draw tokens, record them."""
        t0 = time.perf_counter()
        run = None
        self.drain()                                 # a row whose requests have all ended is waited for and forgotten
        if self._in_flight is not None:
            step, run = self._in_flight
            self._in_flight = None
        if run is None:
            step = self.scheduler.schedule()
            if step is None:
                return None
            seqs = self._seq_steps(step)
            if step.repeat > 1 and self.executor.can_repeat(len(seqs)):
                run = self.executor.launch_repeated(seqs, step.repeat, *self._sampling_arrays(step))
        if run is not None:
            self._launch_ahead(step, run)
            drawn = run.tokens()
            sampled = [[int(t) for t in drawn[:, i]] for i in range(len(step.seqs))]
        elif step.repeat > 1:
            sampled = self._run_repeated(step, seqs)
        else:
            logits = self.executor.step(seqs)
            drawing = [s.request for s in step.seqs if s.sample]
            tokens = self.sampler.sample(logits, [r.sampling_params for r in drawing],
                                         [self._seeds[r.id] for r in drawing],
                                         [r.num_completion_tokens for r in drawing])
            it = iter(tokens)
            sampled = [next(it) if s.sample else None for s in step.seqs]
        done = self.scheduler.update(step, sampled)
        for r in done:
            self._seeds.pop(r.id, None)
        self.metrics.update(step, done, time.perf_counter() - t0)
        self.metrics.preemptions = self.scheduler.num_preemptions
        step.finished = done
        return step

    def drain(self) -> None:
        """Waits for decode steps that were launched ahead for requests that have all ended since
        (their tokens are dropped). ``step()`` does the same when it is called again."""
        if self._in_flight is not None and all(r.state == RequestState.FINISHED for r in self._in_flight[0].requests):
            self._in_flight[1].tokens()
            self._in_flight = None

    def _seq_steps(self, step: ScheduledStep, further: int = 0) -> List[SeqStep]:
        """What the executor runs for a scheduled step. ``further``: the step was scheduled ahead of
        one that draws that many tokens per request first; its own input tokens are on the device."""
        groups = range(len(self.manager.groups))
        seqs = []
        for s in step.seqs:
            r = s.request
            cache = self.manager.sequence(r.id)
            tokens = [0] * s.num_tokens if further else r.tokens[s.start:s.start + s.num_tokens]
            seqs.append(SeqStep(tokens=tokens, start=s.start, block_tables=[cache.table(g) for g in groups],
                                state_slot=cache.state_slot, want=[s.num_tokens - 1] if s.sample else []))
        return seqs

    def _sampling_arrays(self, step: ScheduledStep, further: int = 0):
        reqs = step.requests
        return Sampler.arrays([r.sampling_params for r in reqs], [self._seeds[r.id] for r in reqs],
                              [r.num_completion_tokens + further for r in reqs])

    def _launch_ahead(self, step: ScheduledStep, run) -> None:
        """While ``run`` (the decode steps of ``step``) is on the device and its tokens are unknown:
        launches the steps after it, if the scheduler can tell what they hold and their graph
        exists; the next ``step()`` waits for them."""
        if not self.config.launch_ahead:
            return
        probe = [SeqStep(tokens=[0], start=s.start + step.repeat, block_tables=[], state_slot=0, want=[0])
                 for s in step.seqs]
        if not self.executor.repeat_ready(probe, step.repeat):
            return                                   # its first use captures the graph, which waits for the device
        ahead = self.scheduler.schedule_ahead(step)
        if ahead is None:
            return
        seqs = self._seq_steps(ahead, further=step.repeat)
        nxt = self.executor.launch_repeated(seqs, ahead.repeat, *self._sampling_arrays(ahead, further=step.repeat),
                                            after=run)
        self._in_flight = (ahead, nxt)

    def _run_repeated(self, step: ScheduledStep, seqs: List[SeqStep]) -> List[List[int]]:
        """A step of decoded tokens that runs ``step.repeat`` times in a row where the executor
        offers no graph for it: run by run from here. Returns the tokens each sequence drew, in
        order."""
        reqs = step.requests
        params = [r.sampling_params for r in reqs]
        seeds = [self._seeds[r.id] for r in reqs]
        counters = [r.num_completion_tokens for r in reqs]
        out: List[List[int]] = [[] for _ in seqs]
        for j in range(step.repeat):
            if j:
                seqs = [SeqStep(tokens=[out[i][-1]], start=s.start + 1, block_tables=s.block_tables,
                                state_slot=s.state_slot, want=[0]) for i, s in enumerate(seqs)]
            logits = self.executor.step(seqs)
            tokens = self.sampler.sample(logits, params, seeds, [c + j for c in counters])
            for i, t in enumerate(tokens):
                out[i].append(int(t))
        return out

    # ---- batch generation ---------------------------------------------------------------------
    def _encode(self, prompt: Union[str, Sequence[int]]) -> List[int]:
        if isinstance(prompt, str):
            if self.tokenizer is None:
                raise ValueError("a text prompt needs a tokenizer in the model folder; pass token ids instead")
            return list(self.tokenizer.encode(prompt))
        return list(prompt)

    def generate(self, prompts: Sequence[Union[str, Sequence[int]]],
                 sampling_params: Union[SamplingParams, Sequence[SamplingParams], None] = None,
                 use_tqdm: bool = True) -> List[RequestOutput]:
        if sampling_params is None:
            sampling_params = SamplingParams()
        if not isinstance(sampling_params, (list, tuple)):
            sampling_params = [sampling_params] * len(prompts)
        if len(sampling_params) != len(prompts):
            raise ValueError("one SamplingParams per prompt is needed")
        requests = [self.submit(self._encode(p), sp) for p, sp in zip(prompts, sampling_params)]
        pbar = None
        if use_tqdm:
            try:
                from tqdm.auto import tqdm
                pbar = tqdm(total=len(prompts), desc="Generating", dynamic_ncols=True)
            except ImportError:
                pbar = None
        finished_before = self.metrics.finished_request_count
        while not self.finished:
            self.step()
            if pbar is not None:
                s = self.metrics.stats()
                pbar.set_postfix({"Prefill(token/s)": f"{s.prefill_throughput:4.0f}",
                                  "Decode(token/s)": f"{s.decode_throughput:4.0f}",
                                  "TTFT": f"{s.time_to_first_token:4.2f}", "ITL": f"{s.inter_token_latency:4.4f}",
                                  "TPS": f"{s.tokens_per_second:4.2f}", "RPS": f"{s.requests_per_second:4.2f}"})
                pbar.update(s.finished_requests - finished_before - pbar.n)
        if pbar is not None:
            pbar.close()
        self.drain()
        return [self._output(r) for r in sorted(requests, key=lambda r: r.id)]

    def _output(self, r: Request) -> RequestOutput:
        prompt_text = completion_text = None
        if self.tokenizer is not None:
            prompt_text = self.tokenizer.decode(r.prompt_tokens)
            completion_text = self.tokenizer.decode(r.completion_tokens)
        return RequestOutput(request_id=r.id, prompt_token_ids=r.prompt_tokens, token_ids=r.completion_tokens,
                             finish_reason=r.finish_reason, prompt=prompt_text, text=completion_text)
