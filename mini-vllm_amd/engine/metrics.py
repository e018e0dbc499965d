"""Running figures of the engine.

Reference: minivllm/engine/metrics.py — the same seven figures under the same names
(``prefill_throughput``, ``decode_throughput``, ``time_to_first_token``,
``inter_token_latency``, ``tokens_per_second``, ``requests_per_second``,
``finished_requests``). A step may hold prompt portions and decoded tokens together; its time
is shared between the two kinds in proportion to their token counts. Time to first token is
measured per request from submission, finished requests are counted in whichever step they
finish, and ``reset`` clears everything (the reference counts prompt tokens after the sampled
token was appended, metrics.py:38, counts finishes only in decode steps, :45-47, and keeps the
token counters across a reset, :49-55).
"""
from __future__ import annotations

import time
from dataclasses import dataclass


@dataclass
class Stats:
    prefill_throughput: float = 0.0
    decode_throughput: float = 0.0
    time_to_first_token: float = 0.0
    inter_token_latency: float = 0.0
    tokens_per_second: float = 0.0
    requests_per_second: float = 0.0
    finished_requests: int = 0
    steps: int = 0
    preemptions: int = 0


class Metrics:
    def __init__(self):
        self.reset()

    def reset(self) -> None:
        self.prefill_time = 0.0
        self.prefill_tokens = 0
        self.decode_time = 0.0
        self.decode_tokens = 0
        self.decode_steps = 0
        self.steps = 0
        self.finished_request_count = 0
        self.ttft_sum = 0.0
        self.ttft_count = 0
        self.preemptions = 0
        self.start_time = time.perf_counter()

    def update(self, step, finished, elapsed: float) -> None:
        """``step`` is the ScheduledStep that ran, ``finished`` the requests it completed,
        ``elapsed`` its wall time in seconds."""
        repeat = getattr(step, "repeat", 1)     # a decode-only step may have run several times in a row
        prefill = sum(s.num_tokens for s in step.seqs if not s.is_decode)
        decode = sum(s.num_tokens for s in step.seqs if s.is_decode) * repeat
        total = max(1, prefill + decode)
        self.prefill_time += elapsed * prefill / total
        self.decode_time += elapsed * decode / total
        self.prefill_tokens += prefill
        self.decode_tokens += decode
        self.decode_steps += repeat if decode else 0
        self.steps += 1
        for s in step.seqs:
            r = s.request
            if s.sample and r.num_completion_tokens == 1 and r.first_token_time is not None:
                self.ttft_sum += r.first_token_time - r.arrival_time
                self.ttft_count += 1
        self.finished_request_count += len(finished)

    def stats(self) -> Stats:
        elapsed = time.perf_counter() - self.start_time
        tokens = self.prefill_tokens + self.decode_tokens
        return Stats(
            prefill_throughput=self.prefill_tokens / self.prefill_time if self.prefill_time > 0 else 0.0,
            decode_throughput=self.decode_tokens / self.decode_time if self.decode_time > 0 else 0.0,
            time_to_first_token=self.ttft_sum / self.ttft_count if self.ttft_count else 0.0,
            inter_token_latency=self.decode_time / self.decode_steps if self.decode_steps else 0.0,
            tokens_per_second=tokens / elapsed if elapsed > 0 else 0.0,
            requests_per_second=self.finished_request_count / elapsed if elapsed > 0 else 0.0,
            finished_requests=self.finished_request_count,
            steps=self.steps,
            preemptions=self.preemptions,
        )
