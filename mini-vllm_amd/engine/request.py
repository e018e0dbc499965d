"""A generation request and what is returned for it.

Reference: minivllm/engine/request.py:7-47 — states WAITING / RUNNING / FINISHED, a global id
counter, ``tokens`` = prompt followed by generated tokens, views of both parts. Here each
request owns its ``SamplingParams`` (the reference shares one default instance between
requests, request.py:14), and the pages it holds are kept by the cache manager, not here.
"""
from __future__ import annotations

import copy
import enum
import time
from dataclasses import dataclass
from itertools import count
from typing import List, Optional

from ..config.sampling_params import SamplingParams


class RequestState(enum.Enum):
    WAITING = 0
    RUNNING = 1
    FINISHED = 2


class Request:
    _counter = count()

    def __init__(self, prompt_token_ids: List[int], sampling_params: Optional[SamplingParams] = None):
        if len(prompt_token_ids) == 0:
            raise ValueError("a request needs at least one prompt token")
        self.id = next(Request._counter)
        self.state = RequestState.WAITING
        self.prompt_token_count = len(prompt_token_ids)
        self.tokens: List[int] = list(prompt_token_ids)
        self.sampling_params = copy.copy(sampling_params) if sampling_params is not None else SamplingParams()
        self.finish_reason: Optional[str] = None
        self.num_preemptions = 0
        self.arrival_time = time.perf_counter()
        self.first_token_time: Optional[float] = None
        self.finish_time: Optional[float] = None

    def __len__(self) -> int:
        return len(self.tokens)

    @property
    def finished(self) -> bool:
        return self.state == RequestState.FINISHED

    def append_output_token(self, token: int) -> None:
        self.tokens.append(int(token))

    @property
    def prompt_tokens(self) -> List[int]:
        return self.tokens[:self.prompt_token_count]

    @property
    def completion_tokens(self) -> List[int]:
        return self.tokens[self.prompt_token_count:]

    @property
    def num_completion_tokens(self) -> int:
        return len(self.tokens) - self.prompt_token_count


@dataclass
class RequestOutput:
    request_id: int
    prompt_token_ids: List[int]
    token_ids: List[int]
    finish_reason: Optional[str]
    prompt: Optional[str] = None
    text: Optional[str] = None

    # the reference's generate() returns dictionaries with these keys (minivllm/engine/engine.py:79-84)
    def __getitem__(self, key: str):
        if key == "prompt":
            return self.prompt
        if key == "completion":
            return self.text
        if key == "tokens":
            return self.token_ids
        raise KeyError(key)
