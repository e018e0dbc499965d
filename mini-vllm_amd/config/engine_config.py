"""Engine-wide options.

Reference: minivllm/config/config.py:6-59. Names and meanings are the reference's where it
has them (``model``, ``max_model_len``, ``max_num_batched_tokens``, ``max_num_batched_seqs``,
``eos_token_ids``, ``kv_cache_num_blocks``, ``kv_cache_block_size``,
``gpu_memory_utilization``, ``use_cuda_graph``). Differences:

* ``max_model_len`` is enforced (the reference never checks it);
* ``kv_cache_num_blocks`` None sizes the cache from free device memory, a number is taken
  as given (the reference treats it as an upper cap, executor.py:46);
* ``use_cuda_graph`` keeps its name; the decode step is captured in a HIP graph;
* the executor never writes into this object (the reference's does, executor.py:49);
* ``prefill_chunk``, ``enable_prefix_caching``, ``num_scheduler_steps``, ``launch_ahead``, ``seed``,
  ``prompt_graph_max_tokens`` have no
  counterpart there (its scheduler runs whole prompts and one decoded token a step, scheduler.py:26-89).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple


COMPUTE_DTYPES = ("bfloat16", "float32")


def compute_dtype_name(engine_dtype: Optional[str], model_dtype: Optional[str], where: str = "config.json") -> str:
    """The precision the engine computes in: the engine option when it is given, else what the
    model's config.json names. The engine computes in bfloat16 or float32 only; a model that
    names anything else (float16) is served only when the caller states which of the two to use
    (the reference takes whatever config.json says, minivllm/executor/executor.py:17)."""
    from .model_config import ConfigError
    name = engine_dtype or model_dtype or "bfloat16"
    if name not in COMPUTE_DTYPES:
        raise ConfigError(f"{where}: the model names the dtype {name!r}; the engine computes in bfloat16 or float32 "
                          f"and picks neither silently: state dtype='bfloat16' or dtype='float32' (--dtype). Tensors "
                          f"stored in {name} are not converted on the way in either: a {name} checkpoint has to be "
                          f"saved again in bfloat16 or float32 before it can be served")
    return name


@dataclass
class EngineConfig:
    # ---- model -------------------------------------------------------------------------
    model: str = ""
    # compute precision: "bfloat16" (serving) or "float32" (everything in IEEE 32-bit);
    # None takes the model's own dtype from config.json
    dtype: Optional[str] = None
    # longest sequence (prompt + generated) a request may reach
    max_model_len: int = 4096

    # ---- scheduler ---------------------------------------------------------------------
    # most tokens in one step, prompt portions and decoded tokens together
    max_num_batched_tokens: int = 16384
    # most requests in one step
    max_num_batched_seqs: int = 512
    # most prompt tokens of one request in one step (None: only the token budget limits it)
    prefill_chunk: Optional[int] = None
    # None takes config.json's eos_token_id
    eos_token_ids: Optional[Tuple[int, ...]] = None

    # ---- cache -------------------------------------------------------------------------
    # pages of the cache pools: None sizes them from the memory left; a number gives every cache group
    # that many; a sequence names one count per group (a group that gives pages back early needs fewer)
    kv_cache_num_blocks: Optional[object] = None
    kv_cache_block_size: int = 16
    gpu_memory_utilization: float = 0.5
    enable_prefix_caching: bool = False

    # ---- executor ----------------------------------------------------------------------
    use_cuda_graph: bool = True
    # decode-only steps run this many times in a row on the device before the host looks at the
    # tokens (1: every step comes back to the host)
    num_scheduler_steps: int = 4
    # such a row of steps is launched before the tokens of the row that runs have been read, where
    # nothing but an end-of-sequence token could change what it holds (what ran on for a request
    # that ended is dropped)
    launch_ahead: bool = True
    # record every decode graph the configuration can ask for when the engine starts (the
    # reference does, minivllm/executor/graph.py:24-58) instead of at a graph's first use, which
    # makes that step wait for the recording
    capture_graphs_at_start: bool = False
    # steps that hold prompt portions (alone or beside decoded tokens) of up to this many tokens are
    # replayed from graphs too, recorded at first use per (token bucket, sequence bucket, context cap):
    # such steps are bound by the host's launches, not by the device (0: only decode steps use graphs)
    prompt_graph_max_tokens: int = 2048
    # debugging: fill a cache page with NaN when it is handed out for new content and (without
    # prefix reuse, which revives given-back pages) when its last holder gives it back, so that a
    # kernel that reads a slot nobody has written since, or a page that is no longer the request's,
    # shows in the logits
    debug_poison_pages: bool = False
    seed: int = 0

    def __post_init__(self) -> None:
        self.validate()

    def validate(self) -> None:
        if self.dtype not in (None, "bfloat16", "float32"):
            raise ValueError(f"dtype must be 'bfloat16' or 'float32', got {self.dtype!r}")
        if self.num_scheduler_steps < 1:
            raise ValueError(f"num_scheduler_steps must be >= 1, got {self.num_scheduler_steps}")
        if self.max_model_len < 1:
            raise ValueError(f"max_model_len must be >= 1, got {self.max_model_len}")
        if self.max_num_batched_tokens < 1:
            raise ValueError(f"max_num_batched_tokens must be >= 1, got {self.max_num_batched_tokens}")
        if self.max_num_batched_seqs < 1:
            raise ValueError(f"max_num_batched_seqs must be >= 1, got {self.max_num_batched_seqs}")
        if self.prompt_graph_max_tokens < 0:
            raise ValueError(f"prompt_graph_max_tokens must be >= 0, got {self.prompt_graph_max_tokens}")
        if self.prefill_chunk is not None and self.prefill_chunk < 1:
            raise ValueError(f"prefill_chunk must be >= 1, got {self.prefill_chunk}")
        if self.kv_cache_block_size < 1:
            raise ValueError(f"kv_cache_block_size must be >= 1, got {self.kv_cache_block_size}")
        if self.kv_cache_num_blocks is not None:
            counts = [self.kv_cache_num_blocks] if isinstance(self.kv_cache_num_blocks, int) else list(self.kv_cache_num_blocks)
            if not counts or any(not isinstance(n, int) or n < 1 for n in counts):
                raise ValueError(f"kv_cache_num_blocks must be >= 1 (one count, or one per cache group), "
                                 f"got {self.kv_cache_num_blocks}")
        if not (0.0 < self.gpu_memory_utilization <= 1.0):
            raise ValueError(f"gpu_memory_utilization must be in (0, 1], got {self.gpu_memory_utilization}")
        if self.eos_token_ids is not None:
            self.eos_token_ids = tuple(int(e) for e in self.eos_token_ids)
