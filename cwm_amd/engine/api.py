"""Options and request/response records, with the reference's names and meanings.

`GenArgs` follows cwm/fastgen/generate.py:37-68 and `Packet` follows
cwm/fastgen/api.py:11-37.  Options that belong to parts this engine does not have
(host prefix cache, CUDA graph buckets, the prefill batching thresholds) are kept
so that a reference configuration still parses; they must hold their neutral
value or are ignored as noted.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, List, Optional


@dataclass
class GenArgs:
    # sampling defaults, each can be overridden per request
    use_sampling: bool = True  # False: greedy argmax for every request
    temperature: float = 0.7  # 0 means greedy for that request (the reference divides by it)
    top_p: float = 1.0

    logprobs: bool = False  # return log-probabilities of the generated tokens
    prompt_logprobs: bool = False  # also of the prompt's tokens (positions 1..)

    max_batch: int = 128  # most requests live at a time
    max_seq: int = -1  # tokens of cache in total, and the longest a sequence may get; negative: from free memory
    max_gen: Optional[int] = None  # most new tokens of a request

    host_cache_gb: float = 0  # host prefix cache: not built, must be 0
    num_cuda_graphs: int = 16  # decode steps kept as HIP graphs, one per number of requests (the reference: one per bucket of
    # batch sizes); 0, or FG_NO_CUDA_GRAPHS in the environment: every step is launched kernel by kernel
    cache_block: int = 256  # tokens in a page
    max_prefill: int = 4096  # token budget of one step
    min_prefill: int = 512  # reference batching threshold: not needed with mixed steps, ignored
    min_prefill_batch: int = 8  # likewise ignored

    expected_seq: int = -1  # not in the reference: tokens a typical request holds; how free memory is split between
    # layer groups when max_seq is negative (negative: the context length the model's configuration names)
    prefill_gb: float = 2  # memory kept free for activations when max_seq is negative
    gpu_gb: float = 74  # the reference's memory budget: ignored, free memory is measured

    sync_freq: int = 10  # decode steps that run back to back, each fed by the tokens the one before sampled on the
    # device, before tokens come to the host (whenever a step holds decoded tokens only and pages for all of them are free)
    handover_frequency: int = 0  # yield None every so many steps (0: never)

    def __post_init__(self) -> None:
        if self.host_cache_gb != 0:
            raise ValueError("host_cache_gb: the host prefix cache is not part of this engine, set it to 0")
        if self.max_batch <= 0:
            raise ValueError("max_batch must be positive")
        if self.cache_block <= 0:
            raise ValueError("cache_block must be positive")
        if self.max_prefill <= 0:
            raise ValueError("max_prefill must be positive")
        if self.temperature < 0:
            raise ValueError("temperature must not be negative")
        if not 0 < self.top_p <= 1:
            raise ValueError("top_p must lie in (0, 1]")


@dataclass
class Packet:
    thread_id: Any
    "An arbitrary identifier to link inputs to outputs."
    tokens: List[int] = field(default_factory=list)
    "The prompt as input, the generated tokens as output."
    text: Optional[str] = None
    "Unused: this engine takes token ids only."
    temperature: Optional[float] = None
    top_p: Optional[float] = None
    stop_str: Optional[str] = None
    "Needs a tokenizer, which this engine does not have: must be None."
    logprobs: Optional[List[float]] = None
    """Output only, when asked for: log softmax(logits)[token] per generated token; with
    prompt_logprobs, preceded by the same for the prompt's tokens 1.. (len(prompt) - 1 values)."""
    sample_logprobs: Optional[List[float]] = None
    "Output only: the same under the temperature / top-p distribution."
    max_gen: Optional[int] = None
    seed: Optional[int] = None
    "Seed of this request's random stream (default: derived from the engine's seed and thread_id)."
    finish_reason: Optional[str] = None
    "Output only: 'stop' (a stop token, kept as the last token), 'length', or 'cache' (the cache cannot hold it)."
