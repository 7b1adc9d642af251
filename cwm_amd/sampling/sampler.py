"""Sampling of next tokens: greedy, temperature and top-p, with a random stream per
request.

The reference draws with torch.multinomial from the global generator
(cwm/fastgen/utils/sampling.py:16,43), so a request's tokens depend on what else
is in the batch.  Here each request owns a counter-based stream (Philox keyed by
the engine's seed and the request's own): its n-th draw is the same whatever the
batch, and a preempted request goes on with its stream where it was.
"""

from __future__ import annotations

import hashlib
from typing import Any, List, Sequence, Tuple

import numpy as np
import torch

from .. import ops


class RequestStream:
    """Uniform numbers in [0, 1) for one request."""

    def __init__(self, engine_seed: int, request_key: Any) -> None:
        digest = hashlib.sha256(f"{engine_seed}:{request_key!r}".encode()).digest()
        key = [int.from_bytes(digest[0:8], "little"), int.from_bytes(digest[8:16], "little")]
        self._gen = np.random.Generator(np.random.Philox(key=key))

    def next_uniform(self) -> float:
        return float(self._gen.random(dtype=np.float32))


def effective_temperature(use_sampling: bool, temperature: float) -> float:
    """0 selects greedy.  cwm/fastgen/generate.py:1002-1014: with use_sampling off
    every request is greedy; a zero temperature, which the reference would divide
    by, means greedy too."""
    return float(temperature) if use_sampling else 0.0


class Sampler:
    def __init__(self, device: torch.device) -> None:
        self.device = device

    def sample_packed(self, logits: torch.Tensor, temperatures: torch.Tensor, top_ps: torch.Tensor, uniforms: torch.Tensor) -> torch.Tensor:
        """One token per row of float32 `logits` [R, V] with parameters and results on the device (float32 [R]
        each in): nothing waits for the host, so that the tokens can feed the next step as they are.  The result is
        one int32 tensor [3, R] (tokens, then the bits of the two log-probabilities that `sample` returns), which
        goes to the host in one copy; `unpack` reads it there."""
        return ops.sample_packed(logits, temperatures, top_ps, uniforms)

    @staticmethod
    def unpack(packed: torch.Tensor) -> Tuple[List[int], List[float], List[float]]:
        tokens, logprob, sample_logprob = ops.unpack_sampled(packed.cpu())
        return tokens.tolist(), logprob.tolist(), sample_logprob.tolist()

    def sample(
        self,
        logits: torch.Tensor,
        temperatures: Sequence[float],
        top_ps: Sequence[float],
        uniforms: Sequence[float],
    ) -> Tuple[List[int], List[float], List[float]]:
        """One token per row of float32 `logits` [R, V]; also log softmax(logits) at
        the token and its log-probability under the sampling distribution."""
        n = logits.shape[0]
        if not (len(temperatures) == len(top_ps) == len(uniforms) == n):
            raise ValueError("one temperature, top_p and uniform number per row of logits")
        params = torch.tensor([list(temperatures), list(top_ps), list(uniforms)], dtype=torch.float32).to(self.device)
        return self.unpack(ops.sample_packed(logits, params[0], params[1], params[2]))
