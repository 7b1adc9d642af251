"""The parts at the two ends of a model: the token embedding and the output head."""

from __future__ import annotations

from typing import Any, Dict, Mapping, Optional

import torch

from .. import ops
from .base import Embedding, Head, Runtime, TensorSpec, register_part
from .linear import LinearWeights


class TokenEmbedding(Embedding):
    """h = scale * table[tokens], as the float32 residual stream (cwm/fastgen/forward.py:543; the reference
    has no scale, which is `scale=None`)."""

    replayable = True

    def __init__(self, vocab_size: int, dim: int, scale: Optional[float] = None) -> None:
        self.vocab_size = vocab_size
        self.dim = dim
        self.scale = 1.0 if scale is None else float(scale)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {"weight": TensorSpec((self.vocab_size, self.dim))}

    def bind(self, tensors: Mapping[str, torch.Tensor], runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        self.table = tensors["weight"].contiguous()

    def forward(self, batch: Any) -> torch.Tensor:
        return ops.embedding(batch.tokens, self.table, self.scale)


class LinearHead(Head):
    """logits = x W^T in float32 (cwm/fastgen/forward.py:820-821).  A model whose head is its embedding table
    gives this part the embedding's prefix: both then name the same tensor."""

    replayable = True

    def __init__(self, vocab_size: int, dim: int) -> None:
        self.vocab_size = vocab_size
        self.dim = dim

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {"weight": TensorSpec((self.vocab_size, self.dim))}

    def bind(self, tensors: Mapping[str, torch.Tensor], runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        self.weights = LinearWeights(tensors["weight"], stream_copy=runtime.stream_copies)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.weights(x, out_dtype=torch.float32)


register_part("embedding", "token_embedding", TokenEmbedding)
register_part("head", "linear_head", LinearHead)
