"""Dense gated feed-forward."""

from __future__ import annotations

from typing import Any, Dict, Mapping

import torch

from .. import ops
from .base import FeedForward, Runtime, TensorSpec, register_part
from .linear import LinearWeights


class SwiGLU(FeedForward):
    """w2(silu(w1 x) * (w3 x)), no biases (cwm/fastgen/forward.py:776-782;
    cwm/model/transformer.py:214-228).  w1 and w3 are joined into one product; the
    gate's SiLU and the product with the up branch are computed in float32 and
    rounded once."""

    replayable = True

    def __init__(self, dim: int, hidden_dim: int) -> None:
        self.dim = dim
        self.hidden_dim = hidden_dim

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {
            "w1.weight": TensorSpec((self.hidden_dim, self.dim)),
            "w2.weight": TensorSpec((self.dim, self.hidden_dim)),
            "w3.weight": TensorSpec((self.hidden_dim, self.dim)),
        }

    def bind(self, tensors: Mapping[str, torch.Tensor], runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        # gate and up rows alternate in groups of 8 where the width allows, so that a decode batch
        # finishes silu(gate) * up in the product's epilogue
        self.grouped = self.hidden_dim % 8 == 0
        self.gate_up = LinearWeights.joined(
            [tensors["w1.weight"], tensors["w3.weight"]], [None, None], group=8 if self.grouped else None,
            stream_copy=runtime.stream_copies,
        )
        self.down = LinearWeights(tensors["w2.weight"], stream_copy=runtime.stream_copies)

    def forward(self, x: torch.Tensor, batch: Any) -> torch.Tensor:
        # the result (or partial sums of it) is added into the residual by the next norm.  (Forming
        # silu(gate) * up inside the down product was tried: every block recomputes it, which costs
        # more than the kernel it saves.)
        hidden = ops.gate_up_silu(x, self.gate_up.weight, self.gate_up.bias, self.grouped, streamed=self.gate_up.streamed)
        return self.down(hidden, partials_ok=True)


register_part("feed_forward", "swiglu", SwiGLU)
