"""RMSNorm fused with the residual sum that precedes it."""

from __future__ import annotations

from typing import Dict, Mapping, Optional

import torch

from .. import ops
from .base import Norm, Runtime, TensorSpec, register_part


class RMSNorm(Norm):
    """y = x * rsqrt(mean(x^2) + eps) * weight, in float32
    (cwm/fastgen/kernels/rmsnorm.py:34-61; call sites cwm/fastgen/forward.py:571,
    772,789).  The residual update that the reference adds just before
    (`h.add_`, forward.py:769,786) is added here, in float32, in the same kernel."""

    replayable = True

    def __init__(self, dim: int, eps: float) -> None:
        self.dim = dim
        self.eps = float(eps)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {"weight": TensorSpec((self.dim,), init="norm", precision="stored")}

    def bind(self, tensors: Mapping[str, torch.Tensor], runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        self.weight = tensors["weight"]

    def forward(self, h: torch.Tensor, delta: Optional[torch.Tensor], rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        return ops.add_rmsnorm(h, delta, self.weight, self.eps, self.runtime.act_dtype, rows)


register_part("norm", "rmsnorm", RMSNorm)
