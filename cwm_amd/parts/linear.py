"""A weight matrix (and optional bias) with its product; not a part of its own,
parts hold these."""

from __future__ import annotations

from typing import Optional, Sequence

import torch

from .. import ops


class LinearWeights:
    """y = x W^T (+ b), W stored [out, in] (cwm/fastgen/forward.py:593-606).  Several
    matrices applied to the same input may be joined row-wise at load time into one
    product (a layout choice: each output column is computed as before)."""

    def __init__(self, weight: torch.Tensor, bias: Optional[torch.Tensor] = None, stream_copy: bool = False) -> None:
        """`stream_copy`: also keep the matrix in the layout that the weight-streaming product of a decode step
        reads fastest (`ops.stream_layout`; bfloat16 matrices on the device only)."""
        self.weight = weight.contiguous()
        self.bias = bias.contiguous() if bias is not None else None
        self.streamed: Optional[torch.Tensor] = None
        if stream_copy and self.weight.is_cuda and self.weight.dtype == torch.bfloat16 and self.weight.shape[1] % 8 == 0:
            self.streamed = ops.stream_layout(self.weight)

    @classmethod
    def joined(
        cls, weights: Sequence[torch.Tensor], biases: Sequence[Optional[torch.Tensor]], group: Optional[int] = None,
        stream_copy: bool = False,
    ) -> "LinearWeights":
        """One matrix from several with the same input.  Rows follow one another matrix
        by matrix, or, with `group` (two matrices of equal height, a multiple of
        `group`), alternate in groups of that many rows: the two results for one output
        column then lie `group` columns apart, within reach of one kernel's epilogue."""
        dtype = torch.float32 if any(w.dtype == torch.float32 for w in weights) else weights[0].dtype
        columns = []
        if any(b is not None for b in biases):
            for w, b in zip(weights, biases):
                columns.append(b.float() if b is not None else torch.zeros(w.shape[0], dtype=torch.float32, device=w.device))
        if group is None:
            weight = torch.cat([w.to(dtype) for w in weights], dim=0)
            bias = torch.cat(columns, dim=0) if columns else None
        else:
            if len(weights) != 2 or weights[0].shape != weights[1].shape or weights[0].shape[0] % group != 0:
                raise ValueError("rows alternate in groups only between two matrices of equal height, a multiple of the group")
            k = weights[0].shape[1]
            weight = torch.stack([w.to(dtype).reshape(-1, group, k) for w in weights], dim=1).reshape(-1, k)
            bias = torch.stack([c.reshape(-1, group) for c in columns], dim=1).reshape(-1) if columns else None
        return cls(weight, bias, stream_copy)

    def __call__(self, x: torch.Tensor, out_dtype: Optional[torch.dtype] = None, partials_ok: bool = False) -> torch.Tensor:
        """With `partials_ok` the result may be float32 partial sums [P, M, N] (a
        product whose K was split) for a consumer that adds them, as the norms do."""
        return ops.linear(x, self.weight, self.bias, out_dtype, partials_ok, streamed=self.streamed)
