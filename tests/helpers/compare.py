"""How close the engine's logits must be to the plain implementation's.

float32: the largest error of a request's logits is at most 3e-5 of its largest
logit (rounding of float32 sums in another order; nothing else differs).

bfloat16: the limit is derived, per request, from the plain implementation itself.
`llama3_plain.forward(..., rounding=ROUND_AS_ENGINE)` computes in float64 and
rounds to bfloat16 wherever the engine stores a bfloat16 tensor; its distance from
the exact float64 logits is what bfloat16 storage costs for these weights and
tokens.  The engine rounds at the same places but sums in other orders, so its
distance from the exact logits is another draw of the same size: over 2,052
requests of random configurations (1 to 24 layers, weights of std 0.02 to 0.1, every
way of cutting the work) the ratio of the two root-mean-square errors had median
1.00 and maximum 1.33, the ratio of the two largest errors median 1.00 and maximum
2.12.  A request passes with ratios of at most 1.5 and 3.  (A later search over 7,491
requests, more of them with 16 and 24 layers, had the same medians, 99th percentiles
of 1.14 and 1.34, and maxima of 1.52 and 1.89: the highest on requests of one or two
tokens and a vocabulary of 97, where both errors are estimated from a few hundred
logits.  The limits are as they were.)
"""

from __future__ import annotations

from typing import Dict, List, Optional

import numpy as np
import torch

from helpers import models
from plain import llama3_plain

FLOAT32_LIMIT = 3e-5
BF16_RMS_RATIO = 1.5
BF16_MAX_RATIO = 3.0


class Expected:
    """Exact logits of a request and, for bfloat16, the error that rounding alone gives."""

    def __init__(self, exact: np.ndarray, rounded: Optional[np.ndarray]) -> None:
        self.exact = exact
        self.rounded = rounded
        if rounded is not None:
            diff = rounded.astype(np.float64) - exact.astype(np.float64)
            self.rms = float(np.sqrt((diff * diff).mean()))
            self.max = float(np.abs(diff).max())


def expected(folder: str, requests: Dict[str, List[int]], dtype: str) -> Dict[str, Expected]:
    config, weights = models.read_folder(folder)
    out = {}
    for rid, toks in requests.items():
        exact = llama3_plain.forward_from_config(weights, config, toks, dtype=torch.float64).to(torch.float32).numpy()
        rounded = None
        if dtype == "bfloat16":
            rounded = (
                llama3_plain.forward_from_config(weights, config, toks, dtype=torch.float64, rounding=llama3_plain.ROUND_AS_ENGINE)
                .to(torch.float32)
                .numpy()
            )
        out[rid] = Expected(exact, rounded)
    return out


def check(got: np.ndarray, want: Expected, dtype: str, what: str) -> None:
    """`got` [positions, vocab] against the request's expectation; raises AssertionError
    naming the first position over the limit."""
    assert got.shape == want.exact.shape, f"{what}: logits {got.shape}, expected {want.exact.shape}"
    assert not np.isnan(got).any(), f"{what}: missing or NaN logits"
    diff = got.astype(np.float64) - want.exact.astype(np.float64)
    err = np.abs(diff).max(axis=1)
    if dtype == "float32":
        limit = FLOAT32_LIMIT * float(np.abs(want.exact).max())
        assert err.max() <= limit, (
            f"{what}: first position over the limit {int(np.argmax(err > limit))}, worst position {int(err.argmax())}, "
            f"error {err.max():.3e} vs limit {limit:.3e}"
        )
        return
    rms = float(np.sqrt((diff * diff).mean()))
    limit = BF16_MAX_RATIO * want.max
    assert err.max() <= limit, (
        f"{what}: first position over the limit {int(np.argmax(err > limit))}, worst position {int(err.argmax())}, "
        f"error {err.max():.3e} is {err.max() / want.max:.2f} times what bfloat16 rounding gives ({want.max:.3e})"
    )
    assert rms <= BF16_RMS_RATIO * want.rms, (
        f"{what}: root-mean-square error {rms:.3e} is {rms / want.rms:.2f} times what bfloat16 rounding gives ({want.rms:.3e}); "
        f"worst position {int(err.argmax())}"
    )
