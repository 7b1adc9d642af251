"""Rotary position encodings: tables of inverse frequencies."""

from __future__ import annotations

import math
from typing import Mapping, Optional

import torch

from .base import PositionEncoding, Runtime, register_part


def rotary_inverse_frequencies(head_dim: int, theta: float) -> torch.Tensor:
    """float32 [head_dim / 2]: theta ** -(2i / head_dim).  cwm/fastgen/forward.py:1025-1026."""
    exponents = torch.arange(0, head_dim, 2).float() / head_dim
    return 1.0 / (theta ** exponents)


def llama3_scale_frequencies(
    freqs: torch.Tensor,
    scale_factor: float,
    old_context_len: int,
    low_freq_factor: float,
    high_freq_factor: float,
) -> torch.Tensor:
    """llama3 long-context scaling of a frequency table (cwm/fastgen/forward.py:1031-1047).

    Wavelengths longer than old_context_len / low_freq_factor are divided by the
    factor, those shorter than old_context_len / high_freq_factor stay, and the
    band between is blended; the band's rule is applied after the first and from
    the unscaled value, as the reference's loop does.
    """
    low_wavelen = old_context_len / low_freq_factor
    high_wavelen = old_context_len / high_freq_factor
    scaled = freqs.clone()
    for i in range(freqs.numel()):
        freq = freqs[i]
        wavelen = 2 * math.pi / freq
        if wavelen > low_wavelen:
            scaled[i] = freq / scale_factor
        if high_wavelen <= wavelen <= low_wavelen:
            blend = (old_context_len / wavelen - low_freq_factor) / (high_freq_factor - low_freq_factor)
            scaled[i] = (1 - blend) * freq / scale_factor + blend * freq
    return scaled


class RotaryEncoding(PositionEncoding):
    """Rotation of adjacent pairs (2i, 2i+1) of queries and keys by
    position * inv_freq[i] (cwm/fastgen/kernels/rope.py:55-90).  The table is all a
    kernel needs; a scaling scheme only changes the table."""

    replayable = True

    def __init__(self, head_dim: int, theta: float, llama3_scaling: Optional[Mapping[str, float]] = None) -> None:
        if head_dim % 2 != 0:
            raise ValueError("rotary pairs need an even head size")
        self.head_dim = head_dim
        self.theta = float(theta)
        self.llama3_scaling = dict(llama3_scaling) if llama3_scaling else None
        table = rotary_inverse_frequencies(head_dim, self.theta)
        if self.llama3_scaling:
            table = llama3_scale_frequencies(
                table,
                self.llama3_scaling["scale_factor"],
                self.llama3_scaling["old_context_len"],
                self.llama3_scaling["low_freq_factor"],
                self.llama3_scaling["high_freq_factor"],
            )
        self.host_table = table.contiguous()
        self._table: Optional[torch.Tensor] = None

    def bind(self, tensors: Mapping[str, torch.Tensor], runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        self._table = self.host_table.to(runtime.device)

    def rotary_table(self) -> Optional[torch.Tensor]:
        return self._table


class NoPositionEncoding(PositionEncoding):
    """Queries and keys are used as they are."""

    replayable = True


register_part("position_encoding", "rotary", RotaryEncoding)
register_part("position_encoding", "none", NoPositionEncoding)
