"""Arrangements of parts in one layer."""

from __future__ import annotations

from typing import Any, Mapping, Optional

import torch

from .base import Block, FeedForward, Mixer, Norm, register_part


class PreNormBlock(Block):
    """h += mixer(norm1(h)); h += feed_forward(norm2(h))  (cwm/fastgen/forward.py:563-786).

    Each residual sum is done by the norm that follows it, in float32: the block
    takes the previous layer's pending update and returns its own.
    """

    def __init__(self, names: Mapping[str, str], norm1: Norm, mixer: Mixer, norm2: Norm, feed_forward: FeedForward) -> None:
        super().__init__(names, norm1=norm1, mixer=mixer, norm2=norm2, feed_forward=feed_forward)
        self.norm1 = norm1
        self.mixer = mixer
        self.norm2 = norm2
        self.feed_forward = feed_forward

    def forward(self, h: torch.Tensor, delta: Optional[torch.Tensor], batch: Any, cache: Any, write_cache: bool = True) -> torch.Tensor:
        x = self.norm1.forward(h, delta)
        mixed = self.mixer.forward(x, batch, cache, write_cache)
        x = self.norm2.forward(h, mixed)
        return self.feed_forward.forward(x, batch)


register_part("block", "pre_norm", PreNormBlock)
