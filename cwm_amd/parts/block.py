"""Arrangements of parts in one layer."""

from __future__ import annotations

from typing import Any, Dict, Mapping, Optional

import torch

from .base import Block, FeedForward, Mixer, Norm, Runtime, TensorSpec, register_part


class PreNormBlock(Block):
    """h += mixer(norm1(h)); h += feed_forward(norm2(h))  (cwm/fastgen/forward.py:563-786).

    Each residual sum is done by the norm that follows it, in float32: the block
    takes the previous layer's pending update and returns its own.
    """

    def __init__(self, norm1: Norm, mixer: Mixer, norm2: Norm, feed_forward: FeedForward, names: Mapping[str, str]) -> None:
        self.norm1 = norm1
        self.mixer = mixer
        self.norm2 = norm2
        self.feed_forward = feed_forward
        self.names = dict(names)
        self._parts = {"norm1": norm1, "mixer": mixer, "norm2": norm2, "feed_forward": feed_forward}

    @property
    def replayable(self) -> bool:
        return all(part.replayable for part in self._parts.values())

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs: Dict[str, TensorSpec] = {}
        for role, part in self._parts.items():
            for name, spec in part.tensor_specs().items():
                specs[self.names[role] + name] = spec
        return specs

    def bind(self, tensors: Mapping[str, torch.Tensor], runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        for role, part in self._parts.items():
            prefix = self.names[role]
            part.bind({n[len(prefix):]: t for n, t in tensors.items() if n.startswith(prefix)}, runtime)

    def forward(self, h: torch.Tensor, delta: Optional[torch.Tensor], batch: Any, cache: Any, write_cache: bool = True) -> torch.Tensor:
        x = self.norm1.forward(h, delta)
        mixed = self.mixer.forward(x, batch, cache, write_cache)
        x = self.norm2.forward(h, mixed)
        return self.feed_forward.forward(x, batch)


register_part("block", "pre_norm", PreNormBlock)
