"""The step function: one batch of (request, its next tokens) through the model.

It runs only the tokens it is given, as one batch, reading earlier tokens from the
cache, and returns float32 logits at the wanted places.  Portions of prompts and
single decoded tokens may share a step and a portion may be cut anywhere.  The
reference has two entry points for this, `prefill` for ragged new tokens and
`decode` for one token per lane (cwm/fastgen/forward.py:824-961), and never mixes
them in one call (cwm/fastgen/generate.py:480-498).
"""

from __future__ import annotations

from typing import Callable, Hashable, List, Optional, Sequence

import torch

from ..cache.manager import CacheManager
from ..cache.storage import CacheStorage
from ..models.model import Model
from .batch import Portion, build_batch


class ModelRunner:
    def __init__(self, model: Model, manager: CacheManager, storage: CacheStorage) -> None:
        if model.runtime is None:
            raise RuntimeError("the model has no weights yet (Model.bind)")
        self.model = model
        self.manager = manager
        self.storage = storage
        self.device = model.runtime.device
        # called as on_pages_freed(group, pages) whenever pages go back to a pool
        self.on_pages_freed: Optional[Callable[[int, List[int]], None]] = None

    # ---- requests ------------------------------------------------------------- #
    def admit(self, rid: Hashable) -> int:
        slot = self.manager.admit(rid)
        self.storage.zero_state(slot)
        return slot

    def release(self, rid: Hashable) -> None:
        freed = self.manager.release(rid)
        self._report(freed)

    def _report(self, freed: Sequence[Sequence[int]]) -> None:
        if self.on_pages_freed is not None:
            for group, pages in enumerate(freed):
                if pages:
                    self.on_pages_freed(group, list(pages))

    # ---- the step ---------------------------------------------------------------- #
    @torch.inference_mode()
    def step(self, portions: Sequence[Portion], tokens_device: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
        """Run `portions` (pages already reserved with `CacheManager.extend`) and
        return logits [R, V], rows ordered by portion and then by `want`; None if no
        place is wanted.  Afterwards every request's length has grown by its portion
        and window groups have given back the pages that fell out of reach.  With
        `tokens_device` the token ids come from that device tensor (see `build_batch`)."""
        batch = build_batch(portions, self.manager, self.device, self.model.vocab_size, tokens_device)
        logits = self.model.forward(batch, self.storage)
        for portion in portions:
            self._report(self.manager.advance(portion.rid, len(portion.tokens)))
        return logits
