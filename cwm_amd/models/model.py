"""A model assembled from a plan: embedding, layers in their run order, final norm
and output head.  Nothing here is specific to an architecture."""

from __future__ import annotations

from typing import Dict, List, Mapping, Optional

import torch

from .. import ops
from ..parts.base import BLOCKS, Block, CacheSpec, LayerCall, ModelPlan, Norm, Runtime, TensorSpec
from ..parts.linear import LinearWeights


class Model:
    def __init__(self, plan: ModelPlan) -> None:
        self.plan = plan
        self.vocab_size = plan.vocab_size
        self.dim = plan.dim
        self.blocks: List[Block] = []
        for layer in plan.layers:
            if layer.block not in BLOCKS:
                raise KeyError(f"no block arrangement named {layer.block!r}; registered: {', '.join(sorted(BLOCKS))}")
            self.blocks.append(
                BLOCKS[layer.block](
                    norm1=layer.norm.build("norm"),
                    mixer=layer.mixer.build("mixer"),
                    norm2=(layer.norm2 or layer.norm).build("norm"),
                    feed_forward=layer.feed_forward.build("feed_forward"),
                    names=layer.names,
                )
            )
        self.final_norm: Norm = plan.final_norm.build("norm")
        # run order: entry i runs block `layer` on cache slot `cache_slot[i]`
        self.run_order: List[LayerCall] = list(plan.run_order)
        self.cache_slot: List[int] = []
        self.writes_cache: List[bool] = []
        self.cache_specs: List[CacheSpec] = []
        owner_slot: Dict[int, int] = {}
        for i, call in enumerate(self.run_order):
            if not 0 <= call.layer < len(self.blocks):
                raise ValueError(f"run order entry {i} names layer {call.layer}, the model has {len(self.blocks)}")
            if call.cache_of is None:
                owner_slot[i] = len(self.cache_specs)
                self.cache_slot.append(owner_slot[i])
                self.writes_cache.append(True)
                self.cache_specs.append(self.blocks[call.layer].mixer.cache_spec())
            else:
                if call.cache_of not in owner_slot:
                    raise ValueError(
                        f"run order entry {i} reads the cache of entry {call.cache_of}, "
                        "which is not an earlier entry with a cache of its own"
                    )
                slot = owner_slot[call.cache_of]
                if self.cache_specs[slot] != self.blocks[call.layer].mixer.cache_spec():
                    raise ValueError(f"run order entry {i} cannot read a cache of another shape (entry {call.cache_of})")
                self.cache_slot.append(slot)
                self.writes_cache.append(False)
        self.runtime: Optional[Runtime] = None

    # ---- tensors ---------------------------------------------------------------- #
    def tensor_specs(self) -> Dict[str, TensorSpec]:
        """Every tensor of the model folder by its full name."""
        plan = self.plan
        specs: Dict[str, TensorSpec] = {plan.embedding_name + ".weight": TensorSpec((plan.vocab_size, plan.dim))}
        if not plan.tied_head:
            specs[plan.head_name + ".weight"] = TensorSpec((plan.vocab_size, plan.dim))
        for layer, block in zip(plan.layers, self.blocks):
            for name, spec in block.tensor_specs().items():
                specs[layer.prefix + name] = spec
        for name, spec in self.final_norm.tensor_specs().items():
            specs[plan.final_norm_name + "." + name] = spec
        return specs

    def bind(self, tensors: Mapping[str, torch.Tensor], runtime: Runtime) -> None:
        plan = self.plan
        self.runtime = runtime
        self.embedding = tensors[plan.embedding_name + ".weight"].contiguous()
        self.head = LinearWeights(self.embedding if plan.tied_head else tensors[plan.head_name + ".weight"])
        for layer, block in zip(plan.layers, self.blocks):
            prefix = layer.prefix
            block.bind({n[len(prefix):]: t for n, t in tensors.items() if n.startswith(prefix)}, runtime)
        prefix = plan.final_norm_name + "."
        self.final_norm.bind({n[len(prefix):]: t for n, t in tensors.items() if n.startswith(prefix)}, runtime)

    @property
    def replayable(self) -> bool:
        """Whether a decode step may be captured once and replayed: every part says so (`Part.replayable`)."""
        return all(block.replayable for block in self.blocks) and self.final_norm.replayable

    # ---- one step ------------------------------------------------------------------ #
    def forward(self, batch, cache) -> Optional[torch.Tensor]:
        """Run the batch's tokens through every layer, writing the cache, and return
        float32 logits [R, V] at `batch.logit_rows` (None if no row is wanted).

        Order as cwm/fastgen/forward.py:543-821: embedding, layers, final norm on
        the wanted rows, output projection, float32 logits.
        """
        h = ops.embedding(batch.tokens, self.embedding, 1.0 if self.plan.embedding_scale is None else self.plan.embedding_scale)
        delta = None
        for call, slot, writes in zip(self.run_order, self.cache_slot, self.writes_cache):
            view = cache.view(slot, batch)
            delta = self.blocks[call.layer].forward(h, delta, batch, view, writes)
        if batch.n_logit_rows == 0:
            return None
        x = self.final_norm.forward(h, delta, rows=batch.logit_rows)
        return self.head(x, out_dtype=torch.float32)
