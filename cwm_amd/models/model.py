"""A model assembled from a plan: embedding, layers in their run order, final norm
and output head.  Nothing here is specific to an architecture."""

from __future__ import annotations

from typing import Dict, List, Mapping, Optional, Set, Tuple

import torch

from ..parts.base import BLOCKS, Block, CacheSpec, Embedding, Head, LayerCall, ModelPlan, Norm, Part, Runtime, TensorSpec


class Model:
    def __init__(self, plan: ModelPlan) -> None:
        self.plan = plan
        self.vocab_size = plan.vocab_size
        self.dim = plan.dim
        self.blocks: List[Block] = []
        for layer in plan.layers:
            if layer.block not in BLOCKS:
                raise KeyError(f"no block arrangement named {layer.block!r}; registered: {', '.join(sorted(BLOCKS))}")
            built = {role: slot.build() for role, slot in layer.parts.items()}
            names = {role: slot.prefix for role, slot in layer.parts.items()}
            self.blocks.append(BLOCKS[layer.block](names=names, **built))
        self.embedding: Embedding = plan.embedding.build()  # type: ignore[assignment]
        self.final_norm: Norm = plan.final_norm.build()  # type: ignore[assignment]
        self.head: Head = plan.head.build()  # type: ignore[assignment]
        # the model's own parts with the prefixes of their tensors in the folder
        self._ends: List[Tuple[str, str, Part]] = [
            ("embedding", plan.embedding.prefix, self.embedding),
            ("final_norm", plan.final_norm.prefix, self.final_norm),
            ("head", plan.head.prefix, self.head),
        ]
        # run order: entry i runs block `layer` on the cache slots `cache_slots[i]`, one for each of the block's mixers
        self.run_order: List[LayerCall] = list(plan.run_order)
        self.cache_slots: List[Tuple[int, ...]] = []
        self.writes_cache: List[bool] = []
        self.cache_specs: List[CacheSpec] = []
        owner_slots: Dict[int, Tuple[int, ...]] = {}
        for i, call in enumerate(self.run_order):
            if not 0 <= call.layer < len(self.blocks):
                raise ValueError(f"run order entry {i} names layer {call.layer}, the model has {len(self.blocks)}")
            specs = [mixer.cache_spec() for mixer in self.blocks[call.layer].mixers()]
            if call.cache_of is None:
                owner_slots[i] = tuple(range(len(self.cache_specs), len(self.cache_specs) + len(specs)))
                self.cache_specs.extend(specs)
                self.cache_slots.append(owner_slots[i])
                self.writes_cache.append(True)
            else:
                if call.cache_of not in owner_slots:
                    raise ValueError(
                        f"run order entry {i} reads the cache of entry {call.cache_of}, "
                        "which is not an earlier entry with a cache of its own"
                    )
                slots = owner_slots[call.cache_of]
                if [self.cache_specs[slot] for slot in slots] != specs:
                    raise ValueError(f"run order entry {i} cannot read a cache of another shape (entry {call.cache_of})")
                self.cache_slots.append(slots)
                self.writes_cache.append(False)
        self.runtime: Optional[Runtime] = None

    @property
    def cache_slot(self) -> List[Optional[int]]:
        """For each entry of the run order the cache slot of its block's mixer (the first one's if it has
        several, None if it has none)."""
        return [slots[0] if slots else None for slots in self.cache_slots]

    # ---- tensors ---------------------------------------------------------------- #
    def tensor_specs(self) -> Dict[str, TensorSpec]:
        """Every tensor of the model folder by its full name.  Two parts may name one tensor (a head on the
        embedding's table): they must agree on what it is."""
        specs: Dict[str, TensorSpec] = {}

        def add(name: str, spec: TensorSpec) -> None:
            if name in specs and specs[name] != spec:
                raise ValueError(f"tensor {name!r} is named by two parts that disagree: {specs[name]} and {spec}")
            specs[name] = spec

        for role, prefix, part in self._ends:
            if role == "final_norm":
                continue
            for name, spec in part.tensor_specs().items():
                add(prefix + name, spec)
        for layer, block in zip(self.plan.layers, self.blocks):
            for name, spec in block.tensor_specs().items():
                add(layer.prefix + name, spec)
        for name, spec in self.final_norm.tensor_specs().items():
            add(self.plan.final_norm.prefix + name, spec)
        return specs

    def tensor_names(self, role: str) -> Set[str]:
        """Full names of the tensors of the model's own part `role`: "embedding", "final_norm" or "head"."""
        for r, prefix, part in self._ends:
            if r == role:
                return {prefix + name for name in part.tensor_specs()}
        raise KeyError(f"the model's own parts are embedding, final_norm and head, not {role!r}")

    def bind(self, tensors: Mapping[str, torch.Tensor], runtime: Runtime) -> None:
        self.runtime = runtime
        for layer, block in zip(self.plan.layers, self.blocks):
            prefix = layer.prefix
            block.bind({n[len(prefix):]: t for n, t in tensors.items() if n.startswith(prefix)}, runtime)
        for _role, prefix, part in self._ends:
            names = part.tensor_specs()
            part.bind({name: tensors[prefix + name] for name in names}, runtime)

    @property
    def replayable(self) -> bool:
        """Whether a decode step may be captured once and replayed: every part says so (`Part.replayable`)."""
        return all(block.replayable for block in self.blocks) and all(part.replayable for _r, _p, part in self._ends)

    # ---- one step ------------------------------------------------------------------ #
    def forward(self, batch, cache) -> Optional[torch.Tensor]:
        """Run the batch's tokens through every layer, writing the cache, and return
        float32 logits [R, V] at `batch.logit_rows` (None if no row is wanted).

        Order as cwm/fastgen/forward.py:543-821: embedding, layers, final norm on
        the wanted rows, output projection, float32 logits.
        """
        h = self.embedding.forward(batch)
        delta = None
        for call, slots, writes in zip(self.run_order, self.cache_slots, self.writes_cache):
            views = tuple(cache.view(slot, batch) for slot in slots)
            view = views[0] if len(views) == 1 else (views or None)
            delta = self.blocks[call.layer].forward(h, delta, batch, view, writes)
        if batch.n_logit_rows == 0:
            return None
        x = self.final_norm.forward(h, delta, rows=batch.logit_rows)
        return self.head.forward(x)
