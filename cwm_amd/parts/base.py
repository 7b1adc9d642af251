"""Interfaces of the parts that layers are put together from.

A part is given every size and constant at construction, declares the tensors it
needs by local name (`tensor_specs`) and receives them in `bind`.  No part knows
which model it sits in: the architecture's builder chooses parts per layer and
tells each one the prefix its tensors carry in the model folder.

Kinds of part and their registries (name -> class):
  NORMS               h (fp32 residual) [+ delta] -> normalised activations
  MIXERS              token mixing: attention here; may keep a cache or state
  FEED_FORWARDS       per-token transform [T, D] -> [T, D]
  POSITION_ENCODINGS  what a mixer applies to queries and keys
  BLOCKS              arrangement of the above in one layer
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable, Dict, Hashable, List, Mapping, Optional, Tuple, Union

import torch


# --------------------------------------------------------------------------- #
# tensors a part needs
# --------------------------------------------------------------------------- #
@dataclass(frozen=True)
class TensorSpec:
    shape: Tuple[int, ...]
    kind: str = "float"  # "float" or "int" (integer tables are kept as int32)
    init: str = "normal"  # how the random-weights writer fills it: "normal" | "norm" | "zeros"
    # type a floating tensor is kept in when the model runs in bfloat16: "activation" casts it to
    # bfloat16 whatever it is stored in (matrices: every product then runs on the bfloat16 kernels, as the
    # reference casts every parameter, cwm/model/parallelize_transformer.py:50-59); "stored" keeps a
    # tensor that is stored in 32 bits in float32 (norm weights, tables whose precision matters)
    precision: str = "activation"


# --------------------------------------------------------------------------- #
# what a mixer asks of the cache manager
# --------------------------------------------------------------------------- #
@dataclass(frozen=True)
class PagedKVSpec:
    """Keys and values in pages.  `window` is the number of keys a query reads, its
    own included; None keeps every key."""

    n_kv_heads: int
    head_dim: int
    window: Optional[int] = None

    # What the cache manager asks.  A mixer with another rule (keys pinned at the start
    # of a sequence beside a window, say) passes a subclass that answers differently;
    # the manager, the scheduler and the pool sizes know these four methods only.
    def retention(self) -> Hashable:
        """Cache slots whose values are equal keep the same keys: they share a pool and
        block tables.  It is also the key under which a pool size is given."""
        return self.window

    def first_key_needed(self, length: int) -> int:
        """Lowest position, pinned keys apart, that a query at position >= `length` can
        still read.  A layer with window W lets the query at position p read keys
        p-(W-1)..p (cwm/model/transformer.py:253-270)."""
        if self.window is None:
            return 0
        return max(0, length - (self.window - 1))

    def pinned_keys(self) -> int:
        """Keys at the start of a sequence that every later query reads."""
        return 0

    def keys_kept(self, step_tokens: int) -> Optional[int]:
        """Most keys, pinned ones apart, that a request holds at any time when a step
        brings at most `step_tokens`; None if all are kept."""
        if self.window is None:
            return None
        return self.window - 1 + step_tokens


@dataclass(frozen=True)
class StateSpec:
    """Per-request state of fixed size, zero when a request is admitted."""

    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


CacheSpec = Union[PagedKVSpec, StateSpec, None]


@dataclass
class Runtime:
    """Where and in which precision a model runs.

    `act_dtype` is the storage type of activations and of the cache (bfloat16 or
    float32).  The residual stream and the logits are float32 in both modes.
    """

    device: torch.device
    act_dtype: torch.dtype

    @property
    def is_float32(self) -> bool:
        return self.act_dtype == torch.float32


class Part:
    """Base of every part."""

    # Whether a decode step through this part may be captured once and replayed: its `forward` then launches
    # the same kernels with the same arguments for every step of that shape, and reads what changes from step
    # to step (tokens, positions, lengths, block tables, state slots) from the step's device vectors only;
    # nothing goes between host and device in it.  A part that does not say so keeps its model on the path
    # that launches every step kernel by kernel.
    replayable = False

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {}

    def bind(self, tensors: Mapping[str, torch.Tensor], runtime: Runtime) -> None:
        """Receive the tensors named by `tensor_specs` (already on the device)."""
        self.runtime = runtime


class Norm(Part):
    def forward(
        self,
        h: torch.Tensor,
        delta: Optional[torch.Tensor],
        rows: Optional[torch.Tensor] = None,
    ) -> torch.Tensor:
        """`h` is the float32 residual stream [T, D].  If `delta` is given ([T, D], or
        float32 partial sums [P, T, D] to be added in order) it is first added into
        `h` in place (the residual sum, in float32).  Returns the
        normalised rows in the activation type; with `rows` (int32 [R]) only those
        rows are normalised and returned, and `h` is left as it was."""
        raise NotImplementedError


class PositionEncoding(Part):
    """How positions reach a mixer.  A rotary encoding returns its table of inverse
    frequencies (float32 [head_dim / 2]) from `rotary_table`; an encoding that does
    nothing to queries and keys returns None."""

    def rotary_table(self) -> Optional[torch.Tensor]:
        return None

    def rotary_pairing(self) -> str:
        """Which two elements of a head the i-th frequency turns: "adjacent" (2i, 2i + 1), the
        reference's (cwm/fastgen/kernels/rope.py:71-87), or "halves" (i, i + head_dim / 2).  The
        kernels turn adjacent pairs; a mixer serves "halves" by reordering, once at load time, the
        rows of its query and key projections so that each pair lies side by side (scores are sums
        over a head's elements, so a common reordering of queries and keys changes nothing else)."""
        return "adjacent"


class Mixer(Part):
    def cache_spec(self) -> CacheSpec:
        return None

    def forward(self, x: torch.Tensor, batch: Any, cache: Any, write_cache: bool = True) -> torch.Tensor:
        """x: normalised activations [T, D] -> [T, D] to be added to the residual (or
        float32 partial sums [P, T, D] of it, which the next norm adds).
        `batch` is the step's `StepBatch`; `cache` the view of this call's cache
        (a `PagedKVView`, a `StateView` or None).  With `write_cache` false the
        mixer reads a cache that another layer has written in this step."""
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, x: torch.Tensor, batch: Any) -> torch.Tensor:
        raise NotImplementedError


class Block(Part):
    """One layer: an arrangement of norms, a mixer and a feed-forward."""

    mixer: Mixer

    def forward(
        self,
        h: torch.Tensor,
        delta: Optional[torch.Tensor],
        batch: Any,
        cache: Any,
        write_cache: bool = True,
    ) -> Optional[torch.Tensor]:
        """Consumes the pending residual update `delta` of the previous layer and
        returns its own, so that each residual sum is fused with the norm that
        follows it."""
        raise NotImplementedError


# --------------------------------------------------------------------------- #
# registries
# --------------------------------------------------------------------------- #
NORMS: Dict[str, Callable[..., Norm]] = {}
MIXERS: Dict[str, Callable[..., Mixer]] = {}
FEED_FORWARDS: Dict[str, Callable[..., FeedForward]] = {}
POSITION_ENCODINGS: Dict[str, Callable[..., PositionEncoding]] = {}
BLOCKS: Dict[str, Callable[..., Block]] = {}

_REGISTRIES = {
    "norm": NORMS,
    "mixer": MIXERS,
    "feed_forward": FEED_FORWARDS,
    "position_encoding": POSITION_ENCODINGS,
    "block": BLOCKS,
}


def register_part(kind: str, name: str, factory: Callable[..., Part]) -> None:
    """Make `factory` available to architecture builders as part `name` of `kind`
    ("norm", "mixer", "feed_forward", "position_encoding" or "block")."""
    if kind not in _REGISTRIES:
        raise KeyError(f"unknown kind of part {kind!r}; kinds: {', '.join(_REGISTRIES)}")
    _REGISTRIES[kind][name] = factory


@dataclass(frozen=True)
class PartChoice:
    """A part chosen by name with its constructor arguments."""

    name: str
    args: Mapping[str, Any] = field(default_factory=dict)

    def build(self, kind: str) -> Part:
        table = _REGISTRIES[kind]
        if self.name not in table:
            raise KeyError(f"no {kind} named {self.name!r}; registered: {', '.join(sorted(table)) or '(none)'}")
        return table[self.name](**dict(self.args))


# --------------------------------------------------------------------------- #
# the plan of a model: data that an architecture's builder returns
# --------------------------------------------------------------------------- #
@dataclass(frozen=True)
class LayerPlan:
    """One layer: which block arrangement, which parts, and the prefixes of their
    tensors in the model folder.

    The block factory is called as
        BLOCKS[block](norm1=Norm, mixer=Mixer, norm2=Norm, feed_forward=FeedForward, names=names)
    where `names` maps each of these four roles to the prefix of its tensors below
    `prefix` (for instance {"norm1": "attention_norm.", "mixer": "attention.", ...}).
    `norm` is the norm before the mixer and, unless `norm2` names another, also the one
    before the feed-forward.  A position encoding is an argument of the mixer that applies it.
    """

    prefix: str
    block: str
    norm: PartChoice
    mixer: PartChoice
    feed_forward: PartChoice
    names: Mapping[str, str]
    norm2: Optional[PartChoice] = None


@dataclass(frozen=True)
class LayerCall:
    """One entry of the run order.  `layer` indexes `ModelPlan.layers`; a layer may
    be named more than once.  `cache_of` names an earlier entry of the run order
    whose cache this call reads instead of keeping one of its own."""

    layer: int
    cache_of: Optional[int] = None


@dataclass(frozen=True)
class ModelPlan:
    vocab_size: int
    dim: int
    embedding_name: str
    layers: List[LayerPlan]
    run_order: List[LayerCall]
    final_norm: PartChoice
    final_norm_name: str
    head_name: str  # ignored with `tied_head`
    max_positions: Optional[int] = None  # the context length the configuration names (cache sizing reads it)
    embedding_scale: Optional[float] = None  # the embedding is multiplied by it (None: as it is)
    tied_head: bool = False  # the output projection is the embedding table; the folder holds no head tensor
