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
  EMBEDDINGS          token ids (and whatever else of the step) -> the float32 residual stream
  HEADS               normalised rows -> float32 logits
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

    # What the storage, the pool sizes and the measurements ask: how a page of this cache is laid out
    # and what a token costs.  A mixer whose cached row is not a key and a value of equal width (one
    # compressed row a token, say) passes a subclass that answers differently; its own kernels read
    # the pages, nothing else looks inside them.
    def page_shape(self, page_size: int) -> Tuple[int, ...]:
        """Shape of one page of `page_size` tokens; the storage allocates [pages, *page_shape].
        Here: a plane of keys and a plane of values, [2, n_kv_heads, page_size * head_dim]."""
        return (2, self.n_kv_heads, page_size * self.head_dim)

    def bytes_per_token(self, element_size: int) -> int:
        """Bytes that one cached token takes with elements of `element_size` bytes."""
        count = 1
        for n in self.page_shape(1):
            count *= n
        return count * element_size


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
    # Whether matrices keep, beside the row-major tensor that products of many rows read, a second copy laid out
    # for the weight-streaming product of a decode step (`ops.stream_layout`): twice the memory for the matrices,
    # about a tenth less time to stream them.  Whoever loads the model decides, from the memory there is.
    stream_copies: bool = False


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


class Embedding(Part):
    """What starts the residual stream."""

    def forward(self, batch: Any) -> torch.Tensor:
        """The step's `StepBatch` (`tokens` int32 [T], `positions`, ...) -> float32 [T, D], a fresh tensor
        that the layers add into."""
        raise NotImplementedError


class Head(Part):
    """What turns the final norm's rows into logits."""

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        """Normalised rows [R, D] in the activation type -> float32 logits [R, V]."""
        raise NotImplementedError


class Block(Part):
    """One layer: an arrangement of any number of norms, mixers and feed-forwards.

    The model builds the parts that the layer's plan names and calls the block's factory with them by
    role, as keyword arguments, and with `names`, the prefix of each role's tensors:
        BLOCKS[block](names={"norm1": "attention_norm.", ...}, norm1=<Norm>, mixer=<Mixer>, ...)
    A subclass that hands them on to `Block.__init__` gets `tensor_specs`, `bind`, `replayable` and
    `mixers` from here and only has to write `forward` (`replayable` is then what the parts say; a block
    whose own `forward` does not keep to the rule of `Part.replayable` sets it to False)."""

    def __init__(self, names: Mapping[str, str], **parts: Part) -> None:
        self.names = dict(names)
        self.parts: Dict[str, Part] = dict(parts)
        for role in self.parts:
            if role not in self.names:
                raise KeyError(f"no tensor prefix is given for the block's part {role!r}")

    def _own_parts(self) -> Dict[str, Part]:
        parts = getattr(self, "parts", None)
        if parts is None:
            raise NotImplementedError(f"{type(self).__name__} neither calls Block.__init__ nor defines this itself")
        return parts

    @property
    def replayable(self) -> bool:
        parts = getattr(self, "parts", None)
        return parts is not None and all(part.replayable for part in parts.values())

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs: Dict[str, TensorSpec] = {}
        for role, part in self._own_parts().items():
            for name, spec in part.tensor_specs().items():
                specs[self.names[role] + name] = spec
        return specs

    def bind(self, tensors: Mapping[str, torch.Tensor], runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        for role, part in self._own_parts().items():
            prefix = self.names[role]
            part.bind({n[len(prefix):]: t for n, t in tensors.items() if n.startswith(prefix)}, runtime)

    def mixers(self) -> List[Mixer]:
        """The block's mixers in the order in which `forward` gets their caches: each has a cache slot of its
        own per entry of the run order.  By default the mixers among the parts, in the order of the plan (a
        block that keeps its parts itself and has one `mixer` attribute is served too)."""
        parts = getattr(self, "parts", None)
        if parts is None:
            return [self.mixer]  # type: ignore[attr-defined]
        return [part for part in parts.values() if isinstance(part, Mixer)]

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
        follows it.  `cache` is the cache view of the block's mixer; a tuple of views, in the
        order of `mixers()`, if it has several; None if it has none."""
        raise NotImplementedError


# --------------------------------------------------------------------------- #
# registries
# --------------------------------------------------------------------------- #
NORMS: Dict[str, Callable[..., Norm]] = {}
MIXERS: Dict[str, Callable[..., Mixer]] = {}
FEED_FORWARDS: Dict[str, Callable[..., FeedForward]] = {}
POSITION_ENCODINGS: Dict[str, Callable[..., PositionEncoding]] = {}
BLOCKS: Dict[str, Callable[..., Block]] = {}
EMBEDDINGS: Dict[str, Callable[..., Embedding]] = {}
HEADS: Dict[str, Callable[..., Head]] = {}

_REGISTRIES = {
    "norm": NORMS,
    "mixer": MIXERS,
    "feed_forward": FEED_FORWARDS,
    "position_encoding": POSITION_ENCODINGS,
    "block": BLOCKS,
    "embedding": EMBEDDINGS,
    "head": HEADS,
}


def register_part(kind: str, name: str, factory: Callable[..., Part]) -> None:
    """Make `factory` available to architecture builders as part `name` of `kind`
    ("norm", "mixer", "feed_forward", "position_encoding", "block", "embedding" or "head")."""
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
class PartSlot:
    """A place in a plan: the kind of part that fills it (a registry), the part chosen, and the prefix of its
    tensors (below the layer's prefix for a layer's parts, in the model folder for the model's own)."""

    kind: str
    choice: PartChoice
    prefix: str = ""

    def build(self) -> Part:
        return self.choice.build(self.kind)


@dataclass(frozen=True)
class LayerPlan:
    """One layer: which block arrangement, and its parts by role.

    The roles are the block's own: the factory is called as
        BLOCKS[block](names={role: prefix, ...}, **{role: built part, ...})
    so a block may have any number of norms, mixers and feed-forwards under any names.  A position encoding is
    an argument of the mixer that applies it.  Two roles that are given one prefix read the same tensors.
    """

    prefix: str
    block: str
    parts: Mapping[str, PartSlot]

    @classmethod
    def standard(
        cls,
        prefix: str,
        block: str,
        norm: PartChoice,
        mixer: PartChoice,
        feed_forward: PartChoice,
        names: Mapping[str, str],
        norm2: Optional[PartChoice] = None,
    ) -> "LayerPlan":
        """The common layer of four roles: `norm1` before the `mixer`, `norm2` (`norm` again unless another is
        named) before the `feed_forward`; `names` gives each role's prefix."""
        return cls(
            prefix,
            block,
            {
                "norm1": PartSlot("norm", norm, names["norm1"]),
                "mixer": PartSlot("mixer", mixer, names["mixer"]),
                "norm2": PartSlot("norm", norm2 or norm, names["norm2"]),
                "feed_forward": PartSlot("feed_forward", feed_forward, names["feed_forward"]),
            },
        )


@dataclass(frozen=True)
class LayerCall:
    """One entry of the run order.  `layer` indexes `ModelPlan.layers`; a layer may
    be named more than once.  `cache_of` names an earlier entry of the run order
    whose cache this call reads instead of keeping one of its own."""

    layer: int
    cache_of: Optional[int] = None


@dataclass(frozen=True)
class ModelPlan:
    """A model as data: the embedding, the layers and the order in which they run, the final norm and the
    head, each a part chosen by name.  What the embedding does beside the table look-up (a scale, learned
    positions) and what the head does beside the product (a cap on the logits, a bias) belongs to those
    parts; a head that shares the embedding's table is a head whose prefix is the embedding's."""

    vocab_size: int
    dim: int
    layers: List[LayerPlan]
    run_order: List[LayerCall]
    embedding: PartSlot
    final_norm: PartSlot
    head: PartSlot
    max_positions: Optional[int] = None  # the context length the configuration names (cache sizing reads it)

    @classmethod
    def standard(
        cls,
        vocab_size: int,
        dim: int,
        embedding_name: str,
        layers: List[LayerPlan],
        run_order: List[LayerCall],
        final_norm: PartChoice,
        final_norm_name: str,
        head_name: str,
        max_positions: Optional[int] = None,
    ) -> "ModelPlan":
        """A table of token embeddings, the layers, a norm and a linear head, each under its module's name."""
        sizes = {"vocab_size": vocab_size, "dim": dim}
        return cls(
            vocab_size,
            dim,
            layers,
            run_order,
            embedding=PartSlot("embedding", PartChoice("token_embedding", sizes), embedding_name + "."),
            final_norm=PartSlot("norm", final_norm, final_norm_name + "."),
            head=PartSlot("head", PartChoice("linear_head", sizes), head_name + "."),
            max_positions=max_positions,
        )
