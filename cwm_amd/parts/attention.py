"""Causal grouped-query attention over a paged cache."""

from __future__ import annotations

from typing import Any, Dict, Mapping, Optional

import torch

from .. import ops
from .base import Mixer, PagedKVSpec, PartChoice, PositionEncoding, Runtime, TensorSpec, register_part
from .linear import LinearWeights


MAX_HEAD_DIM = 256  # the attention kernels' largest head size (csrc/attention_simple.hip, attention_mfma.hip)


class PagedAttention(Mixer):
    """x -> wo(attention(rope(wq x), cache of rope(wk x), cache of wv x)).

    cwm/fastgen/forward.py:593-656,763: three projections of the same input, heads
    as the slow axis of the projected features, rotation of queries and keys,
    cache write before the attention, softmax(q k^T * scale) v over the sequence's
    cached keys up to the query's own position (and no further back than the
    window), query head h reading key/value head h // (n_heads / n_kv_heads), and
    the output projection.  Every constant is an argument: sizes, `scale`
    (the reference fixes head_dim ** -0.5 at forward.py:651), `window` (keys read
    per query, own included; None for all), `bias` on the three input projections
    (cwm/model/transformer.py:173-187) and the position encoding.
    """

    def __init__(
        self,
        dim: int,
        n_heads: int,
        n_kv_heads: int,
        head_dim: int,
        scale: float,
        window: Optional[int] = None,
        bias: bool = False,
        position_encoding: Optional[PartChoice] = None,
    ) -> None:
        if n_heads % n_kv_heads != 0:
            raise ValueError(f"{n_heads} query heads do not divide into {n_kv_heads} key/value heads")
        if not 1 <= head_dim <= MAX_HEAD_DIM:
            raise ValueError(f"head_dim {head_dim} is outside 1..{MAX_HEAD_DIM}, the sizes the attention kernels take")
        self.dim = dim
        self.n_heads = n_heads
        self.n_kv_heads = n_kv_heads
        self.head_dim = head_dim
        self.scale = float(scale)
        self.window = window
        self.bias = bias
        self.position_encoding: Optional[PositionEncoding] = (
            position_encoding.build("position_encoding") if position_encoding is not None else None
        )

    def cache_spec(self) -> PagedKVSpec:
        return PagedKVSpec(n_kv_heads=self.n_kv_heads, head_dim=self.head_dim, window=self.window)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        q_out = self.n_heads * self.head_dim
        kv_out = self.n_kv_heads * self.head_dim
        specs = {
            "wq.weight": TensorSpec((q_out, self.dim)),
            "wk.weight": TensorSpec((kv_out, self.dim)),
            "wv.weight": TensorSpec((kv_out, self.dim)),
            "wo.weight": TensorSpec((self.dim, q_out)),
        }
        if self.bias:
            specs["wq.bias"] = TensorSpec((q_out,))
            specs["wk.bias"] = TensorSpec((kv_out,))
            specs["wv.bias"] = TensorSpec((kv_out,))
        return specs

    def bind(self, tensors: Mapping[str, torch.Tensor], runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        if self.position_encoding is not None:
            self.position_encoding.bind({}, runtime)
        names = ("wq", "wk", "wv")
        weights = {n: tensors[f"{n}.weight"] for n in names}
        biases = {n: tensors.get(f"{n}.bias") for n in names}
        pairing = self.position_encoding.rotary_pairing() if self.position_encoding is not None else "adjacent"
        # element j of a head as `transform_qk` sees it is element qk_order[j] of the head as the folder's wq and wk give it
        self.qk_order = torch.arange(self.head_dim)
        if pairing == "halves":
            # the kernels turn adjacent elements: bring element i and i + head_dim / 2 of every query and key
            # head side by side, once, by the order of the projections' rows
            half = self.head_dim // 2
            order = torch.stack([torch.arange(half), torch.arange(half) + half], dim=1).reshape(-1)
            self.qk_order = order
            for n, heads in (("wq", self.n_heads), ("wk", self.n_kv_heads)):
                rows = (torch.arange(heads)[:, None] * self.head_dim + order[None, :]).reshape(-1).to(weights[n].device)
                weights[n] = weights[n][rows]
                if biases[n] is not None:
                    biases[n] = biases[n][rows]
        elif pairing != "adjacent":
            raise ValueError(f"rotary pairing {pairing!r}: 'adjacent' and 'halves' are known")
        self.qkv = LinearWeights.joined([weights[n] for n in names], [biases[n] for n in names], stream_copy=runtime.stream_copies)
        self.wo = LinearWeights(tensors["wo.weight"], stream_copy=runtime.stream_copies)
        # a subclass that changes queries and keys between projection and rotation cannot use the fused product
        self._plain_projection = type(self).transform_qk is not PagedAttention.transform_qk

    def transform_qk(self, q: torch.Tensor, k: Optional[torch.Tensor], batch: Any) -> None:
        """The seam between projection and rotation: a subclass may change the projected queries
        `q` [T, Hq, hd] and keys `k` [T, Hkv, hd] (None when this call writes no cache) in place
        here (a norm per head, say) before they are rotated and the keys are cached.  Overriding it
        takes the step off the fused projection + rotation + cache-write kernel, and off captured
        steps unless the subclass sets `transform_replayable`.

        The elements of a head arrive in the order the kernels rotate them, which for a position
        encoding with the "halves" pairing is not the folder's: element j here is element
        `self.qk_order[j]` of the head as wq and wk give it (`qk_order` is the identity for adjacent
        pairs; it is set by `bind`).  A subclass with a tensor per element of a head (the weight of a
        norm) reorders it once, `weight[self.qk_order]`, after calling `bind` of this class."""

    transform_replayable = False  # whether an overriding `transform_qk` keeps to the rule of `Part.replayable`

    @property
    def replayable(self) -> bool:
        own = type(self).transform_qk is PagedAttention.transform_qk or self.transform_replayable
        return own and (self.position_encoding is None or self.position_encoding.replayable)

    def forward(self, x: torch.Tensor, batch: Any, cache: Any, write_cache: bool = True) -> torch.Tensor:
        hd = self.head_dim
        q_out = self.n_heads * hd
        kv_out = self.n_kv_heads * hd
        table = self.position_encoding.rotary_table() if self.position_encoding is not None else None
        if write_cache and not self._plain_projection:
            qkv = ops.qkv_rope_write(
                x, self.qkv.weight, self.qkv.bias, self.n_heads, self.n_kv_heads, hd,
                batch.positions, table, cache.cache, cache.block_table, batch.seq_of_token, streamed=self.qkv.streamed,
            )
            q = qkv[:, :q_out].unflatten(1, (self.n_heads, hd))
        else:
            qkv = self.qkv(x)
            q = qkv[:, :q_out].unflatten(1, (self.n_heads, hd))
            if write_cache:
                k = qkv[:, q_out : q_out + kv_out].unflatten(1, (self.n_kv_heads, hd))
                v = qkv[:, q_out + kv_out :].unflatten(1, (self.n_kv_heads, hd))
                self.transform_qk(q, k, batch)
                ops.rope_kv_write(q, k, v, batch.positions, table, cache.cache, cache.block_table, batch.seq_of_token)
            else:
                # reads a cache that another layer wrote in this step: only the queries are needed
                self.transform_qk(q, None, batch)
                if table is not None:
                    ops.rope_kv_write(q, None, None, batch.positions, table)
        attn = ops.paged_attention(q, cache.cache, cache.block_table, batch, self.window, self.scale)
        return self.wo(attn, partials_ok=True)  # added into the residual by the next norm


register_part("mixer", "paged_attention", PagedAttention)
