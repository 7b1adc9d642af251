"""Typed configuration of the Llama-3 dense decoder.

Key names, meanings and defaults follow the reference's `TransformerArgs`
(cwm/model/transformer.py:88-145) and its nested `ScaledRoPEArgs` (:25-43) and
`WindowAttentionArgs` (:56-85).  The reference reads these from the "model" entry
of params.json (cwm/fastgen/utils/loading.py:39-41); here they are the top-level
keys of the model folder's config.json.  Three keys have no counterpart in the
reference: `architecture` (the registry key), `hidden_dim` (the feed-forward width
given directly instead of by the rounding rule) and `layer_types` (an explicit
per-layer list of "global" / "local" instead of the interleaving rule).
"""

from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import List, Optional

from .schema import ConfigError


@dataclass(frozen=True)
class ScaledRoPEConfig:
    """llama3 frequency scaling (cwm/model/transformer.py:25-43)."""

    scale_factor: float = 8
    old_context_len: int = 8192
    low_freq_factor: float = 1
    high_freq_factor: float = 4
    use_attn_scale: bool = False  # present in the reference, never read by its engine

    def __post_init__(self) -> None:
        if self.scale_factor == 1:
            raise ConfigError("scaled_rope.scale_factor == 1 scales nothing")
        low_wl = self.old_context_len / self.low_freq_factor
        high_wl = self.old_context_len / self.high_freq_factor
        if low_wl < high_wl:
            raise ConfigError(
                f"scaled_rope: low-frequency wavelength {low_wl} is below the high-frequency one {high_wl}"
            )
        if self.high_freq_factor == self.low_freq_factor:
            raise ConfigError("scaled_rope: high_freq_factor equals low_freq_factor")


@dataclass(frozen=True)
class WindowAttentionConfig:
    """Interleaved sliding-window / global layers (cwm/model/transformer.py:56-85)."""

    window_pattern: int = 6
    global_window: Optional[int] = None
    local_window: Optional[int] = None
    global_last_layer: bool = True

    def __post_init__(self) -> None:
        if self.window_pattern <= 0:
            raise ConfigError("window_attn.window_pattern must be positive")
        if not ((self.local_window is not None and self.local_window > 0) or self.window_pattern == 1):
            raise ConfigError("window_attn.local_window must be a positive size unless window_pattern is 1")
        if self.global_window is not None and self.global_window <= 0:
            raise ConfigError("window_attn.global_window must be positive")

    def is_global_layer(self, layer_id: int, n_layers: int) -> bool:
        """cwm/model/transformer.py:79-85."""
        if self.global_last_layer and layer_id == n_layers - 1:
            return True
        return layer_id % self.window_pattern == 0


@dataclass(frozen=True)
class Llama3DenseConfig:
    architecture: str
    dim: int
    n_layers: int
    n_heads: int
    vocab_size: int
    n_kv_heads: Optional[int] = None
    head_dim: Optional[int] = None
    max_seq_len: int = 1024

    ffn_dim_multiplier: Optional[float] = None
    ffn_exp: int = 4
    multiple_of: int = 256
    hidden_dim: Optional[int] = None
    norm_eps: float = 1e-5

    pos_embed_impl: str = "rope"
    rope_theta: float = 10000.0
    scaled_rope: ScaledRoPEConfig = field(default_factory=ScaledRoPEConfig)

    attn_impl: str = "xformers"
    attn_bias_type: Optional[str] = None
    window_attn: Optional[WindowAttentionConfig] = None
    layer_types: Optional[List[str]] = None

    # multi-head latent attention: another architecture, must stay off
    q_lora_rank: int = 0
    kv_lora_rank: int = 0
    qk_nope_head_dim: int = 128
    qk_rope_head_dim: int = 64

    weight_tying: bool = False
    qkv_biases: bool = False
    qk_norm: bool = False

    # storage type that the random-weights writer uses for this model
    dtype: str = "bfloat16"

    def __post_init__(self) -> None:
        for name in ("dim", "n_layers", "n_heads", "vocab_size"):
            if getattr(self, name) <= 0:
                raise ConfigError(f"{name} must be positive, found {getattr(self, name)}")
        if self.n_heads % self.kv_heads != 0:
            raise ConfigError(f"n_heads {self.n_heads} is not a multiple of n_kv_heads {self.kv_heads}")
        if self.head_dim is None and self.dim % self.n_heads != 0:
            raise ConfigError(f"dim {self.dim} is not a multiple of n_heads {self.n_heads} and head_dim is not given")
        if self.head_size % 2 != 0:
            raise ConfigError(f"head_dim {self.head_size} must be even for rotary pairs")
        if self.attn_impl != "xformers":
            # the one value the reference accepts (cwm/model/transformer.py:134); it names the reference's attention
            # library, which this engine's own kernels stand in for, so any other value is a configuration of something else
            raise ConfigError(f"attn_impl must be 'xformers' (cwm/model/transformer.py:134), found {self.attn_impl!r}")
        if self.weight_tying:
            raise ConfigError("weight_tying is not supported (cwm/model/transformer.py:135)")
        if self.q_lora_rank or self.kv_lora_rank:
            raise ConfigError("latent attention (q_lora_rank / kv_lora_rank) is another architecture")
        if self.qk_norm:
            raise ConfigError("qk_norm is not supported (cwm/model/transformer.py:170-171)")
        if self.pos_embed_impl not in ("rope", "scaled_rope"):
            raise ConfigError(f"pos_embed_impl must be 'rope' or 'scaled_rope', found {self.pos_embed_impl!r}")
        if self.attn_bias_type not in (None, "causal"):
            raise ConfigError(f"attn_bias_type {self.attn_bias_type!r}: only causal attention is built")
        if self.norm_eps <= 0 or not math.isfinite(self.norm_eps):
            raise ConfigError("norm_eps must be a positive finite number")
        if self.dtype not in ("bfloat16", "float32"):
            raise ConfigError(f"dtype must be 'bfloat16' or 'float32', found {self.dtype!r}")
        if self.layer_types is not None:
            if len(self.layer_types) != self.n_layers:
                raise ConfigError(f"layer_types has {len(self.layer_types)} entries for {self.n_layers} layers")
            for kind in self.layer_types:
                if kind not in ("global", "local"):
                    raise ConfigError(f"layer_types entries are 'global' or 'local', found {kind!r}")
            if "local" in self.layer_types and (self.window_attn is None or self.window_attn.local_window is None):
                raise ConfigError("layer_types names local layers but window_attn.local_window is not set")
        if self.ffn_width <= 0:
            raise ConfigError("the feed-forward width works out to zero")

    # ---- derived sizes ------------------------------------------------------ #
    @property
    def kv_heads(self) -> int:
        return self.n_kv_heads if self.n_kv_heads is not None else self.n_heads

    @property
    def head_size(self) -> int:
        return self.head_dim if self.head_dim is not None else self.dim // self.n_heads

    @property
    def ffn_width(self) -> int:
        """cwm/model/transformer.py:206-209 applied to ffn_exp * dim (:245-250)."""
        if self.hidden_dim is not None:
            return self.hidden_dim
        hidden = int(2 * (self.ffn_exp * self.dim) / 3)
        if self.ffn_dim_multiplier is not None:
            hidden = int(self.ffn_dim_multiplier * hidden)
        return self.multiple_of * ((hidden + self.multiple_of - 1) // self.multiple_of)

    def layer_windows(self) -> List[Optional[int]]:
        """For each layer the number of keys a query reads, its own included
        (None: all).  cwm/model/transformer.py:253-270."""
        wa = self.window_attn
        if self.layer_types is not None:
            return [
                (wa.local_window if kind == "local" else wa.global_window) if wa is not None else None
                for kind in self.layer_types
            ]
        if wa is None:
            return [None] * self.n_layers
        return [
            wa.global_window if wa.is_global_layer(i, self.n_layers) else wa.local_window
            for i in range(self.n_layers)
        ]
