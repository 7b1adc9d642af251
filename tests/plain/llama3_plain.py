"""Plain implementation of every part of the Llama-3 dense decoder.

Each function is written from the text of the reference (file:line cited in its
docstring), operates on whole sequences with no cache, and imports nothing from
the product package.  All arithmetic runs in the dtype of the inputs (tests use
float32 or float64 on the CPU).

`forward(..., rounding=...)` also emulates a bfloat16 run: the arithmetic stays in
the wide type and the value is rounded to bfloat16 at the places where a
bfloat16 run stores it.  `ROUND_AS_REFERENCE` rounds where the reference does
(every tensor it keeps is bfloat16: cwm/fastgen/forward.py:543-546 embedding, :571
and :772,789 norm outputs, :593-606 projections, :618-619 rotated q and k, :639-655
attention output, :763,769 output projection and the residual sum, :776-781 both
branches, silu and the product, :782,786 down projection and residual sum,
:820-821 logits); `ROUND_AS_ENGINE` rounds where the engine under test keeps a
bfloat16 tensor (the residual stream and the logits stay wide, silu(gate) * up
is rounded once).  In both, the attention probabilities are rounded before
the product with the values, as a matrix-core attention kernel has to.
"""

from __future__ import annotations

import math
from typing import Mapping, Optional, Sequence

import torch


# --------------------------------------------------------------------------- #
# configuration rules
# --------------------------------------------------------------------------- #
def hidden_size(dim: int, ffn_exp: int, ffn_dim_multiplier: Optional[float], multiple_of: int) -> int:
    """SwiGLU hidden width.

    cwm/model/transformer.py:206-209 (rule) with hidden_dim = ffn_exp * dim
    passed in at cwm/model/transformer.py:245-250.
    """
    hidden = int(2 * (ffn_exp * dim) / 3)
    if ffn_dim_multiplier is not None:
        hidden = int(ffn_dim_multiplier * hidden)
    return multiple_of * ((hidden + multiple_of - 1) // multiple_of)


def layer_is_global(layer_id: int, n_layers: int, global_last_layer: bool, window_pattern: int) -> bool:
    """cwm/model/transformer.py:79-85."""
    if global_last_layer and layer_id == n_layers - 1:
        return True
    return layer_id % window_pattern == 0


def window_left_of_layer(
    layer_id: int,
    n_layers: int,
    window_attn: Optional[Mapping[str, object]],
) -> int:
    """Number of keys before its own position a query may read (-1: all of them).

    cwm/model/transformer.py:253-270: a layer with window W reads W keys, its
    own included, so window_left = W - 1.
    """
    if not window_attn:
        return -1
    pattern = int(window_attn.get("window_pattern", 6))
    last = bool(window_attn.get("global_last_layer", True))
    if layer_is_global(layer_id, n_layers, last, pattern):
        gw = window_attn.get("global_window")
        return -1 if gw is None else int(gw) - 1
    lw = window_attn.get("local_window")
    return -1 if lw is None else int(lw) - 1


ROUND_AS_REFERENCE = "reference"
ROUND_AS_ENGINE = "engine"


# --------------------------------------------------------------------------- #
# parts
# --------------------------------------------------------------------------- #
def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """y = x * rsqrt(mean(x^2) + eps) * w.

    cwm/fastgen/kernels/rmsnorm.py:34-61 (mean of squares over the last axis, eps
    added to the mean inside the root, weight a plain multiplier); call sites
    cwm/fastgen/forward.py:571,772,789.
    """
    mean_sq = (x * x).sum(dim=-1, keepdim=True) / x.shape[-1]
    return x * torch.rsqrt(mean_sq + eps) * weight


def rope_frequencies(
    head_dim: int,
    theta: float,
    scaled: Optional[Mapping[str, float]] = None,
) -> torch.Tensor:
    """Inverse frequencies, float32 [head_dim / 2].

    cwm/fastgen/forward.py:1018-1047.  The table is built in float32 as the
    reference does; the llama3 scaling loop runs element by element, first the
    'divide long wavelengths' branch, then the smoothing branch, both reading the
    unscaled value.
    """
    pows = torch.arange(0, head_dim, 2).float() / head_dim
    freqs = 1.0 / (theta ** pows)
    if scaled is None:
        return freqs
    low_ff = scaled["low_freq_factor"]
    high_ff = scaled["high_freq_factor"]
    old_ctx = scaled["old_context_len"]
    scaling = scaled["scale_factor"]
    low_wl = old_ctx / low_ff
    high_wl = old_ctx / high_ff
    out = freqs.clone()
    for idx in range(freqs.numel()):
        freq = freqs[idx]
        wavelen = 2 * math.pi / freq
        if wavelen > low_wl:
            out[idx] = freq / scaling
        if high_wl <= wavelen <= low_wl:
            x = old_ctx / wavelen - low_ff
            x = x / (high_ff - low_ff)
            out[idx] = (1 - x) * freq / scaling + x * freq
    return out


def rope_apply(x: torch.Tensor, positions: torch.Tensor, freqs: torch.Tensor) -> torch.Tensor:
    """Rotate adjacent pairs (2i, 2i+1) of the last axis by positions * freqs[i].

    cwm/fastgen/kernels/rope.py:55-90: angle = pos * freq in float32;
    re' = re cos - im sin, im' = im cos + re sin; the same rotation for every head.
    x: [T, H, hd]; positions: [T]; freqs: [hd/2].
    """
    angles = positions.to(x.device, torch.float32)[:, None] * freqs.to(x.device, torch.float32)[None, :]  # [T, hd/2]
    cos = torch.cos(angles).to(x.dtype)[:, None, :]
    sin = torch.sin(angles).to(x.dtype)[:, None, :]
    re = x[..., 0::2]
    im = x[..., 1::2]
    out = torch.empty_like(x)
    out[..., 0::2] = re * cos - im * sin
    out[..., 1::2] = im * cos + re * sin
    return out


def round_bf16(x: torch.Tensor) -> torch.Tensor:
    """x rounded to the nearest bfloat16 (ties to even), in x's own type."""
    return x.to(torch.bfloat16).to(x.dtype)


def attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    window_left: int = -1,
    scale: Optional[float] = None,
    round_probabilities: bool = False,
) -> torch.Tensor:
    """Causal grouped-query attention over one whole sequence.

    cwm/fastgen/forward.py:638-655: softmax(q k^T * hd^-1/2) v over keys j <= p and,
    with window_left = w >= 0, j >= p - w; query head h reads key/value head
    h // (Hq / Hkv).  q: [T, Hq, hd]; k, v: [T, Hkv, hd]; returns [T, Hq, hd].
    With `round_probabilities` the unnormalised probabilities exp(s - max) are
    rounded to bfloat16 for the sum over the values while their own sum is not, as
    in an attention kernel that feeds them to a bfloat16 matrix product.
    """
    n_tok, n_q, hd = q.shape
    n_kv = k.shape[1]
    group = n_q // n_kv
    if scale is None:
        scale = hd ** -0.5
    pos = torch.arange(n_tok, device=q.device)
    distance = pos[:, None] - pos[None, :]  # query position - key position
    allowed = distance >= 0
    if window_left >= 0:
        allowed &= distance <= window_left
    out = torch.empty_like(q)
    for h in range(n_q):
        g = h // group
        scores = (q[:, h, :] @ k[:, g, :].T) * scale  # [T, T]
        scores = scores.masked_fill(~allowed, float("-inf"))
        if round_probabilities:
            e = torch.exp(scores - scores.max(dim=-1, keepdim=True).values)
            out[:, h, :] = (round_bf16(e) @ v[:, g, :]) / e.sum(dim=-1, keepdim=True)
        else:
            out[:, h, :] = torch.softmax(scores, dim=-1) @ v[:, g, :]
    return out


def swiglu(
    x: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor, w3: torch.Tensor, rounding: Optional[str] = None
) -> torch.Tensor:
    """(silu(x w1^T) * (x w3^T)) w2^T.  cwm/fastgen/forward.py:776-782.

    In a bfloat16 run the reference stores x1, x3, silu(x1) (in place) and the
    product (in place), each rounded (:776-781); the engine stores both branches
    and the finished product."""
    rnd = round_bf16 if rounding else (lambda t: t)
    gate = rnd(x @ w1.T)
    up = rnd(x @ w3.T)
    act = gate * torch.sigmoid(gate)
    if rounding == ROUND_AS_REFERENCE:
        act = rnd(act)
    return rnd(rnd(act * up) @ w2.T)


def linear(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """y = x W^T (+ b), weight [out, in].  cwm/fastgen/forward.py:593-606."""
    y = x @ weight.T
    if bias is not None:
        y = y + bias
    return y


# --------------------------------------------------------------------------- #
# whole model
# --------------------------------------------------------------------------- #
def forward(
    weights: Mapping[str, torch.Tensor],
    tokens: Sequence[int],
    *,
    n_layers: int,
    n_heads: int,
    n_kv_heads: int,
    head_dim: int,
    norm_eps: float,
    rope_freqs: torch.Tensor,
    window_left: Sequence[int],
    first_position: int = 0,
    dtype: torch.dtype = torch.float32,
    rounding: Optional[str] = None,
) -> torch.Tensor:
    """Logits [T, V] of one whole sequence.

    Order of operations from cwm/fastgen/forward.py:543-821: embedding; per layer
    h += wo(attn(rope(wq x), rope(wk x), wv x)) with x = norm(h), then
    h += w2(silu(w1 x) * w3 x) with x = norm(h); final norm; output projection.
    Weight names are the module names of cwm/model/transformer.py:173-193,214-228,
    244-252,301-313.  `first_position` shifts every position (used by tests of the
    rotation's dependence on distances only).  `rounding`: None, or one of
    ROUND_AS_REFERENCE / ROUND_AS_ENGINE (see the module's text): the weights are
    rounded to bfloat16 and so is every tensor that such a run stores.
    """
    if rounding not in (None, ROUND_AS_REFERENCE, ROUND_AS_ENGINE):
        raise ValueError(f"unknown rounding {rounding!r}")
    rnd = round_bf16 if rounding else (lambda t: t)
    # the residual stream: bfloat16 in the reference (h.add_ at forward.py:769,786), wide in the engine
    rnd_h = round_bf16 if rounding == ROUND_AS_REFERENCE else (lambda t: t)
    weights = {name: (t.to(torch.bfloat16) if rounding and t.is_floating_point() else t) for name, t in weights.items()}
    w = {name: t.to(dtype) for name, t in weights.items()}
    table = w["tok_embeddings.weight"]
    tok = torch.as_tensor(list(tokens), dtype=torch.long, device=table.device)
    positions = torch.arange(len(tok), device=table.device) + first_position
    h = table[tok]
    for i in range(n_layers):
        pre = f"layers.{i}."
        x = rnd(rms_norm(h, w[pre + "attention_norm.weight"], norm_eps))
        xq = rnd(linear(x, w[pre + "attention.wq.weight"], w.get(pre + "attention.wq.bias")))
        xk = rnd(linear(x, w[pre + "attention.wk.weight"], w.get(pre + "attention.wk.bias")))
        xv = rnd(linear(x, w[pre + "attention.wv.weight"], w.get(pre + "attention.wv.bias")))
        xq = xq.view(-1, n_heads, head_dim)
        xk = xk.view(-1, n_kv_heads, head_dim)
        xv = xv.view(-1, n_kv_heads, head_dim)
        xq = rnd(rope_apply(xq, positions, rope_freqs))
        xk = rnd(rope_apply(xk, positions, rope_freqs))
        att = rnd(attention(xq, xk, xv, window_left=window_left[i], round_probabilities=bool(rounding)))
        h = rnd_h(h + rnd(linear(att.reshape(len(tok), -1), w[pre + "attention.wo.weight"])))
        x = rnd(rms_norm(h, w[pre + "ffn_norm.weight"], norm_eps))
        h = rnd_h(
            h
            + swiglu(
                x,
                w[pre + "feed_forward.w1.weight"],
                w[pre + "feed_forward.w2.weight"],
                w[pre + "feed_forward.w3.weight"],
                rounding,
            )
        )
    h = rnd(rms_norm(h, w["norm.weight"], norm_eps))
    logits = linear(h, w["output.weight"])
    # the reference's head writes bfloat16 before `.float()` (forward.py:820-821); the engine's writes float32
    return round_bf16(logits) if rounding == ROUND_AS_REFERENCE else logits


def forward_from_config(
    weights: Mapping[str, torch.Tensor],
    config: Mapping[str, object],
    tokens: Sequence[int],
    dtype: torch.dtype = torch.float32,
    first_position: int = 0,
    rounding: Optional[str] = None,
) -> torch.Tensor:
    """`forward` with its constants taken from a config.json dictionary.

    Key names and defaults: cwm/model/transformer.py:88-145.  Two keys of the
    model-folder format have no counterpart there and are read here too:
    `hidden_dim` is not needed (weights carry it) and `layer_types`, an explicit
    per-layer list of "global" / "local" that replaces the reference rule.
    """
    n_layers = int(config["n_layers"])
    n_heads = int(config["n_heads"])
    n_kv = int(config.get("n_kv_heads") or n_heads)
    head_dim = int(config.get("head_dim") or int(config["dim"]) // n_heads)
    scaled = None
    if config.get("pos_embed_impl", "rope") == "scaled_rope":
        sr = dict(config.get("scaled_rope") or {})
        scaled = {
            "scale_factor": sr.get("scale_factor", 8),
            "old_context_len": sr.get("old_context_len", 8192),
            "low_freq_factor": sr.get("low_freq_factor", 1),
            "high_freq_factor": sr.get("high_freq_factor", 4),
        }
    freqs = rope_frequencies(head_dim, float(config.get("rope_theta", 10000.0)), scaled)
    wa = config.get("window_attn")
    kinds = config.get("layer_types")
    if kinds is not None:
        lefts = []
        for kind in kinds:
            size = (wa or {}).get("local_window" if kind == "local" else "global_window")
            lefts.append(-1 if size is None else int(size) - 1)
    else:
        lefts = [window_left_of_layer(i, n_layers, wa) for i in range(n_layers)]
    return forward(
        weights,
        tokens,
        n_layers=n_layers,
        n_heads=n_heads,
        n_kv_heads=n_kv,
        head_dim=head_dim,
        norm_eps=float(config.get("norm_eps", 1e-5)),
        rope_freqs=freqs,
        window_left=lefts,
        first_position=first_position,
        dtype=dtype,
        rounding=rounding,
    )


# --------------------------------------------------------------------------- #
# sampling
# --------------------------------------------------------------------------- #
def sampling_probabilities(logits: torch.Tensor, temperature: float, top_p: float) -> torch.Tensor:
    """Distribution the reference draws from, [V].

    cwm/fastgen/generate.py:1003 (softmax(logits / T) in float32) and
    cwm/fastgen/utils/sampling.py:38-45 (sort descending, cumulate, drop entries
    whose preceding mass exceeds top_p, renormalise).
    """
    probs = torch.softmax(logits.float() / temperature, dim=-1)
    if top_p >= 1.0:
        return probs
    sorted_p, order = torch.sort(probs, dim=-1, descending=True)
    csum = torch.cumsum(sorted_p, dim=-1)
    sorted_p = sorted_p.clone()
    sorted_p[csum - sorted_p > top_p] = 0.0
    sorted_p = sorted_p / sorted_p.sum(-1, keepdim=True)
    out = torch.zeros_like(probs)
    out[order] = sorted_p
    return out


def sample_inverse_cdf(probs: torch.Tensor, u: float) -> int:
    """First index whose cumulative probability (vocabulary order, float64)
    reaches u * total: a draw from `probs` given a uniform u in [0, 1)."""
    c = torch.cumsum(probs.double(), dim=-1)
    target = u * float(c[-1])
    idx = int(torch.searchsorted(c, torch.tensor(target, dtype=torch.float64), right=True))
    nz = torch.nonzero(probs > 0).flatten()
    idx = min(idx, int(nz[-1]))
    while probs[idx] <= 0:
        idx += 1
    return idx


def greedy(logits: torch.Tensor) -> int:
    """cwm/fastgen/generate.py:1012 (argmax when use_sampling is off)."""
    return int(torch.argmax(logits, dim=-1))
