"""Stand-ins for the HIP kernels, written with torch on the CPU.

The product has no CPU path.  These functions exist so that tests which run without
a GPU can exercise everything *around* the kernels (batch descriptors, block
tables, page reuse, the scheduler) by patching `cwm_amd.ops`; they follow the same
signatures and the same cache layout as the kernels' wrappers.
"""

from __future__ import annotations

import math
from typing import Optional

import torch

from helpers import cache_layout


def embedding(tokens, table, scale=1.0):
    return table[tokens.long()].float() * scale


def add_rmsnorm(h, delta, weight, eps, out_dtype, rows=None):
    if delta is not None and delta.dim() == 3:
        delta = delta.float().sum(0)
    if delta is not None:
        if rows is None:
            h += delta.float()
            x = h
        else:
            x = h + delta.float()
    else:
        x = h
    if rows is not None:
        x = x[rows.long()]
    y = x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps) * weight.float()
    return y.to(out_dtype)


def silu_mul(gate_up, out_dtype=None, grouped=False):
    if gate_up.dim() == 3:
        gate_up = gate_up.sum(0).to(out_dtype or torch.float32)
    f = gate_up.shape[1] // 2
    if grouped:
        pairs = gate_up.reshape(gate_up.shape[0], f // 8, 2, 8)
        g, u = pairs[:, :, 0].reshape(-1, f).float(), pairs[:, :, 1].reshape(-1, f).float()
    else:
        g, u = gate_up[:, :f].float(), gate_up[:, f:].float()
    return (g * torch.sigmoid(g) * u).to(gate_up.dtype)


def gate_up_silu(x, weight, bias, grouped, streamed=None):
    return silu_mul(linear(x, weight, bias), grouped=grouped)


def linear(x, weight, bias=None, out_dtype=None, partials_ok=False, streamed=None):
    y = x.float() @ weight.float().T
    if bias is not None:
        y = y + bias.float()
    return y.to(out_dtype or x.dtype)


gemm_f32 = linear
gemm_bf16 = linear


def _rotate(x, positions, inv_freq):
    ang = positions.float()[:, None] * inv_freq[None, :]
    c = torch.cos(ang)[:, None, :]
    s = torch.sin(ang)[:, None, :]
    xf = x.float()
    re, im = xf[..., 0::2], xf[..., 1::2]
    out = torch.empty_like(xf)
    out[..., 0::2] = re * c - im * s
    out[..., 1::2] = im * c + re * s
    return out.to(x.dtype)


def rope_kv_write(q, k, v, positions, inv_freq, cache=None, block_table=None, seq_of_token=None):
    if inv_freq is not None:
        q.copy_(_rotate(q, positions, inv_freq))
        if k is not None:
            k.copy_(_rotate(k, positions, inv_freq))
    if cache is None:
        return
    n_tokens, n_kv, hd = k.shape
    page_size = cache.shape[3] // hd
    for t in range(n_tokens):
        pos = int(positions[t])
        page = int(block_table[int(seq_of_token[t]), pos // page_size])
        assert page >= 0, "write to a page that is not held"
        slot = pos % page_size
        cache_layout.write_kv(cache, page, slot, k[t], v[t], hd)


def qkv_rope_write(x, weight, bias, n_q_heads, n_kv_heads, head_dim, positions, inv_freq, cache, block_table, seq_of_token, streamed=None):
    qkv = linear(x, weight, bias)
    q_out, kv_out = n_q_heads * head_dim, n_kv_heads * head_dim
    q = qkv[:, :q_out].unflatten(1, (n_q_heads, head_dim))
    k = qkv[:, q_out : q_out + kv_out].unflatten(1, (n_kv_heads, head_dim))
    v = qkv[:, q_out + kv_out :].unflatten(1, (n_kv_heads, head_dim))
    rope_kv_write(q, k, v, positions, inv_freq, cache, block_table, seq_of_token)
    return qkv


def paged_attention(q, cache, block_table, batch, window, scale):
    n_tokens, n_q, hd = q.shape
    n_kv = cache.shape[2]
    page_size = cache.shape[3] // hd
    group = n_q // n_kv
    out = torch.empty((n_tokens, n_q, hd), dtype=torch.float32)
    for t in range(n_tokens):
        p = int(batch.positions[t])
        b = int(batch.seq_of_token[t])
        lo = 0 if window is None else max(0, p - (window - 1))
        keys, vals = [], []
        for j in range(lo, p + 1):
            page = int(block_table[b, j // page_size])
            assert page >= 0, f"key {j} of sequence {b} has no page"
            slot = j % page_size
            kk_, vv_ = cache_layout.read_kv(cache, page, slot, hd)
            keys.append(kk_.float())
            vals.append(vv_.float())
        kk = torch.stack(keys, 1)  # [n_kv, n, hd]
        vv = torch.stack(vals, 1)
        for h in range(n_q):
            g = h // group
            s = (kk[g] @ q[t, h].float()) * scale
            w = torch.softmax(s, -1)
            out[t, h] = w @ vv[g]
    return out.reshape(n_tokens, n_q * hd).to(q.dtype)


def sample(logits, temperature, top_p, uniform):
    n, vocab = logits.shape
    toks = torch.empty(n, dtype=torch.int32)
    lp = torch.empty(n)
    slp = torch.empty(n)
    for r in range(n):
        x = logits[r].float()
        logp = torch.log_softmax(x, -1)
        t = float(temperature[r])
        if not t > 0:
            tok = int(torch.argmax(x))
            toks[r], lp[r], slp[r] = tok, logp[tok], 0.0
            continue
        probs = torch.softmax(x / t, -1)
        tp = float(top_p[r])
        if tp < 1.0:
            sp, order = torch.sort(probs, descending=True)
            cs = torch.cumsum(sp, -1)
            sp[cs - sp > tp] = 0.0
            kept = torch.zeros_like(probs)
            kept[order] = sp
            probs = kept
        c = torch.cumsum(probs.double(), -1)
        target = float(uniform[r]) * float(c[-1])
        tok = int(torch.searchsorted(c, torch.tensor(target, dtype=torch.float64), right=True))
        tok = min(tok, vocab - 1)
        while probs[tok] <= 0:
            tok -= 1
        toks[r], lp[r], slp[r] = tok, logp[tok], math.log(float(probs[tok] / probs.sum()))
    return toks, lp, slp


def sample_packed(logits, temperature, top_p, uniform):
    toks, lp, slp = sample(logits, temperature, top_p, uniform)
    return torch.stack([toks, lp.float().view(torch.int32), slp.float().view(torch.int32)])


def token_logprobs(logits, rows, targets):
    lp = torch.log_softmax(logits.float()[rows.long()], -1)
    return lp.gather(1, targets.long()[:, None])[:, 0]


def install(monkeypatch) -> None:
    """Patch every kernel entry point of `cwm_amd.ops` with its stand-in."""
    import cwm_amd.ops as ops

    for name in (
        "embedding", "add_rmsnorm", "silu_mul", "gate_up_silu", "linear", "gemm_f32", "gemm_bf16",
        "rope_kv_write", "qkv_rope_write", "paged_attention", "sample", "sample_packed", "token_logprobs",
    ):
        monkeypatch.setattr(ops, name, globals()[name])
