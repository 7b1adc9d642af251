"""Each HIP kernel alone against the plain implementation, at sizes other than the
tiny models': widths and vocabularies that are no power of two, several head
sizes in steps of 16, odd head counts, page sizes from 1 token up."""

import math

import numpy as np
import pytest
import torch

from helpers import cache_layout
from plain import llama3_plain as plain

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


def tol(dtype):
    return dict(rtol=2e-5, atol=2e-6) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)


def rnd(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


@pytest.mark.parametrize("table_dtype", DTYPES)
@pytest.mark.parametrize("vocab,dim", [(263, 120), (1000, 6144), (17, 7)])
def test_embedding(table_dtype, vocab, dim):
    from cwm_amd import ops

    table = rnd((vocab, dim), table_dtype, 1)
    tokens = torch.tensor([0, vocab - 1, 5 % vocab, 3 % vocab, vocab - 1], dtype=torch.int32)
    out = ops.embedding(tokens.to(DEV), table.to(DEV)).cpu()
    assert out.dtype == torch.float32
    torch.testing.assert_close(out, table[tokens.long()].float(), rtol=0, atol=0)


@pytest.mark.parametrize("out_dtype", DTYPES)
@pytest.mark.parametrize("w_dtype", DTYPES)
@pytest.mark.parametrize("dim,eps", [(120, 1e-5), (6144, 1e-6), (1000, 3e-3), (7, 1e-5)])
def test_add_rmsnorm(out_dtype, w_dtype, dim, eps):
    from cwm_amd import ops

    n = 9
    h = rnd((n, dim), torch.float32, 2, 3.0)
    delta = rnd((n, dim), out_dtype, 3)
    w = (rnd((dim,), torch.float32, 4) * 0.2 + 1.0).to(w_dtype)
    want_h = h.double() + delta.double()
    want = plain.rms_norm(want_h, w.double(), eps)
    hd = h.to(DEV).clone()
    got = ops.add_rmsnorm(hd, delta.to(DEV), w.to(DEV), eps, out_dtype).cpu()
    torch.testing.assert_close(hd.cpu().double(), want_h, rtol=1e-6, atol=1e-6)  # the residual sum itself is float32
    torch.testing.assert_close(got.double(), want, **tol(out_dtype))
    # without a delta, and on chosen rows only (h untouched)
    got2 = ops.add_rmsnorm(h.to(DEV), None, w.to(DEV), eps, out_dtype).cpu()
    torch.testing.assert_close(got2.double(), plain.rms_norm(h.double(), w.double(), eps), **tol(out_dtype))
    rows = torch.tensor([4, 0, 8], dtype=torch.int32)
    hd = h.to(DEV).clone()
    got3 = ops.add_rmsnorm(hd, delta.to(DEV), w.to(DEV), eps, out_dtype, rows=rows.to(DEV)).cpu()
    torch.testing.assert_close(hd.cpu(), h, rtol=0, atol=0)
    torch.testing.assert_close(got3.double(), want[rows.long()], **tol(out_dtype))


def test_rmsnorm_eps_placement_shows():
    """With tiny inputs eps dominates: y = x / sqrt(eps) * w.  An eps added outside the
    root or to the sum instead of the mean gives another number."""
    from cwm_amd import ops

    dim, eps = 96, 1e-2
    h = torch.full((1, dim), 1e-4, dtype=torch.float32)
    w = torch.ones(dim)
    got = ops.add_rmsnorm(h.to(DEV), None, w.to(DEV), eps, torch.float32).cpu()
    want = 1e-4 / math.sqrt(1e-8 + eps)
    np.testing.assert_allclose(got.numpy(), want, rtol=1e-5)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden", [296, 21504 // 8, 5])
def test_silu_mul(dtype, hidden):
    from cwm_amd import ops

    x = rnd((7, 2 * hidden), dtype, 5, 2.0)
    got = ops.silu_mul(x.to(DEV)).cpu()
    g, u = x[:, :hidden].double(), x[:, hidden:].double()
    want = g * torch.sigmoid(g) * u
    torch.testing.assert_close(got.double(), want, **tol(dtype))
    # gate and up are not interchangeable
    swapped = torch.cat([x[:, hidden:], x[:, :hidden]], 1)
    assert not torch.allclose(ops.silu_mul(swapped.to(DEV)).cpu().double(), want, atol=1e-2)


def _grouped(gate, up):
    """[T, F] gate and up -> [T, 2F] with gate and up alternating in groups of 8 columns."""
    t, f = gate.shape
    return torch.stack([gate.reshape(t, f // 8, 8), up.reshape(t, f // 8, 8)], dim=2).reshape(t, 2 * f)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden", [8, 40, 296])
def test_silu_mul_grouped_layout(dtype, hidden):
    """Gate and up in alternating groups of 8 columns give the same bits as the two halves."""
    from cwm_amd import ops

    x = rnd((7, 2 * hidden), dtype, 5, 2.0)
    halves = ops.silu_mul(x.to(DEV))
    grouped = ops.silu_mul(_grouped(x[:, :hidden], x[:, hidden:]).contiguous().to(DEV), grouped=True)
    assert torch.equal(halves, grouped)
    p = rnd((3, 7, 2 * hidden), torch.float32, 6, 1.5)
    pg = torch.stack([_grouped(q[:, :hidden], q[:, hidden:]) for q in p]).contiguous()
    assert torch.equal(ops.silu_mul(p.to(DEV), out_dtype=dtype), ops.silu_mul(pg.to(DEV), out_dtype=dtype, grouped=True))
    with pytest.raises(ops.KernelError, match="multiple of 8"):
        ops.silu_mul(rnd((2, 20), dtype, 1).to(DEV), grouped=True)


@pytest.mark.parametrize("m,f,k,bias", [(1, 24, 64, False), (8, 21504 // 8, 6144 // 4, False), (16, 296, 120, True), (5, 8, 8, True)])
def test_gate_up_silu_in_the_products_epilogue(m, f, k, bias):
    """The streaming product with the gated epilogue against the product followed by the
    activation kernel (the same bits), and against float64."""
    from cwm_amd import ops

    x = rnd((m, k), torch.bfloat16, 1)
    wg, wu = rnd((f, k), torch.bfloat16, 2, 0.2), rnd((f, k), torch.bfloat16, 3, 0.2)
    bg, bu = (rnd((f,), torch.bfloat16, 4), rnd((f,), torch.bfloat16, 5)) if bias else (None, None)
    w = torch.stack([wg.reshape(f // 8, 8, k), wu.reshape(f // 8, 8, k)], dim=1).reshape(2 * f, k).contiguous()
    b = torch.stack([bg.reshape(f // 8, 8), bu.reshape(f // 8, 8)], dim=1).reshape(2 * f).contiguous() if bias else None
    dev = lambda t: None if t is None else t.to(DEV)
    fused = ops.gemm_bf16_stream(dev(x), dev(w), dev(b), torch.bfloat16, glu=True)
    assert fused.shape == (m, f)
    two_steps = ops.silu_mul(ops.gemm_bf16_stream(dev(x), dev(w), dev(b), torch.bfloat16), grouped=True)
    assert torch.equal(fused, two_steps)
    assert torch.equal(ops.gate_up_silu(dev(x), dev(w), dev(b), True), fused)
    g = x.double() @ wg.double().T + (bg.double() if bias else 0)
    u = x.double() @ wu.double().T + (bu.double() if bias else 0)
    want = g * torch.sigmoid(g) * u
    torch.testing.assert_close(fused.cpu().double(), want, rtol=3e-2, atol=3e-2 * float(want.abs().max()))


@pytest.mark.parametrize("out_dtype", DTYPES)
@pytest.mark.parametrize("hidden,parts", [(40, 3), (132, 1), (21, 2)])
def test_silu_mul_of_partial_sums(out_dtype, hidden, parts):
    """Partial sums of a gate/up product go straight into the activation: the same bits as
    adding them, rounding to the output type and applying the kernel for whole sums."""
    from cwm_amd import ops

    p = rnd((parts, 9, 2 * hidden), torch.float32, 12, 1.5).to(DEV)
    got = ops.silu_mul(p, out_dtype=out_dtype)
    assert got.dtype == out_dtype and got.shape == (9, hidden)
    two_steps = ops.silu_mul(ops.sum_partials(p, out_dtype))
    assert torch.equal(got, two_steps)
    whole = p.double().sum(0).cpu()
    g, u = whole[:, :hidden], whole[:, hidden:]
    torch.testing.assert_close(got.cpu().double(), g * torch.sigmoid(g) * u, **tol(out_dtype))


@pytest.mark.parametrize("a_dtype,w_dtype,c_dtype", [
    (torch.float32, torch.float32, torch.float32),
    (torch.bfloat16, torch.float32, torch.bfloat16),
    (torch.bfloat16, torch.bfloat16, torch.float32),
    (torch.float32, torch.bfloat16, torch.float32),
])
@pytest.mark.parametrize("m,n,k", [(1, 263, 120), (5, 64, 64), (67, 130, 17), (130, 509, 296), (3, 1, 1)])
def test_gemm_f32(a_dtype, w_dtype, c_dtype, m, n, k):
    from cwm_amd import ops

    a = rnd((m, k), a_dtype, 6)
    w = rnd((n, k), w_dtype, 7)
    b = rnd((n,), w_dtype, 8)
    got = ops.gemm_f32(a.to(DEV), w.to(DEV), b.to(DEV), out_dtype=c_dtype).cpu()
    want = a.double() @ w.double().T + b.double()
    # float32 sums of k products of unit-variance numbers: rounding grows with k
    t = dict(rtol=1e-5, atol=2e-7 * k + 1e-6) if c_dtype == torch.float32 else dict(rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(got.double(), want, **t)


def test_gemm_f32_is_true_float32():
    """Products of numbers that need all 24 bits: a reduced-precision matrix mode
    (bfloat16 or tf32 inputs) would lose the low bits."""
    from cwm_amd import ops

    k = 4  # short enough that the float32 sum itself is exact
    a = torch.full((2, k), 1.0 + 2.0 ** -20, dtype=torch.float32)
    w = torch.full((3, k), 1.0 - 2.0 ** -21, dtype=torch.float32)
    got = ops.gemm_f32(a.to(DEV), w.to(DEV)).cpu().double()
    want = a.double() @ w.double().T
    assert (got - want).abs().max() < 1e-7
    assert (got - float(k)).abs().min() > 1e-6  # not rounded to 1.0 * 1.0


@pytest.mark.parametrize("c_dtype", DTYPES)
@pytest.mark.parametrize("m,n,k", [(1, 263, 120), (8, 6144, 6144), (5, 64, 64), (16, 509, 296), (7, 130, 4), (3, 1000, 21504), (16, 48, 3080), (2, 7, 40)])
def test_gemm_f32_stream(c_dtype, m, n, k):
    """The weight-streaming float32 product for up to 16 rows: against float64, with and without
    partial sums of a split K, and a row's bits do not depend on how many rows the call has."""
    from cwm_amd import ops

    a = rnd((m, k), torch.float32, 6)
    w = rnd((n, k), torch.float32, 7)
    b = rnd((n,), torch.float32, 8)
    want = a.double() @ w.double().T + b.double()
    t = dict(rtol=1e-5, atol=2e-7 * k + 1e-6) if c_dtype == torch.float32 else dict(rtol=1e-2, atol=1e-2)
    got = ops.gemm_f32_stream(a.to(DEV), w.to(DEV), b.to(DEV), out_dtype=c_dtype).cpu()
    assert got.dtype == c_dtype
    torch.testing.assert_close(got.double(), want, **t)
    parts = ops.gemm_f32_stream(a.to(DEV), w.to(DEV), b.to(DEV), out_dtype=c_dtype, partials_ok=True).cpu()
    if parts.dim() == 3:
        assert parts.dtype == torch.float32
        parts = parts.sum(0)
    torch.testing.assert_close(parts.double(), want, **t)
    fewer = max(1, m // 2)
    one = ops.gemm_f32_stream(a[m - fewer :].contiguous().to(DEV), w.to(DEV), b.to(DEV), out_dtype=c_dtype).cpu()
    assert torch.equal(one, got[m - fewer :])
    # through `linear`: float32 operands of few rows take this kernel
    via = ops.linear(a.to(DEV), w.to(DEV), b.to(DEV), c_dtype).cpu()
    assert torch.equal(via, got)


def test_gemm_f32_stream_is_true_float32_and_refuses_what_it_does_not_take():
    from cwm_amd import ops

    k = 4
    a = torch.full((2, k), 1.0 + 2.0 ** -20, dtype=torch.float32)
    w = torch.full((3, k), 1.0 - 2.0 ** -21, dtype=torch.float32)
    got = ops.gemm_f32_stream(a.to(DEV), w.to(DEV)).cpu().double()
    want = a.double() @ w.double().T
    assert (got - want).abs().max() < 1e-7
    assert (got - float(k)).abs().min() > 1e-6  # not rounded to 1.0 * 1.0
    with pytest.raises(ops.KernelError):
        ops.gemm_f32_stream(torch.zeros(17, 8, device=DEV), torch.zeros(4, 8, device=DEV))
    with pytest.raises(ops.KernelError):
        ops.gemm_f32_stream(torch.zeros(2, 6, device=DEV), torch.zeros(4, 6, device=DEV))
    # a row length that is no multiple of 4 goes to the other float32 kernel through `linear`
    x, y = rnd((3, 6), torch.float32, 1), rnd((5, 6), torch.float32, 2)
    torch.testing.assert_close(ops.linear(x.to(DEV), y.to(DEV)).cpu().double(), x.double() @ y.double().T, rtol=1e-5, atol=1e-5)


def test_gemm_rows_do_not_depend_on_batch():
    from cwm_amd import ops

    a = rnd((70, 120), torch.float32, 9).to(DEV)
    w = rnd((263, 120), torch.float32, 10).to(DEV)
    full = ops.gemm_f32(a, w)
    one = ops.gemm_f32(a[33:34].contiguous(), w)
    assert torch.equal(full[33:34], one)


def _paged_setup(dtype, n_kv, hd, page_size, lens_old, lens_new, seed):
    """Random k/v for sequences; returns per-sequence full q, k, v and a shuffled
    page assignment."""
    g = torch.Generator().manual_seed(seed)
    seqs = []
    for n0, n1 in zip(lens_old, lens_new):
        n = n0 + n1
        seqs.append(dict(n0=n0, n1=n1, k=torch.randn((n, n_kv, hd), generator=g).to(dtype), v=torch.randn((n, n_kv, hd), generator=g).to(dtype)))
    total_pages = sum((s["n0"] + s["n1"] + page_size - 1) // page_size for s in seqs) + 3
    perm = torch.randperm(total_pages, generator=g).tolist()
    width = max((s["n0"] + s["n1"] + page_size - 1) // page_size for s in seqs)
    table = torch.full((len(seqs), width), -1, dtype=torch.int32)
    for b, s in enumerate(seqs):
        for lp in range((s["n0"] + s["n1"] + page_size - 1) // page_size):
            table[b, lp] = perm.pop()
    return seqs, table, total_pages


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n_q,n_kv,hd,page_size", [(4, 2, 16, 4), (3, 1, 32, 16), (5, 5, 48, 1), (12, 2, 128, 64), (2, 1, 256, 8), (6, 3, 80, 5)])
def test_rope_kv_write_and_attention(dtype, n_q, n_kv, hd, page_size):
    """Rotation + cache write + paged attention for a mixed batch (a fresh prompt, a
    continued portion, a single decoded token) against the plain functions on whole
    sequences; pages are handed out in a shuffled order."""
    from cwm_amd import ops

    lens_old, lens_new = [0, 37, 70], [29, 21, 1]
    for window in (None, 9):
        seqs, table, total_pages = _paged_setup(dtype, n_kv, hd, page_size, lens_old, lens_new, seed=hd + n_q)
        inv_freq = plain.rope_frequencies(hd, 10000.0)
        cache = torch.full((total_pages, 2, n_kv, page_size * hd), float("nan"), dtype=dtype)
        g = torch.Generator().manual_seed(11)
        scale = hd ** -0.5
        want_rows, q_rows, k_rows, v_rows, pos_rows, seq_rows = [], [], [], [], [], []
        for b, s in enumerate(seqs):
            n = s["n0"] + s["n1"]
            q_full = torch.randn((n, n_q, hd), generator=g).to(dtype)
            pos = torch.arange(n)
            q_rot = plain.rope_apply(q_full.double(), pos, inv_freq)
            k_rot = plain.rope_apply(s["k"].double(), pos, inv_freq)
            want = plain.attention(q_rot, k_rot.to(dtype).double(), s["v"].double(), window_left=-1 if window is None else window - 1, scale=scale)
            want_rows.append(want[s["n0"]:].reshape(s["n1"], -1))
            # the old part is already in the cache (rotated keys, rounded to the storage type)
            for j in range(s["n0"]):
                page, slot = int(table[b, j // page_size]), j % page_size
                cache_layout.write_kv(cache, page, slot, k_rot[j].to(dtype), s["v"][j], hd)
            q_rows.append(q_full[s["n0"]:])
            k_rows.append(s["k"][s["n0"]:])
            v_rows.append(s["v"][s["n0"]:])
            pos_rows.append(pos[s["n0"]:])
            seq_rows.append(torch.full((s["n1"],), b))
        # q, k, v as views of one joined projection output, as the model has them
        q = torch.cat(q_rows).flatten(1)
        k = torch.cat(k_rows).flatten(1)
        v = torch.cat(v_rows).flatten(1)
        qkv = torch.cat([q, k, v], 1).to(DEV)
        positions = torch.cat(pos_rows).to(torch.int32).to(DEV)
        seq_of_token = torch.cat(seq_rows).to(torch.int32).to(DEV)
        qv = qkv[:, : n_q * hd].unflatten(1, (n_q, hd))
        kv = qkv[:, n_q * hd : (n_q + n_kv) * hd].unflatten(1, (n_kv, hd))
        vv = qkv[:, (n_q + n_kv) * hd :].unflatten(1, (n_kv, hd))
        cache_d = cache.to(DEV)
        table_d = table.to(DEV)
        ops.rope_kv_write(qv, kv, vv, positions, inv_freq.to(DEV), cache_d, table_d, seq_of_token)
        got = ops.paged_attention_simple(qv, cache_d, table_d, positions, seq_of_token, window, scale).cpu()
        want = torch.cat(want_rows)
        t = dict(rtol=1e-4, atol=1e-5) if dtype == torch.float32 else dict(rtol=3e-2, atol=3e-2)
        torch.testing.assert_close(got.double(), want, **t)
        # the new keys and values sit where the table says, values transposed
        cache_h = cache_d.cpu()
        for b, s in enumerate(seqs):
            j = s["n0"] + s["n1"] - 1
            page, slot = int(table[b, j // page_size]), j % page_size
            k_rot = plain.rope_apply(s["k"][j : j + 1].double(), torch.tensor([j]), inv_freq)[0]
            k_got, v_got = cache_layout.read_kv(cache_h, page, slot, hd)
            torch.testing.assert_close(k_got.double(), k_rot, **t)
            assert torch.equal(v_got, s["v"][j])


def test_attention_far_key_stands_out():
    """One far key among hundreds is made to dominate (its key equals the scaled
    query): the output must be that key's value."""
    from cwm_amd import ops

    n_q, n_kv, hd, page_size, n = 2, 1, 64, 16, 600
    g = torch.Generator().manual_seed(5)
    k = torch.randn((n, n_kv, hd), generator=g) * 0.1
    v = torch.randn((n, n_kv, hd), generator=g)
    q = torch.randn((1, n_q, hd), generator=g)
    far = 3
    k[far, 0] = q[0, 1] * 40.0
    pages = (n + page_size - 1) // page_size
    table = torch.arange(pages, dtype=torch.int32).flip(0).reshape(1, pages).contiguous()
    cache = torch.zeros((pages, 2, n_kv, page_size * hd))
    for j in range(n):
        page, slot = int(table[0, j // page_size]), j % page_size
        cache_layout.write_kv(cache, page, slot, k[j], v[j], hd)
    positions = torch.tensor([n - 1], dtype=torch.int32).to(DEV)
    seq = torch.zeros(1, dtype=torch.int32).to(DEV)
    out = ops.paged_attention_simple(q.to(DEV), cache.to(DEV), table.to(DEV), positions, seq, None, hd ** -0.5).cpu().view(n_q, hd)
    torch.testing.assert_close(out[1], v[far, 0], rtol=1e-3, atol=1e-3)
    # with a window that ends before the far key it is not seen
    out_w = ops.paged_attention_simple(q.to(DEV), cache.to(DEV), table.to(DEV), positions, seq, n - far - 1, hd ** -0.5).cpu().view(n_q, hd)
    assert (out_w[1] - v[far, 0]).abs().max() > 0.1
    out_w2 = ops.paged_attention_simple(q.to(DEV), cache.to(DEV), table.to(DEV), positions, seq, n - far, hd ** -0.5).cpu().view(n_q, hd)
    torch.testing.assert_close(out_w2[1], v[far, 0], rtol=1e-3, atol=1e-3)


def _simple_segments(n_keys):
    """The plain kernel's rule for cutting a token's keys (the comment at the head of
    cwm_amd/csrc/attention_simple.hip): one segment up to 2,048 keys, then ceil(n / 1,024) segments, at most
    16, of equal length in chunks of 64."""
    n_seg = 1 if n_keys <= 2048 else min(16, -(-n_keys // 1024))
    return n_seg, -(-(-(-n_keys // n_seg)) // 64) * 64


def _loud_keys_case(lengths, page_size, seed):
    """Sequences of the given lengths in a float32 cache (one key/value head of 64, eight query heads), pages
    in reverse order.  For the last token of every sequence each query head has a key of its own that answers
    it loudly: at position 0, at the last and the first key of adjacent segments, at the query's own position."""
    n_q, hd = 8, 64
    g = torch.Generator().manual_seed(seed)
    pages_of = [(n + page_size - 1) // page_size for n in lengths]
    table = torch.full((len(lengths), max(pages_of)), -1, dtype=torch.int32)
    total = sum(pages_of)
    cache = torch.full((total, 2, 1, page_size * hd), float("nan"))
    kc = cache[:, 0].view(total, 1, page_size, hd)
    vc = cache[:, 1].view(total, 1, page_size // 8, hd, 8)
    used, seqs = 0, []
    for b, n in enumerate(lengths):
        n_seg, seg_len = _simple_segments(n)
        if n_seg > 1:
            loud = [0, seg_len - 1, seg_len, (n_seg - 1) * seg_len - 1, (n_seg - 1) * seg_len, n - 1, n // 2, seg_len // 2]
        else:
            loud = [0, 63, 64, 255, 256, n - 1, n // 2, n - 2]
        assert len(set(loud)) == n_q and max(loud) < n
        k = torch.randn((n, hd), generator=g) * 0.1
        v = torch.randn((n, hd), generator=g)
        q = torch.randn((n_q, hd), generator=g)
        for h, j in enumerate(loud):
            k[j] = q[h] * 40.0
        table[b, :pages_of[b]] = torch.arange(total - used - 1, total - used - 1 - pages_of[b], -1, dtype=torch.int32)
        used += pages_of[b]
        pos = torch.arange(n)
        pages, slots = table[b, pos // page_size].long(), pos % page_size
        kc[pages, 0, slots, :] = k
        vc[pages, 0, slots // 8, :, slots % 8] = v
        seqs.append(dict(n=n, k=k, v=v, q=q, loud=loud))
    return seqs, cache, table


def _exact_last_row(s, window):
    n, hd = s["n"], 64
    scores = (s["q"].double() @ s["k"].double().T) * hd ** -0.5  # [heads, keys]
    if window is not None:
        scores[:, : max(0, n - window)] = float("-inf")
    return torch.softmax(scores, -1) @ s["v"].double()


def test_attention_simple_segments_and_their_edges():
    """The plain kernel's segmented path in float32: one launch with tokens of 1, 3, 5 and 16 segments (600,
    2,049, 5,000 and 17,000 keys; the last is held at the cap of 16), `max_keys` given.  Every query head has
    its own loud key: the first key, the last key of a segment and the first of the next, the query's own.  A
    key dropped or counted twice at an edge changes that head's output by the whole of a value."""
    from cwm_amd import ops

    lengths, page_size, hd = [600, 2049, 5000, 17000], 16, 64
    assert [_simple_segments(n)[0] for n in lengths] == [1, 3, 5, 16]
    seqs, cache, table = _loud_keys_case(lengths, page_size, seed=21)
    q = torch.stack([s["q"] for s in seqs]).to(DEV)
    positions = torch.tensor([n - 1 for n in lengths], dtype=torch.int32).to(DEV)
    seq = torch.arange(len(lengths), dtype=torch.int32).to(DEV)
    cache_d, table_d = cache.to(DEV), table.to(DEV)
    out = ops.paged_attention_simple(q, cache_d, table_d, positions, seq, None, hd ** -0.5, max_keys=max(lengths)).cpu().view(len(lengths), 8, hd)
    for b, s in enumerate(seqs):
        torch.testing.assert_close(out[b].double(), _exact_last_row(s, None), rtol=1e-4, atol=1e-4)
        for h, j in enumerate(s["loud"]):
            torch.testing.assert_close(out[b, h], s["v"][j], rtol=1e-3, atol=1e-3)
    # the same rows one sequence at a time, `max_keys` from the positions: bit-equal (the cut depends on the token alone)
    for b in range(len(lengths)):
        alone = ops.paged_attention_simple(q[b:b + 1], cache_d, table_d, positions[b:b + 1], seq[b:b + 1], None, hd ** -0.5).cpu().view(8, hd)
        assert torch.equal(alone, out[b])


@pytest.mark.parametrize("n,far", [(5000, 100), (17000, 0), (17000, 613), (2700, 7)])
def test_attention_simple_window_edge_on_the_segmented_path(n, far):
    """A window whose first key is the loud one sees it; one key shorter does not; both windows hold more than
    2,048 keys, so the window's first key is a segment's first key."""
    from cwm_amd import ops

    page_size, hd = 8, 64
    seqs, cache, table = _loud_keys_case([n], page_size, seed=n + far)
    s = seqs[0]
    s["k"][far] = s["q"][3] * 40.0  # head 3 has a second loud key, at `far`; its own lies at (n_seg-1)*seg_len-1
    own = s["loud"][3]
    page, slot = int(table[0, far // page_size]), far % page_size
    cache[page, 0].view(1, page_size, hd)[0, slot] = s["k"][far]
    positions = torch.tensor([n - 1], dtype=torch.int32).to(DEV)
    seq = torch.zeros(1, dtype=torch.int32).to(DEV)
    for window, sees in ((n - far, True), (n - far - 1, False)):
        assert _simple_segments(window)[0] > 1
        out = ops.paged_attention_simple(s["q"][None].to(DEV), cache.to(DEV), table.to(DEV), positions, seq, window, hd ** -0.5, max_keys=n).cpu().view(8, hd)
        torch.testing.assert_close(out.double(), _exact_last_row(s, window), rtol=1e-4, atol=1e-4)
        both = (s["v"][far] + s["v"][own]) / 2  # two keys equally loud share the row
        if sees:
            torch.testing.assert_close(out[3], both, rtol=1e-3, atol=1e-3)
        else:
            torch.testing.assert_close(out[3], s["v"][own], rtol=1e-3, atol=1e-3)


def test_attention_simple_with_too_small_max_keys_gives_nan_and_ends_normally():
    """`max_keys` below what a token reads leaves no block or no scratch for its segments: its rows are NaN,
    the other tokens' rows are right, and every kernel ends normally (the next call works)."""
    from cwm_amd import ops

    lengths, page_size, hd = [600, 5000], 16, 64
    seqs, cache, table = _loud_keys_case(lengths, page_size, seed=4)
    q = torch.stack([s["q"] for s in seqs]).to(DEV)
    positions = torch.tensor([n - 1 for n in lengths], dtype=torch.int32).to(DEV)
    seq = torch.arange(2, dtype=torch.int32).to(DEV)
    cache_d, table_d = cache.to(DEV), table.to(DEV)
    for max_keys in (1000, 3000):  # no scratch at all; scratch, but three segments where five are needed
        out = ops.paged_attention_simple(q, cache_d, table_d, positions, seq, None, hd ** -0.5, max_keys=max_keys).cpu().view(2, 8, hd)
        assert torch.isnan(out[1]).all()
        torch.testing.assert_close(out[0].double(), _exact_last_row(seqs[0], None), rtol=1e-4, atol=1e-4)
    out = ops.paged_attention_simple(q, cache_d, table_d, positions, seq, None, hd ** -0.5, max_keys=5000).cpu().view(2, 8, hd)
    torch.testing.assert_close(out[1].double(), _exact_last_row(seqs[1], None), rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("vocab", [263, 1000, 128256])
def test_sampling(vocab):
    from cwm_amd import ops

    g = torch.Generator().manual_seed(vocab)
    rows = 6
    logits = torch.randn((rows, vocab), generator=g) * 3.0
    temps = torch.tensor([0.0, 0.7, 1.0, 0.6, 1.3, 0.7])
    top_ps = torch.tensor([1.0, 1.0, 0.9, 0.5, 1e-6, 0.95])
    us = torch.tensor([0.3, 0.25, 0.5, 0.999, 0.7, 0.0])
    toks, lp, slp = ops.sample(logits.to(DEV), temps.to(DEV), top_ps.to(DEV), us.to(DEV))
    toks, lp, slp = toks.cpu(), lp.cpu(), slp.cpu()
    logp = torch.log_softmax(logits.double(), -1)
    for r in range(rows):
        tok = int(toks[r])
        assert 0 <= tok < vocab
        np.testing.assert_allclose(float(lp[r]), float(logp[r, tok]), rtol=1e-4, atol=1e-4)
        if temps[r] <= 0:
            assert tok == plain.greedy(logits[r])
            continue
        probs = plain.sampling_probabilities(logits[r], float(temps[r]), float(top_ps[r]))
        assert probs[tok] > 0, f"row {r}: token {tok} lies outside the nucleus"
        np.testing.assert_allclose(float(slp[r]), math.log(float(probs[tok])), rtol=1e-3, atol=1e-3)
        # inverse CDF: the mass before the token is at most u, the mass through it more than u
        c = torch.cumsum(probs.double(), -1)
        before = float(c[tok] - probs[tok])
        assert before <= float(us[r]) + 1e-4 and float(c[tok]) >= float(us[r]) - 1e-4
    assert int(toks[4]) == plain.greedy(logits[4])  # a vanishing nucleus keeps the top token


@pytest.mark.parametrize("top_p", [1.0, 0.8])
@pytest.mark.parametrize("vocab", [70, 1000, 5003, 128256])
def test_sampling_draws_follow_the_inverse_cdf(vocab, top_p):
    """512 uniform numbers over [0, 1), 0 and the largest float below 1 among them, on one row of logits:
    every token has mass, the mass before it is at most u and the mass through it more than u (the search
    goes through regions, parts and groups of 64 entries, and every edge between them is crossed here)."""
    from cwm_amd import ops

    g = torch.Generator().manual_seed(vocab + 1)
    n = 512
    logits = torch.randn(vocab, generator=g) * 2.0
    us = torch.cat([torch.tensor([0.0, 1.0 - 2.0 ** -24]), torch.rand(n - 2, generator=g)])
    toks, _, slp = ops.sample(logits.repeat(n, 1).to(DEV), torch.full((n,), 0.9).to(DEV), torch.full((n,), top_p).to(DEV), us.to(DEV))
    toks, slp = toks.cpu().long(), slp.cpu()
    probs = plain.sampling_probabilities(logits, 0.9, top_p).double()
    c = torch.cumsum(probs, -1)
    assert (probs[toks] > 0).all()
    before = c[toks] - probs[toks]
    assert (before <= us.double() + 1e-5).all() and (c[toks] >= us.double() - 1e-5).all()
    torch.testing.assert_close(slp.double(), probs[toks].log(), rtol=1e-3, atol=1e-3)
    assert len(set(toks.tolist())) > min(int((probs > 0).sum()), n) // 8  # the draws spread over the entries with mass


def test_sampling_keeps_all_entries_equal_to_the_nucleus_threshold():
    """Where entries are exactly equal at the nucleus' edge the reference's sort keeps some of them, whichever
    come first (cwm/fastgen/utils/sampling.py:38-45); the kernel keeps all of them, so that the draw does not
    depend on an order among equals.  Two equal largest logits and a vanishing nucleus: both are kept, each with
    probability one half, and the uniform number picks between them in vocabulary order."""
    from cwm_amd import ops

    vocab = 1000
    logits = torch.randn(vocab, generator=torch.Generator().manual_seed(3))
    logits[[17, 640]] = 9.0
    us = torch.tensor([0.0, 0.49, 0.51, 0.99])
    n = us.numel()
    toks, _, slp = ops.sample(logits.repeat(n, 1).to(DEV), torch.full((n,), 0.7).to(DEV), torch.full((n,), 1e-6).to(DEV), us.to(DEV))
    assert toks.cpu().tolist() == [17, 17, 640, 640]
    torch.testing.assert_close(slp.cpu(), torch.full((n,), math.log(0.5)), rtol=1e-5, atol=1e-5)


def test_sampling_frequencies():
    """Draws with many uniform numbers follow the distribution (chi-square)."""
    from cwm_amd import ops

    vocab, n = 50, 20000
    g = torch.Generator().manual_seed(1)
    logits = torch.randn(vocab, generator=g)
    probs = plain.sampling_probabilities(logits, 0.8, 0.9).double()
    us = torch.rand(n, generator=g)
    toks, _, _ = ops.sample(logits.repeat(n, 1).to(DEV), torch.full((n,), 0.8).to(DEV), torch.full((n,), 0.9).to(DEV), us.to(DEV))
    counts = torch.bincount(toks.cpu().long(), minlength=vocab).double()
    assert counts[probs == 0].sum() == 0
    keep = probs > 0
    chi2 = (((counts[keep] - n * probs[keep]) ** 2) / (n * probs[keep])).sum()
    assert chi2 < 2.5 * keep.sum()


@pytest.mark.parametrize("n_q,n_kv,hd,page_size", [
    (4, 2, 16, 8), (3, 1, 32, 16), (5, 5, 48, 8), (12, 2, 128, 64), (48, 8, 128, 256), (2, 1, 256, 8), (6, 3, 80, 16),
    (16, 1, 64, 32), (40, 2, 32, 8),
])
@pytest.mark.parametrize("window", [None, 9, 300])
def test_attention_mfma(n_q, n_kv, hd, page_size, window):
    """The matrix-core kernel on a mixed batch: a fresh prompt, a continued portion, a
    decoded token, a decoded token far into a long sequence (split over chunks), a
    short portion far in (split, several rows per head) and a long portion (many row
    tiles, not split).  Pages are shuffled and every slot that holds no key is NaN."""
    from types import SimpleNamespace

    from cwm_amd import ops

    dtype = torch.bfloat16
    lens_old, lens_new = [0, 37, 70, 700, 520, 13], [29, 21, 1, 1, 3, 200]
    seqs, table, total_pages = _paged_setup(dtype, n_kv, hd, page_size, lens_old, lens_new, seed=hd + n_q)
    cache = torch.full((total_pages, 2, n_kv, page_size * hd), float("nan"), dtype=dtype)
    g = torch.Generator().manual_seed(12)
    scale = hd ** -0.5
    want_rows, q_rows = [], []
    for b, s in enumerate(seqs):
        n = s["n0"] + s["n1"]
        q_full = torch.randn((n, n_q, hd), generator=g).to(dtype)
        want = plain.attention(q_full.double(), s["k"].double(), s["v"].double(), window_left=-1 if window is None else window - 1, scale=scale)
        want_rows.append(want[s["n0"]:].reshape(s["n1"], -1))
        for jpos in range(n):
            page, slot = int(table[b, jpos // page_size]), jpos % page_size
            cache_layout.write_kv(cache, page, slot, s["k"][jpos], s["v"][jpos], hd)
        q_rows.append(q_full[s["n0"]:])
    q = torch.cat(q_rows).to(DEV)
    q_lens, kv_lens = lens_new, [a + b for a, b in zip(lens_old, lens_new)]
    cu = [0]
    for n in q_lens:
        cu.append(cu[-1] + n)
    batch = SimpleNamespace(
        q_lens=q_lens, kv_lens=kv_lens, n_seqs=len(seqs), n_tokens=sum(q_lens), scratch={},
        cu_q=torch.tensor(cu, dtype=torch.int32).to(DEV), kv_len=torch.tensor(kv_lens, dtype=torch.int32).to(DEV),
    )
    got = ops.paged_attention_mfma(q, cache.to(DEV), table.to(DEV), batch, window, scale).cpu()
    want = torch.cat(want_rows)
    assert torch.isfinite(got).all()
    torch.testing.assert_close(got.double(), want, rtol=3e-2, atol=3e-2)
    # and it agrees with the plain kernel on the same cache, more tightly
    positions = torch.cat([torch.arange(a, a + b) for a, b in zip(lens_old, lens_new)]).to(torch.int32).to(DEV)
    seq_of = torch.cat([torch.full((n,), b) for b, n in enumerate(q_lens)]).to(torch.int32).to(DEV)
    simple = ops.paged_attention_simple(q, cache.to(DEV), table.to(DEV), positions, seq_of, window, scale).cpu()
    torch.testing.assert_close(got.float(), simple.float(), rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("window", [None, 20000])
def test_attention_mfma_long_ranges(window):
    """Decoded tokens and short portions far into long sequences: uncut ranges of up to 2,048 keys (four
    wavefronts of a block combine), every chunk length of the split (512, 1,024 and 2,048 keys) and the
    merge of up to 35 partial results, against
    float32 torch on the device.  One far key stands out in the longest sequence.  The last two
    sequences bring portions of many rows but too few blocks for the chip: their blocks' keys
    are cut (at multiples of 2,048 and of 8,192) and merged as well."""
    from types import SimpleNamespace

    from cwm_amd import ops

    n_q, n_kv, hd, page_size = 6, 2, 64, 64
    lens_old, lens_new = [9000, 70000, 3000, 5000, 1500, 20000, 9000], [1, 3, 1, 2, 1, 150, 1400]
    g = torch.Generator().manual_seed(5)
    scale = hd ** -0.5
    total_pages = sum((a + b + page_size - 1) // page_size for a, b in zip(lens_old, lens_new)) + 1
    perm = torch.randperm(total_pages, generator=g)
    width = max((a + b + page_size - 1) // page_size for a, b in zip(lens_old, lens_new))
    table = torch.full((len(lens_old), width), -1, dtype=torch.int32)
    cache = torch.full((total_pages, 2, n_kv, page_size * hd), float("nan"), dtype=torch.bfloat16)
    kc = cache[:, 0].view(total_pages, n_kv, page_size, hd)
    vc = cache[:, 1].view(total_pages, n_kv, page_size // 8, hd, 8)
    used, q_rows, want_rows = 0, [], []
    for b, (n0, n1) in enumerate(zip(lens_old, lens_new)):
        n = n0 + n1
        k = torch.randn((n, n_kv, hd), generator=g).to(torch.bfloat16)
        v = torch.randn((n, n_kv, hd), generator=g).to(torch.bfloat16)
        q = torch.randn((n1, n_q, hd), generator=g).to(torch.bfloat16)
        if b == 1:  # key 12,345 answers the last query's head 0 loudly
            k[12345, 0] = (q[-1, 0].float() * 4.0).to(torch.bfloat16)
        n_pages = (n + page_size - 1) // page_size
        table[b, :n_pages] = perm[used:used + n_pages].to(torch.int32)
        used += n_pages
        pos = torch.arange(n)
        pages, slots = table[b, pos // page_size].long(), pos % page_size
        kc[pages, :, slots, :] = k
        vc[pages, :, slots // 8, :, slots % 8] = v
        kd, vd, qd = k.float().to(DEV), v.float().to(DEV), q.float().to(DEV)
        group = n_q // n_kv
        scores = torch.einsum("thd,khd->htk", qd, kd.repeat_interleave(group, dim=1)) * scale
        qpos = torch.arange(n0, n, device=DEV).view(1, -1, 1)
        kpos = torch.arange(n, device=DEV).view(1, 1, -1)
        ok = kpos <= qpos
        if window is not None:
            ok = ok & (kpos >= qpos - (window - 1))
        probs = torch.softmax(scores.masked_fill(~ok, float("-inf")), dim=-1)
        if b == 1 and window is None:
            assert probs[0, -1, 12345] > 0.9
        want_rows.append(torch.einsum("htk,khd->thd", probs, vd.repeat_interleave(group, dim=1)).reshape(n1, -1).cpu())
        q_rows.append(q)
    kv_lens = [a + b for a, b in zip(lens_old, lens_new)]
    cu = [0]
    for n in lens_new:
        cu.append(cu[-1] + n)
    batch = SimpleNamespace(
        q_lens=lens_new, kv_lens=kv_lens, n_seqs=len(kv_lens), n_tokens=sum(lens_new), scratch={},
        cu_q=torch.tensor(cu, dtype=torch.int32).to(DEV), kv_len=torch.tensor(kv_lens, dtype=torch.int32).to(DEV),
    )
    got = ops.paged_attention_mfma(torch.cat(q_rows).to(DEV), cache.to(DEV), table.to(DEV), batch, window, scale).cpu()
    assert torch.isfinite(got).all()
    torch.testing.assert_close(got.float(), torch.cat(want_rows), rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("window", [None, 8192])
def test_attention_mfma_long_ranges_with_heads_of_128_and_pages_of_256(window):
    """The geometry of a long-context decode step of the 32B shape (48 query heads on 8 key/value heads
    of 128, pages of 256 keys): decoded tokens after 32,767 and 131,071 keys (chunks of 1,024 and 2,048 keys,
    up to 64 partial results a row) and a portion of three rows after 100,000, against float32 torch on
    the device.  Everything is made on the device; one far key stands out for the longest sequence."""
    from types import SimpleNamespace

    from cwm_amd import ops

    n_q, n_kv, hd, page_size = 48, 8, 128, 256
    group = n_q // n_kv
    lens_old, lens_new = [32767, 131071, 100000, 700], [1, 1, 3, 1]
    g = torch.Generator(device=DEV).manual_seed(7)
    scale = hd ** -0.5
    total_pages = sum((a + b + page_size - 1) // page_size for a, b in zip(lens_old, lens_new)) + 1
    perm = torch.randperm(total_pages, generator=torch.Generator().manual_seed(7))
    width = max((a + b + page_size - 1) // page_size for a, b in zip(lens_old, lens_new))
    table = torch.full((len(lens_old), width), -1, dtype=torch.int32)
    cache = torch.full((total_pages, 2, n_kv, page_size * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
    kc = cache[:, 0].view(total_pages, n_kv, page_size, hd)
    vc = cache[:, 1].view(total_pages, n_kv, page_size // 8, hd, 8)
    used, q_rows, want_rows = 0, [], []
    for b, (n0, n1) in enumerate(zip(lens_old, lens_new)):
        n = n0 + n1
        k = torch.randn((n, n_kv, hd), generator=g, device=DEV).to(torch.bfloat16)
        v = torch.randn((n, n_kv, hd), generator=g, device=DEV).to(torch.bfloat16)
        q = torch.randn((n1, n_q, hd), generator=g, device=DEV).to(torch.bfloat16)
        far = 777 if window is None else n - 8000
        if b == 1:  # one key answers the query's head 7 (key/value head 1) loudly
            k[far, 1] = (q[-1, 7].float() * 4.0).to(torch.bfloat16)
        n_pages = (n + page_size - 1) // page_size
        table[b, :n_pages] = perm[used:used + n_pages].to(torch.int32)
        used += n_pages
        pos = torch.arange(n, device=DEV)
        pages, slots = table[b].to(DEV)[pos // page_size].long(), pos % page_size
        kc[pages, :, slots, :] = k
        vc[pages, :, slots // 8, :, slots % 8] = v
        want = torch.empty((n1, n_q, hd), dtype=torch.float32, device=DEV)
        qpos = torch.arange(n0, n, device=DEV).view(-1, 1)
        ok = pos.view(1, -1) <= qpos
        if window is not None:
            ok = ok & (pos.view(1, -1) >= qpos - (window - 1))
        for h in range(n_kv):  # head by head: the scores of all 48 heads at once would be large
            scores = torch.einsum("tgd,kd->tgk", q[:, h * group:(h + 1) * group].float(), k[:, h].float()) * scale
            probs = torch.softmax(scores.masked_fill(~ok[:, None, :], float("-inf")), dim=-1)
            if b == 1 and h == 1:
                assert probs[-1, 1, far] > 0.9
            want[:, h * group:(h + 1) * group] = torch.einsum("tgk,kd->tgd", probs, v[:, h].float())
        want_rows.append(want.reshape(n1, -1).cpu())
        q_rows.append(q)
    kv_lens = [a + b for a, b in zip(lens_old, lens_new)]
    cu = [0]
    for n in lens_new:
        cu.append(cu[-1] + n)
    batch = SimpleNamespace(
        q_lens=lens_new, kv_lens=kv_lens, n_seqs=len(kv_lens), n_tokens=sum(lens_new), scratch={},
        cu_q=torch.tensor(cu, dtype=torch.int32).to(DEV), kv_len=torch.tensor(kv_lens, dtype=torch.int32).to(DEV),
    )
    got = ops.paged_attention_mfma(torch.cat(q_rows), cache, table.to(DEV), batch, window, scale).cpu()
    assert torch.isfinite(got).all()
    torch.testing.assert_close(got.float(), torch.cat(want_rows), rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("n_q,n_kv,hd,page_size", [(6, 2, 64, 32), (12, 2, 128, 64), (6, 3, 48, 8)])
def test_missing_page_shows_as_nan_in_both_attention_kernels(n_q, n_kv, hd, page_size):
    """A block-table entry of -1 (or past the pool) for a page that a query reads must not pass
    for page 0: every row that reads it comes out NaN, from the matrix-core kernels (decoded
    token, split and merged; short portion; long portion through LDS, with and without direct
    loads) as from the plain kernel; rows of other sequences, and rows whose window has passed
    the page, stay finite."""
    from types import SimpleNamespace

    from cwm_amd import ops

    dtype = torch.bfloat16
    lens_old, lens_new = [2000, 100, 0, 40, 900], [1, 1, 300, 5, 1]
    n_seqs = len(lens_old)
    kv_lens = [a + b for a, b in zip(lens_old, lens_new)]
    width = max((n + page_size - 1) // page_size for n in kv_lens)
    total_pages = sum((n + page_size - 1) // page_size for n in kv_lens)
    table = torch.full((n_seqs, width), -1, dtype=torch.int32)
    used = 0
    for b, n in enumerate(kv_lens):
        n_pages = (n + page_size - 1) // page_size
        table[b, :n_pages] = torch.arange(used, used + n_pages, dtype=torch.int32)
        used += n_pages
    g = torch.Generator().manual_seed(3)
    cache = torch.randn((total_pages, 2, n_kv, page_size * hd), generator=g).to(dtype).to(DEV)
    q = torch.randn((sum(lens_new), n_q, hd), generator=g).to(dtype).to(DEV)
    cu = [0]
    for n in lens_new:
        cu.append(cu[-1] + n)
    positions = torch.cat([torch.arange(a, a + b) for a, b in zip(lens_old, lens_new)]).to(torch.int32).to(DEV)
    seq_of = torch.cat([torch.full((n,), b) for b, n in enumerate(lens_new)]).to(torch.int32).to(DEV)

    def run(tbl, window):
        batch = SimpleNamespace(
            q_lens=lens_new, kv_lens=kv_lens, n_seqs=n_seqs, n_tokens=sum(lens_new), scratch={},
            cu_q=torch.tensor(cu, dtype=torch.int32).to(DEV), kv_len=torch.tensor(kv_lens, dtype=torch.int32).to(DEV),
        )
        mfma = ops.paged_attention_mfma(q, cache, tbl.to(DEV), batch, window, hd ** -0.5).float().cpu()
        simple = ops.paged_attention_simple(q, cache, tbl.to(DEV), positions, seq_of, window, hd ** -0.5).float().cpu()
        return mfma, simple

    for out in run(table, None):
        assert torch.isfinite(out).all()
    # no window: everyone reads logical page 0 of their sequence
    for b in range(n_seqs):
        broken = table.clone()
        broken[b, 0] = -1 if b % 2 == 0 else total_pages + 5
        for name, out in zip(("matrix-core", "plain"), run(broken, None)):
            rows = slice(cu[b], cu[b + 1])
            assert torch.isnan(out[rows]).all(), f"{name}: sequence {b} read a missing page and shows no NaN"
            rest = torch.cat([out[: cu[b]], out[cu[b + 1] :]])
            assert torch.isfinite(rest).all(), f"{name}: a missing page of sequence {b} reached other sequences"
    # a window of 70 keys: page 0 of the long sequences is out of reach, the page of key 1,960 is not
    window = 70
    broken = table.clone()
    broken[0, 0] = -1
    broken[4, 0] = -1
    for name, out in zip(("matrix-core", "plain"), run(broken, window)):
        assert torch.isfinite(out).all(), f"{name}: a page that the window has passed was read"
    broken[0, 1960 // page_size] = -1
    for name, out in zip(("matrix-core", "plain"), run(broken, window)):
        assert torch.isnan(out[0]).all() and torch.isfinite(out[1:]).all(), name


def test_attention_mfma_builds_agree_bit_for_bit(monkeypatch):
    """The wrapper picks between builds of the same arithmetic by the shape of the work (two or
    three blocks a compute unit for long portions; the wavefront index declared uniform or not
    for decoded tokens): whichever it picks, the result is the same bits."""
    from types import SimpleNamespace

    from cwm_amd import ops

    n_q, n_kv, hd, page_size = 8, 2, 64, 32
    lens_old, lens_new = [700, 0, 3000], [1, 900, 2]
    kv_lens = [a + b for a, b in zip(lens_old, lens_new)]
    g = torch.Generator().manual_seed(4)
    width = max((n + page_size - 1) // page_size for n in kv_lens)
    n_pages = len(kv_lens) * width
    table = torch.randperm(n_pages, generator=g).to(torch.int32).view(len(kv_lens), width)
    cache = torch.randn((n_pages, 2, n_kv, page_size * hd), generator=g).to(torch.bfloat16).to(DEV)
    q = torch.randn((sum(lens_new), n_q, hd), generator=g).to(torch.bfloat16).to(DEV)
    cu = [0]
    for n in lens_new:
        cu.append(cu[-1] + n)

    def run():
        batch = SimpleNamespace(
            q_lens=lens_new, kv_lens=kv_lens, n_seqs=len(kv_lens), n_tokens=sum(lens_new), scratch={},
            cu_q=torch.tensor(cu, dtype=torch.int32).to(DEV), kv_len=torch.tensor(kv_lens, dtype=torch.int32).to(DEV),
        )
        return ops.paged_attention_mfma(q, cache, table.to(DEV), batch, None, hd ** -0.5).cpu()

    base = run()
    assert torch.isfinite(base).all()
    for three in (0, 1):
        monkeypatch.setattr(ops, "_three_blocks_a_unit", lambda n_blocks, shape, device, three=three: three)
        assert torch.equal(run(), base)
    monkeypatch.undo()
    plan_of = ops._attention_plan
    for keys in (64, 4096):  # below and above the length at which the other build of the split kernel runs

        def forced(*args, keys=keys, **kwargs):
            plan = plan_of(*args, **kwargs)
            plan.work_keys = keys
            return plan

        monkeypatch.setattr(ops, "_attention_plan", forced)
        assert torch.equal(run(), base)


@pytest.mark.parametrize("window", [None, 1000])
def test_attention_mfma_many_blocks(window):
    """A portion long enough, over enough heads, for the launch that puts three blocks on a
    compute unit (1,536 blocks of 128 rows and more): 3,072 tokens after 45 cached ones, 64
    heads of 64.  The reference is float32 torch on the device, whole sequence, no cache; slots
    that hold no key, and pages that a window has given back, are NaN."""
    from types import SimpleNamespace

    from cwm_amd import ops

    n_q = n_kv = 64
    hd, page_size, n0, n1 = 64, 32, 45, 3072
    n = n0 + n1
    g = torch.Generator().manual_seed(77)
    q_full = torch.randn((n, n_q, hd), generator=g).to(torch.bfloat16)
    k = torch.randn((n, n_kv, hd), generator=g).to(torch.bfloat16)
    v = torch.randn((n, n_kv, hd), generator=g).to(torch.bfloat16)
    n_pages = (n + page_size - 1) // page_size
    perm = torch.randperm(n_pages + 2, generator=g)
    table = perm[:n_pages].to(torch.int32).view(1, n_pages).clone()
    cache = torch.full((n_pages + 2, 2, n_kv, page_size * hd), float("nan"), dtype=torch.bfloat16)
    first_needed = 0 if window is None else max(0, n0 - (window - 1))
    pos = torch.arange(n)
    live = pos // page_size >= first_needed // page_size
    pages, slots = table[0, pos // page_size].long(), pos % page_size
    kc = cache[:, 0].view(n_pages + 2, n_kv, page_size, hd)
    vc = cache[:, 1].view(n_pages + 2, n_kv, page_size // 8, hd, 8)
    kc[pages[live], :, slots[live], :] = k[live]
    vc[pages[live], :, slots[live] // 8, :, slots[live] % 8] = v[live]
    table[0, : first_needed // page_size] = -1
    scale = hd ** -0.5
    # reference on the device in float32
    qd, kd, vd = q_full[n0:].float().to(DEV), k.float().to(DEV), v.float().to(DEV)
    scores = torch.einsum("thd,khd->htk", qd, kd) * scale
    qpos = torch.arange(n0, n, device=DEV).view(1, -1, 1)
    kpos = torch.arange(n, device=DEV).view(1, 1, -1)
    ok = kpos <= qpos
    if window is not None:
        ok = ok & (kpos >= qpos - (window - 1))
    scores = scores.masked_fill(~ok, float("-inf"))
    want = torch.einsum("htk,khd->thd", torch.softmax(scores, dim=-1), vd).reshape(n1, -1).cpu()
    del scores
    batch = SimpleNamespace(
        q_lens=[n1], kv_lens=[n], n_seqs=1, n_tokens=n1, scratch={},
        cu_q=torch.tensor([0, n1], dtype=torch.int32).to(DEV), kv_len=torch.tensor([n], dtype=torch.int32).to(DEV),
    )
    got = ops.paged_attention_mfma(q_full[n0:].to(DEV), cache.to(DEV), table.to(DEV), batch, window, scale).cpu()
    assert torch.isfinite(got).all()
    torch.testing.assert_close(got.float(), want, rtol=3e-2, atol=3e-2)


@pytest.mark.parametrize("n_q,n_kv,hd,page_size", [(4, 2, 64, 32), (12, 2, 128, 64), (6, 3, 48, 16)])
def test_attention_mfma_window_with_pages_given_back(n_q, n_kv, hd, page_size):
    """Under a window the pages that lie wholly before every query's reach have been given
    back: their block-table entries are -1 and whatever they held is gone (NaN here).  A
    long portion (many row tiles), a short one and a decoded token far into a sequence."""
    from types import SimpleNamespace

    from cwm_amd import ops

    dtype, window = torch.bfloat16, 70
    lens_old, lens_new = [200, 333, 900], [120, 5, 1]
    seqs, table, total_pages = _paged_setup(dtype, n_kv, hd, page_size, lens_old, lens_new, seed=3 * hd + n_q)
    cache = torch.full((total_pages, 2, n_kv, page_size * hd), float("nan"), dtype=dtype)
    g = torch.Generator().manual_seed(21)
    scale = hd ** -0.5
    want_rows, q_rows = [], []
    table = table.clone()
    for b, s in enumerate(seqs):
        n = s["n0"] + s["n1"]
        q_full = torch.randn((n, n_q, hd), generator=g).to(dtype)
        want = plain.attention(q_full.double(), s["k"].double(), s["v"].double(), window_left=window - 1, scale=scale)
        want_rows.append(want[s["n0"]:].reshape(s["n1"], -1))
        first_needed = max(0, s["n0"] - (window - 1))
        for jpos in range(n):
            if jpos // page_size < first_needed // page_size:
                continue  # this page has been given back: nothing is written there
            page, slot = int(table[b, jpos // page_size]), jpos % page_size
            cache_layout.write_kv(cache, page, slot, s["k"][jpos], s["v"][jpos], hd)
        table[b, : first_needed // page_size] = -1
        q_rows.append(q_full[s["n0"]:])
    q = torch.cat(q_rows).to(DEV)
    kv_lens = [a + b for a, b in zip(lens_old, lens_new)]
    cu = [0]
    for n in lens_new:
        cu.append(cu[-1] + n)
    batch = SimpleNamespace(
        q_lens=lens_new, kv_lens=kv_lens, n_seqs=len(seqs), n_tokens=sum(lens_new), scratch={},
        cu_q=torch.tensor(cu, dtype=torch.int32).to(DEV), kv_len=torch.tensor(kv_lens, dtype=torch.int32).to(DEV),
    )
    got = ops.paged_attention_mfma(q, cache.to(DEV), table.to(DEV), batch, window, scale).cpu()
    assert torch.isfinite(got).all()
    torch.testing.assert_close(got.double(), torch.cat(want_rows), rtol=3e-2, atol=3e-2)


def test_attention_mfma_far_key_and_window_edge():
    """A far key made to dominate must be found through chunks and pages, and must
    vanish exactly when the window ends one key short of it."""
    from types import SimpleNamespace

    from cwm_amd import ops

    n_q, n_kv, hd, page_size, n = 6, 1, 128, 16, 1500
    g = torch.Generator().manual_seed(5)
    k = (torch.randn((n, n_kv, hd), generator=g) * 0.1).to(torch.bfloat16)
    v = torch.randn((n, n_kv, hd), generator=g).to(torch.bfloat16)
    q = torch.randn((1, n_q, hd), generator=g).to(torch.bfloat16)
    far = 261
    k[far, 0] = (q[0, 4].float() * 4.0).to(torch.bfloat16)
    pages = (n + page_size - 1) // page_size
    table = torch.arange(pages, dtype=torch.int32).flip(0).reshape(1, pages).contiguous()
    cache = torch.full((pages, 2, n_kv, page_size * hd), float("nan"), dtype=torch.bfloat16)
    for jpos in range(n):
        page, slot = int(table[0, jpos // page_size]), jpos % page_size
        cache_layout.write_kv(cache, page, slot, k[jpos], v[jpos], hd)

    def run(window):
        batch = SimpleNamespace(q_lens=[1], kv_lens=[n], n_seqs=1, n_tokens=1, scratch={},
                                cu_q=torch.tensor([0, 1], dtype=torch.int32).to(DEV), kv_len=torch.tensor([n], dtype=torch.int32).to(DEV))
        return ops.paged_attention_mfma(q.to(DEV), cache.to(DEV), table.to(DEV), batch, window, hd ** -0.5).cpu().view(n_q, hd).float()

    torch.testing.assert_close(run(None)[4], v[far, 0].float(), rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(run(n - far)[4], v[far, 0].float(), rtol=2e-2, atol=2e-2)
    assert (run(n - far - 1)[4] - v[far, 0].float()).abs().max() > 0.1


def test_gemm_bf16_many_rows_float32_out():
    from cwm_amd import ops

    a = rnd((150, 96), torch.bfloat16, 1)
    w = rnd((509, 96), torch.bfloat16, 2, 0.1)
    got = ops.gemm_bf16(a.to(DEV), w.to(DEV), None, torch.float32).cpu()
    want = a.double() @ w.double().T
    assert got.dtype == torch.float32 and (got.double() - want).abs().max() < 1e-4
    got_bf = ops.gemm_bf16(a.to(DEV), w.to(DEV), None, torch.bfloat16).cpu()
    torch.testing.assert_close(got_bf.double(), want, rtol=2e-2, atol=2e-2)
    # with a bias, in both output types
    b = rnd((509,), torch.bfloat16, 3, 2.0)
    for out_dtype in (torch.float32, torch.bfloat16):
        got_b = ops.gemm_bf16(a.to(DEV), w.to(DEV), b.to(DEV), out_dtype).cpu()
        assert got_b.dtype == out_dtype
        torch.testing.assert_close(got_b.double(), want + b.double(), rtol=2e-2, atol=2e-2)


def test_gemm_bf16_many_rows_is_the_same_in_every_call():
    """More than 64 rows go to the library in one call, with nothing timed or chosen at run time:
    the result is the product, and bit for bit the same from call to call."""
    from cwm_amd import ops

    n = 2 * 8192 + 48
    a = rnd((130, 64), torch.bfloat16, 1)
    w = rnd((n, 64), torch.bfloat16, 2, 0.1)
    want = a.double() @ w.double().T
    first = ops.gemm_bf16(a.to(DEV), w.to(DEV), None, torch.bfloat16).cpu()
    torch.testing.assert_close(first.double(), want, rtol=2e-2, atol=2e-2)
    assert torch.equal(ops.gemm_bf16(a.to(DEV), w.to(DEV), None, torch.bfloat16).cpu(), first)


@pytest.mark.parametrize("out_dtype", DTYPES)
@pytest.mark.parametrize("m,n,k", [(1, 263, 120), (8, 6144, 6144), (5, 64, 64), (16, 509, 296), (7, 130, 8), (3, 1000, 21504), (16, 48, 4104), (2, 7, 40),
                                   (17, 130, 8), (33, 1000, 21504 // 4), (64, 48, 4104), (50, 7, 40), (64, 2048, 6144)])
def test_gemm_bf16_stream(out_dtype, m, n, k):
    """The persistent weight-streaming product, with and without a split K."""
    from cwm_amd import ops

    a = rnd((m, k), torch.bfloat16, 6)
    w = rnd((n, k), torch.bfloat16, 7, 0.05)
    b = rnd((n,), torch.bfloat16, 8)
    want = a.double() @ w.double().T + b.double()
    scale = float(want.abs().max())
    got = ops.gemm_bf16_stream(a.to(DEV), w.to(DEV), b.to(DEV), out_dtype=out_dtype).cpu()
    assert got.shape == (m, n) and got.dtype == out_dtype
    if out_dtype == torch.float32:
        assert (got.double() - want).abs().max() <= 1e-5 * scale * (1 + k / 512)
    else:
        torch.testing.assert_close(got.double(), want, rtol=1e-2, atol=1e-2 * scale)
    parts = ops.gemm_bf16_stream(a.to(DEV), w.to(DEV), b.to(DEV), out_dtype=out_dtype, partials_ok=True).cpu()
    if parts.dim() == 3:
        assert parts.dtype == torch.float32
        assert (parts.double().sum(0) - want).abs().max() <= 1e-5 * scale * (1 + k / 512)
    # a row's result does not depend on how many rows there are (among calls of one block shape)
    fewer = 17 if m > 17 else 1
    one = ops.gemm_bf16_stream(a[m - fewer :].contiguous().to(DEV), w.to(DEV), b.to(DEV), out_dtype=out_dtype).cpu()
    assert torch.equal(one[-1], got[m - 1])
    # views with a wider row stride (as the q/k/v and gate/up products are used)
    wide = torch.zeros((m, k + 24), dtype=torch.bfloat16)
    wide[:, 8 : 8 + k] = a
    got2 = ops.gemm_bf16_stream(wide.to(DEV)[:, 8 : 8 + k], w.to(DEV), b.to(DEV), out_dtype).cpu()
    assert torch.equal(got2, got)


def _stream_layout_by_hand(w):
    """The streaming copy as its definition reads: [tiles of 16 rows, steps of 32 columns, 64, 8], lane 16 j + r
    of a step holding W[16 tile + r][32 step + 8 j ..+8], zeros past the matrix."""
    n, k = w.shape
    tiles, steps = -(-n // 16), -(-k // 32)
    padded = torch.zeros((tiles * 16, steps * 32), dtype=w.dtype)
    padded[:n, :k] = w
    return padded.view(tiles, 16, steps, 4, 8).permute(0, 2, 3, 1, 4).reshape(tiles, steps, 64, 8).contiguous()


@pytest.mark.parametrize("out_dtype", DTYPES)
@pytest.mark.parametrize("m,n,k", [(1, 263, 120), (8, 6144, 6144), (5, 64, 64), (16, 509, 296), (7, 130, 8), (3, 1000, 21504), (16, 48, 4104), (2, 7, 40),
                                   (33, 1000, 21504 // 4), (64, 48, 4104)])
def test_gemm_bf16_stream_from_the_streaming_copy(out_dtype, m, n, k):
    """The product from the matrix's streaming copy: the copy is what its definition says (also for sizes that
    fill no whole tile or step, and for a view with a wider row stride), and the product from it gives the bits
    of the product from the row-major matrix: the same values meet in the same order."""
    from cwm_amd import ops

    a = rnd((m, k), torch.bfloat16, 16).to(DEV)
    w = rnd((n, k), torch.bfloat16, 17, 0.05)
    b = rnd((n,), torch.bfloat16, 18).to(DEV)
    copy = ops.stream_layout(w.to(DEV))
    assert torch.equal(copy.cpu(), _stream_layout_by_hand(w))
    wide = torch.zeros((n, k + 16), dtype=torch.bfloat16)
    wide[:, 8 : 8 + k] = w
    assert torch.equal(ops.stream_layout(wide.to(DEV)[:, 8 : 8 + k]).cpu(), copy.cpu())
    for partials_ok in (False, True):
        plain = ops.gemm_bf16_stream(a, w.to(DEV), b, out_dtype=out_dtype, partials_ok=partials_ok)
        # the row-major matrix is not read: a matrix of NaN in its place changes nothing
        nan = torch.full((n, k), float("nan"), dtype=torch.bfloat16, device=DEV)
        got = ops.gemm_bf16_stream(a, nan, b, out_dtype=out_dtype, partials_ok=partials_ok, streamed=copy)
        assert got.shape == plain.shape and torch.equal(got, plain)
    with pytest.raises(ops.KernelError, match="streaming copy"):
        ops.gemm_bf16_stream(a, w.to(DEV), b, out_dtype=out_dtype, streamed=copy[:, :-1].contiguous() if copy.shape[1] > 1 else copy[:-1].contiguous())


@pytest.mark.parametrize("m,f,k", [(1, 24, 64), (8, 21504 // 8, 6144 // 4), (16, 296, 120), (5, 8, 8)])
def test_gated_epilogue_from_the_streaming_copy(m, f, k):
    from cwm_amd import ops

    x = rnd((m, k), torch.bfloat16, 21).to(DEV)
    w = rnd((2 * f, k), torch.bfloat16, 22, 0.1).to(DEV)
    plain = ops.gate_up_silu(x, w, None, True)
    got = ops.gate_up_silu(x, torch.full_like(w, float("nan")), None, True, streamed=ops.stream_layout(w))
    assert torch.equal(got, plain)


def test_add_rmsnorm_takes_partial_sums():
    from cwm_amd import ops

    for dim in (6144, 120, 7):
        h = rnd((5, dim), torch.float32, 1)
        parts = rnd((4, 5, dim), torch.float32, 2)
        w = rnd((dim,), torch.float32, 3) * 0.1 + 1.0
        hd = h.to(DEV).clone()
        got = ops.add_rmsnorm(hd, parts.to(DEV), w.to(DEV), 1e-5, torch.float32).cpu()
        total = h.double() + parts.double().sum(0)
        torch.testing.assert_close(hd.cpu().double(), total, rtol=1e-6, atol=1e-6)
        torch.testing.assert_close(got.double(), plain.rms_norm(total, w.double(), 1e-5), rtol=2e-5, atol=2e-6)
        torch.testing.assert_close(ops.sum_partials(parts.to(DEV), torch.float32).cpu().double(), parts.double().sum(0), rtol=1e-6, atol=1e-6)


def test_token_logprobs():
    from cwm_amd import ops

    g = torch.Generator().manual_seed(3)
    logits = torch.randn((7, 1000), generator=g) * 4
    rows = torch.tensor([6, 0, 3, 3], dtype=torch.int32)
    targets = torch.tensor([999, 0, 17, 500], dtype=torch.int32)
    got = ops.token_logprobs(logits.to(DEV), rows.to(DEV), targets.to(DEV)).cpu()
    want = torch.log_softmax(logits.double(), -1)[rows.long(), targets.long()]
    torch.testing.assert_close(got.double(), want, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("n_q,n_kv,hd,page_size,dim,bias", [(4, 2, 16, 8, 64, False), (3, 1, 32, 16, 96, True), (5, 5, 48, 5, 120, True), (12, 2, 128, 64, 256, False)])
def test_qkv_rope_write_fused_equals_separate(n_q, n_kv, hd, page_size, dim, bias):
    """The streaming product's q/k/v epilogue (rotation + cache write) gives the bits of
    the product followed by the rotation + cache-write kernel."""
    from cwm_amd import ops

    m = 7
    n_out = (n_q + 2 * n_kv) * hd
    x = rnd((m, dim), torch.bfloat16, 1).to(DEV)
    w = rnd((n_out, dim), torch.bfloat16, 2, 0.1).to(DEV)
    b = rnd((n_out,), torch.bfloat16, 3).to(DEV) if bias else None
    inv_freq = plain.rope_frequencies(hd, 10000.0).to(DEV)
    positions = torch.tensor([0, 5, 17, 3, 40, 8, 63], dtype=torch.int32).to(DEV)
    seq = torch.tensor([0, 1, 2, 3, 4, 5, 6], dtype=torch.int32).to(DEV)
    width = 64 // page_size + 1
    table = torch.randperm(7 * width).to(torch.int32).reshape(7, width).contiguous().to(DEV)
    caches = [torch.zeros((7 * width, 2, n_kv, page_size * hd), dtype=torch.bfloat16, device=DEV) for _ in range(2)]
    fused = ops.qkv_rope_write(x, w, b, n_q, n_kv, hd, positions, inv_freq, caches[0], table, seq)
    qkv = ops.gemm_bf16_stream(x, w, b, torch.bfloat16)
    q = qkv[:, : n_q * hd].unflatten(1, (n_q, hd))
    k = qkv[:, n_q * hd : (n_q + n_kv) * hd].unflatten(1, (n_kv, hd))
    v = qkv[:, (n_q + n_kv) * hd :].unflatten(1, (n_kv, hd))
    ops.rope_kv_write(q, k, v, positions, inv_freq, caches[1], table, seq)
    assert torch.equal(fused, qkv)
    assert torch.equal(caches[0], caches[1])
    assert caches[0].abs().sum() > 0
    # and from the matrix's streaming copy (the row-major matrix is then not read)
    third = torch.zeros_like(caches[0])
    streamed = ops.qkv_rope_write(x, torch.full_like(w, float("nan")), b, n_q, n_kv, hd, positions, inv_freq, third, table, seq, streamed=ops.stream_layout(w))
    assert torch.equal(streamed, fused) and torch.equal(third, caches[0])


@pytest.mark.parametrize(
    "m,n,k,units",
    [
        (17, 16, 64, 4), (64, 208, 192, 3), (40, 1072, 256, 7), (65, 1072, 256, 7), (128, 5376, 512, 16), (100, 6144, 1024, None),
        (200, 512, 128, 5), (256, 3072, 640, None), (33, 128256, 64, None), (64, 8192, 6144, None), (129, 96, 64, 2), (512, 192, 128, 3),
    ],
)
def test_gemm_bf16_tile(m, n, k, units):
    """The tiled product: whole tiles and tiles shared between blocks, against float64; `units`
    stands in for the number of blocks that run at once, so that few blocks cut small products
    the way 256 cut large ones."""
    from cwm_amd import ops

    a = rnd((m, k), torch.bfloat16, 6)
    w = rnd((n, k), torch.bfloat16, 7, 0.05)
    want = a.double() @ w.double().T
    scale = float(want.abs().max())
    limit = 1e-5 * scale * (1 + k / 512)
    ad, wd = a.to(DEV), w.to(DEV)
    # memory that the next result is likely to be given, full of NaN: what the kernel does not write shows
    junk = torch.full((8, m, n), float("nan"), dtype=torch.float32, device=DEV)
    del junk
    parts = ops.gemm_bf16_tile(ad, wd, None, torch.float32, partials_ok=True, units=units).cpu()
    assert parts.dtype == torch.float32
    total = parts.double().sum(0) if parts.dim() == 3 else parts.double()
    assert (total - want).abs().max() <= limit
    got = ops.gemm_bf16_tile(ad, wd, None, torch.float32, units=units).cpu()
    assert got.shape == (m, n) and (got.double() - want).abs().max() <= limit
    got_bf = ops.gemm_bf16_tile(ad, wd, None, torch.bfloat16, units=units).cpu()
    assert got_bf.dtype == torch.bfloat16
    torch.testing.assert_close(got_bf.double(), want, rtol=1e-2, atol=1e-2 * scale)
    # a row's result does not depend on the other rows, among calls of one block height
    fewer = m - 1 if m > 65 and (m - 1 + 127) // 128 == (m + 127) // 128 else (17 if 17 < m <= 64 else m)
    if fewer != m:
        one = ops.gemm_bf16_tile(ad[m - fewer :].contiguous(), wd, None, torch.float32, units=units).cpu()
        assert torch.equal(one[-1], got[m - 1])
    # a bias is added after the kernel
    b = rnd((n,), torch.bfloat16, 8, 2.0)
    got_b = ops.gemm_bf16_tile(ad, wd, b.to(DEV), torch.float32, units=units).cpu()
    assert (got_b.double() - want - b.double()).abs().max() <= limit + 1e-6 * float(b.abs().max())
    # views with a wider row stride
    wide = torch.zeros((m, k + 24), dtype=torch.bfloat16)
    wide[:, 8 : 8 + k] = a
    assert torch.equal(ops.gemm_bf16_tile(wide.to(DEV)[:, 8 : 8 + k], wd, None, torch.float32, units=units).cpu(), got)


@pytest.mark.parametrize("m,f,k,units", [(17, 48, 64, 1), (64, 21504 // 8, 6144 // 4, 16), (128, 1000, 192, 8), (100, 296, 128, 2), (30, 8, 64, 1)])
def test_gemm_bf16_tile_gated_epilogue(m, f, k, units):
    """The tiled product with silu(gate) * up in its epilogue against the product followed by the
    activation kernel (the same bits), whichever cut the sizes get, and against float64."""
    from cwm_amd import ops

    x = rnd((m, k), torch.bfloat16, 1)
    wg, wu = rnd((f, k), torch.bfloat16, 2, 0.2), rnd((f, k), torch.bfloat16, 3, 0.2)
    w = torch.stack([wg.reshape(f // 8, 8, k), wu.reshape(f // 8, 8, k)], dim=1).reshape(2 * f, k).contiguous()
    fused = ops.gemm_bf16_tile(x.to(DEV), w.to(DEV), None, torch.bfloat16, glu=True, units=units)
    assert fused.shape == (m, f) and fused.dtype == torch.bfloat16
    two_steps = ops.silu_mul(ops.gemm_bf16_tile(x.to(DEV), w.to(DEV), None, torch.bfloat16, units=units), grouped=True)
    assert torch.equal(fused, two_steps)
    g = x.double() @ wg.double().T
    u = x.double() @ wu.double().T
    want = g * torch.sigmoid(g) * u
    torch.testing.assert_close(fused.cpu().double(), want, rtol=3e-2, atol=3e-2 * float(want.abs().max()))


def test_products_of_9_to_128_rows_take_the_tiled_kernel():
    """`linear` and `gate_up_silu` route the sizes the tiled kernel takes to it, and the others as before."""
    from cwm_amd import ops

    x = rnd((40, 128), torch.bfloat16, 1).to(DEV)
    w = rnd((208, 128), torch.bfloat16, 2, 0.1).to(DEV)
    assert torch.equal(ops.linear(x, w), ops.gemm_bf16_tile(x, w))
    assert torch.equal(ops.gate_up_silu(x, w, None, True), ops.gemm_bf16_tile(x, w, glu=True))
    odd = rnd((208, 120), torch.bfloat16, 3, 0.1).to(DEV)  # K no multiple of 64
    xo = rnd((40, 120), torch.bfloat16, 4).to(DEV)
    assert torch.equal(ops.linear(xo, odd), ops.gemm_bf16_stream(xo, odd))
    with pytest.raises(ops.KernelError, match="tiled product takes"):
        ops.gemm_bf16_tile(xo, odd)
    # up to 8 rows the streaming product is preferred; its epilogues serve up to 16 where the tiled kernel refuses
    x8, x12 = x[:8].contiguous(), x[:12].contiguous()
    assert torch.equal(ops.linear(x8, w), ops.gemm_bf16_stream(x8, w))
    assert torch.equal(ops.linear(x12, w), ops.gemm_bf16_tile(x12, w))
    assert torch.equal(ops.gate_up_silu(x12, w, None, True), ops.gemm_bf16_tile(x12, w, glu=True))
    assert torch.equal(ops.gate_up_silu(xo[:12].contiguous(), odd, None, True), ops.gemm_bf16_stream(xo[:12].contiguous(), odd, None, torch.bfloat16, glu=True))


def test_few_rows_of_a_large_matrix_take_the_tiled_kernel_unless_it_has_a_streaming_copy():
    """Up to 8 rows: a large matrix (2**24 entries and more) without a streaming copy goes to the tiled kernel,
    which reads the row-major matrix in whole cache lines past the caches; with the copy, and for small
    matrices, the streaming kernel stays.  Each choice gives the bits of the kernel it names, and all of
    them the right product."""
    from cwm_amd import ops

    x = rnd((5, 4096), torch.bfloat16, 31).to(DEV)
    w = rnd((4096, 4096), torch.bfloat16, 32, 0.05).to(DEV)
    assert w.numel() >= ops.TILE_FEW_ROWS_ENTRIES
    want = x.double() @ w.double().T
    tiled = ops.gemm_bf16_tile(x, w)
    assert torch.equal(ops.linear(x, w), tiled)
    copy = ops.stream_layout(w)
    streamed = ops.gemm_bf16_stream(x, w, streamed=copy)
    assert torch.equal(ops.linear(x, w, streamed=copy), streamed)
    for got in (tiled, streamed):
        torch.testing.assert_close(got.double(), want, rtol=2e-2, atol=2e-2 * float(want.abs().max()))
    # a gated product likewise: the tiled kernel's epilogue without the copy, the streaming kernel's with it
    assert torch.equal(ops.gate_up_silu(x, w, None, True), ops.gemm_bf16_tile(x, w, glu=True))
    assert torch.equal(ops.gate_up_silu(x, w, None, True, streamed=copy), ops.gemm_bf16_stream(x, w, None, torch.bfloat16, glu=True, streamed=copy))
    small = w[:2048].contiguous()
    assert torch.equal(ops.linear(x, small), ops.gemm_bf16_stream(x, small))


@pytest.mark.parametrize("n_q,n_kv,hd,page_size,dim,m", [(4, 2, 16, 8, 64, 40), (6, 1, 64, 16, 128, 70), (12, 2, 128, 64, 256, 33), (3, 3, 48, 8, 192, 100)])
def test_rope_kv_write_from_partial_sums(n_q, n_kv, hd, page_size, dim, m):
    """The q/k/v projection of 17 to 128 rows leaves partial sums; rotation and cache write take them
    as they are and give the bits of adding them first."""
    from cwm_amd import ops

    n_out = (n_q + 2 * n_kv) * hd
    x = rnd((m, dim), torch.bfloat16, 1).to(DEV)
    w = rnd((n_out, dim), torch.bfloat16, 2, 0.1).to(DEV)
    inv_freq = plain.rope_frequencies(hd, 10000.0).to(DEV)
    g = torch.Generator().manual_seed(5)
    positions = torch.randint(0, 64, (m,), generator=g).to(torch.int32).to(DEV)
    seq = torch.arange(m, dtype=torch.int32).to(DEV)
    width = 64 // page_size + 1
    table = torch.randperm(m * width, generator=g).to(torch.int32).reshape(m, width).contiguous().to(DEV)
    caches = [torch.zeros((m * width, 2, n_kv, page_size * hd), dtype=torch.bfloat16, device=DEV) for _ in range(3)]
    parts = rnd((3, m, n_out), torch.float32, 9, 1.5).to(DEV)
    fused = ops.rope_kv_write_partials(parts, n_q, n_kv, hd, positions, inv_freq, caches[0], table, seq)
    qkv = ops.sum_partials(parts, torch.bfloat16)
    q = qkv[:, : n_q * hd].unflatten(1, (n_q, hd))
    k = qkv[:, n_q * hd : (n_q + n_kv) * hd].unflatten(1, (n_kv, hd))
    v = qkv[:, (n_q + n_kv) * hd :].unflatten(1, (n_kv, hd))
    ops.rope_kv_write(q, k, v, positions, inv_freq, caches[1], table, seq)
    assert torch.equal(fused, qkv)
    assert torch.equal(caches[0], caches[1]) and caches[0].abs().sum() > 0
    # and through the entry that the attention part calls, whatever the product leaves for these sizes
    whole = ops.qkv_rope_write(x, w, None, n_q, n_kv, hd, positions, inv_freq, caches[2], table, seq)
    plain_qkv = ops.linear(x, w)
    q = plain_qkv[:, : n_q * hd].unflatten(1, (n_q, hd))
    k = plain_qkv[:, n_q * hd : (n_q + n_kv) * hd].unflatten(1, (n_kv, hd))
    v = plain_qkv[:, (n_q + n_kv) * hd :].unflatten(1, (n_kv, hd))
    ops.rope_kv_write(q, k, v, positions, inv_freq, caches[1], table, seq)
    assert torch.equal(whole, plain_qkv)
    assert torch.equal(caches[2], caches[1])


@pytest.mark.parametrize("seed", range(6))
def test_gemm_bf16_tile_random_sizes(seed):
    """Random row counts, widths, lengths of K and numbers of blocks: every cut of the work (tiles of
    uneven width, tiles shared by many blocks or by none, blocks that run out of work) gives the product."""
    import random

    from cwm_amd import ops

    rng = random.Random(seed)
    for case in range(8):
        m = rng.choice([1, 16, 17, 63, 64, 65, 127, 128, 129, 255, 300, 512])
        n = 16 * rng.choice([1, 2, 5, 8, 9, 13, 24, 25, 77, 150, 333])
        k = 64 * rng.choice([1, 2, 3, 7, 16, 33])
        units = rng.choice([1, 2, 3, 5, 8, 13, 64, 256, 304])
        a = rnd((m, k), torch.bfloat16, 100 * seed + case)
        w = rnd((n, k), torch.bfloat16, 100 * seed + case + 50, 0.05)
        want = a.double() @ w.double().T
        limit = 1e-5 * float(want.abs().max()) * (1 + k / 512)
        junk = torch.full((40, m, n), float("nan"), dtype=torch.float32, device=DEV)
        del junk
        parts = ops.gemm_bf16_tile(a.to(DEV), w.to(DEV), None, torch.float32, partials_ok=True, units=units).cpu()
        total = parts.double().sum(0) if parts.dim() == 3 else parts.double()
        assert (total - want).abs().max() <= limit, (m, n, k, units, tuple(parts.shape))
        if n % 32 == 0:  # gate and up in groups of 8
            got = ops.gemm_bf16_tile(a.to(DEV), w.to(DEV), None, torch.bfloat16, glu=True, units=units)
            two = ops.silu_mul(ops.gemm_bf16_tile(a.to(DEV), w.to(DEV), None, torch.bfloat16, units=units), grouped=True)
            assert torch.equal(got, two), (m, n, k, units)


@pytest.mark.parametrize("n_q,n_kv,hd", [(16, 8, 64), (48, 8, 128), (6, 3, 48)])
def test_attention_of_a_decoded_token_does_not_depend_on_the_batch(n_q, n_kv, hd):
    """Decoded tokens of 200 sequences in one call (another shape of block and another way of reading the work
    items than a few sequences get) and the same sequences ten at a time: the same bits, and what float32 torch
    gives."""
    from types import SimpleNamespace

    from cwm_amd import ops

    page_size, n_seqs = 16, 200
    g = torch.Generator().manual_seed(n_q + hd)
    lens = [int(x) for x in torch.randint(70, 1400, (n_seqs,), generator=g)]
    lens[3], lens[7] = 2049, 4100  # other chunk lengths
    scale = hd ** -0.5
    pages_of = [(n + page_size - 1) // page_size for n in lens]
    total_pages = sum(pages_of) + 1
    perm = torch.randperm(total_pages, generator=g)
    width = max(pages_of)
    table = torch.full((n_seqs, width), -1, dtype=torch.int32)
    cache = torch.full((total_pages, 2, n_kv, page_size * hd), float("nan"), dtype=torch.bfloat16)
    kc = cache[:, 0].view(total_pages, n_kv, page_size, hd)
    vc = cache[:, 1].view(total_pages, n_kv, page_size // 8, hd, 8)
    q = torch.randn((n_seqs, n_q, hd), generator=g).to(torch.bfloat16)
    want, used = [], 0
    for b, n in enumerate(lens):
        k = torch.randn((n, n_kv, hd), generator=g).to(torch.bfloat16)
        v = torch.randn((n, n_kv, hd), generator=g).to(torch.bfloat16)
        table[b, : pages_of[b]] = perm[used : used + pages_of[b]].to(torch.int32)
        used += pages_of[b]
        pos = torch.arange(n)
        pages, slots = table[b, pos // page_size].long(), pos % page_size
        kc[pages, :, slots, :] = k
        vc[pages, :, slots // 8, :, slots % 8] = v
        if b % 20 == 0:
            group = n_q // n_kv
            scores = torch.einsum("hd,khd->hk", q[b].float(), k.float().repeat_interleave(group, dim=1)) * scale
            want.append((b, torch.einsum("hk,khd->hd", torch.softmax(scores, -1), v.float().repeat_interleave(group, dim=1)).reshape(-1)))
    cache_d, table_d = cache.to(DEV), table.to(DEV)

    def run(which):
        batch = SimpleNamespace(
            q_lens=[1] * len(which), kv_lens=[lens[b] for b in which], n_seqs=len(which), n_tokens=len(which), scratch={},
            cu_q=torch.arange(len(which) + 1, dtype=torch.int32).to(DEV), kv_len=torch.tensor([lens[b] for b in which], dtype=torch.int32).to(DEV),
        )
        rows = torch.tensor(which)
        return ops.paged_attention_mfma(q[rows].to(DEV), cache_d, table_d[rows.to(DEV)].contiguous(), batch, None, scale).cpu()

    together = run(list(range(n_seqs)))
    assert torch.isfinite(together).all()
    for start in range(0, n_seqs, 10):
        assert torch.equal(run(list(range(start, start + 10))), together[start : start + 10]), f"sequences {start}.. differ"
    for b, w in want:
        torch.testing.assert_close(together[b].float(), w, rtol=2e-2, atol=2e-2)


def test_ceiling_kernels_run_and_give_plausible_rates():
    """The two kernels that say what the GPU reaches (not on the model's path): a read of 64 MB windows of a
    256 MB buffer and a short loop of matrix instructions; sizes that the entry points do not take are refused."""
    from cwm_amd import ops

    buffer = torch.zeros(256 << 20, dtype=torch.uint8, device=DEV)
    rate = ops.measure_read_rate(buffer, 64 << 20, 8, 2048)
    assert 500.0 < rate < 20000.0, rate  # GB/s: far from nothing, not beyond any memory
    with pytest.raises(ops.KernelError):
        ops.measure_read_rate(buffer, (64 << 20) + 8, 2, 256)
    for shape in (16, 32):
        flops = ops.measure_mfma_rate(DEV, 512, 2000, launches=2, shape=shape)
        assert 0.05 < flops < 5.0, flops  # PFLOP/s
    with pytest.raises(ops.KernelError, match="shape"):
        ops.measure_mfma_rate(DEV, 512, 10, shape=8)
