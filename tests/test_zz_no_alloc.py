"""The sampling entry point that allocates nothing (`cwm_sample_static`), called
through ctypes, against the entry point with a workspace argument (`cwm_sample`):
two calls in a row on one GPU, the second with a smaller input, so that it runs over
what the first left in the fixed scratch array."""

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _inputs(seed, rows, vocab, device):
    gen = torch.Generator().manual_seed(seed)
    logits = (3.0 * torch.randn(rows, vocab, generator=gen)).to(device)
    temperature = torch.tensor([0.0 if r % 3 == 2 else 0.5 + 0.25 * r for r in range(rows)], device=device)
    top_p = torch.tensor([1.0 if r % 2 == 0 else 0.8 for r in range(rows)], device=device)
    uniform = torch.rand(rows, generator=gen).to(device)
    return logits, temperature, top_p, uniform


def _outputs(rows, device):
    return (
        torch.full((rows,), -7, dtype=torch.int32, device=device),
        torch.full((rows,), float("nan"), device=device),
        torch.full((rows,), float("nan"), device=device),
    )


# a large call first, then a smaller one (fewer rows, a shorter vocabulary): once with vocabularies that are no
# multiple of 4 (rows read entry by entry) and once with multiples of 4, as real vocabularies are (rows read 16
# bytes at a time); rows 1, 3, ... have a nucleus of 0.8, so the second call of each pair has one too
@pytest.mark.parametrize("calls", [[(7, 4099), (3, 1237)], [(5, 4096), (2, 1024)]])
def test_sample_static_equals_sample_on_two_calls_in_a_row(calls):
    from cwm_amd.ops import build

    lib = build.load("sampling")
    assert lib.cwm_sample_static_init() == 0, lib.cwm_error_message()
    lib.cwm_sample_static_capacity.restype = ctypes.c_long
    capacity = lib.cwm_sample_static_capacity()
    device = torch.device("cuda:0")
    stream = ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)
    for seed, (rows, vocab) in enumerate(calls):
        assert rows * vocab <= capacity
        logits, temperature, top_p, uniform = _inputs(seed, rows, vocab, device)
        want = _outputs(rows, device)
        workspace = torch.empty((rows, vocab), dtype=torch.float32, device=device)
        status = lib.cwm_sample(
            _ptr(logits), ctypes.c_long(vocab), ctypes.c_int(rows), ctypes.c_int(vocab), _ptr(temperature), _ptr(top_p),
            _ptr(uniform), _ptr(workspace), _ptr(want[0]), _ptr(want[1]), _ptr(want[2]), stream,
        )
        assert status == 0, lib.cwm_error_message()
        got = _outputs(rows, device)
        status = lib.cwm_sample_static(
            _ptr(logits), ctypes.c_long(vocab), ctypes.c_int(rows), ctypes.c_int(vocab), _ptr(temperature), _ptr(top_p),
            _ptr(uniform), _ptr(got[0]), _ptr(got[1]), _ptr(got[2]), stream,
        )
        assert status == 0, lib.cwm_error_message()
        torch.cuda.synchronize()
        assert torch.equal(got[0].cpu(), want[0].cpu())
        assert (got[0] >= 0).all() and (got[0] < vocab).all()
        assert torch.equal(got[1].cpu(), want[1].cpu())
        assert torch.equal(got[2].cpu(), want[2].cpu())
        # greedy rows are the argmax
        greedy = [r for r in range(rows) if float(temperature[r]) == 0.0]
        assert got[0][greedy].cpu().tolist() == logits[greedy].argmax(dim=1).cpu().tolist()
        # the other rows against the distribution itself (softmax at the temperature, the nucleus of
        # cwm/fastgen/utils/sampling.py:38-41, inverse CDF in the order of the vocabulary),
        # so that a mistake shared by both entry points would show
        for r in range(rows):
            if r in greedy:
                continue
            probs = torch.softmax(logits[r].double().cpu() / float(temperature[r]), -1)
            order = torch.argsort(probs, descending=True)
            before = torch.cumsum(probs[order], 0) - probs[order]
            keep = torch.zeros_like(probs, dtype=torch.bool)
            keep[order[before <= float(top_p[r])]] = True  # an entry stays while the mass before it is within top_p
            probs = torch.where(keep, probs, torch.zeros_like(probs))
            probs = probs / probs.sum()
            cdf = torch.cumsum(probs, 0)
            tok, u = int(got[0][r]), float(uniform[r])
            assert probs[tok] > 0 and float(cdf[tok] - probs[tok]) <= u + 1e-4 and float(cdf[tok]) >= u - 1e-4


def test_sample_static_refuses_more_than_its_array_holds():
    from cwm_amd.ops import build

    lib = build.load("sampling")
    lib.cwm_sample_static_capacity.restype = ctypes.c_long
    capacity = lib.cwm_sample_static_capacity()
    device = torch.device("cuda:0")
    rows, vocab = 3, capacity // 2  # 1.5 times the array
    small = torch.zeros(4, device=device)
    tokens = torch.zeros(4, dtype=torch.int32, device=device)
    # the size check comes before any launch: the logits pointer is never read
    status = lib.cwm_sample_static(
        _ptr(small), ctypes.c_long(vocab), ctypes.c_int(rows), ctypes.c_int(vocab), _ptr(small), _ptr(small),
        _ptr(small), _ptr(tokens), _ptr(small), _ptr(small), ctypes.c_void_p(0),
    )
    assert status != 0
    assert b"scratch" in lib.cwm_error_message()
