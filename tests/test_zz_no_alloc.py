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


def test_sample_static_equals_sample_on_two_calls_in_a_row():
    from cwm_amd.ops import build

    lib = build.load("sampling")
    lib.cwm_sample_static_capacity.restype = ctypes.c_long
    capacity = lib.cwm_sample_static_capacity()
    device = torch.device("cuda:0")
    stream = ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)
    # a large call first, then a smaller one (fewer rows, a shorter vocabulary that is no power of two)
    for seed, (rows, vocab) in enumerate([(7, 4099), (3, 1237)]):
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
