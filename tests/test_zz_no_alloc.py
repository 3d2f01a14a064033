"""The sampling entry point that allocates nothing (`ts_sample_static`), called through
ctypes as a caller that cannot allocate would, against `ts_sample` on the same inputs:
two calls in a row, the second with a smaller input, so that what the first call left in
the library's scratch cannot pass for the second's result."""

import ctypes
from ctypes import c_int, c_void_p

import pytest
import torch

pytestmark = pytest.mark.gpu


def _library():
    from tokensprint_amd.kernels.build import build, find_library
    lib = ctypes.CDLL(str(find_library() or build()))
    lib.ts_last_error.restype = ctypes.c_char_p
    return lib


def _inputs(rows, vocab, seed, device):
    g = torch.Generator().manual_seed(seed)
    logits = (torch.randn(rows, vocab, generator=g) * 3).to(device)
    temps = torch.tensor([0.0 if r % 3 == 0 else 0.5 + 0.25 * r for r in range(rows)],
                         dtype=torch.float32, device=device)
    keys = torch.randint(-(1 << 62), 1 << 62, (rows,), generator=g, dtype=torch.int64).to(device)
    return logits, temps, keys


def _both(lib, logits, temps, keys):
    """(tokens of ts_sample with a caller's workspace, tokens of ts_sample_static)."""
    rows, vocab = logits.shape
    device = logits.device
    stream = c_void_p(torch.cuda.current_stream(device).cuda_stream)
    slices = lib.ts_pick_slices(vocab)
    part_v = torch.empty(rows * slices, dtype=torch.float32, device=device)
    part_i = torch.empty(rows * slices, dtype=torch.int32, device=device)
    want = torch.full((rows,), -1, dtype=torch.int32, device=device)
    got = torch.full((rows,), -2, dtype=torch.int32, device=device)
    p = lambda t: c_void_p(t.data_ptr())
    rc = lib.ts_sample(p(logits), p(temps), p(keys), p(want), p(part_v), p(part_i),
                       c_int(rows), c_int(vocab), stream)
    assert rc == 0, lib.ts_last_error().decode()
    rc = lib.ts_sample_static(p(logits), p(temps), p(keys), p(got), c_int(rows), c_int(vocab),
                              stream)
    assert rc == 0, lib.ts_last_error().decode()
    torch.cuda.synchronize(device)
    return want.tolist(), got.tolist()


def test_sample_static_matches_sample_on_two_calls_in_a_row(gpu_device):
    lib = _library()
    big = _inputs(37, 20011, 0, gpu_device)          # 5 slices of the vocabulary a row
    small = _inputs(5, 4099, 1, gpu_device)          # 2 slices: fewer rows, fewer slices
    want_big, got_big = _both(lib, *big)
    want_small, got_small = _both(lib, *small)
    assert got_big == want_big
    assert got_small == want_small
    # the greedy rows are the plain argmax, so the comparison is not of two equal mistakes
    for (logits, temps, _), got in ((big, got_big), (small, got_small)):
        greedy = (temps <= 1e-10).nonzero().flatten().tolist()
        assert [got[r] for r in greedy] == logits[greedy].argmax(-1).tolist()
    # and the first input once more: the smaller call has not spoilt anything
    assert _both(lib, *big)[1] == want_big


def test_sample_static_refuses_more_than_its_scratch_holds(gpu_device):
    lib = _library()
    cap = lib.ts_sample_static_capacity()
    vocab = 4096 * 8
    rows = cap // 8 + 1
    one = torch.zeros(1, dtype=torch.float32, device=gpu_device)
    # refused on the host before any pointer is used, so small dummies are enough
    rc = lib.ts_sample_static(c_void_p(one.data_ptr()), c_void_p(one.data_ptr()),
                              c_void_p(one.data_ptr()), c_void_p(one.data_ptr()), c_int(rows),
                              c_int(vocab), c_void_p(0))
    assert rc != 0
    assert "exceed" in lib.ts_last_error().decode()
