"""The sampling entry point that allocates nothing (`ts_sample_static`), called through
ctypes as a caller that cannot allocate would, against `ts_sample` on the same inputs:
two calls in a row, the second with a smaller input, so that what the first call left in
the library's scratch cannot pass for the second's result.  Both are also checked against
the draw written out in Python (the counter hash of `sampling.sampler.mix64`, exponential
noise, argmax), and the device's memory is read before and after a call."""

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


def _python_draw_scores(logits, temps, keys):
    """Per row the scores whose argmax the kernels draw, in float64: the logits for a
    greedy row, else logit / T - log E with E = -log U (at least 1e-10) and U uniform in
    (0, 1) from the top 24 bits of mix64(key + 0x9E3779B97F4A7C15 * (index + 1))."""
    import numpy as np
    from tokensprint_amd.sampling.sampler import mix64
    rows, vocab = logits.shape
    out = logits.double().cpu().numpy().copy()
    index = np.arange(1, vocab + 1, dtype=np.uint64)
    with np.errstate(over="ignore"):
        for r in range(rows):
            t = float(temps[r])
            if t <= 1e-10:
                continue
            z = np.uint64(int(keys[r]) & ((1 << 64) - 1)) + np.uint64(0x9E3779B97F4A7C15) * index
            z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
            z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
            z = z ^ (z >> np.uint64(31))
            # the vectorised hash is the sampler module's, entry by entry
            k = int(keys[r]) & ((1 << 64) - 1)
            assert all(int(z[i]) == mix64(k + 0x9E3779B97F4A7C15 * (i + 1)) for i in (0, 7, vocab - 1))
            u = ((z >> np.uint64(40)).astype(np.float64) + 0.5) / 16777216.0
            out[r] = out[r] * float(np.float32(1.0) / np.float32(t)) \
                - np.log(np.maximum(-np.log(u), 1e-10))
    return out


def _assert_drawn_as_python_draws(logits, temps, keys, tokens):
    scores = _python_draw_scores(logits, temps, keys)
    for r, token in enumerate(tokens):
        # float32 logarithms on the device, float64 here: the drawn entry is the best one up
        # to that rounding
        assert scores[r, token] >= scores[r].max() - 1e-4, \
            f"row {r}: drew {token} with score {scores[r, token]}, best is {scores[r].max()}"
        if float(temps[r]) > 1e-10:
            assert token != int(logits[r].argmax()) or scores[r].argmax() == token


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
    # and against the draw written out in Python: not two equal mistakes on noisy rows either
    _assert_drawn_as_python_draws(*big, got_big)
    _assert_drawn_as_python_draws(*small, got_small)
    assert any(got_big[r] != int(big[0][r].argmax()) for r in range(37) if r % 3)   # noise acts
    # and the first input once more: the smaller call has not spoilt anything
    assert _both(lib, *big)[1] == want_big


def test_sample_static_takes_no_device_memory(gpu_device):
    """Around a call (not the first, which may load the library's code object): the
    allocator's books and the device's free memory are what they were."""
    lib = _library()
    logits, temps, keys = _inputs(9, 20011, 2, gpu_device)
    out = torch.full((9,), -1, dtype=torch.int32, device=gpu_device)
    stream = c_void_p(torch.cuda.current_stream(gpu_device).cuda_stream)
    p = lambda t: c_void_p(t.data_ptr())
    call = lambda: lib.ts_sample_static(p(logits), p(temps), p(keys), p(out), c_int(9),
                                        c_int(20011), stream)
    assert call() == 0
    torch.cuda.synchronize(gpu_device)
    allocated, reserved = torch.cuda.memory_allocated(gpu_device), torch.cuda.memory_reserved(gpu_device)
    free = torch.cuda.mem_get_info(gpu_device)[0]
    for _ in range(3):
        assert call() == 0
    torch.cuda.synchronize(gpu_device)
    assert torch.cuda.memory_allocated(gpu_device) == allocated
    assert torch.cuda.memory_reserved(gpu_device) == reserved
    assert torch.cuda.mem_get_info(gpu_device)[0] == free
    _assert_drawn_as_python_draws(logits, temps, keys, out.tolist())


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
