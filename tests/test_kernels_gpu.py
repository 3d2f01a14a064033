"""Each HIP kernel alone against its plain torch reference (tests/kernel_refs.py), in
float32 and bfloat16, at sizes other than the engine's tiny models: widths and
vocabularies that are no power of two, head sizes in steps of 16, odd head groupings."""

import ctypes

import pytest
import torch

from kernel_refs import TorchOps
from scenarios import paged_scenario

pytestmark = pytest.mark.gpu

REF = TorchOps()
DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(scope="module")
def ops(gpu_device):
    from tokensprint_amd.kernels import load_hip_ops
    return load_hip_ops(gpu_device)


@pytest.fixture(autouse=True)
def default_product_choices(ops, monkeypatch):
    """The provider is one per device and process; what an engine's warm-up in another test
    chose for the products of few rows with large weights is not these tests' business."""
    monkeypatch.setattr(ops, "_large_rows", {})
    monkeypatch.setattr(ops, "_large_undecided", set())


def tol(dtype):
    return dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=1.6e-2, atol=1.6e-2)


def rand(shape, dtype, device, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype).to(device)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("vocab,width", [(389, 96), (1000, 1030)])
def test_embed_and_gather(ops, gpu_device, dtype, vocab, width):
    table = rand((vocab, width), dtype, gpu_device, 0)
    ids = torch.randint(0, vocab, (77,), dtype=torch.int32, device=gpu_device)
    out = ops.embed(table, ids)
    assert out.dtype == torch.float32
    torch.testing.assert_close(out, REF.embed(table, ids), rtol=0, atol=0)
    rows = torch.tensor([5, 0, 76, 5], dtype=torch.int32, device=gpu_device)
    x = out.to(dtype)
    torch.testing.assert_close(ops.gather_rows(x, rows), REF.gather_rows(x, rows), rtol=0, atol=0)


# shapes (257,1024) and (4*73,1024), weights U(-1,1), eps 1e-6 are the reference's own
# parity vectors (tests/test_kernel_parity.py:234-262 of the reference)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,width", [(257, 1024), (292, 1024), (33, 96), (5, 5120), (7, 50)])
def test_rmsnorm(ops, gpu_device, dtype, rows, width):
    x = rand((rows, width), dtype, gpu_device, 1)
    w = (torch.rand(width, generator=torch.Generator().manual_seed(2)) * 2 - 1).to(gpu_device)
    out = ops.rmsnorm(x, w, 1e-6, dtype)
    torch.testing.assert_close(out.float(), REF.rmsnorm(x, w, 1e-6, dtype).float(), **tol(dtype))
    torch.testing.assert_close(
        out.float(), torch.nn.functional.rms_norm(x.float(), (width,), w, 1e-6),
        **(tol(dtype) if dtype == torch.float32 else dict(rtol=1e-2, atol=3.2e-2)))


@pytest.mark.parametrize("dtype", DTYPES)
def test_add_rmsnorm_updates_the_residual(ops, gpu_device, dtype):
    rows, width = 19, 1030
    resid = rand((rows, width), torch.float32, gpu_device, 3)
    delta = rand((rows, width), dtype, gpu_device, 4)
    w = 1 + 0.1 * rand((width,), torch.float32, gpu_device, 5)
    ref_resid = resid.clone()
    ref = REF.add_rmsnorm(ref_resid, delta, w, 1e-5, dtype)
    out = ops.add_rmsnorm(resid, delta, w, 1e-5, dtype)
    torch.testing.assert_close(resid, ref_resid, rtol=0, atol=0)
    torch.testing.assert_close(out.float(), ref.float(), **tol(dtype))


def test_take_tokens(ops, gpu_device):
    ids = torch.arange(100, 109, dtype=torch.int32, device=gpu_device)
    drawn = torch.tensor([7, 8, 9, 10], dtype=torch.int32, device=gpu_device)
    src = torch.tensor([-1, 3, 0, -1, 2, 2, 4, -5, 1], dtype=torch.int32, device=gpu_device)
    ops.take_tokens(ids, src, drawn)
    # a lane without a source, or with one outside the drawn tokens, keeps its own
    assert ids.tolist() == [100, 10, 7, 103, 9, 9, 106, 107, 8]


@pytest.mark.parametrize("dtype", DTYPES)
def test_silu_mul(ops, gpu_device, dtype):
    gu = rand((37, 2 * 150), dtype, gpu_device, 6, scale=3.0)
    torch.testing.assert_close(ops.silu_mul(gu).float(), REF.silu_mul(gu).float(), **tol(dtype))
    g, u = gu[:, :150].float(), gu[:, 150:].float()
    torch.testing.assert_close(ops.silu_mul(gu).float(), torch.nn.functional.silu(g) * u,
                               **tol(dtype))


def from_library(M, N, K):
    """Whether a plain bfloat16 product of this shape goes to the vendor library: above 64
    rows, from 17 rows on where the kernels here lay their waves along N (a short K), from
    5 rows on at a very wide N (the output head), from 9 at weights above 2^23 elements."""
    return (M > 64 or (M > 16 and K < 512) or (M > 4 and N >= 16384)
            or (M > 8 and N * K > 2 ** 23))


@pytest.mark.parametrize("out_dtype", DTYPES)
@pytest.mark.parametrize("x_dtype,w_dtype", [(torch.float32, torch.float32),
                                             (torch.bfloat16, torch.bfloat16),
                                             (torch.bfloat16, torch.float32)])
@pytest.mark.parametrize("M,N,K", [(1, 389, 96), (7, 130, 50), (64, 64, 64), (100, 301, 1030),
                                   (300, 77, 17)])
def test_linear(ops, gpu_device, x_dtype, w_dtype, out_dtype, M, N, K):
    x = rand((M, K), x_dtype, gpu_device, 7)
    w = rand((N, K), w_dtype, gpu_device, 8, scale=0.1)
    out = ops.linear(x, w, out_dtype)
    ref = x.double() @ w.double().T
    # every kernel sums in float32, the vendor library's too, and a float32 result leaves
    # unrounded: held to float32 rounding whatever the operands' types; a bfloat16 result
    # to bfloat16's
    t = dict(rtol=1e-5, atol=1e-5) if out_dtype == torch.float32 else dict(rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(out.double(), ref, **t)


@pytest.mark.parametrize("out_dtype", DTYPES)
@pytest.mark.parametrize("M,N,K", [(1, 1024, 1024), (8, 4096, 1024), (8, 1024, 3072),
                                   (17, 1000, 2048), (64, 6144, 1024), (3, 151936, 1024),
                                   (130, 389, 96), (33, 50, 520), (70, 20000, 64),
                                   (48, 1024, 3072), (64, 1024, 2048), (40, 3000, 1096),
                                   (16, 300, 2056), (23, 520, 640), (4, 20000, 1024),
                                   (8, 4096, 4096), (12, 4096, 4096),
                                   (6, 20000, 1024)])
def test_linear_bf16_matrix_core_shapes(ops, gpu_device, out_dtype, M, N, K):
    x = rand((M, K), torch.bfloat16, gpu_device, 17)
    w = rand((N, K), torch.bfloat16, gpu_device, 18, scale=0.05)
    out = ops.linear(x, w, out_dtype)
    ref = x.float() @ w.float().T
    ours = not from_library(M, N, K)
    t = dict(rtol=2e-3, atol=2e-3) if out_dtype == torch.float32 and ours \
        else dict(rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(out.float(), ref, **t)
    # a row does not depend on the rest of the batch, bit for bit, while our own kernels
    # serve it; beyond that the vendor library does, and rows agree to rounding
    one = ops.linear(x[M // 2:M // 2 + 1].contiguous(), w, out_dtype)
    if ours:
        assert torch.equal(out[M // 2:M // 2 + 1], one)
        last = ops.linear(x[M - 1:].contiguous(), w, out_dtype)
        assert torch.equal(out[M - 1:], last)
    else:
        torch.testing.assert_close(out[M // 2:M // 2 + 1].float(), one.float(), rtol=1e-2, atol=1e-2)


def test_library_plan_chosen_by_timing(ops, gpu_device):
    """A few rows against a large weight with the plan chosen by timing the library's
    candidates (as the engine does for the decode steps it captures): whichever algorithm
    wins, the product is the same to rounding, also for later calls with the kept plan
    and inside a captured graph."""
    M, N, K = 24, 4096 + 64, 4096         # a shape no other test has planned already
    x = rand((M, K), torch.bfloat16, gpu_device, 60)
    w = rand((N, K), torch.bfloat16, gpu_device, 61, scale=0.05)
    ref = x.float() @ w.float().T
    ops.timed_plans(True)
    try:
        out = ops.linear(x, w, torch.bfloat16)
    finally:
        ops.timed_plans(False)
    torch.testing.assert_close(out.float(), ref, rtol=1e-2, atol=1e-2)
    again = ops.linear(x, w, torch.bfloat16)
    assert torch.equal(out, again)
    side = torch.cuda.Stream(gpu_device)
    graph = torch.cuda.CUDAGraph()
    side.wait_stream(torch.cuda.current_stream(gpu_device))
    with torch.cuda.stream(side):
        ops.linear(x, w, torch.bfloat16)
    torch.cuda.current_stream(gpu_device).wait_stream(side)
    with torch.cuda.graph(graph):
        captured = ops.linear(x, w, torch.bfloat16)
    for _ in range(3):
        captured.zero_()
        graph.replay()
        torch.cuda.synchronize(gpu_device)
        assert torch.equal(captured, out)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,I,K", [(8, 3072, 1024), (1, 160, 96), (40, 112, 80), (70, 1000, 520),
                                   (40, 3072, 1024), (64, 1000, 2056), (33, 200, 520),
                                   (5, 304, 3080), (130, 3072, 1024), (300, 1008, 320)])
def test_linear_silu_mul(ops, gpu_device, dtype, M, I, K):
    x = rand((M, K), dtype, gpu_device, 19)
    w = rand((2 * I, K), dtype, gpu_device, 20, scale=0.1)
    out = ops.linear_silu_mul(x, w, dtype)
    if dtype == torch.float32:
        # float64 reference; float32 sums of K products err by about K * 2^-24 * |x||w|
        gu = x.double() @ w.double().T
        ref = torch.nn.functional.silu(gu[:, :I]) * gu[:, I:]
        bound = 1e-5 * float(ref.abs().max())
        torch.testing.assert_close(out.double(), ref, rtol=1e-5, atol=bound)
    else:
        ref = REF.linear_silu_mul(x, w, dtype)
        torch.testing.assert_close(out.float(), ref.float(), **tol(dtype))


@pytest.mark.parametrize("out_dtype", DTYPES)
@pytest.mark.parametrize("M,N,K", [(300, 400, 320), (70, 1040, 256), (2051, 1024, 2048),
                                   (513, 4096, 1024), (1000, 48, 4096), (640, 1296, 640)])
def test_gemm_tiled(ops, gpu_device, out_dtype, M, N, K):
    """The LDS-tiled product at sizes whose edges cut tiles in both directions and whose
    tile grids do not divide into the eight regions evenly, with every tile size: against
    float32 sums of the same bfloat16 operands, and every tile size the same to the bit
    (one accumulator per element sums K in index order whatever the tile)."""
    x = rand((M, K), torch.bfloat16, gpu_device, 50)
    w = rand((N, K), torch.bfloat16, gpu_device, 51, scale=0.05)
    ref = x.float() @ w.float().T
    t = dict(rtol=2e-3, atol=2e-3) if out_dtype == torch.float32 else dict(rtol=1e-2, atol=1e-2)
    first = None
    for tile in (0, 1, 2, 3, 4, 5):
        out = ops.gemm_tiled(x, w, out_dtype, tile=tile)
        torch.testing.assert_close(out.float(), ref, **t)
        first = out if first is None else first
        assert torch.equal(out, first), f"tile {tile} differs"
    # a row does not depend on the rows beside it
    one = ops.gemm_tiled(x[M // 3:M // 3 + 1].contiguous(), w, out_dtype)
    assert torch.equal(one, first[M // 3:M // 3 + 1])


@pytest.mark.parametrize("M,I,K", [(130, 112, 256), (2051, 3072, 1024), (300, 1008, 320),
                                   (65, 16, 256), (700, 2000, 4096)])
def test_gemm_tiled_with_silu_mul(ops, gpu_device, M, I, K):
    """Stacked gate and up weights: the tiles interleave their columns per wave and the
    epilogue multiplies.  One gate column is made to dominate so that a column paired with
    the wrong partner, or a tile's columns in the wrong place, shows."""
    x = rand((M, K), torch.bfloat16, gpu_device, 52)
    w = rand((2 * I, K), torch.bfloat16, gpu_device, 53, scale=0.05)
    w[I // 2] *= 8                      # one gate column far above the others
    w[I + I // 3] *= 8                  # and one up column elsewhere
    ref = REF.linear_silu_mul(x, w, torch.bfloat16)
    first = None
    for tile in (0, 1, 2, 3, 4, 5):
        out = ops.gemm_tiled(x, w, torch.bfloat16, pair=True, tile=tile)
        torch.testing.assert_close(out.float(), ref.float(), rtol=2e-2, atol=2e-2)
        first = out if first is None else first
        assert torch.equal(out, first), f"tile {tile} differs"
    # the engine's entry takes this kernel from 65 rows on at weights of this size
    if 2 * I * K <= ops.dispatch.tiled_pair_weight:
        assert torch.equal(ops.linear_silu_mul(x, w, torch.bfloat16), first)


@pytest.mark.parametrize("M,N,K,next_n,silu", [(2051, 1024, 2048, 3072, True),
                                               (513, 320, 1024, 400, False),
                                               (700, 576, 4096, 112, True),
                                               (1030, 1024, 3072, 4096, False),
                                               (520, 4096, 256, 64, False),
                                               (8200, 1024, 2048, 3072, True)])
def test_gemm_tiled_into_stream(ops, gpu_device, M, N, K, next_n, silu):
    """The tiled product's tail form (adds itself into the float32 stream, hands the stream
    on times the norm's weight, with the rows' sums of squares in slices) and the scaled
    form behind it, each against float32 arithmetic on what it was given, every tile the
    same to the bit; then the two through the provider's entry points against the
    separate product, add-and-norm and product.  The stream's rows differ a hundredfold
    in size, so that a factor taken from another row shows.  (The last case has 128 slices
    a row: more than the scaled form asks for at a time.)"""
    from tokensprint_amd.kernels.hip_ops import _ptr
    from tokensprint_amd.kernels.stream import NormHint, PreparedRows
    bf = torch.bfloat16
    x = rand((M, K), bf, gpu_device, 60)
    w = rand((N, K), bf, gpu_device, 61, scale=0.03)
    resid0 = rand((M, N), torch.float32, gpu_device, 62)
    resid0 *= torch.logspace(-1, 1, M, device=gpu_device)[torch.randperm(M, device=gpu_device)][:, None]
    g = rand((N,), torch.float32, gpu_device, 63).abs() + 0.5
    wn = rand((next_n * (2 if silu else 1), N), bf, gpu_device, 64, scale=0.05)
    eps = 1e-5
    delta = (x.float() @ w.float().T)
    parts = ops.lib.ts_gemm_tiled_tail_parts(N)
    first = None
    for tile in (0, 1, 2, 3, 4, 5):
        resid = resid0.clone()
        rows = torch.empty(M, N, dtype=bf, device=gpu_device)
        sumsq = torch.empty(parts, M, dtype=torch.float32, device=gpu_device)
        ops._call(ops.lib.ts_gemm_tiled_tail_bf16, _ptr(x), _ptr(w), _ptr(resid), _ptr(g), _ptr(rows),
                  _ptr(sumsq), M, N, K, tile, ops._stream())
        if first is None:
            # the product is rounded to bfloat16 before it is added: half an ulp of it off
            # where the sums' order rounds the other way
            torch.testing.assert_close(resid - resid0, delta, rtol=1e-2, atol=1e-2)
            assert torch.equal(rows, (resid * g).to(bf))
            torch.testing.assert_close(sumsq.double().sum(0), (resid.double() ** 2).sum(1),
                                       rtol=1e-5, atol=0)
            first = (resid, rows, sumsq)
        for got, want in zip((resid, rows, sumsq), first):
            assert torch.equal(got, want), f"tail tile {tile} differs"
    resid, rows, sumsq = first
    rstd = torch.rsqrt((resid.double() ** 2).sum(1, keepdim=True) / N + eps)
    prod = (rows.double() @ wn.double().T * rstd).float()
    if silu:
        gate, up = prod[:, :next_n].to(bf).float(), prod[:, next_n:].to(bf).float()
        want = gate * torch.sigmoid(gate) * up
    else:
        want = prod
    first_out = None
    for tile in (0, 1, 2, 3, 4, 5):
        out = torch.empty(M, next_n, dtype=bf, device=gpu_device)
        ops._call(ops.lib.ts_gemm_tiled_scaled_bf16, _ptr(rows), _ptr(sumsq), parts, ctypes.c_float(eps),
                  _ptr(wn), _ptr(out), 1, M, next_n, N, int(silu), tile, ops._stream())
        torch.testing.assert_close(out.float(), want, rtol=2e-2, atol=2e-2)
        first_out = out if first_out is None else first_out
        assert torch.equal(out, first_out), f"scaled tile {tile} differs"
    # through the provider, where its table sends these sizes to the two forms
    hint = NormHint(g, eps, wn, silu)
    if ops._tiled_stream_ok(M, N, K, hint):
        stream = resid0.clone()
        prepared = ops.linear_into_stream(x, w, stream, hint)
        assert isinstance(prepared, PreparedRows)
        assert torch.equal(stream, resid)
        out, stream_out = ops.norm_linear(stream, prepared, g, eps, wn, bf, silu_mul=silu)
        assert torch.equal(out, first_out) and stream_out is stream
        apart, stream_apart = ops.norm_linear(resid0.clone(), ops.linear(x, w, bf), g, eps, wn, bf,
                                              silu_mul=silu)
        torch.testing.assert_close(stream_apart, stream, rtol=1e-2, atol=1e-2)
        # The two round the normed rows to bfloat16 at different places (before or after the
        # division by the root mean square), so each is compared with the exact function of
        # the stream.  A sum of N products of operands 2^-9 off has noise of about
        # 2^-9 * sqrt(N) * rms(h) * rms(w) (0.003 at N = 1,024 here); six of those, since
        # millions of elements are compared, plus the result's own rounding; and
        # silu(gate) * up carries both factors' noise.
        s64 = stream.double()
        h = s64 * torch.rsqrt((s64 ** 2).mean(1, keepdim=True) + eps) * g.double()
        exact = h @ wn.double().T
        sigma = 2.0 ** -9 * (N ** 0.5) * float(h.pow(2).mean().sqrt() * wn.double().pow(2).mean().sqrt())
        if silu:
            gate, up = exact[:, :next_n], exact[:, next_n:]
            exact, slack = gate * torch.sigmoid(gate) * up, 6 * sigma * (1 + gate.abs() + up.abs())
        else:
            slack = 6 * sigma
        for name, got in (("fused", out), ("apart", apart)):
            excess = ((got.double() - exact).abs() - slack - 0.01 * exact.abs()).max().item()
            assert excess <= 0, f"{name}: {excess} beyond the rounding bound"


def test_gemm_tiled_refuses_what_it_cannot_take(ops, gpu_device):
    x = rand((100, 200), torch.bfloat16, gpu_device, 54)
    w = rand((64, 200), torch.bfloat16, gpu_device, 55)
    with pytest.raises(RuntimeError, match="gemm_tiled"):
        ops.gemm_tiled(x, w, torch.bfloat16)                  # K not a multiple of 64
    x = rand((100, 256), torch.bfloat16, gpu_device, 54)
    w = rand((2 * 24, 256), torch.bfloat16, gpu_device, 55)
    with pytest.raises(RuntimeError, match="gemm_tiled"):
        ops.gemm_tiled(x, w, torch.bfloat16, pair=True)       # 24 columns: not a multiple of 16
    with pytest.raises(RuntimeError, match="bfloat16"):
        ops.gemm_tiled(x, rand((64, 256), torch.bfloat16, gpu_device, 56), torch.float32, pair=True)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("silu", [False, True])
@pytest.mark.parametrize("M,N,K", [(8, 4096, 1024), (1, 160, 96), (16, 112, 80), (3, 1024, 3072),
                                   (20, 96, 64), (5, 20000, 64), (16, 1000, 2056),
                                   (9, 3072, 4096), (12, 520, 1096), (4, 1000, 2056),
                                   (1, 3072, 4096), (3, 5000, 4096)])
def test_norm_linear(ops, gpu_device, dtype, silu, M, N, K):
    """Against float64.  In bfloat16 both the operand of the product (the normalised row)
    and its results are rounded to 8 bits; which value exactly is rounded differs between
    correct implementations (the fused kernel rounds x*w and divides by the root mean
    square afterwards), so the bound is the rounding noise itself: a sum of K products of
    operands with relative error 2^-9 has noise about 2^-9 * sqrt(K) * rms(x) * rms(w), a
    rounded result 2^-9 of itself, and silu(g)*u inherits |u| times the noise of g plus
    |silu(g)| times the noise of u."""
    resid = rand((M, K), torch.float32, gpu_device, 40)
    delta = rand((M, K), dtype, gpu_device, 41)
    nw = 1 + 0.1 * rand((K,), torch.float32, gpu_device, 42)
    w = rand((N, K), dtype, gpu_device, 43, scale=0.05)
    for d in (delta, None):
        x = resid.double() + (0 if d is None else d.double())
        h = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-5) * nw.double()
        y = h @ w.double().T
        # float32: sums in index order err by up to about sqrt(K) * 2^-24 per term magnitude
        eps = 2.0 ** -9 if dtype == torch.bfloat16 else 2.0 ** -19
        dot_noise = eps * (K ** 0.5) * float(h.pow(2).mean().sqrt() * w.double().pow(2).mean().sqrt())
        noise = 4 * (dot_noise + eps * y.abs())
        if silu:
            g, u = y[:, :N // 2], y[:, N // 2:]
            ref = torch.nn.functional.silu(g) * u
            sg = torch.nn.functional.silu(g).abs()
            bound = 1.2 * (u.abs() + noise[:, N // 2:]) * noise[:, :N // 2] + sg * noise[:, N // 2:] \
                + 4 * eps * ref.abs()
        else:
            ref, bound = y, noise
        r_in = resid.clone()
        out, r_out = ops.norm_linear(r_in, d, nw, 1e-5, w, dtype, silu_mul=silu)
        torch.testing.assert_close(r_out.double(), x, rtol=1e-6, atol=1e-6)
        excess = ((out.double() - ref).abs() - bound).max()
        assert excess <= 0, f"error exceeds the rounding bound by {float(excess):.3e}"


@pytest.mark.parametrize("silu", [False, True])
@pytest.mark.parametrize("M,W,K,N", [(8, 1024, 2048, 4096), (1, 1024, 3072, 6144), (64, 1024, 2048, 4096),
                                     (33, 520, 1096, 1392), (16, 1000, 2056, 112), (17, 4096, 512, 160),
                                     (7, 2048, 4096, 528), (40, 1000, 520, 2000),
                                     (8, 1280, 1024, 512), (4, 1536, 512, 1024), (2, 3000, 520, 264),
                                     (3, 1024, 2048, 4096), (12, 1024, 3072, 6144)])
def test_linear_into_stream_then_norm_linear(ops, gpu_device, silu, M, W, K, N):
    """The norm split over two products (bfloat16 only): the first adds bf16(x Wo^T) into
    the stream [M, W] in place and prepares the rows, the second is norm_linear over them.
    Against float64 from the stream the first one must leave, with norm_linear's bound."""
    from tokensprint_amd.kernels.stream import NormHint, PreparedRows
    bf = torch.bfloat16
    resid = rand((M, W), torch.float32, gpu_device, 50)
    x = rand((M, K), bf, gpu_device, 51)
    wo = rand((W, K), bf, gpu_device, 52, scale=0.05)
    nw = 1 + 0.1 * rand((W,), torch.float32, gpu_device, 53)
    w = rand((N, W), bf, gpu_device, 54, scale=0.05)
    hint = NormHint(nw, 1e-5, w, silu)
    r = resid.clone()
    prepared = ops.linear_into_stream(x, wo, r, hint)
    assert isinstance(prepared, PreparedRows), "these shapes are ones the fused kernels take"
    delta = (x.double() @ wo.double().T)
    # the product is rounded to bfloat16 (unit roundoff 2^-8) before the add, as the
    # separate kernels do
    eps = 2.0 ** -9
    dnoise = 2 * eps * delta.abs() + 4 * 2.0 ** -24 * (K ** 0.5) * float(
        x.double().pow(2).mean().sqrt() * wo.double().pow(2).mean().sqrt())
    assert ((r.double() - (resid.double() + delta)).abs() <= 1.01 * dnoise + 1e-6).all()
    xs = r.double()
    assert prepared.sumsq.shape == (M, -(-prepared.slices // 4) * 4)     # a row's slices side by side
    assert torch.allclose(prepared.sumsq[:, :prepared.slices].double().sum(1), xs.pow(2).sum(-1), rtol=1e-5)
    torch.testing.assert_close(prepared.rows.float(), (r * nw).to(bf).float(), rtol=2 ** -7, atol=1e-30)
    h = xs * torch.rsqrt(xs.pow(2).mean(-1, keepdim=True) + 1e-5) * nw.double()
    y = h @ w.double().T
    dot_noise = eps * (W ** 0.5) * float(h.pow(2).mean().sqrt() * w.double().pow(2).mean().sqrt())
    noise = 4 * (dot_noise + eps * y.abs())
    if silu:
        g, u = y[:, :N // 2], y[:, N // 2:]
        ref = torch.nn.functional.silu(g) * u
        sg = torch.nn.functional.silu(g).abs()
        bound = 1.2 * (u.abs() + noise[:, N // 2:]) * noise[:, :N // 2] + sg * noise[:, N // 2:] \
            + 4 * eps * ref.abs()
    else:
        ref, bound = y, noise
    out, r_out = ops.norm_linear(r, prepared, nw, 1e-5, w, bf, silu_mul=silu)
    assert r_out is r
    # The bound is four standard deviations of the rounding noise: it is for the number of
    # results that the other product tests hold, so it is applied to the first 16 rows;
    # the rest is covered by the next check, bit for bit.
    excess = ((out.double() - ref).abs() - bound)[:16].max()
    assert excess <= 0, f"error exceeds the rounding bound by {float(excess):.3e}"
    # a row's result does not depend on the other rows of the step, nor on the tile of
    # rows it lands in: fewer rows at a time give the same bits (up to 16 rows a product
    # of few columns is cut into narrower slices, whose sums of squares add up in another
    # order: the same bits on either side of 16 rows, not across)
    some = 8 if M <= 16 else max(17, (M + 1) // 2)
    for m0 in (range(0, M, some) if M <= 16 else (0, M - some)):
        r8 = resid[m0:m0 + some].clone()
        p8 = ops.linear_into_stream(x[m0:m0 + some].contiguous(), wo, r8, hint)
        out8, _ = ops.norm_linear(r8, p8, nw, 1e-5, w, bf, silu_mul=silu)
        assert torch.equal(r8, r[m0:m0 + some]) and torch.equal(out8, out[m0:m0 + some]), m0
    # rows prepared for one norm are refused by another
    with pytest.raises(ValueError):
        ops.norm_linear(r, prepared, nw.clone(), 1e-5, w, bf, silu_mul=silu)


def test_linear_into_stream_declines_what_it_cannot_fuse(ops, gpu_device):
    from tokensprint_amd.kernels.stream import NormHint
    bf = torch.bfloat16
    nw = torch.ones(1024, device=gpu_device)
    w = rand((4096, 1024), bf, gpu_device, 1)
    wo = rand((1024, 2048), bf, gpu_device, 2)
    for M, dt in ((65, bf), (8, torch.float32)):
        x = rand((M, 2048), dt, gpu_device, 3)
        r = rand((M, 1024), torch.float32, gpu_device, 4)
        before = r.clone()
        assert ops.linear_into_stream(x, wo if dt == bf else wo.float(), r, NormHint(nw, 1e-6, w)) is None
        assert torch.equal(r, before)
    assert ops.linear_into_stream(rand((8, 2048), bf, gpu_device, 3), wo,
                                  rand((8, 1024), torch.float32, gpu_device, 4), None) is None


def test_linear_rows_do_not_depend_on_the_batch(ops, gpu_device):
    x = rand((70, 200), torch.float32, gpu_device, 9)
    w = rand((150, 200), torch.float32, gpu_device, 10)
    full = ops.linear(x, w, torch.float32)
    one = ops.linear(x[33:34].contiguous(), w, torch.float32)
    assert torch.equal(full[33:34], one)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq,nkv,hd,page", [(4, 2, 16, 4), (8, 2, 32, 16), (6, 3, 48, 8),
                                            (16, 8, 128, 16), (5, 5, 80, 3), (8, 1, 256, 64)])
@pytest.mark.parametrize("spans", [[(0, 9), (13, 1), (5, 20), (31, 2)],
                                   [(3, 70), (0, 33), (40, 1)]], ids=["short", "long"])
def test_qk_norm_rope_store(ops, gpu_device, dtype, nq, nkv, hd, page, spans):
    batch, cache, table, _ = paged_scenario(gpu_device, dtype, nkv=nkv, hd=hd, page_size=page,
                                            spans=spans, seed=11)
    T = batch.num_tokens
    qkv = rand((T, (nq + 2 * nkv) * hd), dtype, gpu_device, 12)
    wq = 1 + 0.1 * rand((hd,), torch.float32, gpu_device, 13)
    wk = 1 + 0.1 * rand((hd,), torch.float32, gpu_device, 14)
    angles = torch.outer(torch.arange(80, dtype=torch.float32),
                         1.0 / (10000.0 ** (torch.arange(0, hd, 2, dtype=torch.float32) / hd)))
    cos_sin = (angles.cos().to(gpu_device), angles.sin().to(gpu_device))
    ref_cache = type(cache)(cache.group, cache.page_size, cache.num_pages,
                            cache.k_pages.clone(), cache.v_pages.clone())
    kw = dict(num_heads=nq, num_kv_heads=nkv, head_dim=hd, q_weight=wq, k_weight=wk, eps=1e-5,
              cos_sin=cos_sin)
    q_ref = REF.qk_norm_rope_store(qkv, batch, table, ref_cache, **kw)
    q = ops.qk_norm_rope_store(qkv, batch, table, cache, **kw)
    torch.testing.assert_close(q.float(), q_ref.float(), **tol(dtype))
    torch.testing.assert_close(cache.k_pages.float(), ref_cache.k_pages.float(), **tol(dtype))
    torch.testing.assert_close(cache.v_pages.float(), ref_cache.v_pages.float(), rtol=0, atol=0)
    # pieces alone: norm-only split, rotation in place, store
    q2, k2, v2 = ops.qk_norm_split(qkv, num_heads=nq, num_kv_heads=nkv, head_dim=hd,
                                   q_weight=wq, k_weight=wk, eps=1e-5)
    q2r, k2r, v2r = REF.qk_norm_split(qkv, num_heads=nq, num_kv_heads=nkv, head_dim=hd,
                                      q_weight=wq, k_weight=wk, eps=1e-5)
    torch.testing.assert_close(q2.float(), q2r.float(), **tol(dtype))
    torch.testing.assert_close(k2.float(), k2r.float(), **tol(dtype))
    torch.testing.assert_close(v2.float(), v2r.float(), rtol=0, atol=0)
    ops.rope_inplace(q2, batch.positions, *cos_sin)
    REF.rope_inplace(q2r, batch.positions, *cos_sin)
    torch.testing.assert_close(q2.float(), q2r.float(), **tol(dtype))
    cache.k_pages.zero_(); ref_cache.k_pages.zero_()
    ops.kv_store(k2, v2, batch, table, cache)
    REF.kv_store(k2r, v2r, batch, table, ref_cache)
    torch.testing.assert_close(cache.k_pages.float(), ref_cache.k_pages.float(), **tol(dtype))


# the reference's rotary parity vector: 257 tokens, 16/8 heads of 128, positions below
# 4096, theta 1e6 (tests/test_kernel_parity.py:71-109 of the reference)
@pytest.mark.parametrize("dtype", DTYPES)
def test_rope_reference_shape(ops, gpu_device, dtype):
    hd, max_pos = 128, 4096
    angles = torch.outer(torch.arange(max_pos, dtype=torch.float32),
                         1.0 / (1e6 ** (torch.arange(0, hd, 2, dtype=torch.float32) / hd)))
    cos, sin = angles.cos().to(gpu_device), angles.sin().to(gpu_device)
    pos = torch.randint(0, max_pos, (257,), dtype=torch.int32, device=gpu_device)
    for heads in (16, 8):
        x = rand((257, heads, hd), dtype, gpu_device, 15 + heads)
        ref = x.clone()
        ops.rope_inplace(x, pos, cos, sin)
        REF.rope_inplace(ref, pos, cos, sin)
        t = tol(dtype) if dtype == torch.float32 else dict(rtol=1e-2, atol=2e-2)
        torch.testing.assert_close(x.float(), ref.float(), **t)


ATTN_SHAPES = [(4, 2, 16, 4), (8, 2, 32, 16), (6, 3, 48, 8), (16, 8, 128, 16), (5, 5, 80, 3),
               (8, 1, 64, 64), (4, 4, 256, 16), (14, 2, 112, 32), (32, 1, 64, 16),
               (40, 2, 32, 8), (3, 1, 96, 12)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [None, 7, 40])
@pytest.mark.parametrize("nq,nkv,hd,page", ATTN_SHAPES)
def test_paged_attention(ops, gpu_device, dtype, nq, nkv, hd, page, window):
    spans = [(0, 9), (70, 1), (5, 33), (130, 2), (0, 1), (63, 1), (64, 1), (65, 70)]
    batch, cache, table, _ = paged_scenario(gpu_device, dtype, nkv=nkv, hd=hd, page_size=page,
                                            spans=spans, seed=21)
    q = rand((batch.num_tokens, nq, hd), dtype, gpu_device, 22)
    kw = dict(num_heads=nq, num_kv_heads=nkv, head_dim=hd, scale=hd ** -0.5, window=window)
    out = ops.paged_attention(q, batch, table, cache, **kw)
    ref = REF.paged_attention(q, batch, table, cache, **kw)
    torch.testing.assert_close(out.float(), ref.float(), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [None, 300])
def test_paged_attention_long_contexts(ops, gpu_device, dtype, window):
    """Contexts of many key chunks: decode tokens beside a long portion, so both the
    walk over chunks and the split over waves with its merge are used."""
    nq, nkv, hd, page = 16, 8, 128, 16
    for spans in ([(1500, 1), (129, 1), (0, 1)], [(900, 200), (1030, 1)], [(2047, 1)] * 3):
        batch, cache, table, _ = paged_scenario(gpu_device, dtype, nkv=nkv, hd=hd,
                                                page_size=page, spans=spans, seed=31)
        q = rand((batch.num_tokens, nq, hd), dtype, gpu_device, 32)
        kw = dict(num_heads=nq, num_kv_heads=nkv, head_dim=hd, scale=hd ** -0.5, window=window)
        out = ops.paged_attention(q, batch, table, cache, **kw)
        # reference on a sample of tokens (the plain loop is slow)
        ref = REF.paged_attention(q, batch, table, cache, **kw) if batch.num_tokens < 20 else None
        if ref is None:
            pick = [0, 1, 57, 128, 199, 200]
            import copy
            sub = copy.copy(batch)
            sub.positions = batch.positions[pick].contiguous()
            sub.entry_of_token = batch.entry_of_token[pick].contiguous()
            ref = REF.paged_attention(q[pick].contiguous(), sub, table, cache, **kw)
            out = out[pick]
        torch.testing.assert_close(out.float(), ref.float(), **tol(dtype))


@pytest.mark.parametrize("window", [None, 100])
@pytest.mark.parametrize("nq,nkv,hd,page", [(16, 8, 128, 16), (8, 2, 64, 16), (6, 3, 48, 8),
                                            (4, 4, 256, 32), (32, 1, 32, 16), (6, 2, 64, 32),
                                            (10, 2, 32, 12), (40, 2, 32, 16), (3, 1, 128, 64)])
def test_paged_attention_long_portions(ops, gpu_device, nq, nkv, hd, page, window):
    """Portions long enough for the kernels in which a wavefront walks several query tiles
    (bfloat16; pages that are powers of two share blocks through LDS, others do not),
    with and without cached context before them, beside a decode token.  Groups of 3, 5
    and 20 heads: 16 rows are then not a whole number of tokens."""
    dtype = torch.bfloat16
    group = nq // nkv
    per_tile = 16 // min(group, 16)
    need = -(-2048 // (nkv * -(-group // 16))) * per_tile          # tokens for 2048 wave tiles
    spans = [(0, need // 2 + 188), (333, 1), (50, need // 2 + 3)]
    batch, cache, table, _ = paged_scenario(gpu_device, dtype, nkv=nkv, hd=hd, page_size=page,
                                            spans=spans, seed=33)
    assert ops._prefill_tiles(batch, nkv, group) is not None
    q = rand((batch.num_tokens, nq, hd), dtype, gpu_device, 34)
    kw = dict(num_heads=nq, num_kv_heads=nkv, head_dim=hd, scale=hd ** -0.5, window=window)
    out = ops.paged_attention(q, batch, table, cache, **kw)
    T, first = batch.num_tokens, spans[0][1]
    if T <= 3000:
        pick = list(range(T))
    else:       # the first tokens, both portions' ends and starts, and tile borders all over
        step = 4 * per_tile
        pick = sorted(set(list(range(0, 70)) + list(range(first - 40, first + 70)) +
                          list(range(T - 70, T)) +
                          [t + d for t in range(step * 7, T - step, step * 29)
                           for d in (-1, 0, 1, per_tile - 1, per_tile)]))
    import copy
    sub = copy.copy(batch)
    sub.positions = batch.positions[pick].contiguous()
    sub.entry_of_token = batch.entry_of_token[pick].contiguous()
    ref = REF.paged_attention(q[pick].contiguous(), sub, table, cache, **kw)
    torch.testing.assert_close(out[pick].float(), ref.float(), **tol(dtype))


@pytest.mark.parametrize("window", [40, 100, 333])
@pytest.mark.parametrize("spans,kernel", [
    ([(0, 1212), (333, 1), (50, 1027), (700, 700)], 2),     # many items: turns of 32 keys
    ([(0, 700), (333, 1), (50, 500), (700, 300)], 2),       # few items: turns of 64, two sets
    ([(0, 1212), (333, 1), (50, 1027), (700, 700)], 3),     # turns of 64, eight tiles an item
], ids=["turns-of-32", "two-sets", "eight-tiles"])
def test_long_portions_under_a_window_come_out_the_same_every_time(ops, gpu_device, window, spans,
                                                                   kernel):
    """Under a window the waves of a workgroup have different blocks to skip, so some run a
    turn ahead of the others; a block sent for into a buffer that a slower wave still reads
    would show as a result that differs from launch to launch.  Each of the three kernels
    for long portions of this head size."""
    dtype, nq, nkv, hd, page = torch.bfloat16, 16, 8, 128, 16
    batch, cache, table, _ = paged_scenario(gpu_device, dtype, nkv=nkv, hd=hd, page_size=page,
                                            spans=spans, seed=35)
    assert ops._prefill_tiles(batch, nkv, nq // nkv) is not None
    q = rand((batch.num_tokens, nq, hd), dtype, gpu_device, 36)
    kw = dict(num_heads=nq, num_kv_heads=nkv, head_dim=hd, scale=hd ** -0.5, window=window)
    ops.lib.ts_attention_prefill_variant(kernel)
    try:
        first = ops.paged_attention(q, batch, table, cache, **kw).clone()
        ref = REF.paged_attention(q, batch, table, cache, **kw)
        torch.testing.assert_close(first.float(), ref.float(), **tol(dtype))
        for _ in range(30):
            assert torch.equal(ops.paged_attention(q, batch, table, cache, **kw), first)
    finally:
        ops.lib.ts_attention_prefill_variant(2)


DECODE_SPANS = [(0, 1), (1, 1), (31, 1), (32, 1), (127, 1), (128, 1), (129, 1), (255, 1),
                (256, 1), (700, 1), (1023, 1)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [None, 40, 300])
@pytest.mark.parametrize("nq,nkv,hd,page", ATTN_SHAPES + [(16, 8, 128, 32), (8, 8, 64, 128),
                                                          (6, 2, 160, 16), (20, 1, 32, 16)])
def test_attend_in_a_decode_step(ops, gpu_device, dtype, nq, nkv, hd, page, window):
    attend_decode_case(ops, gpu_device, dtype, nq, nkv, hd, page, window, DECODE_SPANS)


@pytest.mark.parametrize("window", [None, 300])
def test_attend_in_a_large_decode_step(ops, gpu_device, window):
    """Enough entries that a tile's keys are not split over workgroups, and more than the
    decode kernel takes at all."""
    assert ops._decode_splits(8 * 3 * len(DECODE_SPANS), 1024) == 1
    attend_decode_case(ops, gpu_device, torch.bfloat16, 16, 8, 128, 16, window, DECODE_SPANS * 3)
    attend_decode_case(ops, gpu_device, torch.bfloat16, 16, 8, 128, 16, window, DECODE_SPANS * 7)
    # and so many that the kernel for long portions takes the single tokens as its items
    many = DECODE_SPANS * 13
    batch, _, _, _ = paged_scenario(gpu_device, torch.bfloat16, nkv=8, hd=128, page_size=16,
                                    spans=many, seed=51, fill=False)
    assert ops._prefill_tiles(batch, 8, 2) is not None
    attend_decode_case(ops, gpu_device, torch.bfloat16, 16, 8, 128, 16, window, many)


def attend_decode_case(ops, gpu_device, dtype, nq, nkv, hd, page, window, spans):
    """One new token per entry: norm, rotation, cache write and attention in one call (in
    bfloat16 with a head size in steps of 32 and a power-of-two page: one kernel).  The
    new key's slot holds garbage before the call, so a kernel that reads it instead of
    using the step's own key shows."""
    batch, cache, table, _ = paged_scenario(gpu_device, dtype, nkv=nkv, hd=hd, page_size=page,
                                            spans=spans, seed=51)
    T = batch.num_tokens
    wq = 1 + 0.1 * rand((hd,), torch.float32, gpu_device, 53)
    wk = 1 + 0.1 * rand((hd,), torch.float32, gpu_device, 54)
    angles = torch.outer(torch.arange(1100, dtype=torch.float32),
                         1.0 / (10000.0 ** (torch.arange(0, hd, 2, dtype=torch.float32) / hd)))
    cos_sin = (angles.cos().to(gpu_device), angles.sin().to(gpu_device))
    for b, (start, _) in enumerate(spans):               # poison the slots to be written
        phys = int(table[b, start // page])
        cache.k_pages[phys, :, start % page] = 1e4
        cache.v_pages[phys, :, :, start % page] = -1e4
    for kv_in_row, norm, rot in ((nkv, True, True), (nkv, False, True), (nkv, True, False),
                                 (0, True, True)):
        qkv = rand((T, (nq + 2 * kv_in_row) * hd), dtype, gpu_device, 52)
        mine = type(cache)(cache.group, cache.page_size, cache.num_pages,
                           cache.k_pages.clone(), cache.v_pages.clone())
        theirs = type(cache)(cache.group, cache.page_size, cache.num_pages,
                             cache.k_pages.clone(), cache.v_pages.clone())
        if not kv_in_row:   # a run that reads another run's cache: the keys are there
            for c in (mine, theirs):
                c.k_pages.clamp_(-3, 3); c.v_pages.clamp_(-3, 3)
        kw = dict(num_heads=nq, num_kv_heads=nkv, kv_in_row=kv_in_row, head_dim=hd,
                  q_weight=wq if norm else None, k_weight=wk if norm else None, eps=1e-5,
                  cos_sin=cos_sin if rot else None, scale=hd ** -0.5, window=window)
        out = ops.attend(qkv, batch, table, mine, bool(kv_in_row), **kw)
        ref = REF.attend(qkv, batch, table, theirs, bool(kv_in_row), **kw)
        torch.testing.assert_close(mine.k_pages.float(), theirs.k_pages.float(), **tol(dtype))
        torch.testing.assert_close(mine.v_pages.float(), theirs.v_pages.float(), rtol=0, atol=0)
        torch.testing.assert_close(out.float(), ref.float(), **tol(dtype))


@pytest.mark.parametrize("nq,nkv,hd,spans", [
    (16, 8, 128, [(5000, 1), (2047, 1), (3, 1), (2049, 1), (130, 1)]),
    (32, 8, 128, [(900, 1)] * 7), (64, 8, 128, [(4000, 1), (129, 1)]),
    (12, 2, 64, [(3000, 1), (0, 1), (257, 1)]), (40, 1, 96, [(1500, 1), (700, 1)]),
    (6, 3, 48, [(2100, 1), (127, 1), (640, 1)]), (10, 2, 80, [(900, 1), (1300, 1)]),
    (4, 4, 256, [(1000, 1), (130, 1)])])
@pytest.mark.parametrize("window", [None, 1000])
def test_decode_kernel_merges_its_key_splits_as_the_merge_kernel_does(ops, gpu_device, monkeypatch,
                                                                      nq, nkv, hd, spans, window):
    """The workgroup of an item that finishes last merges the item's key splits; the result
    is, bit for bit, the merge kernel's, time after time (the arrival counts are left at
    zero), with splits that hold no keys beside full ones."""
    dtype, page = torch.bfloat16, 16
    batch, cache, table, _ = paged_scenario(gpu_device, dtype, nkv=nkv, hd=hd, page_size=page,
                                            spans=spans, seed=71)
    assert ops._decode_splits(len(spans) * nkv * -(-(nq // nkv) // 16), batch.max_ctx_len) > 1
    qkv = rand((batch.num_tokens, (nq + 2 * nkv) * hd), dtype, gpu_device, 72)
    wq = 1 + 0.1 * rand((hd,), torch.float32, gpu_device, 73)
    angles = torch.outer(torch.arange(5100, dtype=torch.float32),
                         1.0 / (1e6 ** (torch.arange(0, hd, 2, dtype=torch.float32) / hd)))
    cos_sin = (angles.cos().to(gpu_device), angles.sin().to(gpu_device))
    kw = dict(num_heads=nq, num_kv_heads=nkv, head_dim=hd, q_weight=wq, k_weight=wq, eps=1e-6,
              cos_sin=cos_sin, scale=hd ** -0.5, window=window, kv_in_row=nkv)
    assert ops.fold_merge
    folded = [ops.attend(qkv, batch, table, cache, True, **kw).clone() for _ in range(3)]
    assert int(ops._arrivals.abs().sum()) == 0
    monkeypatch.setattr(ops, "fold_merge", False)
    apart = ops.attend(qkv, batch, table, cache, True, **kw)
    for out in folded:
        assert torch.equal(out, apart)


def test_decode_kernel_merge_over_hundreds_of_launches(ops, gpu_device, monkeypatch):
    """The in-kernel merge rests on an order of memory operations (partial results by
    device-scope stores that each wave waits for, then the count; the last workgroup reads
    them back by device-scope loads).  Hundreds of launches back to back over many items
    (up to 16 entries x 8 heads, two to ten splits each, contexts that change from launch to
    launch), with other kernels' traffic between them, each compared bit for bit with the
    merge kernel's result; stops at the first launch that differs."""
    dtype, page, nq, nkv, hd = torch.bfloat16, 16, 16, 8, 128
    g = torch.Generator().manual_seed(5)
    cases = []
    for n in (3, 16, 9):
        spans = [(int(torch.randint(130, 3000, (1,), generator=g)), 1) for _ in range(n)]
        batch, cache, table, _ = paged_scenario(gpu_device, dtype, nkv=nkv, hd=hd,
                                                page_size=page, spans=spans, seed=90 + n)
        assert ops._decode_splits(n * nkv, batch.max_ctx_len) > 1
        qkv = rand((batch.num_tokens, (nq + 2 * nkv) * hd), dtype, gpu_device, 91 + n)
        cases.append((batch, cache, table, qkv))
    wq = 1 + 0.1 * rand((hd,), torch.float32, gpu_device, 73)
    angles = torch.outer(torch.arange(3100, dtype=torch.float32),
                         1.0 / (1e6 ** (torch.arange(0, hd, 2, dtype=torch.float32) / hd)))
    cos_sin = (angles.cos().to(gpu_device), angles.sin().to(gpu_device))
    kw = dict(num_heads=nq, num_kv_heads=nkv, head_dim=hd, q_weight=wq, k_weight=wq, eps=1e-6,
              cos_sin=cos_sin, scale=hd ** -0.5, window=None, kv_in_row=nkv)
    monkeypatch.setattr(ops, "fold_merge", False)
    apart = [ops.attend(qkv, batch, table, cache, True, **kw).clone()
             for batch, cache, table, qkv in cases]
    monkeypatch.setattr(ops, "fold_merge", True)
    filler = rand((4096, 4096), torch.float32, gpu_device, 7)
    outs = []
    for launch in range(240):
        batch, cache, table, qkv = cases[launch % 3]
        outs.append(ops.attend(qkv, batch, table, cache, True, **kw))
        if launch % 4 == 0:
            filler.mul_(1.0)                   # other traffic through the caches
        if launch % 40 == 39:                  # compared in groups: the launches stay back to back
            for k, out in enumerate(outs):
                assert torch.equal(out, apart[(launch - 39 + k) % 3]), \
                    f"launch {launch - 39 + k} differs from the merge kernel's result"
            outs.clear()
    assert int(ops._arrivals.abs().sum()) == 0
    # counts left behind by a launch that did not finish would make later merges wrong:
    # `reset_scratch` (after every failed call, before warm-up and capture) clears them
    ops._arrivals[:5] = 3
    ops.reset_scratch()
    assert int(ops._arrivals.abs().sum()) == 0
    batch, cache, table, qkv = cases[1]
    assert torch.equal(ops.attend(qkv, batch, table, cache, True, **kw), apart[1])


@pytest.mark.parametrize("window", [None, 1000])
@pytest.mark.parametrize("fused", [True, False])
def test_attend_decode_long_contexts_split_and_merge(ops, gpu_device, window, fused):
    """Contexts long enough that a decode step's keys are split over workgroups and merged,
    beside short ones whose later splits are empty."""
    dtype = torch.bfloat16
    nq, nkv, hd, page = 16, 8, 128, 16
    spans = [(5000, 1), (2047, 1), (3, 1), (2049, 1)]
    batch, cache, table, _ = paged_scenario(gpu_device, dtype, nkv=nkv, hd=hd, page_size=page,
                                            spans=spans, seed=61)
    assert ops._decode_splits(len(spans) * nkv, batch.max_ctx_len) > 3
    T = batch.num_tokens
    qkv = rand((T, (nq + 2 * nkv) * hd), dtype, gpu_device, 62)
    wq = 1 + 0.1 * rand((hd,), torch.float32, gpu_device, 63)
    angles = torch.outer(torch.arange(5100, dtype=torch.float32),
                         1.0 / (1e6 ** (torch.arange(0, hd, 2, dtype=torch.float32) / hd)))
    cos_sin = (angles.cos().to(gpu_device), angles.sin().to(gpu_device))
    theirs = type(cache)(cache.group, cache.page_size, cache.num_pages,
                         cache.k_pages.clone(), cache.v_pages.clone())
    kw = dict(num_heads=nq, num_kv_heads=nkv, head_dim=hd, q_weight=wq, k_weight=wq, eps=1e-6,
              cos_sin=cos_sin)
    akw = dict(num_heads=nq, num_kv_heads=nkv, head_dim=hd, scale=hd ** -0.5, window=window)
    ref = REF.attend(qkv, batch, table, theirs, True, kv_in_row=nkv, **kw,
                     scale=hd ** -0.5, window=window)
    if fused:
        out = ops.attend(qkv, batch, table, cache, True, kv_in_row=nkv, **kw,
                         scale=hd ** -0.5, window=window)
    else:
        q = ops.qk_norm_rope_store(qkv, batch, table, cache, **kw)
        out = ops.paged_attention(q, batch, table, cache, **akw)
    torch.testing.assert_close(cache.k_pages.float(), theirs.k_pages.float(), **tol(dtype))
    torch.testing.assert_close(out.float(), ref.float(), **tol(dtype))


@pytest.mark.parametrize("window", [None, 1000])
@pytest.mark.parametrize("nq,nkv,hd,hidden,spans", [
    (16, 8, 128, 1024, [(5000, 1), (2047, 1), (3, 1), (2049, 1)]),
    (16, 8, 128, 1024, [(777, 1)]),
    (32, 8, 128, 4096, [(3000, 1), (129, 1), (4100, 1), (0, 1), (640, 1), (2500, 1), (77, 1),
                        (1024, 1)]),
    (16, 8, 128, 1024, [(3000, 1), (129, 1), (4100, 1), (0, 1), (640, 1), (2500, 1), (77, 1),
                        (1024, 1), (900, 1), (31, 1), (4000, 1)]),
    (40, 2, 64, 520, [(1500, 1), (300, 1)]),
])
def test_output_projection_merges_the_key_splits_itself(ops, gpu_device, monkeypatch, nq, nkv, hd,
                                                        hidden, spans, window):
    """A decode step whose keys are split over workgroups: with the merge deferred, the
    output projection in its tail form merges the partial results as it loads its rows.
    Stream, prepared rows and sums of squares must be, bit for bit, what the merge kernel
    followed by the tail form leaves; and a deferred merge that another call meets (a
    plain product here) is run before that call."""
    from tokensprint_amd.kernels.stream import NormHint, UnmergedRows
    dtype, page = torch.bfloat16, 16
    batch, cache, table, _ = paged_scenario(gpu_device, dtype, nkv=nkv, hd=hd, page_size=page,
                                            spans=spans, seed=81)
    T = batch.num_tokens
    group = nq // nkv
    assert ops._decode_splits(T * nkv * -(-group // 16), batch.max_ctx_len) > 1
    qkv = rand((T, (nq + 2 * nkv) * hd), dtype, gpu_device, 82)
    wq = 1 + 0.1 * rand((hd,), torch.float32, gpu_device, 83)
    angles = torch.outer(torch.arange(5100, dtype=torch.float32),
                         1.0 / (1e6 ** (torch.arange(0, hd, 2, dtype=torch.float32) / hd)))
    cos_sin = (angles.cos().to(gpu_device), angles.sin().to(gpu_device))
    kw = dict(num_heads=nq, num_kv_heads=nkv, kv_in_row=nkv, head_dim=hd, q_weight=wq,
              k_weight=wq, eps=1e-6, cos_sin=cos_sin, scale=hd ** -0.5, window=window)
    w_o = rand((hidden, nq * hd), dtype, gpu_device, 84, scale=0.05)
    norm_w = 1 + 0.1 * rand((hidden,), torch.float32, gpu_device, 85)
    w_next = rand((2 * 96, hidden), dtype, gpu_device, 86, scale=0.05)
    hint = NormHint(norm_w, 1e-6, w_next, True)
    resid0 = rand((T, hidden), torch.float32, gpu_device, 87)

    # (the provider defers only up to the few rows for which it pays; here every size)
    monkeypatch.setattr(ops, "merged_rows", 16)

    def run(defer):
        mine = type(cache)(cache.group, cache.page_size, cache.num_pages,
                           cache.k_pages.clone(), cache.v_pages.clone())
        o = ops.attend(qkv, batch, table, mine, True, defer_merge=defer, **kw).view(T, nq * hd)
        assert isinstance(o, UnmergedRows) == defer and tuple(o.shape) == (T, nq * hd)
        resid = resid0.clone()
        prepared = ops.linear_into_stream(o, w_o, resid, hint)
        if defer:
            assert not o.is_merged          # the product's kernel merged the rows itself
        return o, resid, prepared

    o_ref, resid_ref, prep_ref = run(False)
    o_new, resid_new, prep_new = run(True)
    assert prep_ref is not None and prep_new is not None
    assert torch.equal(resid_new, resid_ref)
    assert torch.equal(prep_new.rows, prep_ref.rows)
    assert prep_new.slices == prep_ref.slices
    assert torch.equal(prep_new.sumsq[:, :prep_new.slices], prep_ref.sumsq[:, :prep_ref.slices])
    # deferred, then met by another call: merged first, the same attention output
    mine = type(cache)(cache.group, cache.page_size, cache.num_pages,
                       cache.k_pages.clone(), cache.v_pages.clone())
    o = ops.attend(qkv, batch, table, mine, True, defer_merge=True, **kw).view(T, nq * hd)
    y = ops.linear(o, w_o, dtype)
    assert o.is_merged
    assert torch.equal(o.merged(), o_ref)
    assert torch.equal(y, ops.linear(o_ref, w_o, dtype))
    # the handle is no tensor: code that is not this provider's cannot read unmerged rows
    o = ops.attend(qkv, batch, table, mine, True, defer_merge=True, **kw)
    with pytest.raises(TypeError):
        torch.matmul(o, w_o.T)
    with pytest.raises(TypeError, match="unmerged"):
        ops.silu_mul(o.view(T, nq * hd))
    assert torch.equal(o.view(T, nq * hd).merged(), o_ref)


@pytest.mark.parametrize("dtype", DTYPES)
def test_paged_attention_finds_one_far_key(ops, gpu_device, dtype):
    """One key among hundreds, at a page's edge, is made to dominate: the output must be
    its value row.  A kernel that skips a tile, a page or the last key of a page fails."""
    nq, nkv, hd, page = 4, 2, 64, 16
    for far in (0, 15, 16, 255, 256, 511, 700):
        batch, cache, table, _ = paged_scenario(gpu_device, dtype, nkv=nkv, hd=hd, page_size=page,
                                                spans=[(700, 1)], seed=23)
        q = rand((1, nq, hd), dtype, gpu_device, 24)
        phys = int(table[0, far // page])
        for kvh in range(nkv):
            # key = 4 * q of the first head of the group: score is far above the others
            cache.k_pages[phys, kvh, far % page] = (4.0 * q[0, kvh * 2]).to(dtype)
        out = ops.paged_attention(q, batch, table, cache, num_heads=nq, num_kv_heads=nkv,
                                  head_dim=hd, scale=1.0, window=None)
        for kvh in range(nkv):
            torch.testing.assert_close(out[0, kvh * 2].float(),
                                       cache.v_pages[phys, kvh, :, far % page].float(),
                                       rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("nq,nkv,hd,page,window", [(16, 8, 128, 16, None), (16, 8, 128, 64, 700),
                                                   (8, 8, 96, 16, None), (6, 2, 64, 32, None),
                                                   (40, 2, 32, 16, 300)])
@pytest.mark.parametrize("kernel", [2, 0, 3], ids=["default", "turns-of-32", "eight-tiles"])
def test_attend_long_portions(ops, gpu_device, nq, nkv, hd, page, window, kernel):
    """Portions of prompts long enough for the kernels in which a wavefront walks several
    query tiles: with and without norm weights, rotation, and keys in the row; groups of
    3 and 20 heads, whose 16 rows are not a whole number of tokens (a row past a tile's
    tokens must not be computed with that tile's key range and stored).  Head sizes 64 and
    128 have three kernels for this (turns of 64 keys with two sets of waves an item, with
    eight tiles an item, and turns of 32 keys), chosen by the number of items: each is
    made to take the same step."""
    if kernel != 2 and hd not in (64, 128):
        pytest.skip("one kernel for this head size")
    ops.lib.ts_attention_prefill_variant(kernel)
    try:
        _attend_long_portions(ops, gpu_device, nq, nkv, hd, page, window)
    finally:
        ops.lib.ts_attention_prefill_variant(2)


def _attend_long_portions(ops, gpu_device, nq, nkv, hd, page, window):
    dtype = torch.bfloat16
    group = nq // nkv
    per_tile = 16 // min(group, 16)
    need = -(-2048 // (nkv * -(-group // 16))) * per_tile          # tokens for 2048 wave tiles
    spans = [(0, need // 2 + 37), (300, need // 2 + 100), (17, 150)]
    batch, cache, table, _ = paged_scenario(gpu_device, dtype, nkv=nkv, hd=hd, page_size=page,
                                            spans=spans, seed=71)
    tiles16 = sum(-(-n // per_tile) for _, n in spans)
    assert tiles16 * nkv * -(-group // 16) >= 2048
    T = batch.num_tokens
    wq = 1 + 0.1 * rand((hd,), torch.float32, gpu_device, 73)
    wk = 1 + 0.1 * rand((hd,), torch.float32, gpu_device, 74)
    angles = torch.outer(torch.arange(batch.max_ctx_len + 8, dtype=torch.float32),
                         1.0 / (10000.0 ** (torch.arange(0, hd, 2, dtype=torch.float32) / hd)))
    cos_sin = (angles.cos().to(gpu_device), angles.sin().to(gpu_device))
    variants = [(nkv, True, True), (0, True, True)]
    if (nq, hd) == (16, 128):
        variants += [(nkv, False, True), (nkv, True, False)]
    for kv_in_row, norm, rot in variants:
        qkv = rand((T, (nq + 2 * kv_in_row) * hd), dtype, gpu_device, 72)
        mine = type(cache)(cache.group, cache.page_size, cache.num_pages,
                           cache.k_pages.clone(), cache.v_pages.clone())
        theirs = type(cache)(cache.group, cache.page_size, cache.num_pages,
                             cache.k_pages.clone(), cache.v_pages.clone())
        kw = dict(num_heads=nq, num_kv_heads=nkv, kv_in_row=kv_in_row, head_dim=hd,
                  q_weight=wq if norm else None, k_weight=wk if norm else None, eps=1e-6,
                  cos_sin=cos_sin if rot else None, scale=hd ** -0.5, window=window)
        out = ops.attend(qkv, batch, table, mine, bool(kv_in_row), **kw)
        ref = REF.attend(qkv, batch, table, theirs, bool(kv_in_row), **kw)
        torch.testing.assert_close(mine.k_pages.float(), theirs.k_pages.float(), **tol(dtype))
        torch.testing.assert_close(mine.v_pages.float(), theirs.v_pages.float(), **tol(dtype))
        torch.testing.assert_close(out.float(), ref.float(), **tol(dtype))


@pytest.mark.parametrize("page", [16, 64])
@pytest.mark.parametrize("kernel", [2, 0, 3], ids=["default", "turns-of-32", "eight-tiles"])
def test_long_portion_finds_one_far_key(ops, gpu_device, kernel, page):
    """Random keys would hide a block that a kernel for long portions skips, reads from the
    wrong page or masks by mistake: among two thousand keys one more changes a bfloat16
    result by less than the tolerance.  Here one key at a time, at the edges of pages, of
    32-key sub-blocks, of 64-key turns and of the sets' alternating turns, is made to
    dominate every later query's scores: rows from that position on must return its value
    row, rows before it must not."""
    dtype = torch.bfloat16
    nq, nkv, hd, S = 16, 8, 128, 1100          # 1100 tokens: 552 tiles of 16 rows, 4,416 wave tiles
    batch, cache, table, _ = paged_scenario(gpu_device, dtype, nkv=nkv, hd=hd, page_size=page,
                                            spans=[(0, S)], seed=31)
    assert ops._prefill_tiles(batch, nkv, nq // nkv) is not None
    q = rand((S, nq, hd), dtype, gpu_device, 32)
    direction = rand((hd,), torch.float32, gpu_device, 33)
    direction = direction / direction.norm()
    # every query gets a large component along one direction; a key that is 6 x that
    # direction scores about 6 * 8 above the rest (scale 1)
    q = (q.float() * 0.2 + 8.0 * direction).to(dtype)
    ops.lib.ts_attention_prefill_variant(kernel)
    try:
        for far in (0, 15, 16, 31, 32, 63, 64, 65, 127, 128, 191, 192, 511, 512, 1023, 1024, 1087, 1099):
            k_pages = cache.k_pages.clone()
            phys = int(table[0, far // page])
            k_pages[phys, :, far % page] = (6.0 * direction).to(dtype)
            mine = type(cache)(cache.group, cache.page_size, cache.num_pages, k_pages, cache.v_pages)
            out = ops.paged_attention(q, batch, table, mine, num_heads=nq, num_kv_heads=nkv,
                                      head_dim=hd, scale=1.0, window=None).float()
            want = cache.v_pages[phys, :, :, far % page].float()           # [nkv, hd]
            want = want.repeat_interleave(nq // nkv, dim=0)                # [nq, hd]
            later = out[far:]                                               # rows that see the key
            assert (later - want).abs().max() < 3e-2, f"key {far}: {(later - want).abs().max():.3f}"
            if far:
                earlier = out[:far]
                assert (earlier - want).abs().max() > 0.3, f"key {far} shows to rows before it"
    finally:
        ops.lib.ts_attention_prefill_variant(2)


@pytest.mark.parametrize("ctx", [700, 2500])
def test_attend_finds_one_far_key_in_a_decode_step(ops, gpu_device, ctx):
    """The same through the fused decode call (no norm, no rotation, so the query is the
    row's own): one key at a page's, a block's or a split's edge dominates, or the step's
    own key does, which is not in the cache when the walk starts."""
    dtype = torch.bfloat16
    nq, nkv, hd, page = 4, 2, 128, 16
    kw = dict(num_heads=nq, num_kv_heads=nkv, kv_in_row=nkv, head_dim=hd, q_weight=None,
              k_weight=None, eps=0.0, cos_sin=None, scale=1.0, window=None)
    for far in (0, 15, 16, 31, 32, 127, 128, 255, 256, 511, 512, ctx - 2, ctx - 1, ctx):
        batch, cache, table, _ = paged_scenario(gpu_device, dtype, nkv=nkv, hd=hd, page_size=page,
                                                spans=[(ctx, 1)], seed=23)
        qkv = rand((1, (nq + 2 * nkv) * hd), dtype, gpu_device, 24)
        row = qkv.view(nq + 2 * nkv, hd)
        if far == ctx:       # the step's own key: 4 * q of the first head of its group
            for kvh in range(nkv):
                row[nq + kvh] = (4.0 * row[kvh * 2].float()).to(dtype)
            want = [row[nq + nkv + kvh].float() for kvh in range(nkv)]
        else:
            phys = int(table[0, far // page])
            for kvh in range(nkv):
                cache.k_pages[phys, kvh, far % page] = (4.0 * row[kvh * 2].float()).to(dtype)
            want = [cache.v_pages[phys, kvh, :, far % page].float() for kvh in range(nkv)]
        out = ops.attend(qkv, batch, table, cache, True, **kw).view(1, nq, hd)
        for kvh in range(nkv):
            torch.testing.assert_close(out[0, kvh * 2].float(), want[kvh], rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("lo", [512, 528, 544, 531, 700])
def test_window_edge_in_a_decode_step(ops, gpu_device, dtype, lo):
    """A window's lower edge, with a key made to dominate on either side of it: the key
    at p-W+1 must be found (the output is its value row) and the key at p-W ignored.  The
    edge is put on a 128-key chunk's, a page's and a 32-key block's first key, inside a
    block, and on the step's own key (W = 1).  With random keys alone one key more or
    less moves a row by about 1/W, which a tolerance hides."""
    nq, nkv, hd, page, ctx = 4, 2, 128, 16, 700
    W = ctx + 1 - lo                       # the query is at position ctx
    kw = dict(num_heads=nq, num_kv_heads=nkv, kv_in_row=nkv, head_dim=hd, q_weight=None,
              k_weight=None, eps=0.0, cos_sin=None, scale=1.0, window=W)
    for planted in (lo - 1, lo):
        batch, cache, table, _ = paged_scenario(gpu_device, dtype, nkv=nkv, hd=hd, page_size=page,
                                                spans=[(ctx, 1)], seed=23)
        qkv = rand((1, (nq + 2 * nkv) * hd), dtype, gpu_device, 24)
        row = qkv.view(nq + 2 * nkv, hd)
        if planted == ctx:                 # the step's own key
            for kvh in range(nkv):
                row[nq + kvh] = (4.0 * row[kvh * 2].float()).to(dtype)
            value = [row[nq + nkv + kvh].float() for kvh in range(nkv)]
        else:
            phys = int(table[0, planted // page])
            for kvh in range(nkv):
                cache.k_pages[phys, kvh, planted % page] = (4.0 * row[kvh * 2].float()).to(dtype)
            value = [cache.v_pages[phys, kvh, :, planted % page].float() for kvh in range(nkv)]
        theirs = type(cache)(cache.group, cache.page_size, cache.num_pages,
                             cache.k_pages.clone(), cache.v_pages.clone())
        out = ops.attend(qkv, batch, table, cache, True, **kw).view(1, nq, hd).float()
        ref = REF.attend(qkv, batch, table, theirs, True, **kw).view(1, nq, hd).float()
        torch.testing.assert_close(out, ref, rtol=2e-2, atol=2e-2)
        for kvh in range(nkv):
            if planted == lo:
                torch.testing.assert_close(out[0, kvh * 2], value[kvh], rtol=2e-2, atol=2e-2)
            else:
                assert (out[0, kvh * 2] - value[kvh]).abs().max() > 0.5


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("start,n,picks", [(683, 2, [0]), (619, 2, [0]), (603, 2, [0]), (601, 2, [0]),
                                           (600, 2200, [0, 3, 19, 83, 1000, 2198])])
def test_window_edge_in_portions(ops, gpu_device, dtype, start, n, picks):
    """The same for portions of prompts, through `paged_attention`: two tokens (each query
    has an edge of its own, one key apart) and a portion long enough for the kernels in
    which a wavefront walks several query tiles.  For a picked query at position p the
    key at p-W+1, its window's first, is aligned with the first head of each group, and
    the next token gets the same query vector: the picked query's output is that key's
    value row, the next token's, one position on, is not; both equal the plain reference.
    The edges fall on a chunk's, a block's and a page's first key and between."""
    nq, nkv, hd, page, W = 16, 8, 128, 16, 300
    if dtype == torch.float32 and n > 2:
        pytest.skip("the long-portion kernels are bfloat16 only; float32 takes the general one")
    batch, cache, table, _ = paged_scenario(gpu_device, dtype, nkv=nkv, hd=hd, page_size=page,
                                            spans=[(start, n)], seed=31)
    q = rand((n, nq, hd), dtype, gpu_device, 32)
    group = nq // nkv
    value = {}
    for i in picks:
        where = start + i - W + 1
        q[i + 1] = q[i]
        phys = int(table[0, where // page])
        for kvh in range(nkv):
            cache.k_pages[phys, kvh, where % page] = (4.0 * q[i, kvh * group].float()).to(dtype)
            value[(i, kvh * group)] = cache.v_pages[phys, kvh, :, where % page].float()
    kw = dict(num_heads=nq, num_kv_heads=nkv, head_dim=hd, scale=1.0, window=W)
    out = ops.paged_attention(q, batch, table, cache, **kw).float()
    rows = sorted(picks + [i + 1 for i in picks])
    ref = REF.paged_attention(q, batch, table, cache, only=rows, **kw).float()
    torch.testing.assert_close(out[rows], ref[rows], rtol=2e-2, atol=2e-2)
    for (i, head), row in value.items():
        torch.testing.assert_close(out[i, head], row, rtol=2e-2, atol=2e-2)
        assert (out[i + 1, head] - row).abs().max() > 0.5, (i, head)


def test_argmax_and_ties(ops, gpu_device):
    logits = rand((9, 151936), torch.float32, gpu_device, 30)
    assert torch.equal(ops.argmax(logits).long(), logits.argmax(-1))
    logits = torch.zeros(3, 389, device=gpu_device)
    logits[0, 17] = logits[0, 300] = 2.0
    logits[1, 388] = 1.0
    assert ops.argmax(logits).tolist() == [17, 388, 0]


def test_sample_is_keyed_and_follows_the_distribution(ops, gpu_device):
    vocab = 11
    logits = torch.linspace(-2, 2, vocab, device=gpu_device).repeat(4000, 1).contiguous()
    temps = torch.full((4000,), 0.7, device=gpu_device)
    keys = torch.arange(4000, dtype=torch.int64, device=gpu_device) * 7919 + 5
    a = ops.sample(logits, temps, keys)
    # same key, other batch: same token
    b = ops.sample(logits[100:200].contiguous(), temps[100:200].contiguous(),
                   keys[100:200].contiguous())
    assert torch.equal(a[100:200], b)
    freq = torch.bincount(a.long(), minlength=vocab).float() / 4000
    probs = torch.softmax(logits[0] / 0.7, -1)
    assert (freq - probs).abs().max() < 0.03
    # temperature 0 rows are greedy
    temps[:10] = 0.0
    assert (ops.sample(logits, temps, keys)[:10] == vocab - 1).all()
