"""GPU dequant-GEMV / dequant-GEMM against the CPU oracle.

Parity is judged on the fp32-output variant of each kernel (same accumulation,
final cast skipped) against an fp64 evaluation of the oracle, with the north-star
tolerances max-abs <= 1e-2 and relative Frobenius <= 2e-3.  The bf16 output is
checked separately: it must be the round-to-nearest-even of the kernel's own fp32
result, lie within half a bf16 ulp (plus the fp32 error just measured) of the
oracle's fp64 value, and be inside the Frobenius bound.  (An output of magnitude
>= 2 has a bf16 ulp of 2^-6 > 1e-2, so max-abs <= 1e-2 cannot be asked of any bf16
output, the oracle's own included.)
"""

import numpy as np
import pytest
import torch

from oracle import qspec
from tests.helpers import MAX_ABS_TOL, REL_FRO_TOL, bf16_rounding_excess, errors, make_activations, make_weight

pytestmark = pytest.mark.gpu

_cache: dict = {}


def _quantized(scheme: str, n: int, k: int, seed: int, cuda):
    """(oracle dequantized weight fp64 on CPU, private GPU tensors) for one seeded weight."""
    key = (scheme, n, k, seed)
    if key not in _cache:
        from ajllm_amd import repack_w4, repack_w8

        w = make_weight(n, k, seed).numpy()
        if scheme == "w4":
            q, s, z = qspec.quantize_w4_g128(w)
            qw = qspec.pack_int4(q)
            w_hat = torch.from_numpy(qspec.dequantize_w4(qw, s, z))
            wq, meta = repack_w4(torch.from_numpy(qw).to(cuda), torch.from_numpy(s).to(cuda), torch.from_numpy(z).to(cuda))
        else:
            q, s = qspec.quantize_w8(w)
            w_hat = torch.from_numpy(qspec.dequantize_w8(q, s))
            wq, meta = repack_w8(torch.from_numpy(q).to(cuda)), torch.from_numpy(s).to(cuda)
        _cache.clear()  # keep one weight resident at a time
        _cache[key] = (w_hat, wq, meta)
    return _cache[key]


def _run(scheme, x, wq, meta, out_dtype, kernel):
    from ajllm_amd import w4a16_matmul, w8a16_matmul

    fn = w4a16_matmul if scheme == "w4" else w8a16_matmul
    return fn(x, wq, meta, out_dtype, kernel=kernel)


def _check(scheme, kernel, m, n, k, seed, cuda, outliers=False, max_rows=None):
    w_hat, wq, meta = _quantized(scheme, n, k, seed, cuda)
    x = make_activations(m, k, seed + 100, outliers)
    xg = x.to(cuda)
    y32 = _run(scheme, xg, wq, meta, torch.float32, kernel)
    y16 = _run(scheme, xg, wq, meta, torch.bfloat16, kernel)
    torch.cuda.synchronize()
    assert y32.shape == (m, n) and y16.shape == (m, n)
    rows = torch.arange(m)
    if max_rows is not None and m > max_rows:
        rows = torch.randperm(m, generator=torch.Generator().manual_seed(seed))[:max_rows].sort().values
    want64 = qspec.quant_linear(x[rows], w_hat, accumulate=torch.float64, out_dtype=torch.float64)
    max_abs, rel_fro = errors(y32.cpu()[rows], want64)
    assert max_abs <= MAX_ABS_TOL and rel_fro <= REL_FRO_TOL, (max_abs, rel_fro)
    # the kernel's fp32 result is far inside the tolerance: fp32 accumulation noise only
    assert max_abs <= 2e-3, max_abs
    got16 = y16.cpu()[rows]
    assert bf16_rounding_excess(got16, want64, max_abs) <= 0
    assert errors(got16, want64)[1] <= REL_FRO_TOL
    # bf16 output is the rounding of the fp32 output
    assert torch.equal(y16.cpu(), y32.cpu().to(torch.bfloat16))
    return y32


GEMV_SHAPES = [(4096, 4096), (14336, 4096), (4096, 14336)]  # (N, K)


@pytest.mark.parametrize("n,k", GEMV_SHAPES)
@pytest.mark.parametrize("m", [1, 4, 16])
def test_w4a16_gemv(cuda, m, n, k):
    _check("w4", "gemv", m, n, k, seed=11, cuda=cuda)


@pytest.mark.parametrize("n,k", GEMV_SHAPES)
@pytest.mark.parametrize("m", [1, 4, 16])
def test_w8a16_gemv(cuda, m, n, k):
    _check("w8", "gemv", m, n, k, seed=12, cuda=cuda)


@pytest.mark.parametrize("m", [2, 3, 7, 13])
@pytest.mark.parametrize("scheme", ["w4", "w8"])
def test_gemv_ragged_m_and_small_shapes(cuda, scheme, m):
    _check(scheme, "gemv", m, 48, 384, seed=13, cuda=cuda)
    _check(scheme, "gemv", m, 2048, 5632, seed=14, cuda=cuda)


@pytest.mark.parametrize("m", [5, 8, 11, 16])
@pytest.mark.parametrize("scheme", ["w4", "w8"])
def test_gemv_wide_matrix_with_ragged_last_workgroup(cuda, scheme, m):
    """N / 16 = 517 row tiles at K = 4096: several row tiles per workgroup, the last workgroup short."""
    _check(scheme, "gemv", m, 16 * 517, 4096, seed=15, cuda=cuda)
    w_hat, wq, meta = _quantized(scheme, 16 * 517, 4096, 15, cuda)
    x = make_activations(m, 4096, 6).to(cuda)
    first = _run(scheme, x, wq, meta, torch.float32, "gemv")
    for _ in range(5):
        assert torch.equal(_run(scheme, x, wq, meta, torch.float32, "gemv"), first)


@pytest.mark.parametrize("m", [8, 13, 16])
@pytest.mark.parametrize("n", [6144, 16 * 2001])
@pytest.mark.parametrize("scheme", ["w4", "w8"])
def test_gemv_wide_matrix_at_k_2048(cuda, scheme, m, n):
    """More row tiles than CUs at K = 2048 (q|k|v and the head of the 12-layer model at batch 8 and up; N = 32016 is no
    multiple of the CU count), 8 to 16 rows."""
    _check(scheme, "gemv", m, n, 2048, seed=17, cuda=cuda)
    w_hat, wq, meta = _quantized(scheme, n, 2048, 17, cuda)
    x = make_activations(m, 2048, 8).to(cuda)
    first = _run(scheme, x, wq, meta, torch.float32, "gemv")
    assert torch.equal(_run(scheme, x, wq, meta, torch.float32, "gemv"), first)


@pytest.mark.parametrize("scheme", ["w4", "w8"])
def test_gemv_is_deterministic(cuda, scheme):
    w_hat, wq, meta = _quantized(scheme, 4096, 4096, 11 if scheme == "w4" else 12, cuda)
    x = make_activations(4, 4096, 5).to(cuda)
    first = _run(scheme, x, wq, meta, torch.float32, "gemv")
    for _ in range(10):
        assert torch.equal(_run(scheme, x, wq, meta, torch.float32, "gemv"), first)


@pytest.mark.parametrize("scheme", ["w4", "w8"])
def test_one_hot_activation_reads_back_dequantized_weights(cuda, scheme):
    """x = e_k picks column k of W_hat: every entry must be the exact fp32 dequantized weight."""
    n, k = 64, 512
    w_hat, wq, meta = _quantized(scheme, n, k, 21, cuda)
    cols = [0, 1, 7, 8, 127, 128, 255, 300, 511, 37, 64, 65, 190, 256, 383, 448]
    x = torch.zeros((16, k), dtype=torch.bfloat16)
    for i, c in enumerate(cols):
        x[i, c] = 1.0
    for kernel in ("gemv", "gemm"):
        y = _run(scheme, x.to(cuda), wq, meta, torch.float32, kernel).cpu()
        assert torch.equal(y, w_hat[:, cols].t().contiguous()), kernel


GEMM_CASES = [(256, 4096, 4096), (2048, 4096, 4096), (256, 14336, 4096), (2048, 14336, 4096)]


@pytest.mark.parametrize("m,n,k", GEMM_CASES)
@pytest.mark.parametrize("scheme", ["w4", "w8"])
def test_prefill_gemm(cuda, scheme, m, n, k):
    _check(scheme, "gemm", m, n, k, seed=31, cuda=cuda, outliers=True, max_rows=256)


@pytest.mark.parametrize("m,n,k", [(1024, 4096, 4096), (1000, 3088, 4096), (640, 6144, 4096)])
@pytest.mark.parametrize("scheme", ["w4", "w8"])
def test_prefill_gemm_few_tiles(cuda, scheme, m, n, k):
    """Shapes with fewer 256 x 128 tiles than CUs: the library's cost model takes the 128 x 128 tile
    kernel (ring of three tile buffers); ragged M (last row tile shifted up) and an N whose last
    column tile is partly outside the matrix."""
    _check(scheme, "gemm", m, n, k, seed=33, cuda=cuda, outliers=True, max_rows=192)


@pytest.mark.parametrize("scheme", ["w4", "w8"])
@pytest.mark.parametrize("n", [4096, 14336])
def test_prefill_gemm_m8192(cuda, scheme, n):
    _check(scheme, "gemm", 8192, n, 4096, seed=32, cuda=cuda, outliers=True, max_rows=128)


@pytest.mark.parametrize("scheme", ["w4", "w8"])
@pytest.mark.parametrize("m,n,k", [(4096, 4096, 14336), (2300, 7168, 640), (4096, 3856, 384)])
def test_prefill_gemm_on_256x256_tiles(cuda, scheme, m, n, k):
    """Shapes with enough tiles for the 256 x 256 kernel: the longest K of the benchmark models, ragged M (the last
    row tile shifted up) with an odd number of 128-k rounds, and an N whose last column tile is mostly outside the
    matrix; fp32 and bf16 outputs."""
    _check(scheme, "gemm", m, n, k, seed=35, cuda=cuda, outliers=True, max_rows=96)


def test_w4_gemm_on_256_row_tiles_takes_no_workspace(cuda):
    """The 256-row tile kernels subtract the zero-points while unpacking: no group sums, a NULL workspace is fine."""
    from ajllm_amd import _lib
    lib = _lib.load()
    for m, n, k in ((2048, 4096, 1024), (4096, 4096, 512)):  # 256 x 128 and 256 x 256 tiles
        assert lib.ajq_w4a16_gemm_workspace_bytes_for(m, n, k) == 0
        w_hat, wq, meta = _quantized("w4", n, k, 41, cuda)
        x = make_activations(m, k, 6, True).to(cuda)
        y = torch.empty((m, n), dtype=torch.float32, device=cuda)
        _lib.check(lib.ajq_w4a16_gemm(x.data_ptr(), m, k, wq.data_ptr(), meta.data_ptr(), n, y.data_ptr(), _lib.AJQ_OUT_F32,
                                      None, 0, torch.cuda.current_stream().cuda_stream), "w4 gemm without workspace")
        torch.cuda.synchronize()
        want = x.double() @ w_hat.to(cuda).double().t()
        assert errors(y.double().cpu(), want.cpu())[1] <= 1e-5


@pytest.mark.parametrize("m,n,k", [(2048, 4096, 512), (2048, 4096, 1280), (4096, 4096, 640), (300, 512, 1024), (40, 512, 1024),
                                   (4, 512, 1024)])
def test_w4_group_scales_far_apart_and_zero(cuda, m, n, k):
    """W4 columns whose group scales differ by six orders of magnitude from one group to the next, with
    constant-zero groups (scale 0) and constant non-zero groups (scale 0 too: they dequantize to 0) in
    between, first and last.  The tile kernels carry their accumulators in units of the current group's
    scale, so a wrong rescale at a group boundary, or a zero scale, shows as an O(1) error here.  Shapes:
    256 x 128 tiles (an even and an odd number of groups), 256 x 256 tiles (M = 4096), 128 x 128 tiles, the
    weight-streaming kernel and the GEMV."""
    from ajllm_amd import repack_w4, w4a16_matmul

    gen = torch.Generator().manual_seed(m + n + k)
    groups = k // 128
    magnitude = torch.tensor([1e-3, 1.0, 0.0, 30.0, 1e-4, 3.0, 0.0, 0.0, 1e2, 1e-2])[
        torch.randint(0, 10, (n, groups), generator=gen)
    ]
    magnitude[:, 0] = torch.where(torch.arange(n) % 3 == 0, 0.0, magnitude[:, 0])     # zero scale first
    magnitude[:, -1] = torch.where(torch.arange(n) % 5 == 0, 0.0, magnitude[:, -1])   # and last
    w = (torch.randn(n, groups, 128, generator=gen) * magnitude[:, :, None]).reshape(n, k)
    w[7::11, 128:256] = 0.5  # constant non-zero groups
    q, s, z = qspec.quantize_w4_g128(w.numpy())
    assert (s == 0).any() and (s > 1).any()
    qw = qspec.pack_int4(q)
    w_hat = torch.from_numpy(qspec.dequantize_w4(qw, s, z))
    wq, meta = repack_w4(torch.from_numpy(qw).to(cuda), torch.from_numpy(s).to(cuda), torch.from_numpy(z).to(cuda))
    x = make_activations(m, k, 77, True)
    y = w4a16_matmul(x.to(cuda), wq, meta, torch.float32).cpu()
    rows = torch.arange(0, m, max(1, m // 128))
    want = qspec.quant_linear(x[rows], w_hat, accumulate=torch.float64, out_dtype=torch.float64)
    assert torch.isfinite(y).all()
    rel = float((y[rows].double() - want).norm() / want.norm())
    assert rel <= 1e-5, rel
    # columns are independent: a column's error is judged against that column's own magnitude
    col_err = (y[rows].double() - want).norm(dim=0)
    col_ref = want.norm(dim=0)
    live = col_ref > 0
    assert float((col_err[live] / col_ref[live]).max()) <= 1e-4
    if (~live).any():
        assert float(col_err[~live].max()) <= 1e-10


@pytest.mark.parametrize("m", [1, 17, 63, 65, 100, 129, 300])
@pytest.mark.parametrize("scheme", ["w4", "w8"])
def test_gemm_ragged_m(cuda, scheme, m):
    _check(scheme, "gemm", m, 272, 640, seed=33, cuda=cuda, outliers=True)


@pytest.mark.parametrize("n,k", [(4096, 4096), (4096, 14336)])
@pytest.mark.parametrize("m", [32, 40, 64, 128, 255])
@pytest.mark.parametrize("scheme", ["w4", "w8"])
def test_batched_decode_matmul(cuda, scheme, m, n, k):
    """17 <= M < 256 (several sequences decoded together): the weight-streaming kernel with
    32-, 48- and 64-row activation blocks, at the sweep's matrix sizes."""
    _check(scheme, "gemm", m, n, k, seed=31, cuda=cuda, outliers=True, max_rows=64)


@pytest.mark.parametrize("scheme", ["w4", "w8"])
def test_batched_decode_matmul_is_deterministic(cuda, scheme):
    w_hat, wq, meta = _quantized(scheme, 4096, 4096, 31, cuda)
    x = make_activations(32, 4096, 9).to(cuda)
    runs = [_run(scheme, x, wq, meta, torch.float32, "gemm") for _ in range(3)]
    assert torch.equal(runs[0], runs[1]) and torch.equal(runs[0], runs[2])


class _LentWorkspace:
    """A zeroed buffer lent to the library's matmuls for the duration of a ``with`` block."""

    def __init__(self, cuda):
        from ajllm_amd import _lib

        self.lib = _lib.load()
        self.buffer = torch.zeros(int(self.lib.ajq_matmul_workspace_bytes()), dtype=torch.uint8, device=cuda)

    def __enter__(self):
        from ajllm_amd import _lib

        _lib.check(self.lib.ajq_matmul_workspace_set(self.buffer.data_ptr(), self.buffer.numel()), "matmul_workspace_set")
        return self

    def __exit__(self, *exc):
        self.lib.ajq_matmul_workspace_set(None, 0)

    def tickets(self) -> torch.Tensor:
        return self.buffer[:4096]


@pytest.mark.parametrize("m,n,k", [(32, 4096, 14336), (17, 4096, 14336), (32, 4000, 8192), (24, 1040, 16384),
                                   (32, 64, 8704), (16, 4096, 14336), (9, 4000, 14336), (13, 64, 14336)])
@pytest.mark.parametrize("scheme", ["w4", "w8"])
def test_batched_decode_matmul_split_along_k(cuda, scheme, m, n, k):
    """The weight-streaming kernel with four workgroups per group of four row tiles, a quarter of K each, and the
    partial sums exchanged through a lent buffer (17 <= M <= 32, K >= 8192, N <= 4096): against the oracle like
    every other kernel; against the unsplit kernel within fp32 reassociation; identical from run to run; the
    buffer's ticket words zero again afterwards; no trace of the previous call's partial sums when calls on
    different matrices alternate on one buffer.  K = 14336 and 16384 take the straight-line kernels (seven and eight
    waves' runs of four groups), 8192 and 8704 the loop; N = 4000 and 1040 end in a group of fewer than four row
    tiles.  With 9 <= M <= 16 at K = 14336 the same exchange runs behind the resident-activation form with one
    16-row block (in place of the GEMV)."""
    w_hat, wq, meta = _quantized(scheme, n, k, 31, cuda)
    x = make_activations(m, k, 131, True).to(cuda)
    plain = _run(scheme, x, wq, meta, torch.float32, "gemm")
    with _LentWorkspace(cuda) as ws:
        split = _check(scheme, "gemm", m, n, k, seed=31, cuda=cuda, outliers=True)
        again = _run(scheme, x, wq, meta, torch.float32, "gemm")
        # another matrix through the same buffer, then the first again
        other_wq = torch.roll(wq, 1, 0)
        other = _run(scheme, x, other_wq, meta, torch.float32, "gemm")
        third = _run(scheme, x, wq, meta, torch.float32, "gemm")
        torch.cuda.synchronize()
        assert int(ws.tickets().max()) == 0
    assert not torch.equal(plain, split)  # (the split form did run: its sums associate differently)
    assert errors(split.cpu(), plain.cpu().double())[0] <= 1e-4
    assert torch.equal(split, again) and torch.equal(split, third) and not torch.equal(split, other)
    # without the buffer the unsplit kernel runs again
    assert torch.equal(plain, _run(scheme, x, wq, meta, torch.float32, "gemm"))


@pytest.mark.parametrize("m", [32, 16, 11])
@pytest.mark.parametrize("scheme", ["w4", "w8"])
def test_split_along_k_with_the_residual_epilogue(cuda, scheme, m):
    """ajq_w*a16_gemv_residual (w2 of a batched decode step: K = 14336) through the split form: the new residual
    stream is the plain split matmul's output added to h_in bit for bit, its bf16 image and the sums of squares
    follow from it."""
    from ajllm_amd import _lib
    lib = _lib.load()
    st = torch.cuda.current_stream().cuda_stream
    d, k = 4096, 14336
    w_hat, wq, meta = _quantized(scheme, d, k, 31, cuda)
    g = torch.Generator().manual_seed(5)
    x = make_activations(m, k, 17, True).to(cuda)
    h_in = (torch.randn((m, d), generator=g) * 3.0).to(cuda)
    gain = (torch.rand(d, generator=g) + 0.5).to(cuda)
    h_out = torch.zeros((m, d), dtype=torch.float32, device=cuda)
    xt = torch.zeros((m, d), dtype=torch.bfloat16, device=cuda)
    ssq = torch.zeros((m, d // 16), dtype=torch.float32, device=cuda)
    res_fn = lib.ajq_w4a16_gemv_residual if scheme == "w4" else lib.ajq_w8a16_gemv_residual
    with _LentWorkspace(cuda) as ws:
        y = _run(scheme, x, wq, meta, torch.float32, "gemm")
        _lib.check(res_fn(x.data_ptr(), m, k, wq.data_ptr(), meta.data_ptr(), d, h_in.data_ptr(), gain.data_ptr(),
                          h_out.data_ptr(), xt.data_ptr(), ssq.data_ptr(), st), "gemv_residual")
        torch.cuda.synchronize()
        assert int(ws.tickets().max()) == 0
    assert torch.equal(h_out, h_in + y)
    assert torch.equal(xt, (h_out * gain).to(torch.bfloat16))
    tiles = h_out.double().square().reshape(m, d // 16, 16).sum(-1)
    assert float((ssq.double() - tiles).abs().max() / tiles.max()) <= 1e-6


@pytest.mark.parametrize("m,n,k", [(32, 28672, 4096), (17, 14336, 4096), (64, 16 * 1001, 4096), (33, 16 * 513, 2048),
                                   (100, 8192, 2048), (127, 16 * 131, 4096), (17, 16, 2048), (31, 48, 4096),
                                   (127, 4096 + 16, 4096), (16, 16 * 257, 2048), (9, 16 * 4100, 4096), (12, 16 * 700, 4096)])
@pytest.mark.parametrize("scheme", ["w4", "w8"])
def test_batched_decode_matmul_many_row_tiles(cuda, scheme, m, n, k):
    """Several 16-row tiles of N per CU at K = 2048 / 4096: the weight-streaming form that keeps a workgroup's
    activation block resident in registers and walks a run of 4, 7 or 8 row tiles past it (w1 | w3 of config 5 at
    32 rows, a run count that does not divide the tiles, several row blocks, the last one ragged; a single row tile;
    more workgroups than one round of the chip holds; with 9 to 16 rows the form with one 16-row block that takes the
    GEMV's wide matrices, up to its longest run of 16 row tiles).  The plain
    product against the oracle, then ajq_w*a16_gemv_gated on the same operands: bf16(silu(a) * u) over tiles of
    8 gate rows and 8 up rows, from the same fp32 values."""
    from ajllm_amd import _lib
    lib = _lib.load()
    y32 = _check(scheme, "gemm", m, n, k, seed=47, cuda=cuda, outliers=True, max_rows=48)
    _, wq, meta = _quantized(scheme, n, k, 47, cuda)
    x = make_activations(m, k, 147, True).to(cuda)
    gated = torch.full((m, n // 2), 7.0, dtype=torch.bfloat16, device=cuda)
    fn = lib.ajq_w4a16_gemv_gated if scheme == "w4" else lib.ajq_w8a16_gemv_gated
    _lib.check(fn(x.data_ptr(), m, k, wq.data_ptr(), meta.data_ptr(), n, gated.data_ptr(),
                  torch.cuda.current_stream().cuda_stream), "gemv_gated")
    again = torch.empty_like(y32)
    fn32 = lib.ajq_w4a16_gemm if scheme == "w4" else lib.ajq_w8a16_gemm
    args = (x.data_ptr(), m, k, wq.data_ptr(), meta.data_ptr(), n, again.data_ptr(), _lib.AJQ_OUT_F32)
    tail = (None, 0, torch.cuda.current_stream().cuda_stream) if scheme == "w4" else (torch.cuda.current_stream().cuda_stream,)
    _lib.check(fn32(*args, *tail), "gemm")
    torch.cuda.synchronize()
    assert torch.equal(again, y32)  # run-to-run identical
    pairs = y32.cpu().reshape(m, n // 16, 2, 8).double()
    want = (torch.nn.functional.silu(pairs[:, :, 0]) * pairs[:, :, 1]).reshape(m, n // 2)
    assert bf16_rounding_excess(gated.cpu(), want, 4e-6 * float(want.abs().max())) <= 0


@pytest.mark.parametrize("scheme", ["w4", "w8"])
def test_gemv_and_gemm_agree(cuda, scheme):
    w_hat, wq, meta = _quantized(scheme, 2048, 2048, 41, cuda)
    x = make_activations(16, 2048, 6).to(cuda)
    a = _run(scheme, x, wq, meta, torch.float32, "gemv")
    b = _run(scheme, x, wq, meta, torch.float32, "gemm")
    assert errors(a, b)[0] <= 1e-4


def test_linearity_at_full_size(cuda):
    """Size-independent property: the kernel is linear in x (checked in fp32 output)."""
    w_hat, wq, meta = _quantized("w4", 14336, 4096, 31, cuda)
    x1 = make_activations(512, 4096, 1).to(cuda)
    x2 = (x1.float() * 2).to(torch.bfloat16)  # exact doubling in bf16
    y1 = _run("w4", x1, wq, meta, torch.float32, "gemm")
    y2 = _run("w4", x2, wq, meta, torch.float32, "gemm")
    assert errors(y2, 2 * y1)[0] <= 1e-3


def test_mfma_rate_probe_runs_and_reports_clocks(cuda):
    """The device yardstick of the bench-only library: a short launch finishes, counts its flops and reports a
    plausible shader clock (the rate itself is a measurement, not a pass criterion); bad arguments
    are refused."""
    import ctypes

    from ajllm_amd import _lib
    lib = _lib.load_bench()
    sink = torch.zeros(8 * 512, dtype=torch.float32, device=cuda)
    clocks = torch.zeros(2, dtype=torch.int64, device=cuda)
    flops = ctypes.c_double(0.0)
    for random_operands in (0, 1):
        status = lib.ajqb_mfma_rate(random_operands, 2000, 8, sink.data_ptr(), clocks.data_ptr(),
                                    ctypes.addressof(flops), torch.cuda.current_stream().cuda_stream)
        assert status == 0
        torch.cuda.synchronize()
        assert flops.value == 8 * 8 * 2000 * 4 * 32768.0
        cycles, ticks = (int(v) for v in clocks.tolist())
        assert ticks > 0 and 0.3 < cycles / ticks * 0.1 < 3.5  # GHz
        assert cycles >= 2000 * 4 * 32 * 0.9  # four 32-cycle MFMAs per iteration, issued in order
    assert lib.ajqb_mfma_rate(0, 0, 8, sink.data_ptr(), clocks.data_ptr(), None, None) == -2
    assert lib.ajqb_mfma_rate(0, 10, 8, None, clocks.data_ptr(), None, None) == -1


def _random_shapes(count: int, seed: int):
    """Seeded (M, N, K) with N a multiple of 16 and K of 128, spread over the ranges where the
    dispatch changes kernel (M = 16 / 17, 127 / 128, 255 / 256; few and many tiles)."""
    gen = torch.Generator().manual_seed(seed)
    pick = lambda values: values[int(torch.randint(0, len(values), (1,), generator=gen))]
    shapes = []
    for _ in range(count):
        m = pick([1, 5, 16, 17, 31, 33, 64, 127, 128, 129, 200, 255, 256, 257, 384, 500, 640, 1000, 1100])
        n = 16 * int(torch.randint(1, 400, (1,), generator=gen))
        k = 128 * pick([1, 2, 3, 5, 8, 16, 24, 32])
        shapes.append((m, n, k))
    return shapes


# three more whose size sends them to the tile kernels with ragged M and a partial last column tile
_TILE_SHAPES = [(1000, 3088, 1024), (640, 4112, 2048), (1100, 6400, 640)]


@pytest.mark.parametrize("m,n,k", _random_shapes(14, seed=2024) + _TILE_SHAPES)
@pytest.mark.parametrize("scheme", ["w4", "w8"])
def test_matmul_random_shapes(cuda, scheme, m, n, k):
    """Whatever kernel the library picks for the shape (GEMV, weight-streaming, 128 x 128 or 256 x 128
    tiles), the result is the oracle's within fp32 accumulation noise; all rows are checked, the
    reference product is formed in fp64 on the GPU from the oracle's dequantized weight."""
    w_hat, wq, meta = _quantized(scheme, n, k, 900 + n + k, cuda)
    x = make_activations(m, k, 7 * m + n, True).to(cuda)
    y32 = _run(scheme, x, wq, meta, torch.float32, "auto")
    y16 = _run(scheme, x, wq, meta, torch.bfloat16, "auto")
    want = x.double() @ w_hat.to(cuda).double().t()
    max_abs, rel_fro = errors(y32.double().cpu(), want.cpu())
    assert max_abs <= 2e-3 and rel_fro <= 1e-5, (max_abs, rel_fro)
    assert torch.equal(y16, y32.to(torch.bfloat16))


@pytest.mark.parametrize("m,f,k", [(256, 7168, 1024), (2048, 2048, 2048), (1000, 3072, 4096), (200, 14336, 4096),
                                   (4096, 2048, 512), (2300, 3584, 640)])  # the last two: 256 x 256 tiles
@pytest.mark.parametrize("scheme", ["w4", "w8"])
def test_gemm_with_gate_epilogue_equals_gemm_then_swiglu(cuda, scheme, m, f, k):
    """ajq_w*a16_gemm_gate on the (w1 | w3) rows: bit for bit the fp32 GEMM followed by ajq_swiglu
    (both tile kernels, ragged M), and the oracle's silu(a) * u within bf16 rounding; shapes the tile
    kernels do not take are refused."""
    from ajllm_amd import _lib
    from ajllm_amd.decoding import _FusedLinear
    lib = _lib.load()
    w_hat, wq, meta = _quantized(scheme, 2 * f, k, 77 + f, cuda)
    x = make_activations(m, k, 5, True).to(cuda)
    fused = _FusedLinear.__new__(_FusedLinear)
    fused.scheme, fused.wq, fused.meta = ("w4a16_g128" if scheme == "w4" else "w8a16"), wq, meta
    fused.in_features, fused.rows16 = k, 2 * f
    assert fused.gate_fusable(m)
    got = fused.gated(x)
    ab = _run(scheme, x, wq, meta, torch.float32, "gemm")
    want = torch.empty((m, f), dtype=torch.bfloat16, device=cuda)
    _lib.check(lib.ajq_swiglu(ab.data_ptr(), want.data_ptr(), m, f, torch.cuda.current_stream().cuda_stream), "swiglu")
    torch.cuda.synchronize()
    assert got.shape == (m, f) and torch.equal(got, want)
    ref = x.double() @ w_hat.to(cuda).double().t()
    gate = torch.nn.functional.silu(ref[:, :f]) * ref[:, f:]
    assert errors(got.double().cpu(), gate.cpu())[1] <= 4e-3  # bf16 output
    assert not fused.gate_fusable(64) and lib.ajq_gemm_gate_supported(m, 2 * f + 16, k, 1) == 0


@pytest.mark.parametrize("scheme", ["w4", "w8"])
@pytest.mark.parametrize("m,k", [(1, 1024), (3, 2048), (16, 2048), (1, 4096), (8, 4096), (2, 5632), (8, 5632)])
def test_gemv_with_norm_or_gate_prologue_against_the_oracle(cuda, scheme, m, k):
    """ajq_w*a16_gemv_norm / _gate against the oracle product: the activations are formed on the CPU
    exactly as the model code forms them (RMSNorm in fp32 then a bf16 cast, layers.py:70-74 behind the
    residual add of transformer.py:45-50; silu(a) * u, activations.py:24-25) and multiplied with the
    oracle's dequantized weight in fp64.  Tolerances are the north-star ones (max-abs 1e-2, relative
    Frobenius 2e-3); a differently ordered sum of squares on the GPU may round a few activations to
    the neighbouring bf16 value, which is far inside them."""
    from ajllm_amd import _lib
    lib = _lib.load()
    st = torch.cuda.current_stream().cuda_stream
    n = 272
    w_hat, wq, meta = _quantized(scheme, n, k, 300 + k, cuda)
    assert lib.ajq_gemv_fused_supported(m, k) == 1
    g = torch.Generator().manual_seed(9 * m + k)
    h = torch.randn((m, k), generator=g)
    d = torch.randn((m, k), generator=g) * 0.5
    gain = torch.rand(k, generator=g) + 0.5
    eps = 1e-5
    norm_fn = lib.ajq_w4a16_gemv_norm if scheme == "w4" else lib.ajq_w8a16_gemv_norm
    gate_fn = lib.ajq_w4a16_gemv_gate if scheme == "w4" else lib.ajq_w8a16_gemv_gate
    for delta in (d, None):
        hg, gg = h.to(cuda), gain.to(cuda)
        dg = delta.to(cuda) if delta is not None else None
        h_out = torch.zeros((m, k), dtype=torch.float32, device=cuda)
        y = torch.empty((m, n), dtype=torch.float32, device=cuda)
        _lib.check(norm_fn(hg.data_ptr(), dg.data_ptr() if dg is not None else None, gg.data_ptr(), eps,
                           h_out.data_ptr(), m, k, wq.data_ptr(), meta.data_ptr(), n, y.data_ptr(), _lib.AJQ_OUT_F32, st),
                   "gemv_norm")
        torch.cuda.synchronize()
        s = h + delta if delta is not None else h.clone()
        assert torch.equal(h_out.cpu(), s)                      # the updated residual stream, one fp32 add
        rms = torch.sqrt(torch.mean(s.square(), dim=-1, keepdim=True) + eps)
        x = ((s / rms) * gain).to(torch.bfloat16)
        want = qspec.quant_linear(x, w_hat, accumulate=torch.float64, out_dtype=torch.float64)
        max_abs, rel = errors(y.cpu(), want)
        assert max_abs <= MAX_ABS_TOL and rel <= REL_FRO_TOL, (max_abs, rel)
        assert max_abs <= 3e-3, max_abs
    ab = torch.randn((m, 2 * k), generator=g) * 2
    y = torch.empty((m, n), dtype=torch.float32, device=cuda)
    abg = ab.to(cuda)
    _lib.check(gate_fn(abg.data_ptr(), m, k, wq.data_ptr(), meta.data_ptr(), n, y.data_ptr(), _lib.AJQ_OUT_F32, st),
               "gemv_gate")
    torch.cuda.synchronize()
    a, u = ab[:, :k], ab[:, k:]
    x = (a * torch.sigmoid(a) * u).to(torch.bfloat16)           # silu(a) * u as activations.py:11-25 writes it
    want = qspec.quant_linear(x, w_hat, accumulate=torch.float64, out_dtype=torch.float64)
    max_abs, rel = errors(y.cpu(), want)
    assert max_abs <= MAX_ABS_TOL and rel <= REL_FRO_TOL, (max_abs, rel)


@pytest.mark.parametrize("scheme", ["w4", "w8"])
@pytest.mark.parametrize("m,k1,d,n2", [(8, 2048, 2048, 6144), (5, 5632, 2048, 11264), (16, 2048, 2048, 512),
                                      (8, 4096, 4096, 1024), (13, 4096, 4096, 2048), (1, 2048, 2048, 256),
                                      (32, 14336, 4096, 6144), (40, 4096, 4096, 28672), (17, 1024, 2048, 512),
                                      (100, 2048, 4096, 4096), (12, 5632, 2048, 1024), (3, 1024, 1024, 512)])
def test_gemv_residual_then_rowscale_against_the_oracle(cuda, scheme, m, k1, d, n2):
    """h_out = h_in + x W1^T (ajq_w*a16_gemv_residual) followed by y = (RMSNorm(h_out) * gain) W2^T
    (ajq_w*a16_gemv_rowscale) without a norm kernel between them: the residual add and the RMSNorm of
    transformer.py:45-50 / layers.py:70-74 around two Linears.  Each output is checked against the
    oracle's dequantized weights in fp64: the new residual stream, its bf16 image (bit for bit the
    rounding of the kernel's own fp32 values), the per-tile sums of squares, the row-scaled product, and
    the product against the REFERENCE order (normalise, round to bf16, multiply) within bf16 rounding.
    With gate = 1 the rows of W2 count as tiles of 8 gate rows and 8 up rows: silu(a) * u in bf16."""
    from ajllm_amd import _lib
    lib = _lib.load()
    st = torch.cuda.current_stream().cuda_stream
    assert lib.ajq_gemv_epilogue_supported(m, k1) == 1 and lib.ajq_gemv_epilogue_supported(m, d) == 1
    w1_hat, wq1, meta1 = _quantized(scheme, d, k1, 500 + k1, cuda)
    w2_hat, wq2, meta2 = _quantized(scheme, n2, d, 600 + n2, cuda)
    g = torch.Generator().manual_seed(31 * m + d)
    x = make_activations(m, k1, 11, True)
    h_in = torch.randn((m, d), generator=g) * 3.0
    gain = torch.rand(d, generator=g) + 0.5
    eps = 1e-5
    res_fn = lib.ajq_w4a16_gemv_residual if scheme == "w4" else lib.ajq_w8a16_gemv_residual
    row_fn = lib.ajq_w4a16_gemv_rowscale if scheme == "w4" else lib.ajq_w8a16_gemv_rowscale
    xg, hg, gg = x.to(cuda), h_in.to(cuda), gain.to(cuda)
    h_out = torch.zeros((m, d), dtype=torch.float32, device=cuda)
    xt = torch.zeros((m, d), dtype=torch.bfloat16, device=cuda)
    ssq = torch.zeros((max(16, m), d // 16), dtype=torch.float32, device=cuda)
    _lib.check(res_fn(xg.data_ptr(), m, k1, wq1.data_ptr(), meta1.data_ptr(), d, hg.data_ptr(), gg.data_ptr(),
                      h_out.data_ptr(), xt.data_ptr(), ssq.data_ptr(), st), "gemv_residual")
    y = torch.empty((m, n2), dtype=torch.float32, device=cuda)
    _lib.check(row_fn(xt.data_ptr(), ssq.data_ptr(), d // 16, eps, m, d, wq2.data_ptr(), meta2.data_ptr(), n2,
                      y.data_ptr(), _lib.AJQ_OUT_F32, 0, st), "gemv_rowscale")
    y16 = torch.empty((m, n2), dtype=torch.bfloat16, device=cuda)
    _lib.check(row_fn(xt.data_ptr(), ssq.data_ptr(), d // 16, eps, m, d, wq2.data_ptr(), meta2.data_ptr(), n2,
                      y16.data_ptr(), _lib.AJQ_OUT_BF16, 0, st), "gemv_rowscale")
    yg = torch.empty((m, n2 // 2), dtype=torch.bfloat16, device=cuda)
    _lib.check(row_fn(xt.data_ptr(), ssq.data_ptr(), d // 16, eps, m, d, wq2.data_ptr(), meta2.data_ptr(), n2,
                      yg.data_ptr(), _lib.AJQ_OUT_BF16, 1, st), "gemv_rowscale gate")
    torch.cuda.synchronize()
    h_out, xt, ssq, y, y16, yg = h_out.cpu(), xt.cpu(), ssq.cpu(), y.cpu(), y16.cpu(), yg.cpu()

    # the residual stream
    h_ref = h_in.double() + qspec.quant_linear(x, w1_hat, accumulate=torch.float64, out_dtype=torch.float64)
    max_abs, rel = errors(h_out, h_ref)
    assert max_abs <= 2e-3 and rel <= 1e-5, (max_abs, rel)
    # its bf16 image and the sums of squares, from the kernel's own fp32 values
    assert torch.equal(xt, (h_out * gain).to(torch.bfloat16))
    assert torch.equal(ssq[m:], torch.zeros_like(ssq[m:]))
    tiles = h_out.double().square().reshape(m, d // 16, 16).sum(-1)
    assert float((ssq[:m].double() - tiles).abs().max() / tiles.max()) <= 1e-6
    # the row-scaled product
    rstd = torch.rsqrt(h_out.double().square().mean(-1, keepdim=True) + eps)
    want = rstd * qspec.quant_linear(xt, w2_hat, accumulate=torch.float64, out_dtype=torch.float64)
    max_abs, rel = errors(y, want)
    assert max_abs <= MAX_ABS_TOL and rel <= 1e-5, (max_abs, rel)
    assert torch.equal(y16, y.to(torch.bfloat16))
    # the reference order: normalise in fp32, round to bf16, multiply
    x_ref = ((h_ref.float() * torch.rsqrt(h_ref.float().square().mean(-1, keepdim=True) + eps)) * gain).to(torch.bfloat16)
    ordered = qspec.quant_linear(x_ref, w2_hat, accumulate=torch.float64, out_dtype=torch.float64)
    # (two independent bf16 roundings of every activation: 2^-9 / sqrt(3) each, relative, which does not
    # average out over K; the bound is twice the expected 1.6e-3)
    assert errors(y, ordered)[1] <= 3.2e-3
    # the same consumer with the activations rounded where the reference rounds them (ajq_w*a16_gemv_norm_sums: the
    # norm prologue fed with the producer's sums of squares): against the reference order within fp32 noise, up
    # to a few activations that a differently ordered sum of squares moves to the neighbouring bf16 value
    if lib.ajq_gemv_fused_supported(m, d):
        ns_fn = lib.ajq_w4a16_gemv_norm_sums if scheme == "w4" else lib.ajq_w8a16_gemv_norm_sums
        h_dev = h_out.to(cuda)
        ssq_dev = ssq.to(cuda)
        y_ns = torch.empty((m, n2), dtype=torch.float32, device=cuda)
        _lib.check(ns_fn(h_dev.data_ptr(), ssq_dev.data_ptr(), d // 16, gg.data_ptr(), eps, m, d, wq2.data_ptr(),
                         meta2.data_ptr(), n2, y_ns.data_ptr(), _lib.AJQ_OUT_F32, 0, st), "gemv_norm_sums")
        yg_ns = torch.empty((m, n2 // 2), dtype=torch.bfloat16, device=cuda)
        _lib.check(ns_fn(h_dev.data_ptr(), ssq_dev.data_ptr(), d // 16, gg.data_ptr(), eps, m, d, wq2.data_ptr(),
                         meta2.data_ptr(), n2, yg_ns.data_ptr(), _lib.AJQ_OUT_BF16, 1, st), "gemv_norm_sums gate")
        torch.cuda.synchronize()
        x_own = ((h_out / torch.sqrt(h_out.square().mean(-1, keepdim=True) + eps)) * gain).to(torch.bfloat16)
        own = qspec.quant_linear(x_own, w2_hat, accumulate=torch.float64, out_dtype=torch.float64)
        assert errors(y_ns.cpu(), own)[1] <= 2e-4
        pairs_ns = y_ns.cpu().reshape(m, n2 // 16, 2, 8)
        gate_ns = (torch.nn.functional.silu(pairs_ns[:, :, 0].double()) * pairs_ns[:, :, 1].double()).reshape(m, n2 // 2)
        assert bf16_rounding_excess(yg_ns.cpu(), gate_ns, 4e-6 * float(gate_ns.abs().max())) <= 0
    # the gate: tiles of 8 gate rows and 8 up rows
    pairs = y.reshape(m, n2 // 16, 2, 8)
    gate = (torch.nn.functional.silu(pairs[:, :, 0].double()) * pairs[:, :, 1].double()).reshape(m, n2 // 2)
    assert bf16_rounding_excess(yg, gate, 4e-6 * float(gate.abs().max())) <= 0
    # unsupported shapes and bad arguments are refused
    assert lib.ajq_gemv_epilogue_supported(256, 2048) == 0 and lib.ajq_gemv_epilogue_supported(9, 5632) == 1
    assert row_fn(xt.data_ptr(), ssq.data_ptr(), 6, eps, m, d, wq2.data_ptr(), meta2.data_ptr(), n2, y.data_ptr(),
                  _lib.AJQ_OUT_F32, 0, st) != 0
