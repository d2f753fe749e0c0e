"""The entry point that allocates nothing (``ajq_w4a16_gemm_noalloc``) against the entry point it
is a variant of (``ajq_w4a16_gemm`` with a caller workspace): same kernels, so the outputs must be
equal bit for bit, on two calls in a row, the second with a smaller input (the built-in scratch
keeps the first call's contents)."""

import pytest
import torch

from tests.helpers import make_activations, make_weight

pytestmark = pytest.mark.gpu


def _private_w4(n, k, seed, cuda):
    from ajllm_amd import quantize_w4_g128, repack_w4

    return repack_w4(*quantize_w4_g128(make_weight(n, k, seed).to(cuda)))


def _both(lib, x, wq, meta, n, k, out_dtype):
    from ajllm_amd import _lib

    m = x.shape[0]
    flag = _lib.AJQ_OUT_F32 if out_dtype == torch.float32 else _lib.AJQ_OUT_BF16
    stream = torch.cuda.current_stream().cuda_stream
    nbytes = lib.ajq_w4a16_gemm_workspace_bytes_for(m, n, k)
    workspace = torch.empty((max(nbytes, 16),), dtype=torch.uint8, device=x.device)
    want = torch.empty((m, n), dtype=out_dtype, device=x.device)
    _lib.check(lib.ajq_w4a16_gemm(x.data_ptr(), m, k, wq.data_ptr(), meta.data_ptr(), n, want.data_ptr(), flag,
                                  workspace.data_ptr(), nbytes, stream), "ajq_w4a16_gemm")
    got = torch.full((m, n), float("nan"), dtype=out_dtype, device=x.device)
    if not _both.resolved:
        # the very first call on a device resolves the scratch array's address (no allocation either, but the
        # runtime may load the code object's data then): measured from the second call on
        _lib.check(lib.ajq_w4a16_gemm_noalloc(x.data_ptr(), m, k, wq.data_ptr(), meta.data_ptr(), n, got.data_ptr(),
                                              flag, stream), "ajq_w4a16_gemm_noalloc")
        got.fill_(float("nan"))
        _both.resolved = True
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    free_before, _ = torch.cuda.mem_get_info()      # the driver's count: sees a hipMalloc that torch's allocator cannot
    _lib.check(lib.ajq_w4a16_gemm_noalloc(x.data_ptr(), m, k, wq.data_ptr(), meta.data_ptr(), n, got.data_ptr(), flag,
                                          stream), "ajq_w4a16_gemm_noalloc")
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.cuda.mem_get_info()[0] == free_before
    return got, want


_both.resolved = False


def test_noalloc_gemm_equals_workspace_gemm_twice(cuda):
    from ajllm_amd import _lib

    lib = _lib.load()
    n, k = 4096, 4096
    wq, meta = _private_w4(n, k, 31, cuda)
    # 128 x 128 tiles (M = 1024, then the smaller M = 384: the kernels that keep their group sums in the scratch),
    # then shapes that need none: below the tile kernels (M = 40) and 256 x 128 tiles (M = 2048)
    for m, out_dtype in ((1024, torch.float32), (384, torch.bfloat16), (40, torch.float32), (2048, torch.bfloat16)):
        x = make_activations(m, k, 500 + m, outliers=True).to(cuda)
        got, want = _both(lib, x, wq, meta, n, k, out_dtype)
        assert torch.equal(got, want), (m, out_dtype)
        assert bool(torch.isfinite(got.float()).all())


def test_noalloc_gemm_runs_under_graph_capture(cuda):
    """A call recorded into a HIP graph (where an allocation or a synchronisation fails the capture) and replayed
    three times, with eager work between the replays, gives the eager call's result every time."""
    from ajllm_amd import _lib

    lib = _lib.load()
    n, k, m = 4096, 4096, 1024  # 128 x 128 tiles: the kernels whose group sums live in the scratch
    wq, meta = _private_w4(n, k, 33, cuda)
    x = make_activations(m, k, 77, outliers=True).to(cuda)
    want = torch.empty((m, n), dtype=torch.float32, device=cuda)
    got = torch.zeros_like(want)

    def call(out):
        _lib.check(lib.ajq_w4a16_gemm_noalloc(x.data_ptr(), m, k, wq.data_ptr(), meta.data_ptr(), n, out.data_ptr(),
                                              _lib.AJQ_OUT_F32, torch.cuda.current_stream().cuda_stream), "noalloc")

    call(want)                                    # warm-up: resolves the scratch address outside the capture
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            call(got)
    for replay in range(3):
        got.zero_()
        (x.float() @ x.float().t()).sum().item()  # unrelated eager work and a synchronisation between replays
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(got, want), replay


def test_noalloc_gemm_rejects_what_does_not_fit(cuda):
    from ajllm_amd import _lib

    lib = _lib.load()
    cap = lib.ajq_noalloc_scratch_bytes()
    assert cap == 16 << 20
    k = 14336
    m = cap // (16 * (k // 128)) + 128        # one tile row past the array
    n = 256                                   # few tiles: the 128 x 128 kernel, the one that keeps group sums
    assert lib.ajq_w4a16_gemm_workspace_bytes_for(m, n, k) > cap
    assert lib.ajq_w4a16_gemm_workspace_bytes_for(m, 4096, k) == 0   # 256 x 128 tiles: nothing to hold, any size fits
    wq, meta = _private_w4(n, k, 32, cuda)
    x = torch.zeros((m, k), dtype=torch.bfloat16, device=cuda)
    y = torch.empty((m, n), dtype=torch.bfloat16, device=cuda)
    status = lib.ajq_w4a16_gemm_noalloc(x.data_ptr(), m, k, wq.data_ptr(), meta.data_ptr(), n, y.data_ptr(),
                                        _lib.AJQ_OUT_BF16, torch.cuda.current_stream().cuda_stream)
    assert status == -6
    with pytest.raises(ValueError, match="built-in scratch"):
        _lib.check(status, "ajq_w4a16_gemm_noalloc")
