"""The C-ABI library loads without a GPU, exports every symbol the header declares, and its
argument validation (which runs before any HIP call) reports errors the way the header says."""

import ctypes
import re
from pathlib import Path

import pytest

from ajllm_amd import _lib

HEADER = Path(__file__).resolve().parents[1] / "include" / "ajq.h"


def _declared_functions() -> list[str]:
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(ajq_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound():
    lib = _lib.load()
    names = _declared_functions()
    assert len(names) >= 14
    for name in names:
        assert hasattr(lib, name), f"{name} declared in ajq.h but not exported by libajq.so"
        assert name in _lib.SIGNATURES, f"{name} has no ctypes signature"
    assert sorted(_lib.SIGNATURES) == names


def test_bench_library_exports_what_its_header_declares():
    """libajq_bench.so (the MFMA-rate yardstick for bench.py; include/ajq_bench.h) against its header, and
    no probe is left in the operator library."""
    header = HEADER.with_name("ajq_bench.h")
    text = re.sub(r"/\*.*?\*/", "", header.read_text(), flags=re.S)
    names = sorted(set(re.findall(r"\b(ajqb_[a-z0-9_]+)\s*\(", text)))
    lib = _lib.load_bench()
    assert names == sorted(_lib.BENCH_SIGNATURES) and len(names) >= 2
    for name in names:
        assert hasattr(lib, name), f"{name} declared in ajq_bench.h but not exported by libajq_bench.so"
    assert not any("probe" in name for name in _lib.SIGNATURES)
    assert not hasattr(_lib.load(), "ajqb_mfma_rate")
    assert lib.ajqb_mfma_rate(0, 8, 256, None, None, None, None) == -1             # refused before any GPU call
    assert b"sink" in lib.ajqb_last_error()


def test_version_and_status_strings():
    lib = _lib.load()
    assert lib.ajq_version() >= 1
    assert lib.ajq_status_string(0) == b"ok"
    for code in range(-6, 0):
        assert lib.ajq_status_string(code) not in (b"", b"unknown status")
    assert lib.ajq_status_string(-99) == b"unknown status"


def test_null_pointers_are_rejected_before_any_gpu_work():
    lib = _lib.load()
    assert lib.ajq_quantize_w8(None, 16, 128, None, None, None) == -1
    assert lib.ajq_quantize_w4_g128(None, 16, 128, None, None, None, None) == -1
    assert lib.ajq_w4a16_gemv(None, 1, 128, None, None, 16, None, 0, None) == -1
    assert b"null" in lib.ajq_last_error()
    with pytest.raises(ValueError):
        _lib.check(-1, "probe")


def test_shape_alignment_and_option_errors():
    lib = _lib.load()
    buf = ctypes.create_string_buffer(4096 + 16)
    base = (ctypes.addressof(buf) + 15) & ~15  # host memory: only its address is inspected
    p = ctypes.c_void_p(base)
    odd = ctypes.c_void_p(base + 4)
    assert lib.ajq_quantize_w4_g128(p, 16, 100, p, p, p, None) == -2      # K not a multiple of 128
    assert lib.ajq_quantize_w8(p, 0, 128, p, p, None) == -2
    assert lib.ajq_repack_w4(p, p, p, 10, 128, p, p, None) == -2            # N not a multiple of 16
    assert lib.ajq_w4a16_gemv(p, 17, 128, p, p, 16, p, 0, None) == -2       # M beyond the GEMV range
    assert b"M=17" in lib.ajq_last_error()
    assert lib.ajq_w4a16_gemv(p, 1, 128, p, p, 16, p, 7, None) == -4        # unknown out_dtype
    assert lib.ajq_w4a16_gemv(odd, 1, 128, p, p, 16, p, 0, None) == -3      # misaligned x
    assert lib.ajq_w8a16_gemm(p, 1, 192, p, p, 16, p, 0, None) == -2
    assert lib.ajq_add_rmsnorm(p, None, p, 1e-5, p, 1, 6, None) == -2            # D not a multiple of 4
    assert lib.ajq_attn_decode(p, p, p, 0, p, 1, 16, 16, 48, 8, p, p, 1 << 20, None) == -4  # head_dim 48 is not built
    assert lib.ajq_attn_decode(p, p, p, 0, p, 1, 16, 16, 128, 1024, p, None, 0, None) == -6  # split attention needs its workspace
    assert lib.ajq_attn_decode(p, p, p, 5, p, 1, 16, 16, 128, 8, p, p, 1 << 20, None) == -4  # unknown cache dtype
    assert lib.ajq_swiglu(p, p, 1, 3, None) == -2
    assert lib.ajq_rope_cache(p, p, p, p, p, p, p, 0, 1, 16, 3, 128, 8, None) == -2   # 16 query heads over 3 cache heads
    need = lib.ajq_w4a16_gemm_workspace_bytes(300, 512)
    assert need == 4 * 300 * 16                                             # G=4 groups x 300 rows x 16 bytes
    assert lib.ajq_w4a16_gemm_workspace_bytes(127, 512) == 0                 # below 128 rows no tile kernel runs: no workspace
    assert lib.ajq_attn_decode(p, p, p, 0, p, 1, 16, 2, 128, 8, p, p, 1 << 20, None) == -4  # 8 query heads per cache head
    # only the 128 x 128 tile kernel takes group sums: M = 1024 on 4096 x 4096 runs it, M = 2048 the 256 x 128 kernel
    need = lib.ajq_w4a16_gemm_workspace_bytes_for(1024, 4096, 4096)
    assert need == 32 * 1024 * 16 == lib.ajq_w4a16_gemm_workspace_bytes(1024, 4096)
    assert lib.ajq_w4a16_gemm_workspace_bytes_for(2048, 4096, 4096) == 0
    assert lib.ajq_w4a16_gemm_workspace_bytes_for(40, 4096, 4096) == 0 == lib.ajq_w4a16_gemm_workspace_bytes_for(8, 4096, 4096)
    assert lib.ajq_w4a16_gemm(p, 1024, 4096, p, p, 4096, p, 0, None, 0, None) == -6
    assert lib.ajq_w4a16_gemm(p, 1024, 4096, p, p, 4096, p, 0, p, need - 1, None) == -6
    # matmuls with a residual / row-scale / gate epilogue: which (M, K) are built, and what is refused before any launch
    assert lib.ajq_gemv_epilogue_supported(1, 2048) == 1 and lib.ajq_gemv_epilogue_supported(16, 4096) == 1
    assert lib.ajq_gemv_epilogue_supported(9, 5632) == 1 and lib.ajq_gemv_epilogue_supported(200, 14336) == 1   # streaming kernel
    assert lib.ajq_gemv_epilogue_supported(256, 2048) == 0 and lib.ajq_gemv_epilogue_supported(4, 1000) == 0
    # the row-scale consumer adds K / 16 tile sums: K <= 4096, or K = 5632 on the eleven-wave GEMV (M <= 8)
    assert lib.ajq_gemv_rowscale_supported(1, 2048) == 1 and lib.ajq_gemv_rowscale_supported(32, 4096) == 1
    assert lib.ajq_gemv_rowscale_supported(8, 5632) == 1 and lib.ajq_gemv_rowscale_supported(12, 5632) == 0
    assert lib.ajq_gemv_rowscale_supported(32, 8192) == 0 and lib.ajq_gemv_rowscale_supported(200, 14336) == 0
    # the buffer lent for split-K partial sums: size query, alignment and size checks, NULL ends the loan
    need = lib.ajq_matmul_workspace_bytes()
    assert need == 4096 + 64 * 4 * 4 * 2048
    assert lib.ajq_matmul_workspace_set(odd, need) == -3
    assert lib.ajq_matmul_workspace_set(p, need - 1) == -6 and b"bytes needed" in lib.ajq_last_error()
    assert lib.ajq_matmul_workspace_set(None, 0) == 0
    assert lib.ajq_w4a16_gemv_rowscale(p, p, 352, 1e-5, 12, 5632, p, p, 16, p, 0, 0, None) == -4
    assert lib.ajq_w8a16_gemv_rowscale(p, p, 512, 1e-5, 32, 8192, p, p, 16, p, 0, 0, None) == -4
    assert lib.ajq_w4a16_gemv_rowscale(p, p, 64, 1e-5, 4, 2048, p, p, 16, p, 0, 0, None) == -2     # parts is not K / 16
    assert lib.ajq_w4a16_gemv_norm_sums(p, p, 64, p, 1e-5, 4, 2048, p, p, 16, p, 0, 0, None) == -2
    assert lib.ajq_w4a16_gemv_rowscale(p, p, 128, 1e-5, 300, 2048, p, p, 16, p, 0, 0, None) == -4   # more rows than built
    assert lib.ajq_w4a16_gemv_rowscale(p, p, 130, 1e-5, 4, 2048, p, p, 16, p, 0, 0, None) == -2   # parts not a multiple of 4
    assert lib.ajq_w4a16_gemv_rowscale(p, p, 260, 1e-5, 4, 2048, p, p, 16, p, 0, 0, None) == -2   # more parts than the waves cover
    assert lib.ajq_w4a16_gemv_rowscale(p, None, 128, 1e-5, 4, 2048, p, p, 16, p, 0, 0, None) == -1
    assert lib.ajq_w8a16_gemv_rowscale(p, p, 128, 1e-5, 4, 2048, p, p, 32, p, 1, 1, None) == -4   # the gated output is bf16
    assert lib.ajq_w4a16_gemv_residual(p, 4, 2048, p, p, 16, p, p, p, p, p, None) == -1           # h_out must not be h_in
    assert lib.ajq_w8a16_gemv_residual(p, 4, 2048, p, p, 16, None, p, p, p, p, None) == -1
    assert lib.ajq_w8a16_gemv_residual(p, 4, 2048, p, p, 16, p, p, odd, p, p, None) == -3          # misaligned h_out
    assert lib.ajq_w4a16_gemv_merge_residual(p, 99, 1, 2048, p, p, 16, odd, p, p, p, p, None) == -4  # more chunks than built
    assert lib.ajq_w4a16_gemv_merge_residual(p, 2, 1, 2048, p, p, 16, p, p, p, p, p, None) == -1     # h_out must not be h_in
    with pytest.raises(ValueError):
        _lib.check(-6, "probe")
    with pytest.raises(RuntimeError):
        _lib.check(-5, "probe")


def test_attention_row_chunk_query():
    """Host-side only: how many row chunks per cache head the decode attention uses (1 = a single launch)."""
    lib = _lib.load()
    assert lib.ajq_attn_row_chunks(0, 8, 128) == 0 and lib.ajq_attn_row_chunks(1, 0, 128) == 0
    assert lib.ajq_attn_row_chunks(1, 16, 768) == 16          # few heads: as many chunks as the merge takes
    assert lib.ajq_attn_row_chunks(1, 16, 64) == 2            # a chunk keeps at least 32 rows
    assert lib.ajq_attn_row_chunks(8, 16, 768) == 6           # about 768 workgroups in all
    assert lib.ajq_attn_row_chunks(32, 8, 2176) == 1          # a cache head per CU: whole heads, no merge
    assert lib.ajq_attn_row_chunks(100, 16, 4096) == 1


def test_python_layer_refuses_cpu_tensors():
    """There is no CPU fallback: the host API raises instead of computing elsewhere."""
    import torch

    from ajllm_amd import QuantLinear, quantize_w4_g128, w4a16_matmul

    with pytest.raises(ValueError):
        quantize_w4_g128(torch.zeros(16, 128))
    with pytest.raises(ValueError):
        QuantLinear.from_weight(torch.zeros(16, 128))
    with pytest.raises(ValueError):
        QuantLinear(128, 16, scheme="w2")
    with pytest.raises(RuntimeError):
        QuantLinear(128, 16)(torch.zeros(1, 128))
    assert w4a16_matmul.__module__ == "ajllm_amd.quant"


def test_state_dict_loading_checks_every_canonical_tensor():
    """A checkpoint whose scales or zero-points have another shape or dtype is refused like a size mismatch of
    the reference layer's weight (strict loading, training/checkpoint.py:35-45); the layer stays untouched."""
    import torch

    from ajllm_amd import QuantLinear

    def w4_state(groups=2, scale_dtype=torch.float16):
        return {"qweight": torch.zeros(16, 32, dtype=torch.int32), "scales": torch.ones(16, groups, dtype=scale_dtype),
                "zeros": torch.zeros(16, groups, dtype=torch.uint8)}

    layer = QuantLinear(256, 16)
    layer.load_state_dict(w4_state())                      # the right shapes load (CPU tensors: nothing is repacked)
    assert layer.scales.shape == (16, 2)
    for bad in (w4_state(groups=4), w4_state(scale_dtype=torch.float32)):
        fresh = QuantLinear(256, 16)
        with pytest.raises(RuntimeError, match="mismatch for scales"):
            fresh.load_state_dict(bad)
        assert fresh.qweight is None and fresh.scales is None
    state = w4_state()
    state["zeros"] = torch.zeros(16, 2, dtype=torch.int32)
    with pytest.raises(RuntimeError, match="dtype mismatch for zeros"):
        QuantLinear(256, 16).load_state_dict(state)
    w8 = {"qweight": torch.zeros(16, 256, dtype=torch.int8), "scales": torch.ones(16, 2, dtype=torch.float16)}
    with pytest.raises(RuntimeError, match="size mismatch for scales"):
        QuantLinear(256, 16, scheme="w8a16").load_state_dict(w8)
    w8["scales"] = torch.ones(16, dtype=torch.float16)
    QuantLinear(256, 16, scheme="w8a16").load_state_dict(w8)


def test_bench_refuses_more_than_one_gpu():
    """The quantized linear is a one-GPU path: bench.py says so and exits non-zero for --gpus 2."""
    import subprocess
    import sys
    from pathlib import Path
    proc = subprocess.run([sys.executable, str(Path(__file__).resolve().parents[1] / "bench.py"), "--gpus", "2"],
                          capture_output=True, text=True, timeout=300)
    assert proc.returncode != 0 and "one GPU" in (proc.stderr + proc.stdout)
