"""ctypes binding of ``libajq.so`` (declared in ``include/ajq.h``).

The library is loaded lazily and is never built from here: a missing library is
an error the caller sees (``python -m ajllm_amd.build`` makes it).  There is no
CPU or PyTorch fallback behind any of these calls.
"""

from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_float, c_int, c_size_t, c_void_p
from pathlib import Path

LIBRARY_PATH = Path(__file__).resolve().parent / "libajq.so"

AJQ_OUT_BF16 = 0
AJQ_OUT_F32 = 1
AJQ_KV_F32 = 0
AJQ_KV_BF16 = 1

# status -> exception class; argument errors are ValueError (the reference CLI turns
# ValueError into a clean exit, src/ajllm/cli.py:57-60), runtime errors RuntimeError.
_ARGUMENT_ERRORS = {-1, -2, -3, -4, -6}

# name -> (restype, argtypes); one entry per declaration in include/ajq.h
SIGNATURES: dict[str, tuple] = {
    "ajq_version": (c_int, []),
    "ajq_last_error": (c_char_p, []),
    "ajq_status_string": (c_char_p, [c_int]),
    "ajq_gemm_gate_supported": (c_int, [c_int, c_int, c_int, c_int]),
    "ajq_w4a16_gemm_gate": (c_int, [c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_size_t,
                                    c_void_p]),
    "ajq_w8a16_gemm_gate": (c_int, [c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_void_p, c_void_p]),
    "ajq_quantize_w8": (c_int, [c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p]),
    "ajq_quantize_w4_g128": (c_int, [c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
    "ajq_repack_w4": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p]),
    "ajq_unrepack_w4": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
    "ajq_repack_w8": (c_int, [c_void_p, c_int, c_int, c_void_p, c_void_p]),
    "ajq_unrepack_w8": (c_int, [c_void_p, c_int, c_int, c_void_p, c_void_p]),
    "ajq_w4a16_gemv": (c_int, [c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p]),
    "ajq_w8a16_gemv": (c_int, [c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p]),
    "ajq_w4a16_gemm_workspace_bytes": (c_size_t, [c_int, c_int]),
    "ajq_w4a16_gemm_workspace_bytes_for": (c_size_t, [c_int, c_int, c_int]),
    "ajq_w4a16_gemm": (
        c_int,
        [c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p, c_size_t, c_void_p],
    ),
    "ajq_w8a16_gemm": (c_int, [c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p]),
    "ajq_noalloc_scratch_bytes": (c_size_t, []),
    "ajq_w4a16_gemm_noalloc": (c_int, [c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p]),
    "ajq_add_rmsnorm": (c_int, [c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_int, c_int, c_void_p]),
    "ajq_rope_cache": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int,
         c_int, c_void_p],
    ),
    "ajq_attn_decode_workspace_bytes": (c_size_t, [c_int, c_int]),
    "ajq_attn_row_chunks": (c_int, [c_int, c_int, c_int]),
    "ajq_rope_prefill": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
         c_int, c_void_p],
    ),
    "ajq_attn_prefill": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_int, c_void_p],
    ),
    "ajq_greedy_pick": (
        c_int,
        [c_void_p, c_int, c_int, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
         c_void_p, c_void_p],
    ),
    "ajq_sample_pick": (
        c_int,
        [c_void_p, c_int, c_int, c_int, c_float, c_float, c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p,
         c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p],
    ),
    "ajq_gemv_merge_max_splits": (c_int, [c_int, c_int]),
    "ajq_w4a16_gemv_merge": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p]),
    "ajq_w8a16_gemv_merge": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p]),
    "ajq_attn_step_partial": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
         c_int, c_void_p, c_void_p, c_size_t, c_void_p],
    ),
    "ajq_gemv_fused_supported": (c_int, [c_int, c_int]),
    "ajq_w4a16_gemv_norm": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_void_p, c_int,
         c_void_p],
    ),
    "ajq_w8a16_gemv_norm": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_void_p, c_int,
         c_void_p],
    ),
    "ajq_gemv_epilogue_supported": (c_int, [c_int, c_int]),
    "ajq_gemv_rowscale_supported": (c_int, [c_int, c_int]),
    "ajq_matmul_workspace_bytes": (c_size_t, []),
    "ajq_matmul_workspace_set": (c_int, [c_void_p, c_size_t]),
    "ajq_w4a16_gemv_residual": (c_int, [c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p,
                                        c_void_p, c_void_p, c_void_p]),
    "ajq_w8a16_gemv_residual": (c_int, [c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p,
                                        c_void_p, c_void_p, c_void_p]),
    "ajq_w4a16_gemv_gated": (c_int, [c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_void_p, c_void_p]),
    "ajq_w8a16_gemv_gated": (c_int, [c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_void_p, c_void_p]),
    "ajq_w4a16_gemv_norm_sums": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_float, c_int, c_int, c_void_p, c_void_p,
                                         c_int, c_void_p, c_int, c_int, c_void_p]),
    "ajq_w8a16_gemv_norm_sums": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_float, c_int, c_int, c_void_p, c_void_p,
                                         c_int, c_void_p, c_int, c_int, c_void_p]),
    "ajq_w4a16_gemv_merge_residual": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                                              c_void_p, c_void_p, c_void_p, c_void_p]),
    "ajq_w8a16_gemv_merge_residual": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                                              c_void_p, c_void_p, c_void_p, c_void_p]),
    "ajq_w4a16_gemv_rowscale": (c_int, [c_void_p, c_void_p, c_int, c_float, c_int, c_int, c_void_p, c_void_p, c_int,
                                        c_void_p, c_int, c_int, c_void_p]),
    "ajq_w8a16_gemv_rowscale": (c_int, [c_void_p, c_void_p, c_int, c_float, c_int, c_int, c_void_p, c_void_p, c_int,
                                        c_void_p, c_int, c_int, c_void_p]),
    "ajq_w4a16_gemv_gate": (c_int, [c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p]),
    "ajq_w8a16_gemv_gate": (c_int, [c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p]),
    "ajq_attn_step_workspace_bytes": (c_size_t, [c_int, c_int]),
    "ajq_attn_step": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
         c_void_p, c_void_p, c_size_t, c_void_p],
    ),
    "ajq_attn_decode": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p,
         c_size_t, c_void_p],
    ),
    "ajq_swiglu": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p]),
}

# libajq_bench.so (include/ajq_bench.h): the device yardstick for bench.py, not an operator
BENCH_LIBRARY_PATH = Path(__file__).resolve().parent / "libajq_bench.so"


BENCH_SIGNATURES: dict[str, tuple] = {
    "ajqb_last_error": (c_char_p, []),
    "ajqb_mfma_rate": (c_int, [c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
}

_lib: ctypes.CDLL | None = None
_bench_lib: ctypes.CDLL | None = None


def load_bench() -> ctypes.CDLL:
    """The bench-only probe library, bound on first use (built by ``python -m ajllm_amd.build``)."""
    global _bench_lib
    if _bench_lib is not None:
        return _bench_lib
    if not BENCH_LIBRARY_PATH.exists():
        raise RuntimeError(f"{BENCH_LIBRARY_PATH} is missing: build it with `python -m ajllm_amd.build`")
    lib = ctypes.CDLL(str(BENCH_LIBRARY_PATH))
    for name, (restype, argtypes) in BENCH_SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    _bench_lib = lib
    return lib


def load() -> ctypes.CDLL:
    """Return the loaded library, binding every signature on first use."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIBRARY_PATH.exists():
        raise RuntimeError(
            f"{LIBRARY_PATH} is missing: build it with `python -m ajllm_amd.build` "
            "(the quantized linear has no fallback path)"
        )
    lib = ctypes.CDLL(str(LIBRARY_PATH))
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def check(status: int, what: str) -> None:
    """Raise the exception that matches a negative ajq_status."""
    if status == 0:
        return
    lib = load()
    message = lib.ajq_last_error().decode() or lib.ajq_status_string(status).decode()
    if status in _ARGUMENT_ERRORS:
        raise ValueError(f"{what}: {message}")
    raise RuntimeError(f"{what}: {message}")
