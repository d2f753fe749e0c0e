"""Host side of the library's causal prefill attention (``ajq_attn_prefill``).

Stands where the reference switches to its FlashAttention under ``use_flash_attention``
(src/ajllm/modeling/attention.py:106-117; its own kernels, flash_attention.py:44-108,194-298, need
CUDA/Triton).  Same contract as there: the arithmetic is flash attention's (bf16 products, fp32
online softmax), not bit-for-bit the eager fp32 one, so it is opt-in.
"""

from __future__ import annotations

import torch

from . import _lib


def flash_prefill(q: torch.Tensor, keys: torch.Tensor, values: torch.Tensor, start: int,
                  out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """Causal attention of the ``T`` new positions ``start .. start + T - 1``.

    ``q`` fp32 ``[B, H, T, hd]`` (rotated; hd 128, 64 or 32); ``keys`` / ``values`` ``[B, Hkv, max_len, hd]`` fp32 or
    bf16 whose rows ``0 .. start + T - 1`` are filled (a KV cache, or the keys and values themselves
    with ``start == 0``).  Returns ``[B, T, H * hd]`` in ``out_dtype`` (fp32, or bf16 = its rounding)."""
    if not q.is_cuda:
        raise ValueError("flash_prefill needs tensors on a ROCm device (there is no CPU path)")
    batch, heads, seq, hd = q.shape
    kv_heads, max_len = keys.shape[1], keys.shape[2]
    if hd not in (128, 64, 32) or keys.shape != values.shape or keys.shape[0] != batch or keys.shape[3] != hd:
        raise ValueError("flash_prefill: q [B, H, T, hd] and caches [B, Hkv, max_len, hd] with hd 128, 64 or 32 expected")
    if keys.dtype not in (torch.float32, torch.bfloat16) or values.dtype != keys.dtype:
        raise ValueError("flash_prefill: the caches must be float32 or bfloat16")
    if not (keys.is_contiguous() and values.is_contiguous()):
        raise ValueError("flash_prefill: the caches must be contiguous")
    if out_dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("flash_prefill: out_dtype must be float32 or bfloat16")
    q = q.float().contiguous()
    out = torch.empty((batch, seq, heads * hd), dtype=out_dtype, device=q.device)
    flag = _lib.AJQ_KV_F32 if keys.dtype == torch.float32 else _lib.AJQ_KV_BF16
    with torch.cuda.device(q.device):
        status = _lib.load().ajq_attn_prefill(q.data_ptr(), keys.data_ptr(), values.data_ptr(), flag, batch, heads,
                                              kv_heads, seq, start, max_len, hd, out.data_ptr(),
                                              _lib.AJQ_OUT_F32 if out_dtype == torch.float32 else _lib.AJQ_OUT_BF16,
                                              torch.cuda.current_stream().cuda_stream)
    _lib.check(status, "attn_prefill")
    return out
