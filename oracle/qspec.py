"""CPU oracle for the quantized linear path (test infrastructure, never shipped).

The reference project has no quantized layer: its only linear arithmetic is the
dense, bias-free ``inputs @ weight.T`` of ``Linear.forward``
(reference ``src/ajllm/modeling/layers.py:32-33``).  The quantization scheme is
therefore specified here, from the wording of the benchmark configurations
("int8 per-output-channel symmetric, scale = absmax/127, fp16 scales";
"int4 asymmetric group-size 128 along K, fp16 scale + uint4 zero-point per
group, 8 nibbles packed per int32") and the conventional asymmetric min/max
recipe.  All arithmetic that decides an integer result is IEEE binary32 with
round-to-nearest-even; ``rint`` is round-half-to-even.

Pinning status (what independent evidence each function has, see
``tests/test_oracle_*.py``):

* ``quantize_w8`` / ``quantize_w4_g128`` / ``pack_int4`` / ``unpack_int4``:
  pinned by closed forms (exact grids, ties, constant rows), by a pure-Python
  restatement that uses only ``struct`` rounding and ``fractions``, and by
  exhaustive per-nibble pack patterns.
* ``dequantize_*`` and ``quant_linear``: pinned by one-hot / all-ones
  activations that read single weights and row sums back exactly, by an fp64
  recomputation, and (W8) by ``torch._weight_int8pack_mm``.
* Nothing here is pinned by the reference project's own tests: it holds no
  vector, fixture or known answer for any linear layer -> "parity unpinned by
  the reference"; the checks above are what stand in for it.
"""

from __future__ import annotations

import numpy as np
import torch

GROUP = 128  # int4 group length along K
NIBBLES_PER_WORD = 8


# ----------------------------------------------------------------------------
# W8: int8, per-output-channel, symmetric
# ----------------------------------------------------------------------------
def quantize_w8(weight: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
    """``weight`` fp32 [N, K] -> (q int8 [N, K], scales fp16 [N]).

    amax = max_k |W|;  scale = fp16(amax / 127);  d = fp32(scale) (1 where the
    scale is 0);  q = clamp(rint(W / d), -127, 127).
    """
    w = np.ascontiguousarray(weight, dtype=np.float32)
    if w.ndim != 2:
        raise ValueError("weight must be [N, K]")
    amax = np.max(np.abs(w), axis=1)
    with np.errstate(over="ignore"):
        scales = (amax / np.float32(127.0)).astype(np.float16)
    d = scales.astype(np.float32)
    d = np.where(d == 0, np.float32(1.0), d).astype(np.float32)
    q = np.rint(w / d[:, None])
    q = np.clip(q, -127.0, 127.0).astype(np.int8)
    return q, scales


def dequantize_w8(q: np.ndarray, scales: np.ndarray) -> np.ndarray:
    """fp32 [N, K] = q * fp32(scale[n])."""
    return q.astype(np.float32) * scales.astype(np.float32)[:, None]


# ----------------------------------------------------------------------------
# W4: uint4, asymmetric, groups of 128 along K
# ----------------------------------------------------------------------------
def quantize_w4_g128(weight: np.ndarray) -> tuple[np.ndarray, np.ndarray, np.ndarray]:
    """``weight`` fp32 [N, K], K % 128 == 0 ->
    (q uint8 [N, K] in 0..15, scales fp16 [N, K/128], zeros uint8 [N, K/128] in 0..15).

    Per row and group: mn, mx = min, max;  scale = fp16((mx - mn) / 15);
    d = fp32(scale) (1 where 0);  zero = clamp(rint(-mn / d), 0, 15);
    q = clamp(rint(W / d) + zero, 0, 15).
    """
    w = np.ascontiguousarray(weight, dtype=np.float32)
    if w.ndim != 2 or w.shape[1] % GROUP != 0:
        raise ValueError("weight must be [N, K] with K a multiple of 128")
    n, k = w.shape
    g = w.reshape(n, k // GROUP, GROUP)
    mn = g.min(axis=2)
    mx = g.max(axis=2)
    with np.errstate(over="ignore"):
        scales = ((mx - mn) / np.float32(15.0)).astype(np.float16)
    d = scales.astype(np.float32)
    d = np.where(d == 0, np.float32(1.0), d).astype(np.float32)
    zeros_f = np.clip(np.rint(-mn / d), 0.0, 15.0).astype(np.float32)
    q = np.rint(g / d[:, :, None]) + zeros_f[:, :, None]
    q = np.clip(q, 0.0, 15.0).astype(np.uint8).reshape(n, k)
    return q, scales, zeros_f.astype(np.uint8)


def pack_int4(q: np.ndarray) -> np.ndarray:
    """uint8 [N, K] (values 0..15) -> int32 [N, K/8]; nibble j of a word is
    element 8c+j (little-nibble order): word = sum_j q[8c+j] << 4j."""
    q = np.asarray(q)
    if q.ndim != 2 or q.shape[1] % NIBBLES_PER_WORD != 0:
        raise ValueError("q must be [N, K] with K a multiple of 8")
    if q.size and (q.min() < 0 or q.max() > 15):
        raise ValueError("nibble out of range")
    n, k = q.shape
    v = q.astype(np.uint32).reshape(n, k // 8, 8)
    word = np.zeros((n, k // 8), dtype=np.uint32)
    for j in range(8):
        word |= v[:, :, j] << np.uint32(4 * j)
    return word.view(np.int32)


def unpack_int4(qweight: np.ndarray) -> np.ndarray:
    """int32 [N, K/8] -> uint8 [N, K], inverse of :func:`pack_int4`."""
    word = np.ascontiguousarray(qweight, dtype=np.int32).view(np.uint32)
    n, c = word.shape
    out = np.empty((n, c, 8), dtype=np.uint8)
    for j in range(8):
        out[:, :, j] = (word >> np.uint32(4 * j)) & np.uint32(0xF)
    return out.reshape(n, c * 8)


def dequantize_w4(qweight: np.ndarray, scales: np.ndarray, zeros: np.ndarray) -> np.ndarray:
    """fp32 [N, K] = (q - zero[n, k // 128]) * fp32(scale[n, k // 128])."""
    q = unpack_int4(qweight).astype(np.float32)
    n, k = q.shape
    s = np.repeat(scales.astype(np.float32), GROUP, axis=1)
    z = np.repeat(zeros.astype(np.float32), GROUP, axis=1)
    return (q - z) * s


# ----------------------------------------------------------------------------
# the linear itself
# ----------------------------------------------------------------------------
def quant_linear(x: torch.Tensor, w_hat: torch.Tensor, *, accumulate: torch.dtype = torch.float32,
                 out_dtype: torch.dtype | None = None) -> torch.Tensor:
    """y = x.to(acc) @ w_hat.to(acc).T, cast to ``out_dtype`` (default x.dtype).

    Mirrors ``Linear.forward`` (reference ``src/ajllm/modeling/layers.py:32-33``)
    with the dequantized weight kept in fp32 (never rounded to bf16)."""
    lead = x.shape[:-1]
    y = x.reshape(-1, x.shape[-1]).to(accumulate) @ w_hat.to(accumulate).t()
    return y.to(out_dtype or x.dtype).reshape(*lead, w_hat.shape[0])


class QuantLinearRef(torch.nn.Module):
    """Oracle twin of the product's ``QuantLinear``: same buffers, CPU math.

    ``scheme`` is ``"w4a16_g128"`` or ``"w8a16"``.  ``forward`` dequantizes on
    every call unless ``cache_dequant`` is set."""

    def __init__(self, in_features: int, out_features: int, scheme: str, cache_dequant: bool = True):
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.scheme = scheme
        self.cache_dequant = cache_dequant
        self._w_hat: torch.Tensor | None = None

    @classmethod
    def from_weight(cls, weight: torch.Tensor, scheme: str, cache_dequant: bool = True) -> "QuantLinearRef":
        n, k = weight.shape
        self = cls(k, n, scheme, cache_dequant)
        w = weight.detach().float().cpu().numpy()
        if scheme == "w8a16":
            q, s = quantize_w8(w)
            self.register_buffer("qweight", torch.from_numpy(q))
            self.register_buffer("scales", torch.from_numpy(s))
            self.register_buffer("zeros", torch.empty(0, dtype=torch.uint8))
        elif scheme == "w4a16_g128":
            q, s, z = quantize_w4_g128(w)
            self.register_buffer("qweight", torch.from_numpy(pack_int4(q)))
            self.register_buffer("scales", torch.from_numpy(s))
            self.register_buffer("zeros", torch.from_numpy(z))
        else:
            raise ValueError(f"unknown scheme {scheme}")
        return self

    @classmethod
    def from_linear(cls, linear: torch.nn.Module, scheme: str) -> "QuantLinearRef":
        return cls.from_weight(linear.weight.data, scheme)

    def dequantized(self) -> torch.Tensor:
        if self._w_hat is not None:
            return self._w_hat
        if self.scheme == "w8a16":
            w = dequantize_w8(self.qweight.numpy(), self.scales.numpy())
        else:
            w = dequantize_w4(self.qweight.numpy(), self.scales.numpy(), self.zeros.numpy())
        w = torch.from_numpy(w)
        if self.cache_dequant:
            self._w_hat = w
        return w

    def forward(self, inputs: torch.Tensor) -> torch.Tensor:
        # "A16": the activations the matmul sees are bf16; other input dtypes are rounded to
        # bf16 first and the fp32-accumulated result is returned in the input's dtype.
        x = inputs if inputs.dtype == torch.bfloat16 else inputs.to(torch.bfloat16)
        return quant_linear(x, self.dequantized(), out_dtype=inputs.dtype)
