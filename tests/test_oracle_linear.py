"""Pins the oracle's dequantize + linear (CPU only)."""

import numpy as np
import pytest
import torch

from oracle import qspec
from tests.helpers import make_activations, make_weight


def _w4(n, k, seed):
    q, s, z = qspec.quantize_w4_g128(make_weight(n, k, seed).numpy())
    return q, s, z, qspec.pack_int4(q)


def test_one_hot_activation_reads_single_weights():
    """x = e_k returns column k of W_hat; each entry is (q - z) * s computed by hand in Python floats."""
    n, k = 8, 256
    q, s, z, packed = _w4(n, k, 1)
    w_hat = torch.from_numpy(qspec.dequantize_w4(packed, s, z))
    for col in (0, 127, 128, 255, 77):
        x = torch.zeros((1, k), dtype=torch.bfloat16)
        x[0, col] = 1.0
        y = qspec.quant_linear(x, w_hat, out_dtype=torch.float32)[0]
        for row in range(n):
            want = (int(q[row, col]) - int(z[row, col // 128])) * float(s[row, col // 128])
            assert float(y[row]) == np.float32(want)


def test_w8_one_hot_activation_reads_single_weights():
    """The W8 twin of the test above: x = e_k returns column k of W_hat, and each entry must equal
    int(q) * float(scale) computed in Python floats (an fp32 product of an integer below 2^7 and an
    fp16 value is exact, so any rounding inside dequantize_w8, e.g. a product formed in fp16, fails)."""
    n, k = 8, 256
    w = make_weight(n, k, 11).numpy()
    w[2] *= 37.0   # rows of different magnitude: different fp16 exponents of the scale
    w[5] *= 1e-3
    q, s = qspec.quantize_w8(w)
    w_hat_np = qspec.dequantize_w8(q, s)
    assert w_hat_np.dtype == np.float32
    for row in range(n):
        for col in range(k):
            assert float(w_hat_np[row, col]) == int(q[row, col]) * float(s[row])
    w_hat = torch.from_numpy(w_hat_np)
    for col in (0, 63, 64, 255, 131):
        x = torch.zeros((1, k), dtype=torch.bfloat16)
        x[0, col] = 1.0
        y = qspec.quant_linear(x, w_hat, out_dtype=torch.float32)[0]
        for row in range(n):
            assert float(y[row]) == int(q[row, col]) * float(s[row])
    # the product must differ from one formed in fp16 somewhere, or the test would pin nothing
    in_fp16 = (q.astype(np.float16) * s[:, None]).astype(np.float32)
    assert not np.array_equal(in_fp16, w_hat_np)


def test_w8_all_ones_activation_gives_row_sums():
    n, k = 16, 512
    q, s = qspec.quantize_w8(make_weight(n, k, 12).numpy())
    w_hat = torch.from_numpy(qspec.dequantize_w8(q, s))
    y = qspec.quant_linear(torch.ones((1, k), dtype=torch.bfloat16), w_hat, accumulate=torch.float64,
                           out_dtype=torch.float64)[0]
    for row in range(n):
        want = float(s[row]) * int(q[row].astype(np.int64).sum())
        assert abs(float(y[row]) - want) <= 1e-9 * max(1.0, abs(want))


def test_all_ones_activation_gives_row_sums():
    n, k = 16, 512
    q, s, z, packed = _w4(n, k, 2)
    w_hat = torch.from_numpy(qspec.dequantize_w4(packed, s, z))
    y = qspec.quant_linear(torch.ones((1, k), dtype=torch.bfloat16), w_hat, accumulate=torch.float64,
                           out_dtype=torch.float64)[0]
    for row in range(n):
        want = sum(
            float(s[row, g]) * (int(q[row, 128 * g:128 * (g + 1)].astype(np.int64).sum()) - 128 * int(z[row, g]))
            for g in range(k // 128)
        )
        assert abs(float(y[row]) - want) <= 1e-9


def test_linear_matches_explicit_triple_loop_on_tiny_input():
    n, k, m = 3, 128, 2
    q, s, z, packed = _w4(n, k, 3)
    x = make_activations(m, k, 4)
    w_hat = qspec.dequantize_w4(packed, s, z)
    y = qspec.quant_linear(x, torch.from_numpy(w_hat), accumulate=torch.float64, out_dtype=torch.float64)
    for i in range(m):
        for j in range(n):
            want = sum(float(x[i, t]) * float(w_hat[j, t]) for t in range(k))
            assert abs(float(y[i, j]) - want) <= 1e-12


def test_w8_linear_agrees_with_torch_int8pack_mm():
    """torch's own int8 weight-only matmul (bf16 scales) is the same math up to the scale dtype."""
    if not hasattr(torch, "_weight_int8pack_mm"):
        pytest.skip("torch._weight_int8pack_mm not in this build")
    n, k, m = 64, 256, 4
    w = make_weight(n, k, 5).numpy()
    q, s = qspec.quantize_w8(w)
    # use scales that are exact in bf16 so both paths see the same numbers
    s = (s.astype(np.float32).view(np.uint32) & 0xFFFF0000).view(np.float32).astype(np.float16)
    x = make_activations(m, k, 6)
    ours = qspec.quant_linear(x, torch.from_numpy(qspec.dequantize_w8(q, s)), out_dtype=torch.float32)
    theirs = torch._weight_int8pack_mm(x, torch.from_numpy(q), torch.from_numpy(s.astype(np.float32)).to(torch.bfloat16))
    assert torch.allclose(ours, theirs.float(), rtol=2e-2, atol=2e-2)  # theirs rounds to bf16
    assert (ours - theirs.float()).abs().max() <= 0.02


def test_leading_dimensions_and_output_dtype_follow_the_reference_linear():
    """Linear.forward (reference src/ajllm/modeling/layers.py:32-33) keeps leading dims and dtype."""
    layer = qspec.QuantLinearRef.from_weight(make_weight(32, 128, 7), "w4a16_g128")
    x = make_activations(6, 128, 8).reshape(2, 3, 128)
    y = layer(x)
    assert y.shape == (2, 3, 32) and y.dtype == torch.bfloat16
    dense = torch.nn.functional.linear(x.float(), layer.dequantized())
    assert torch.equal(y, dense.to(torch.bfloat16))
    layer8 = qspec.QuantLinearRef.from_weight(make_weight(32, 128, 7), "w8a16")
    assert layer8(x).shape == (2, 3, 32)
