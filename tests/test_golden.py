"""The committed small fixture (tests/golden/quant_small.npz) against the oracle (CPU) and the
HIP kernels (GPU).  Integer tensors must match bit for bit; matmul outputs within the tolerances."""

from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import qspec
from tests.helpers import MAX_ABS_TOL, REL_FRO_TOL, errors

FIXTURE = Path(__file__).parent / "golden" / "quant_small.npz"


@pytest.fixture(scope="module")
def gold():
    return dict(np.load(FIXTURE))


def _x(gold) -> torch.Tensor:
    return torch.from_numpy(gold["x_bf16_bits"].view(np.int16).copy()).view(torch.bfloat16)


def test_oracle_reproduces_fixture(gold):
    q8, s8 = qspec.quantize_w8(gold["weight"])
    assert np.array_equal(q8, gold["w8_q"]) and np.array_equal(s8.view(np.uint16), gold["w8_scales_bits"])
    q4, s4, z4 = qspec.quantize_w4_g128(gold["weight"])
    assert np.array_equal(qspec.pack_int4(q4), gold["w4_qweight"])
    assert np.array_equal(s4.view(np.uint16), gold["w4_scales_bits"]) and np.array_equal(z4, gold["w4_zeros"])
    w_hat = qspec.dequantize_w4(gold["w4_qweight"], gold["w4_scales_bits"].view(np.float16), gold["w4_zeros"])
    y = qspec.quant_linear(_x(gold), torch.from_numpy(w_hat), accumulate=torch.float64, out_dtype=torch.float64)
    assert np.array_equal(y.numpy(), gold["y_w4_f64"])
    w_hat8 = qspec.dequantize_w8(gold["w8_q"], gold["w8_scales_bits"].view(np.float16))
    y8 = qspec.quant_linear(_x(gold), torch.from_numpy(w_hat8), accumulate=torch.float64, out_dtype=torch.float64)
    assert np.array_equal(y8.numpy(), gold["y_w8_f64"])


def test_fixture_outputs_follow_from_its_integers(gold):
    """The stored fp64 outputs against a sum written out in Python floats from the stored integer
    tensors (no oracle function involved), so the fixture cannot drift together with the oracle."""
    x = _x(gold).double().numpy()
    q8 = gold["w8_q"].astype(np.int64)
    s8 = gold["w8_scales_bits"].view(np.float16).astype(np.float64)
    w_hat8 = (q8 * s8[:, None]).astype(np.float32).astype(np.float64)   # fp32 product is exact: no rounding
    assert np.array_equal(w_hat8, q8 * s8[:, None])
    want8 = x @ w_hat8.T
    assert np.allclose(gold["y_w8_f64"], want8, rtol=0, atol=1e-11)
    words = gold["w4_qweight"].view(np.uint32)
    q4 = np.stack([(words >> (4 * j)) & 15 for j in range(8)], axis=-1).reshape(words.shape[0], -1).astype(np.int64)
    s4 = np.repeat(gold["w4_scales_bits"].view(np.float16).astype(np.float64), 128, axis=1)
    z4 = np.repeat(gold["w4_zeros"].astype(np.int64), 128, axis=1)
    want4 = x @ ((q4 - z4) * s4).T
    assert np.allclose(gold["y_w4_f64"], want4, rtol=0, atol=1e-11)


@pytest.mark.gpu
def test_kernels_reproduce_fixture(gold, cuda):
    from ajllm_amd import quantize_w4_g128, quantize_w8, repack_w4, repack_w8, w4a16_matmul, w8a16_matmul

    w = torch.from_numpy(gold["weight"]).to(cuda)
    q8, s8 = quantize_w8(w)
    assert np.array_equal(q8.cpu().numpy(), gold["w8_q"])
    assert np.array_equal(s8.cpu().numpy().view(np.uint16), gold["w8_scales_bits"])
    qw, s4, z4 = quantize_w4_g128(w)
    assert np.array_equal(qw.cpu().numpy(), gold["w4_qweight"])
    assert np.array_equal(s4.cpu().numpy().view(np.uint16), gold["w4_scales_bits"])
    assert np.array_equal(z4.cpu().numpy(), gold["w4_zeros"])
    x = _x(gold).to(cuda)
    wq, meta = repack_w4(qw, s4, z4)
    wq8 = repack_w8(q8)
    for kernel in ("gemv", "gemm"):
        y4 = w4a16_matmul(x, wq, meta, torch.float32, kernel=kernel)
        y8 = w8a16_matmul(x, wq8, s8, torch.float32, kernel=kernel)
        for got, want in ((y4, gold["y_w4_f64"]), (y8, gold["y_w8_f64"])):
            max_abs, rel = errors(got, torch.from_numpy(want))
            assert max_abs <= MAX_ABS_TOL and rel <= REL_FRO_TOL
            assert max_abs <= 1e-4
