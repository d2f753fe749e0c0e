"""GPU quantize/pack and repack kernels against the CPU oracle: bit-exact."""

import numpy as np
import pytest
import torch

from oracle import qspec
from tests.helpers import make_weight, tie_and_division_rows

pytestmark = pytest.mark.gpu


def _special_rows(k: int) -> torch.Tensor:
    """Rows that hit the corners of the scheme: zeros, constants, ties, tiny and huge values."""
    g = torch.Generator().manual_seed(7)
    rows = [
        torch.zeros(k),
        torch.full((k,), 0.3),
        torch.full((k,), -1e-9),
        torch.linspace(-1.0, 1.0, k),
        torch.arange(k, dtype=torch.float32) % 16 * 0.125,          # exact grid
        (torch.arange(k, dtype=torch.float32) % 31 - 15) * 0.5 * 0.0625,  # half-way points
        torch.randn(k, generator=g) * 1e-7,                          # fp16-subnormal scales
        torch.randn(k, generator=g) * 300.0,
        torch.randn(k, generator=g).abs() * 0.02,                    # one-signed group
        -torch.randn(k, generator=g).abs() * 0.02,
    ]
    return torch.cat([torch.stack(rows).float(), torch.from_numpy(tie_and_division_rows(k))])


@pytest.mark.parametrize("n,k,seed", [(16, 128, 1), (64, 1024, 2), (4096, 4096, 3), (1000, 2048, 4)])
def test_quantize_w8_bit_exact(cuda, n, k, seed):
    from ajllm_amd import quantize_w8

    w = make_weight(n, k, seed)
    q_ref, s_ref = qspec.quantize_w8(w.numpy())
    q, s = quantize_w8(w.to(cuda))
    assert np.array_equal(q.cpu().numpy(), q_ref)
    assert np.array_equal(s.cpu().numpy().view(np.uint16), s_ref.view(np.uint16))


@pytest.mark.parametrize("n,k,seed", [(16, 128, 1), (64, 1024, 2), (4096, 4096, 3), (1000, 2048, 4), (4096, 14336, 5)])
def test_quantize_w4_bit_exact(cuda, n, k, seed):
    from ajllm_amd import quantize_w4_g128

    w = make_weight(n, k, seed)
    q_ref, s_ref, z_ref = qspec.quantize_w4_g128(w.numpy())
    qw, s, z = quantize_w4_g128(w.to(cuda))
    assert np.array_equal(qw.cpu().numpy(), qspec.pack_int4(q_ref))
    assert np.array_equal(s.cpu().numpy().view(np.uint16), s_ref.view(np.uint16))
    assert np.array_equal(z.cpu().numpy(), z_ref)


def test_quantize_special_rows_bit_exact(cuda):
    from ajllm_amd import quantize_w4_g128, quantize_w8

    w = _special_rows(512)
    q_ref, s_ref = qspec.quantize_w8(w.numpy())
    q, s = quantize_w8(w.to(cuda))
    assert np.array_equal(q.cpu().numpy(), q_ref)
    assert np.array_equal(s.cpu().numpy().view(np.uint16), s_ref.view(np.uint16))
    q4_ref, s4_ref, z4_ref = qspec.quantize_w4_g128(w.numpy())
    qw, s4, z4 = quantize_w4_g128(w.to(cuda))
    assert np.array_equal(qw.cpu().numpy(), qspec.pack_int4(q4_ref))
    assert np.array_equal(s4.cpu().numpy().view(np.uint16), s4_ref.view(np.uint16))
    assert np.array_equal(z4.cpu().numpy(), z4_ref)


@pytest.mark.parametrize("n,k", [(16, 128), (48, 512), (4096, 4096), (1000, 256)])
def test_repack_w4_round_trip(cuda, n, k):
    from ajllm_amd import repack_w4, unrepack_w4

    rng = np.random.default_rng(n + k)
    qweight = torch.from_numpy(rng.integers(-2**31, 2**31, size=(n, k // 8), dtype=np.int64).astype(np.int32)).to(cuda)
    scales = torch.from_numpy(rng.integers(0, 0x7C00, size=(n, k // 128), dtype=np.uint16).view(np.float16)).to(cuda)
    zeros = torch.from_numpy(rng.integers(0, 16, size=(n, k // 128), dtype=np.uint8)).to(cuda)
    wq, meta = repack_w4(qweight, scales, zeros)
    assert wq.numel() * 4 == ((n + 15) // 16 * 16) * k // 2
    q2, s2, z2 = unrepack_w4(wq, meta)
    assert torch.equal(q2[:n], qweight)
    assert torch.equal(s2[:n].view(torch.int16), scales.view(torch.int16))
    assert torch.equal(z2[:n], zeros)
    assert int(q2[n:].abs().sum()) == 0


def test_repack_w4_layout_matches_header(cuda):
    """Element (tile, lane=16*kc+nl, dword j) holds k = 128g+32j+8kc+e, weight e in nibble (e>>1)+4*(e&1)."""
    from ajllm_amd import repack_w4

    n, k = 32, 256
    rng = np.random.default_rng(0)
    q = rng.integers(0, 16, size=(n, k), dtype=np.uint8)
    qweight = torch.from_numpy(qspec.pack_int4(q)).to(cuda)
    scales = torch.ones((n, k // 128), dtype=torch.float16, device=cuda)
    zeros = torch.zeros((n, k // 128), dtype=torch.uint8, device=cuda)
    wq, _ = repack_w4(qweight, scales, zeros)
    wq = wq.cpu().numpy().view(np.uint32)
    for nt, g, lane, j in [(0, 0, 0, 0), (1, 1, 63, 3), (0, 1, 17, 2), (1, 0, 40, 1)]:
        nl, kc = lane % 16, lane // 16
        word = int(wq[nt, g, lane, j])
        for e in range(8):
            nib = (word >> (4 * ((e >> 1) + 4 * (e & 1)))) & 0xF
            assert nib == q[16 * nt + nl, 128 * g + 32 * j + 8 * kc + e]


@pytest.mark.parametrize("n,k", [(16, 128), (48, 512), (4096, 4096), (1000, 384)])
def test_repack_w8_round_trip(cuda, n, k):
    from ajllm_amd import repack_w8, unrepack_w8

    rng = np.random.default_rng(n * 3 + k)
    q = torch.from_numpy(rng.integers(-128, 128, size=(n, k), dtype=np.int8)).to(cuda)
    wq = repack_w8(q)
    q2 = unrepack_w8(wq)
    assert torch.equal(q2[:n], q)
    assert int(q2[n:].abs().sum()) == 0
