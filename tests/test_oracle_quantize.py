"""Pins the numpy oracle of the quantize/pack scheme (CPU only).

Three kinds of evidence, none of which retypes the oracle's own expression:
closed forms whose answer is known in advance, an independent pure-Python
restatement (tests/pyspec.py), and invariants every correct quantizer obeys.
"""

import numpy as np
import pytest

from oracle import qspec
from tests import pyspec
from tests.helpers import W4_DIVISION_CASES, W4_ZERO_DIVISION_CASES, W8_DIVISION_CASES


# ------------------------------------------------------------------ W8 closed forms
def test_w8_exact_grid_quantizes_to_itself():
    d = 2.0**-6
    row = np.arange(-127, 128, dtype=np.float32) * d  # absmax = 127 d, so scale = d exactly
    row = np.concatenate([row, np.zeros(1, np.float32)])
    q, s = qspec.quantize_w8(row[None, :])
    assert float(s[0]) == d
    assert np.array_equal(q[0, :255], np.arange(-127, 128))
    assert q[0, 255] == 0


def test_w8_ties_round_half_to_even():
    d = 2.0**-4
    body = (np.arange(-8, 8, dtype=np.float32) + 0.5) * d  # ... -0.5d, 0.5d, 1.5d, 2.5d ...
    row = np.concatenate([body, np.array([127 * d], np.float32)])
    q, s = qspec.quantize_w8(row[None, :])
    assert float(s[0]) == d
    # half-way cases go to the even neighbour: -7.5 -> -8, -0.5 -> -0, 0.5 -> 0, 1.5 -> 2, 2.5 -> 2
    assert list(q[0, :16]) == [-8, -6, -6, -4, -4, -2, -2, 0, 0, 2, 2, 4, 4, 6, 6, 8]


def test_w8_zero_row_and_clamp():
    w = np.zeros((2, 8), np.float32)
    w[1] = [1e30, -1e30, 1.0, -1.0, 0, 0, 0, 0]  # scale overflows fp16 -> inf -> every q is 0
    q, s = qspec.quantize_w8(w)
    assert float(s[0]) == 0.0 and not q[0].any()
    assert np.isinf(s[1]) and not q[1].any()


def test_w8_absmax_element_is_127_or_126_and_error_is_half_a_step():
    rng = np.random.default_rng(5)
    w = (rng.standard_normal((256, 512)) * 0.02).astype(np.float32)
    q, s = qspec.quantize_w8(w)
    d = s.astype(np.float32)
    assert np.abs(q).max() <= 127
    top = np.abs(q).max(axis=1)
    assert set(np.unique(top)) <= {126, 127}  # fp16 rounding of the scale moves absmax/d by < 1
    err = np.abs(w - q.astype(np.float32) * d[:, None])
    unclamped = np.abs(w / d[:, None]) <= 127.0
    assert (err[unclamped] <= d[:, None].repeat(512, 1)[unclamped] * 0.5 * (1 + 1e-6)).all()


def test_w8_scale_is_fp16_of_fp32_quotient_for_every_exponent():
    """Sweep absmax over many magnitudes incl. fp16-subnormal scales; compare with struct rounding."""
    rng = np.random.default_rng(1)
    amax = np.concatenate([2.0 ** rng.uniform(-30, 15, 2000), [6e-8 * 127, 5.96e-8 * 127 * 0.5, 65504.0 * 127]])
    w = np.zeros((len(amax), 4), np.float32)
    w[:, 0] = amax
    _, s = qspec.quantize_w8(w)
    for i in range(len(amax)):
        want = pyspec.f16(pyspec.f32(pyspec.f32(float(w[i, 0])) / 127.0))
        assert float(s[i]) == want or (np.isinf(s[i]) and np.isinf(want))


# ------------------------------------------------------------------ W4 closed forms
def test_w4_exact_grid_gives_known_codes_scale_and_zero():
    d = 2.0**-5
    for zero in (0, 5, 15):
        codes = np.arange(128) % 16
        group = ((codes - zero) * d).astype(np.float32)  # min = -zero*d, max = (15-zero)*d
        q, s, z = qspec.quantize_w4_g128(group[None, :])
        assert float(s[0, 0]) == d and int(z[0, 0]) == zero
        assert np.array_equal(q[0], codes)


def test_w4_ties_round_half_to_even_before_the_zero_point_is_added():
    d = 2.0**-3
    group = np.zeros(128, np.float32)
    group[0], group[1] = -4 * d, 11 * d  # range 15 d -> scale d, zero 4
    group[2:8] = np.array([0.5, 1.5, 2.5, -0.5, -1.5, -2.5], np.float32) * d
    q, s, z = qspec.quantize_w4_g128(group[None, :])
    assert float(s[0, 0]) == d and int(z[0, 0]) == 4
    # rint(0.5)=0, rint(1.5)=2, rint(2.5)=2, rint(-0.5)=-0, rint(-1.5)=-2, rint(-2.5)=-2, then +4
    assert list(q[0, :8]) == [0, 15, 4, 6, 6, 4, 2, 2]


def test_w4_ties_with_an_odd_zero_point_round_before_the_zero_point_is_added():
    """With an odd zero-point rint(x) + zero and rint(x + zero) differ at every tie."""
    d = 2.0**-3
    group = np.zeros(128, np.float32)
    group[0], group[1] = -5 * d, 10 * d  # range 15 d -> scale d, zero 5
    group[2:8] = np.array([0.5, 1.5, 2.5, -0.5, -1.5, -2.5], np.float32) * d
    q, s, z = qspec.quantize_w4_g128(group[None, :])
    assert float(s[0, 0]) == d and int(z[0, 0]) == 5
    # rint: 0.5 -> 0, 1.5 -> 2, 2.5 -> 2, -0.5 -> -0, -1.5 -> -2, -2.5 -> -2, then + 5
    # (rounding x + 5 instead would give 6, 6, 8, 4, 4, 2)
    assert list(q[0, :8]) == [0, 15, 5, 7, 7, 5, 3, 3]
    assert list(q[0, :8]) == pyspec.quantize_w4_group([float(v) for v in group])[0][:8]


@pytest.mark.parametrize("below,zero", [(2.5, 2), (3.5, 4), (4.5, 4), (0.5, 0), (14.5, 14)])
def test_w4_zero_point_ties_round_half_to_even(below, zero):
    """-min/d exactly on a half: the zero-point is the even neighbour (half-up would give floor + 1)."""
    d = 2.0**-4
    group = np.zeros(128, np.float32)
    group[0], group[1] = -below * d, (15 - below) * d  # max - min = 15 d -> scale d
    q, s, z = qspec.quantize_w4_g128(group[None, :])
    assert float(s[0, 0]) == d
    assert int(z[0, 0]) == zero
    assert int(z[0, 0]) == pyspec.quantize_w4_group([float(v) for v in group])[2]


@pytest.mark.parametrize("scale,weight,by_division,by_reciprocal", W8_DIVISION_CASES)
def test_w8_divides_rather_than_multiplying_by_a_reciprocal(scale, weight, by_division, by_reciprocal):
    d = np.float32(np.float16(scale))
    w = np.float32(float.fromhex(weight))
    assert int(np.rint(w * (np.float32(1.0) / d))) == by_reciprocal != by_division  # the case does discriminate
    row = np.zeros(16, np.float32)
    row[0], row[1] = np.float32(127.0) * d, w  # 127 d is exact in binary32, so the scale is d
    q, s = qspec.quantize_w8(row[None, :])
    assert np.float32(s[0]) == d
    assert int(q[0, 1]) == by_division
    q_py, s_py = pyspec.quantize_w8_row([float(v) for v in row])
    assert q_py[1] == by_division and s_py == float(d)


@pytest.mark.parametrize("scale,weight,by_division,by_reciprocal", W4_DIVISION_CASES)
def test_w4_codes_divide_rather_than_multiplying_by_a_reciprocal(scale, weight, by_division, by_reciprocal):
    d = np.float32(np.float16(scale))
    w = np.float32(float.fromhex(weight))
    assert int(np.rint(w * (np.float32(1.0) / d))) + 5 == by_reciprocal != by_division
    group = np.zeros(128, np.float32)
    group[0], group[1], group[2] = np.float32(-5.0) * d, np.float32(10.0) * d, w
    q, s, z = qspec.quantize_w4_g128(group[None, :])
    assert np.float32(s[0, 0]) == d and int(z[0, 0]) == 5
    assert int(q[0, 2]) == by_division
    q_py, s_py, z_py = pyspec.quantize_w4_group([float(v) for v in group])
    assert q_py[2] == by_division and s_py == float(d) and z_py == 5


@pytest.mark.parametrize("scale,mn,mx,by_division,by_reciprocal", W4_ZERO_DIVISION_CASES)
def test_w4_zero_point_divides_rather_than_multiplying_by_a_reciprocal(scale, mn, mx, by_division, by_reciprocal):
    d = np.float32(np.float16(scale))
    lo, hi = np.float32(float.fromhex(mn)), np.float32(float.fromhex(mx))
    assert int(np.rint(-lo * (np.float32(1.0) / d))) == by_reciprocal != by_division
    group = np.zeros(128, np.float32)
    group[0], group[1] = lo, hi
    _, s, z = qspec.quantize_w4_g128(group[None, :])
    assert np.float32(s[0, 0]) == d
    assert int(z[0, 0]) == by_division
    assert pyspec.quantize_w4_group([float(v) for v in group])[2] == by_division


def test_w4_constant_group_and_one_signed_group():
    w = np.zeros((1, 384), np.float32)
    w[0, 128:256] = 0.3            # constant: scale 0 -> divisor 1, zero = clamp(rint(-0.3)) = 0, q = 0
    w[0, 256:384] = np.linspace(1.0, 2.5, 128)  # positive only: zero clamps to 0, codes saturate at 15
    q, s, z = qspec.quantize_w4_g128(w)
    assert float(s[0, 0]) == 0.0 and float(s[0, 1]) == 0.0
    assert not q[0, :256].any() and not z[0, :2].any()
    assert float(s[0, 2]) == float(np.float16(np.float32(1.5) / np.float32(15)))
    # zero clamps to 0, so the codes are rint(w / 0.1) saturated at 15: 1.0 -> 10, >= 1.56 -> 15
    codes = q[0, 256:384].astype(int)
    assert int(z[0, 2]) == 0 and codes[0] == 10 and (np.diff(codes) >= 0).all()
    assert (codes[w[0, 256:384] >= 1.56] == 15).all() and codes.max() == 15


def test_w4_invariants_on_gaussian_weights():
    rng = np.random.default_rng(9)
    w = (rng.standard_normal((64, 1024)) * 0.02).astype(np.float32)
    q, s, z = qspec.quantize_w4_g128(w)
    assert q.min() >= 0 and q.max() <= 15 and z.min() >= 0 and z.max() <= 15
    d = np.repeat(s.astype(np.float32), 128, axis=1)
    zz = np.repeat(z.astype(np.float32), 128, axis=1)
    w_hat = (q.astype(np.float32) - zz) * d
    unclamped = (q > 0) & (q < 15)
    assert (np.abs(w - w_hat)[unclamped] <= d[unclamped] * 0.5 * (1 + 1e-6)).all()
    # both ends of the code range are used in (nearly) every group that straddles zero
    g = q.reshape(64, 8, 128)
    assert (g.min(axis=2) <= 1).all() and (g.max(axis=2) >= 14).all()
    assert np.array_equal(qspec.dequantize_w4(qspec.pack_int4(q), s, z), w_hat)


# ------------------------------------------------------------------ independent restatement
@pytest.mark.parametrize("seed,std", [(0, 0.02), (1, 1.0), (2, 1e-6), (3, 37.0)])
def test_matches_pure_python_restatement(seed, std):
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((6, 256)) * std).astype(np.float32)
    w[1, :128] = np.abs(w[1, :128])       # one-signed group
    w[2, 128:] = w[2, 128]                # constant group
    w[3] = np.round(w[3] / std * 4) * std / 4  # many exact ties
    q8, s8 = qspec.quantize_w8(w)
    q4, s4, z4 = qspec.quantize_w4_g128(w)
    packed = qspec.pack_int4(q4)
    for n in range(w.shape[0]):
        row = [float(v) for v in w[n]]
        q_py, s_py = pyspec.quantize_w8_row(row)
        assert list(q8[n]) == q_py and float(s8[n]) == s_py
        for g in range(2):
            qg, sg, zg = pyspec.quantize_w4_group(row[128 * g:128 * (g + 1)])
            assert list(q4[n, 128 * g:128 * (g + 1)]) == qg
            assert float(s4[n, g]) == sg and int(z4[n, g]) == zg
            for c in range(16):
                assert int(packed[n, 16 * g + c]) == pyspec.pack_word(qg[8 * c:8 * c + 8])


# ------------------------------------------------------------------ pack / unpack
def test_pack_single_nibble_patterns():
    for j in range(8):
        for v in (1, 7, 8, 15):
            q = np.zeros((1, 8), np.uint8)
            q[0, j] = v
            word = int(qspec.pack_int4(q)[0, 0])
            assert word & 0xFFFFFFFF == v << (4 * j)
            assert (word < 0) == (j == 7 and v >= 8)  # top nibble >= 8 sets the int32 sign bit
    assert int(qspec.pack_int4(np.full((1, 8), 15, np.uint8))[0, 0]) == -1
    seq = np.arange(8, dtype=np.uint8)[None, :]
    assert int(qspec.pack_int4(seq)[0, 0]) == 0x76543210


def test_pack_unpack_are_inverse():
    rng = np.random.default_rng(3)
    q = rng.integers(0, 16, size=(33, 512), dtype=np.uint8)
    packed = qspec.pack_int4(q)
    assert packed.dtype == np.int32 and packed.shape == (33, 64)
    assert np.array_equal(qspec.unpack_int4(packed), q)
    words = rng.integers(-2**31, 2**31, size=(5, 40), dtype=np.int64).astype(np.int32)
    assert np.array_equal(qspec.pack_int4(qspec.unpack_int4(words)), words)


def test_argument_errors():
    with pytest.raises(ValueError):
        qspec.quantize_w4_g128(np.zeros((4, 100), np.float32))
    with pytest.raises(ValueError):
        qspec.pack_int4(np.full((1, 8), 16, np.uint8))
    with pytest.raises(ValueError):
        qspec.pack_int4(np.zeros((1, 7), np.uint8))


def test_corner_rows_shared_with_the_gpu_tests_hold_the_expected_codes():
    """The rows the HIP quantizers are given carry the same cases: check the oracle's answer on them."""
    from tests.helpers import tie_and_division_rows

    w = tie_and_division_rows(512)
    q8, _ = qspec.quantize_w8(w)
    q4, _, z4 = qspec.quantize_w4_g128(w)
    assert list(q4[0, :8]) == [0, 15, 5, 7, 7, 5, 3, 3] and int(z4[0, 0]) == 5
    assert list(z4[1]) == [2, 4, 4, 14]
    for i, (_, _, by_division, _) in enumerate(W8_DIVISION_CASES):
        assert int(q8[2 + i, 1]) == by_division
    for g, (_, _, by_division, _) in enumerate(W4_DIVISION_CASES):
        assert int(q4[5, 128 * g + 2]) == by_division and int(z4[5, g]) == 5
    for g, (_, _, _, by_division, _) in enumerate(W4_ZERO_DIVISION_CASES):
        assert int(z4[6, g]) == by_division
