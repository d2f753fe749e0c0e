"""Seeded synthetic inputs and error measures shared by the tests."""

from __future__ import annotations

import numpy as np
import torch


def make_weight(n: int, k: int, seed: int, std: float = 0.02) -> torch.Tensor:
    g = torch.Generator().manual_seed(seed)
    return torch.randn((n, k), generator=g, dtype=torch.float32) * std


def make_activations(m: int, k: int, seed: int, outliers: bool = False) -> torch.Tensor:
    """bf16 [m, k] ~ N(0, 1); with ``outliers`` 0.1 % of the entries are scaled by 20."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn((m, k), generator=g, dtype=torch.float32)
    if outliers:
        mask = torch.rand((m, k), generator=g) < 0.001
        x = torch.where(mask, x * 20.0, x)
    return x.to(torch.bfloat16)


def errors(got: torch.Tensor, want: torch.Tensor) -> tuple[float, float]:
    """(max-abs error, relative Frobenius error) in fp64."""
    g = got.detach().double().cpu()
    w = want.detach().double().cpu()
    diff = g - w
    return float(diff.abs().max()), float(diff.norm() / w.norm().clamp_min(1e-30))


def bf16_rounding_excess(got16: torch.Tensor, want: torch.Tensor, eps: float) -> float:
    """How far ``got16`` lies outside what rounding can explain, elementwise maximum.

    If the kernel's fp32 value is within ``eps`` of ``want`` and the bf16 output is its
    round-to-nearest, then |got16 - want| <= eps + ulp/2, with the bf16 ulp taken at the
    larger of the two magnitudes (8 significant bits: ulp = 2^(floor(log2 |v|) - 7)).
    Returns max(|got16 - want| - bound); a value <= 0 passes."""
    g = got16.detach().double().cpu()
    w = want.detach().double().cpu()
    mag = torch.maximum(g.abs(), w.abs()).clamp_min(2.0**-126)
    half_ulp = torch.exp2(torch.floor(torch.log2(mag)) - 8)
    return float(((g - w).abs() - (half_ulp + eps)).max())


# north-star tolerances for floating-point outputs
MAX_ABS_TOL = 1e-2
REL_FRO_TOL = 2e-3


def compare_greedy(tokens_got: torch.Tensor, tokens_ref: torch.Tensor, margins_ref: torch.Tensor,
                   prompt_len: int, noise: float) -> dict:
    """Compare two greedy decodes of the same prompts.

    Rows are compared up to their first differing token.  A first difference is *attributable*
    when the reference's top-1 minus top-2 logit at that step is below ``noise`` (the two runs
    may then legitimately pick different tokens: their logits differ by accumulation-order
    noise); everything after it is a different context and says nothing.  Returns counts and the
    smallest margin met on the compared prefix."""
    got, ref = tokens_got.cpu(), tokens_ref.cpu()
    rows = ref.shape[0]
    identical_rows, attributable, unexplained = 0, [], []
    min_margin = float("inf")
    for b in range(rows):
        diff = (got[b, prompt_len:] != ref[b, prompt_len:]).nonzero()
        first = int(diff[0]) if len(diff) else None
        upto = first if first is not None else ref.shape[1] - prompt_len
        if upto:
            min_margin = min(min_margin, float(margins_ref[b, :upto].min()))
        if first is None:
            identical_rows += 1
        elif float(margins_ref[b, first]) < noise:
            attributable.append((b, first, float(margins_ref[b, first])))
        else:
            unexplained.append((b, first, float(margins_ref[b, first])))
    return {"rows": rows, "identical_rows": identical_rows, "attributable": attributable,
            "unexplained": unexplained, "min_margin_on_compared_prefix": min_margin}


# ---------------------------------------------------------------- quantizer corner cases
# (fp16 scale, weight, code by IEEE division, code by multiplying with the rounded reciprocal):
# found by search; W / d and W * (1 / d) land on different sides of a half.
W8_DIVISION_CASES = [
    (0.005665, "0x1.67a6p-4", 16, 15),
    (0.003347, "-0x1.ed9802p-7", -5, -4),
    (0.006348, "0x1.b6bffep-2", 67, 68),
]
W4_DIVISION_CASES = [  # groups spanning -5 d ... 10 d (zero-point 5); codes include the zero-point
    (0.003347, "-0x1.ed9802p-7", 0, 1),
    (0.009796, "0x1.692002p-5", 10, 9),
    (0.005737, "0x1.a70002p-6", 10, 9),
]
W4_ZERO_DIVISION_CASES = [  # (fp16 scale, min, max, zero by division, zero by reciprocal)
    (0.0008893, "-0x1.d24002p-12", "0x1.a68ap-7", 1, 0),
    (0.006264, "-0x1.0d64p-4", "0x1.cddp-6", 10, 11),
    (0.006393, "-0x1.7bb8p-4", "0x1.a3p-9", 14, 15),
]


def tie_and_division_rows(k: int = 512) -> np.ndarray:
    """fp32 rows [*, k] (k >= 512, a multiple of 128) holding the quantizers' rounding corners:
    W4 code ties under an odd zero-point, zero-points exactly on a half, and the committed
    (scale, weight) pairs where IEEE division and a multiply by the rounded reciprocal round
    to different integers (per-row absmax for W8, per-group range for W4)."""
    rows = []
    d = np.float32(2.0**-3)
    row = np.zeros(k, np.float32)
    row[0], row[1] = -5 * d, 10 * d
    row[2:8] = np.array([0.5, 1.5, 2.5, -0.5, -1.5, -2.5], np.float32) * d
    rows.append(row)
    d = np.float32(2.0**-4)
    row = np.zeros(k, np.float32)
    for g, below in enumerate((2.5, 3.5, 4.5, 14.5)):
        row[128 * g], row[128 * g + 1] = -below * d, (15 - below) * d
    rows.append(row)
    for scale, weight, _, _ in W8_DIVISION_CASES:
        dd = np.float32(np.float16(scale))
        row = np.zeros(k, np.float32)
        row[0], row[1] = np.float32(127.0) * dd, np.float32(float.fromhex(weight))
        rows.append(row)
    row = np.zeros(k, np.float32)
    for g, (scale, weight, _, _) in enumerate(W4_DIVISION_CASES):
        dd = np.float32(np.float16(scale))
        row[128 * g], row[128 * g + 1] = np.float32(-5.0) * dd, np.float32(10.0) * dd
        row[128 * g + 2] = np.float32(float.fromhex(weight))
    rows.append(row)
    row = np.zeros(k, np.float32)
    for g, (_, mn, mx, _, _) in enumerate(W4_ZERO_DIVISION_CASES):
        row[128 * g], row[128 * g + 1] = np.float32(float.fromhex(mn)), np.float32(float.fromhex(mx))
    rows.append(row)
    return np.stack(rows)
