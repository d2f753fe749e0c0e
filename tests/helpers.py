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
