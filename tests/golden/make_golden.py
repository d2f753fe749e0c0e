"""Writes tests/golden/quant_small.npz: inputs and expected outputs of the quantized-linear
scheme on a small seeded case.

The reference project holds no vector for any linear layer, so the expected values come from
the CPU oracle (oracle/qspec.py) after its known-answer tests passed; the file freezes them so
that neither the oracle nor the kernels can drift unnoticed.  Run from the repository root:
    python tests/golden/make_golden.py
"""

import sys
from pathlib import Path

import numpy as np
import torch

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))

from oracle import qspec  # noqa: E402


def main() -> None:
    g = torch.Generator().manual_seed(20240607)
    n, k, m = 48, 384, 5
    w = (torch.randn((n, k), generator=g) * 0.02).numpy()
    w[3, :128] = np.abs(w[3, :128])        # one-signed group
    w[4, 128:256] = 0.0                    # all-zero group
    w[5] = np.round(w[5] * 400) / 400      # many ties
    x = torch.randn((m, k), generator=g)
    x[1, 7] *= 20.0
    x = x.to(torch.bfloat16)
    q8, s8 = qspec.quantize_w8(w)
    q4, s4, z4 = qspec.quantize_w4_g128(w)
    qweight = qspec.pack_int4(q4)
    y4 = qspec.quant_linear(x, torch.from_numpy(qspec.dequantize_w4(qweight, s4, z4)),
                            accumulate=torch.float64, out_dtype=torch.float64).numpy()
    y8 = qspec.quant_linear(x, torch.from_numpy(qspec.dequantize_w8(q8, s8)),
                            accumulate=torch.float64, out_dtype=torch.float64).numpy()
    out = Path(__file__).with_name("quant_small.npz")
    np.savez_compressed(
        out, weight=w, x_bf16_bits=x.view(torch.int16).numpy().view(np.uint16),
        w8_q=q8, w8_scales_bits=s8.view(np.uint16),
        w4_qweight=qweight, w4_scales_bits=s4.view(np.uint16), w4_zeros=z4,
        y_w4_f64=y4, y_w8_f64=y8,
    )
    print(f"wrote {out} ({out.stat().st_size} bytes)")


if __name__ == "__main__":
    main()
