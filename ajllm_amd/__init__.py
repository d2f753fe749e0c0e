"""MI355X-native quantized linear path (W8A16 / W4A16-g128) for the ajLLM Transformer."""

from .quant import (  # noqa: F401
    QuantLinear,
    quantize_model_,
    quantize_w4_g128,
    quantize_w8,
    repack_w4,
    repack_w8,
    unrepack_w4,
    unrepack_w8,
    w4a16_matmul,
    w8a16_matmul,
)

__all__ = [
    "QuantLinear",
    "quantize_model_",
    "quantize_w4_g128",
    "quantize_w8",
    "repack_w4",
    "repack_w8",
    "unrepack_w4",
    "unrepack_w8",
    "w4a16_matmul",
    "w8a16_matmul",
]
