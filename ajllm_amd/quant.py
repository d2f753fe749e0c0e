"""Quantized linear layer for the ajLLM Transformer on MI355X.

Host-side mirror of the reference's one linear operator,

    class Linear(nn.Module):            # src/ajllm/modeling/layers.py:9-33
        in_features, out_features, weight[out, in]
        forward(inputs[..., in]) -> inputs @ weight.T

with the weight held as int8 (per-output-channel symmetric, "w8a16") or int4
(asymmetric, groups of 128 along K, fp16 scale + uint4 zero-point, "w4a16_g128")
and the matmul done by the HIP kernels of ``libajq.so``.  All tensors live on a
ROCm device; there is no CPU path here.
"""

from __future__ import annotations

import torch
from torch import nn

from . import _lib

SCHEMES = ("w4a16_g128", "w8a16")
GROUP = 128
TILE_N = 16
GEMV_MAX_M = 16


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _require_cuda(*tensors: torch.Tensor) -> None:
    for t in tensors:
        if not t.is_cuda:
            raise ValueError("ajllm_amd.quant works on ROCm device tensors only (got a CPU tensor)")


# --------------------------------------------------------------------------- quantize / pack
def quantize_w8(weight: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """fp32 [N, K] -> (q int8 [N, K], scales fp16 [N]); scale = fp16(absmax / 127)."""
    _require_cuda(weight)
    if weight.dim() != 2:
        raise ValueError("weight must be [N, K]")
    w = weight.detach().to(torch.float32).contiguous()
    n, k = w.shape
    q = torch.empty((n, k), dtype=torch.int8, device=w.device)
    scales = torch.empty((n,), dtype=torch.float16, device=w.device)
    with torch.cuda.device(w.device):
        status = _lib.load().ajq_quantize_w8(w.data_ptr(), n, k, q.data_ptr(), scales.data_ptr(), _stream())
    _lib.check(status, "quantize_w8")
    return q, scales


def quantize_w4_g128(weight: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """fp32 [N, K] -> (qweight int32 [N, K/8], scales fp16 [N, K/128], zeros uint8 [N, K/128])."""
    _require_cuda(weight)
    if weight.dim() != 2:
        raise ValueError("weight must be [N, K]")
    w = weight.detach().to(torch.float32).contiguous()
    n, k = w.shape
    if k % GROUP != 0:
        raise ValueError(f"K={k} must be a multiple of {GROUP} for w4a16_g128")
    qweight = torch.empty((n, k // 8), dtype=torch.int32, device=w.device)
    scales = torch.empty((n, k // GROUP), dtype=torch.float16, device=w.device)
    zeros = torch.empty((n, k // GROUP), dtype=torch.uint8, device=w.device)
    with torch.cuda.device(w.device):
        status = _lib.load().ajq_quantize_w4_g128(
            w.data_ptr(), n, k, qweight.data_ptr(), scales.data_ptr(), zeros.data_ptr(), _stream()
        )
    _lib.check(status, "quantize_w4_g128")
    return qweight, scales, zeros


def _pad_rows(t: torch.Tensor, rows: int) -> torch.Tensor:
    if t.shape[0] == rows:
        return t.contiguous()
    pad = torch.zeros((rows - t.shape[0], *t.shape[1:]), dtype=t.dtype, device=t.device)
    return torch.cat((t, pad), dim=0).contiguous()


def repack_w4(qweight: torch.Tensor, scales: torch.Tensor, zeros: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """Canonical W4 tensors -> (wq uint32-as-int32 [N16/16, K/128, 64, 4], meta int32 [N16/16, K/128, 16]).

    Rows are padded with zeros to a multiple of 16 (N16)."""
    _require_cuda(qweight, scales, zeros)
    n, words = qweight.shape
    k = words * 8
    n16 = (n + TILE_N - 1) // TILE_N * TILE_N
    qweight, scales, zeros = _pad_rows(qweight, n16), _pad_rows(scales, n16), _pad_rows(zeros, n16)
    wq = torch.empty((n16 // TILE_N, k // GROUP, 64, 4), dtype=torch.int32, device=qweight.device)
    meta = torch.empty((n16 // TILE_N, k // GROUP, TILE_N), dtype=torch.int32, device=qweight.device)
    with torch.cuda.device(qweight.device):
        status = _lib.load().ajq_repack_w4(
            qweight.data_ptr(), scales.data_ptr(), zeros.data_ptr(), n16, k, wq.data_ptr(), meta.data_ptr(), _stream()
        )
    _lib.check(status, "repack_w4")
    return wq, meta


def unrepack_w4(wq: torch.Tensor, meta: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Inverse of :func:`repack_w4` (for the padded row count)."""
    _require_cuda(wq, meta)
    n16, k = wq.shape[0] * TILE_N, wq.shape[1] * GROUP
    qweight = torch.empty((n16, k // 8), dtype=torch.int32, device=wq.device)
    scales = torch.empty((n16, k // GROUP), dtype=torch.float16, device=wq.device)
    zeros = torch.empty((n16, k // GROUP), dtype=torch.uint8, device=wq.device)
    with torch.cuda.device(wq.device):
        status = _lib.load().ajq_unrepack_w4(
            wq.data_ptr(), meta.data_ptr(), n16, k, qweight.data_ptr(), scales.data_ptr(), zeros.data_ptr(), _stream()
        )
    _lib.check(status, "unrepack_w4")
    return qweight, scales, zeros


def repack_w8(q: torch.Tensor) -> torch.Tensor:
    """int8 [N, K] -> wq int32 [N16/16, K128/64, 64, 4] (rows zero-padded to a multiple of 16, columns to a
    multiple of 128: per-channel scales put no condition on K, and zero codes add exact zeros to a product whose
    activations are padded with zeros alike)."""
    _require_cuda(q)
    n, k = q.shape
    if k % GROUP != 0:
        q = torch.nn.functional.pad(q, (0, GROUP - k % GROUP))
        k = q.shape[1]
    n16 = (n + TILE_N - 1) // TILE_N * TILE_N
    q = _pad_rows(q, n16)
    wq = torch.empty((n16 // TILE_N, k // 64, 64, 4), dtype=torch.int32, device=q.device)
    with torch.cuda.device(q.device):
        status = _lib.load().ajq_repack_w8(q.data_ptr(), n16, k, wq.data_ptr(), _stream())
    _lib.check(status, "repack_w8")
    return wq


def unrepack_w8(wq: torch.Tensor) -> torch.Tensor:
    _require_cuda(wq)
    n16, k = wq.shape[0] * TILE_N, wq.shape[1] * 64
    q = torch.empty((n16, k), dtype=torch.int8, device=wq.device)
    with torch.cuda.device(wq.device):
        status = _lib.load().ajq_unrepack_w8(wq.data_ptr(), n16, k, q.data_ptr(), _stream())
    _lib.check(status, "unrepack_w8")
    return q


# --------------------------------------------------------------------------- matmul
def _prep_x(x: torch.Tensor, k: int) -> torch.Tensor:
    _require_cuda(x)
    if x.dim() != 2 or x.shape[1] != k:
        raise ValueError(f"x must be [M, {k}], got {tuple(x.shape)}")
    if x.dtype != torch.bfloat16:
        raise ValueError("activations must be bfloat16")
    return x.contiguous()


def _out(m: int, n: int, out_dtype: torch.dtype, device: torch.device) -> tuple[torch.Tensor, int]:
    if out_dtype == torch.bfloat16:
        return torch.empty((m, n), dtype=torch.bfloat16, device=device), _lib.AJQ_OUT_BF16
    if out_dtype == torch.float32:
        return torch.empty((m, n), dtype=torch.float32, device=device), _lib.AJQ_OUT_F32
    raise ValueError("out_dtype must be torch.bfloat16 or torch.float32")


def w4a16_matmul(
    x: torch.Tensor, wq: torch.Tensor, meta: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16,
    kernel: str = "auto",
) -> torch.Tensor:
    """y[M, N16] = x[M, K] @ W_hat^T for private W4 tensors.  ``kernel``: auto | gemv | gemm."""
    n16, k = wq.shape[0] * TILE_N, wq.shape[1] * GROUP
    x = _prep_x(x, k)
    m = x.shape[0]
    y, flag = _out(m, n16, out_dtype, x.device)
    if m == 0:
        return y
    lib = _lib.load()
    use_gemv = (m <= GEMV_MAX_M) if kernel == "auto" else (kernel == "gemv")
    with torch.cuda.device(x.device):
        if use_gemv:
            status = lib.ajq_w4a16_gemv(
                x.data_ptr(), m, k, wq.data_ptr(), meta.data_ptr(), n16, y.data_ptr(), flag, _stream()
            )
        else:
            nbytes = lib.ajq_w4a16_gemm_workspace_bytes_for(m, n16, k)  # 0 unless the 128 x 128 tile kernel runs
            workspace = torch.empty((max(nbytes, 16),), dtype=torch.uint8, device=x.device)
            status = lib.ajq_w4a16_gemm(
                x.data_ptr(), m, k, wq.data_ptr(), meta.data_ptr(), n16, y.data_ptr(), flag,
                workspace.data_ptr(), nbytes, _stream(),
            )
    _lib.check(status, "w4a16_matmul")
    return y


def w8a16_matmul(
    x: torch.Tensor, wq: torch.Tensor, scales: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16,
    kernel: str = "auto",
) -> torch.Tensor:
    """y[M, N16] = x[M, K] @ W_hat^T for private W8 tensors; ``scales`` fp16 [N16]."""
    n16, k = wq.shape[0] * TILE_N, wq.shape[1] * 64
    x = _prep_x(x, k)
    if scales.numel() != n16:
        raise ValueError(f"scales must have {n16} entries (rows padded to a multiple of 16)")
    m = x.shape[0]
    y, flag = _out(m, n16, out_dtype, x.device)
    if m == 0:
        return y
    lib = _lib.load()
    use_gemv = (m <= GEMV_MAX_M) if kernel == "auto" else (kernel == "gemv")
    fn = lib.ajq_w8a16_gemv if use_gemv else lib.ajq_w8a16_gemm
    with torch.cuda.device(x.device):
        status = fn(x.data_ptr(), m, k, wq.data_ptr(), scales.data_ptr(), n16, y.data_ptr(), flag, _stream())
    _lib.check(status, "w8a16_matmul")
    return y


# --------------------------------------------------------------------------- the layer
class QuantLinear(nn.Module):
    """Drop-in for the reference ``Linear`` (src/ajllm/modeling/layers.py:9-33): bias-free,
    ``in_features`` / ``out_features`` attributes, ``forward(inputs[..., in]) -> [..., out]``.

    The fp32 ``weight`` parameter is replaced by buffers ``qweight`` / ``scales`` / ``zeros``
    (canonical, what a checkpoint stores) plus the kernel-private ``wq`` / ``meta`` built from
    them.  Inference only."""

    def __init__(self, in_features: int, out_features: int, scheme: str = "w4a16_g128") -> None:
        super().__init__()
        if scheme not in SCHEMES:
            raise ValueError(f"scheme must be one of {SCHEMES}, got {scheme!r}")
        self.in_features = in_features
        self.out_features = out_features
        self.scheme = scheme
        self.register_buffer("qweight", None)
        self.register_buffer("scales", None)
        self.register_buffer("zeros", None)
        self.register_buffer("wq", None, persistent=False)
        self.register_buffer("meta", None, persistent=False)

    @classmethod
    def from_weight(cls, weight: torch.Tensor, scheme: str = "w4a16_g128") -> "QuantLinear":
        """Quantize an fp32 ``[out, in]`` weight that already lives on the GPU."""
        out_features, in_features = weight.shape
        self = cls(in_features, out_features, scheme)
        if scheme == "w8a16":
            self.qweight, self.scales = quantize_w8(weight)
            self.zeros = torch.empty(0, dtype=torch.uint8, device=weight.device)
        else:
            self.qweight, self.scales, self.zeros = quantize_w4_g128(weight)
        self.prepare()
        return self

    @classmethod
    def from_linear(cls, linear: nn.Module, scheme: str = "w4a16_g128") -> "QuantLinear":
        """Build from a reference-style ``Linear`` (anything with a 2-D ``weight`` and no bias)."""
        if getattr(linear, "bias", None) is not None:
            raise ValueError("the reference Linear is bias-free; a biased layer cannot be swapped")
        return cls.from_weight(linear.weight.data, scheme)

    @property
    def padded_in_features(self) -> int:
        """Columns of the kernel-private weight tensor: ``in_features`` rounded up to a multiple of 128 (W8 only;
        W4 groups need ``in_features`` itself on that grid)."""
        return (self.in_features + GROUP - 1) // GROUP * GROUP

    def prepare(self) -> None:
        """(Re)build the kernel-private tensors from the canonical ones."""
        if self.scheme == "w8a16":
            self.wq = repack_w8(self.qweight)
            n16 = self.wq.shape[0] * TILE_N
            self.meta = _pad_rows(self.scales, n16)
        else:
            self.wq, self.meta = repack_w4(self.qweight, self.scales, self.zeros)

    def _load_from_state_dict(self, state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys,
                              error_msgs):
        """Takes the canonical tensors under ``prefix``; reports an absent one in ``missing_keys`` and
        any other key directly under the prefix (e.g. a dense ``weight`` aimed at this slot) in
        ``unexpected_keys``, so ``load_state_dict(strict=True)`` raises as it does for the reference
        layer (training/checkpoint.py:35-45 loads strictly)."""
        wanted = ("qweight", "scales") + (() if self.scheme == "w8a16" else ("zeros",))
        found = {}
        for name in ("qweight", "scales", "zeros"):
            key = prefix + name
            if key in state_dict:
                found[name] = state_dict[key]
            elif name in wanted:
                missing_keys.append(key)
        for key in state_dict:
            if key.startswith(prefix) and "." not in key[len(prefix):] and key[len(prefix):] not in (
                    "qweight", "scales", "zeros"):
                unexpected_keys.append(key)
        if any(name not in found for name in wanted):
            return  # leave the layer as it was: a partial load must not leave mixed tensors behind
        expect_q = ((self.out_features, self.in_features) if self.scheme == "w8a16"
                    else (self.out_features, self.in_features // 8))
        w8 = self.scheme == "w8a16"
        groups = (self.out_features,) if w8 else (self.out_features, self.in_features // GROUP)
        expect = {"qweight": (expect_q, torch.int8 if w8 else torch.int32), "scales": (groups, torch.float16)}
        if not w8:
            expect["zeros"] = (groups, torch.uint8)
        bad = False
        for name, (shape, dtype) in expect.items():
            got = found[name]
            if tuple(got.shape) != shape:
                error_msgs.append(f"size mismatch for {prefix}{name}: checkpoint {tuple(got.shape)}, "
                                  f"layer ({self.scheme}) expects {shape}")
                bad = True
            elif got.dtype != dtype:
                error_msgs.append(f"dtype mismatch for {prefix}{name}: checkpoint {got.dtype}, "
                                  f"layer ({self.scheme}) expects {dtype}")
                bad = True
        if bad:
            return  # nothing of the layer has been touched
        for name, value in found.items():
            setattr(self, name, value.clone())
        if self.scheme == "w8a16" and "zeros" not in found:
            self.zeros = torch.empty(0, dtype=torch.uint8, device=self.qweight.device)
        if self.qweight.is_cuda:
            self.prepare()

    def forward(self, inputs: torch.Tensor, out_dtype: torch.dtype | None = None) -> torch.Tensor:
        if self.wq is None:
            raise RuntimeError("QuantLinear has no weights: build it with from_linear()/from_weight()")
        lead = inputs.shape[:-1]
        x = inputs.reshape(-1, self.in_features)
        want = out_dtype or inputs.dtype
        if x.dtype != torch.bfloat16:
            x = x.to(torch.bfloat16)
        if self.padded_in_features != self.in_features:  # W8 with in_features off the kernels' 128-column grid
            x = torch.nn.functional.pad(x, (0, self.padded_in_features - self.in_features))
        kernel_out = torch.float32 if want == torch.float32 else torch.bfloat16
        if self.scheme == "w8a16":
            y = w8a16_matmul(x, self.wq, self.meta, kernel_out)
        else:
            y = w4a16_matmul(x, self.wq, self.meta, kernel_out)
        if y.shape[1] != self.out_features:
            y = y[:, : self.out_features]
        if y.dtype != want:
            y = y.to(want)
        return y.reshape(*lead, self.out_features)

    def extra_repr(self) -> str:
        return f"in_features={self.in_features}, out_features={self.out_features}, scheme={self.scheme}"


def _is_reference_linear(module: nn.Module) -> bool:
    weight = getattr(module, "weight", None)
    return (
        not isinstance(module, QuantLinear)
        and hasattr(module, "in_features")
        and hasattr(module, "out_features")
        and isinstance(weight, torch.Tensor)
        and weight.dim() == 2
        and getattr(module, "bias", None) is None
    )


@torch.no_grad()
def quantize_model_(model: nn.Module, scheme: str = "w4a16_g128", skip: tuple[str, ...] = (),
                    untie_head: bool = False) -> nn.Module:
    """Swap every bias-free linear of ``model`` for a :class:`QuantLinear`, in place.

    Matches by duck type, so it finds the reference's ``q_proj/k_proj/v_proj/output_proj``
    (src/ajllm/modeling/attention.py:82-85), ``w1/w2/w3`` (activations.py:20-22) and
    ``lm_head`` (transformer.py:108).  Embeddings are not linears and stay dense.

    A model with tied embeddings has no ``lm_head`` module: its logits are ``hidden @ embedding.T``
    (transformer.py:116-118) and stay a dense product.  With ``untie_head`` such a model gets a
    quantized ``lm_head`` made from the embedding matrix (the embedding itself stays dense for the
    look-up) and stops being tied: the head then runs through the library like every other linear."""
    for parent in list(model.modules()):
        for name, child in list(parent.named_children()):
            if name in skip or not _is_reference_linear(child):
                continue
            setattr(parent, name, QuantLinear.from_linear(child, scheme))
    if (untie_head and getattr(model, "tie_embeddings", False) and getattr(model, "lm_head", None) is None
            and hasattr(model, "token_embeddings") and "lm_head" not in skip):
        model.lm_head = QuantLinear.from_weight(model.token_embeddings.weight.data, scheme)
        model.tie_embeddings = False
    return model
