"""Quantized checkpoints: the canonical tensors of every QuantLinear in one safetensors file.

The reference stores dense training checkpoints with ``torch.save`` as
``{"model_state_dict", "optimizer_state_dict", "step", "metadata"}``
(src/ajllm/training/checkpoint.py:12-45) and reloads them into a freshly built model
(src/ajllm/workflows/common.py:43-53).  A quantized checkpoint keeps the same tensor names for
everything that stays dense (embeddings, norm gains) and replaces each linear's ``weight`` by
``qweight`` / ``scales`` / ``zeros`` (the canonical interchange tensors; the kernel-private layout
is rebuilt at load time).  The file's header carries a manifest: format tag, scheme, group size,
the model configuration and a SHA-256 over the tensor bytes in key order.
"""

from __future__ import annotations

import hashlib
import json
import os
from pathlib import Path
from typing import Any

import torch
from safetensors import safe_open
from safetensors.torch import save_file

from . import modeling
from .quant import SCHEMES, GROUP, QuantLinear, quantize_model_

FORMAT = "ajq-quantized-v1"


def _digest(tensors: dict[str, torch.Tensor]) -> str:
    h = hashlib.sha256()
    for key in sorted(tensors):
        t = tensors[key].detach().cpu().contiguous()
        h.update(key.encode())
        h.update(str(t.dtype).encode())
        h.update(str(tuple(t.shape)).encode())
        h.update(t.view(torch.uint8).numpy().tobytes() if t.numel() else b"")
    return h.hexdigest()


def model_config(model: modeling.TransformerLM) -> dict[str, Any]:
    """The constructor arguments of a ``modeling.TransformerLM`` (what ``build_model`` needs back)."""
    first = model.layers[0]
    return {
        "vocab_size": model.vocab_size, "context_length": model.context_length, "d_model": model.d_model,
        "num_layers": model.num_layers, "num_heads": model.num_heads, "num_kv_heads": model.num_kv_heads,
        "d_ff": model.d_ff, "position_encoding": model.position_encoding,
        "rope_theta": float(first.attention.rope.theta) if first.attention.rope is not None else 10_000.0,
        "normalization": "rmsnorm" if isinstance(first.norm1, modeling.RMSNorm) else "none",
        "norm_placement": first.norm_placement,
        "feed_forward": "swiglu" if isinstance(first.feed_forward, modeling.SwiGLU) else "silu",
        "tie_embeddings": model.tie_embeddings,
    }


def save_quantized(path: str | Path, model: torch.nn.Module, scheme: str, config: dict[str, Any] | None = None,
                   metadata: dict[str, Any] | None = None) -> Path:
    """Write the quantized model's state dict (canonical tensors only) atomically to ``path``."""
    if scheme not in SCHEMES:
        raise ValueError(f"scheme must be one of {SCHEMES}")
    tensors = {k: v.detach().cpu().contiguous() for k, v in model.state_dict().items()}
    if not any(k.endswith(".qweight") for k in tensors):
        raise ValueError("the model holds no quantized linear")
    header = {
        "format": FORMAT, "scheme": scheme, "group_size": str(GROUP if scheme == "w4a16_g128" else 0),
        "config": json.dumps(config or {}), "metadata": json.dumps(metadata or {}), "sha256": _digest(tensors),
    }
    destination = Path(path)
    destination.parent.mkdir(parents=True, exist_ok=True)
    temporary = destination.with_suffix(destination.suffix + ".tmp")
    save_file(tensors, str(temporary), metadata=header)
    os.replace(temporary, destination)
    return destination


def read_quantized(path: str | Path, verify: bool = True) -> tuple[dict[str, torch.Tensor], dict[str, Any]]:
    """``(tensors on the CPU, manifest)``; raises ``ValueError`` on a foreign or corrupted file."""
    with safe_open(str(path), framework="pt", device="cpu") as f:
        header = f.metadata() or {}
        if header.get("format") != FORMAT:
            raise ValueError(f"{path} is not an {FORMAT} checkpoint")
        tensors = {k: f.get_tensor(k) for k in f.keys()}
    if verify and _digest(tensors) != header.get("sha256"):
        raise ValueError(f"{path}: tensor bytes do not match the manifest's SHA-256")
    manifest = {"format": header["format"], "scheme": header["scheme"], "group_size": int(header["group_size"]),
                "config": json.loads(header.get("config", "{}")), "metadata": json.loads(header.get("metadata", "{}")),
                "sha256": header["sha256"]}
    return tensors, manifest


def load_quantized_into(model: torch.nn.Module, tensors: dict[str, torch.Tensor], scheme: str, device) -> torch.nn.Module:
    """Swap the linears that the checkpoint holds in quantized form for empty QuantLinears, move the
    model to ``device`` and load the tensors (which rebuilds the kernel-private layout)."""
    for parent_name, parent in list(model.named_modules()):
        for name, child in list(parent.named_children()):
            full = f"{parent_name}.{name}" if parent_name else name
            if f"{full}.qweight" in tensors and not isinstance(child, QuantLinear):
                setattr(parent, name, QuantLinear(child.in_features, child.out_features, scheme))
    model.to(device)
    missing, unexpected = model.load_state_dict({k: v.to(device) for k, v in tensors.items()}, strict=False)
    leftover = [k for k in missing if not k.endswith((".wq", ".meta"))]
    if leftover or unexpected:
        raise ValueError(f"checkpoint and model disagree: missing {leftover}, unexpected {list(unexpected)}")
    return model.eval()


def load_quantized(path: str | Path, device, verify: bool = True) -> tuple[modeling.TransformerLM, dict[str, Any]]:
    """Rebuild the ``modeling.TransformerLM`` a checkpoint describes and load it on ``device``."""
    tensors, manifest = read_quantized(path, verify)
    cfg = manifest["config"]
    if not cfg:
        raise ValueError("the checkpoint carries no model configuration; build the model and use load_quantized_into")
    with torch.device(device):  # dense skeleton on the target device; its linears are swapped out next
        model = modeling.TransformerLM(**cfg)
    return load_quantized_into(model, tensors, manifest["scheme"], device), manifest


@torch.no_grad()
def convert_dense_checkpoint(dense_path: str | Path, out_path: str | Path, config: dict[str, Any], scheme: str,
                             device) -> Path:
    """Reference-style dense checkpoint (``model_state_dict`` inside a ``torch.save`` file, or a bare
    state dict) -> quantized checkpoint.  Quantization runs on ``device`` (a ROCm device)."""
    blob = torch.load(Path(dense_path), map_location="cpu", weights_only=True)
    state = blob.get("model_state_dict", blob) if isinstance(blob, dict) else blob
    model = modeling.TransformerLM(**config)
    model.load_state_dict(state)
    model.to(device).eval()
    quantize_model_(model, scheme)
    return save_quantized(out_path, model, scheme, config=model_config(model),
                          metadata={"source": str(dense_path), "step": blob.get("step") if isinstance(blob, dict) else None})
