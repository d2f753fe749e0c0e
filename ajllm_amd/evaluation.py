"""Held-out loss and perplexity of a model, and what quantization did to them.

Mirrors the reference's evaluation of a finished run (src/ajllm/evaluation/evaluator.py:14-31):
random contiguous windows of a memory-mapped uint32 token file
(src/ajllm/training/data.py:11-43), mean next-token cross-entropy per batch
(src/ajllm/training/losses.py:8-19), ``perplexity = exp(min(loss, 50))``.  The same seed draws the
same windows, so a dense model and its quantized copy are scored on identical tokens and the
difference of the two losses is the quality cost of the scheme.
"""

from __future__ import annotations

import copy
import math
from pathlib import Path

import numpy as np
import torch

from .quant import quantize_model_


def cross_entropy(logits: torch.Tensor, targets: torch.Tensor) -> torch.Tensor:
    """Mean of ``logsumexp(logits) - logits[target]`` over every leading position, in fp32."""
    rows = logits.reshape(-1, logits.shape[-1]).float()
    picked = rows.gather(1, targets.reshape(-1, 1)).squeeze(1)
    return (torch.logsumexp(rows, dim=-1) - picked).mean()


class TokenFile:
    """A flat file of uint32 token ids, read through a memory map."""

    def __init__(self, path: str | Path) -> None:
        self.path = Path(path)
        if self.path.stat().st_size % 4:
            raise ValueError(f"{self.path}: size is not a whole number of uint32 tokens")
        self.tokens = np.memmap(self.path, dtype=np.uint32, mode="r")

    def __len__(self) -> int:
        return int(self.tokens.shape[0])

    def batch(self, batch_size: int, context_length: int, device, generator: np.random.Generator):
        """``batch_size`` windows at uniformly drawn starts: inputs ``[B, T]`` and the same windows
        moved one token on as targets (one ``generator.integers`` call per batch, as the reference
        draws them)."""
        last_start = len(self) - context_length - 1
        if last_start < 0:
            raise ValueError(f"{self.path} holds {len(self)} tokens, fewer than context_length + 1")
        starts = generator.integers(0, last_start + 1, size=batch_size)
        windows = np.stack([np.asarray(self.tokens[s:s + context_length + 1], dtype=np.int64) for s in starts])
        both = torch.from_numpy(windows).to(device)
        return both[:, :-1].contiguous(), both[:, 1:].contiguous()


@torch.no_grad()
def evaluate_model(model: torch.nn.Module, dataset, batches: int, batch_size: int, context_length: int,
                   device, seed: int) -> dict[str, float]:
    """Average loss over ``batches`` random batches; same keys as the reference's result."""
    if batches < 1:
        raise ValueError("batches must be at least 1")
    model.eval()
    generator = np.random.default_rng(seed)
    total = 0.0
    for _ in range(batches):
        inputs, targets = dataset.batch(batch_size, context_length, device, generator)
        total += float(cross_entropy(model(inputs), targets))
    loss = total / batches
    return {"loss": loss, "perplexity": math.exp(min(loss, 50.0)), "batches": batches}


@torch.no_grad()
def quantization_report(model: torch.nn.Module, dataset, scheme: str, batches: int, batch_size: int,
                        context_length: int, device, seed: int, skip: tuple[str, ...] = ()) -> dict[str, object]:
    """Score ``model`` and a quantized copy of it on the same windows.

    Both scores come from copies moved to ``device`` (the quantized one is quantized there): the
    caller's model stays where and as it was.  ``loss_delta`` is quantized minus dense."""
    dense_copy = copy.deepcopy(model).to(device)
    dense = evaluate_model(dense_copy, dataset, batches, batch_size, context_length, device, seed)
    del dense_copy
    twin = copy.deepcopy(model).to(device)
    quantize_model_(twin, scheme=scheme, skip=skip)
    quant = evaluate_model(twin, dataset, batches, batch_size, context_length, device, seed)
    return {
        "scheme": scheme, "dense": dense, "quantized": quant,
        "loss_delta": quant["loss"] - dense["loss"],
        "perplexity_ratio": quant["perplexity"] / dense["perplexity"],
    }
