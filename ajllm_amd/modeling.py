"""The ajLLM decoder-only Transformer, restated so that this repository is self-contained
on a GPU box, with the two things the reference lacks and the decode benchmarks need:
a KV cache (incremental decoding) and grouped-query attention.

Architecture, module names and state-dict keys follow the reference exactly
(``token_embeddings``, ``layers.{i}.norm1|norm2``, ``layers.{i}.attention.{q,k,v,output}_proj``,
``layers.{i}.feed_forward.w{1,2,3}``, ``final_norm``, ``lm_head``):

* ``Linear`` / ``Embedding`` / ``RMSNorm``   - reference src/ajllm/modeling/layers.py:9-82
* ``SwiGLU`` / ``SiLUFeedForward``           - reference src/ajllm/modeling/activations.py:11-45
* softmax, masked attention, interleaved RoPE, ``MultiHeadSelfAttention``
                                             - reference src/ajllm/modeling/attention.py:13-120
* ``TransformerBlock`` / ``TransformerLM``   - reference src/ajllm/modeling/transformer.py:13-126
* ``build_model``                            - reference src/ajllm/modeling/factory.py:11-35

Every ``Linear`` is the boundary a ``QuantLinear`` drops into (``quantize_model_``).
"""

from __future__ import annotations

import math
from typing import Any

import torch
from torch import nn


class Linear(nn.Module):
    """Bias-free projection, ``y = x @ W^T``; truncated-normal init with std sqrt(2/(in+out)), cut at 3 std."""

    def __init__(self, in_features: int, out_features: int, device=None, dtype=None) -> None:
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.weight = nn.Parameter(torch.empty(out_features, in_features, device=device, dtype=dtype))
        std = math.sqrt(2.0 / (in_features + out_features))
        nn.init.trunc_normal_(self.weight, mean=0.0, std=std, a=-3 * std, b=3 * std)

    def forward(self, inputs: torch.Tensor) -> torch.Tensor:
        return inputs @ self.weight.transpose(-2, -1)


class Embedding(nn.Module):
    """Row lookup; N(0, 1) init cut at +-3."""

    def __init__(self, num_embeddings: int, embedding_dim: int, device=None, dtype=None) -> None:
        super().__init__()
        self.num_embeddings = num_embeddings
        self.embedding_dim = embedding_dim
        self.weight = nn.Parameter(torch.empty(num_embeddings, embedding_dim, device=device, dtype=dtype))
        nn.init.trunc_normal_(self.weight, mean=0.0, std=1.0, a=-3.0, b=3.0)

    def forward(self, token_ids: torch.Tensor) -> torch.Tensor:
        return self.weight[token_ids]


class RMSNorm(nn.Module):
    """x / sqrt(mean(x^2) + eps) * gain, computed in fp32 and cast back."""

    def __init__(self, d_model: int, epsilon: float = 1e-5, device=None, dtype=None) -> None:
        super().__init__()
        self.epsilon = epsilon
        self.weight = nn.Parameter(torch.ones(d_model, device=device, dtype=dtype))

    def forward(self, inputs: torch.Tensor) -> torch.Tensor:
        x = inputs.float()
        rms = torch.sqrt(torch.mean(x.square(), dim=-1, keepdim=True) + self.epsilon)
        return ((x / rms) * self.weight).to(inputs.dtype)


def build_norm(kind: str, d_model: int) -> nn.Module:
    if kind == "rmsnorm":
        return RMSNorm(d_model)
    if kind == "none":
        return nn.Identity()
    raise ValueError(f"Unsupported normalization type: {kind}")


def silu(inputs: torch.Tensor) -> torch.Tensor:
    return inputs * torch.sigmoid(inputs)


class SwiGLU(nn.Module):
    """w2(silu(w1 x) * w3 x)"""

    def __init__(self, d_model: int, d_ff: int) -> None:
        super().__init__()
        self.w1 = Linear(d_model, d_ff)
        self.w2 = Linear(d_ff, d_model)
        self.w3 = Linear(d_model, d_ff)

    def forward(self, inputs: torch.Tensor) -> torch.Tensor:
        return self.w2(silu(self.w1(inputs)) * self.w3(inputs))


class SiLUFeedForward(nn.Module):
    """w2(silu(w1 x))"""

    def __init__(self, d_model: int, d_ff: int) -> None:
        super().__init__()
        self.w1 = Linear(d_model, d_ff)
        self.w2 = Linear(d_ff, d_model)

    def forward(self, inputs: torch.Tensor) -> torch.Tensor:
        return self.w2(silu(self.w1(inputs)))


def build_feed_forward(kind: str, d_model: int, d_ff: int) -> nn.Module:
    if kind == "swiglu":
        return SwiGLU(d_model, d_ff)
    if kind == "silu":
        return SiLUFeedForward(d_model, d_ff)
    raise ValueError(f"Unsupported feed-forward type: {kind}")


def softmax(inputs: torch.Tensor, dimension: int) -> torch.Tensor:
    shifted = inputs - torch.amax(inputs, dim=dimension, keepdim=True)
    exps = torch.exp(shifted)
    return exps / torch.sum(exps, dim=dimension, keepdim=True)


def scaled_dot_product_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                                 mask: torch.Tensor | None = None) -> torch.Tensor:
    scores = q @ k.transpose(-2, -1) / math.sqrt(q.shape[-1])
    if mask is not None:
        scores = scores.masked_fill(~mask, float("-inf"))
    probs = softmax(scores, -1).nan_to_num_(nan=0.0)
    return probs @ v


class RotaryPositionalEmbedding(nn.Module):
    """Interleaved rotary embedding: pairs (x[2i], x[2i+1]) rotate by pos * theta^(-2i/d)."""

    def __init__(self, theta: float, head_dimension: int, max_sequence_length: int) -> None:
        super().__init__()
        if head_dimension % 2 != 0:
            raise ValueError("RoPE requires an even attention head dimension")
        self.theta = theta
        # the tables are not stored in checkpoints: always form them on the host, so that a model
        # built directly on a GPU gets the same values as one built on the host and moved there
        target = torch.empty(0).device
        positions = torch.arange(max_sequence_length, device="cpu").unsqueeze(1)
        freqs = theta ** (-torch.arange(0, head_dimension, 2, device="cpu").float() / head_dimension)
        angles = positions * freqs
        self.register_buffer("cosine", torch.cos(angles).to(target), persistent=False)
        self.register_buffer("sine", torch.sin(angles).to(target), persistent=False)

    def forward(self, inputs: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        cos, sin = self.cosine[positions], self.sine[positions]
        if cos.dtype != inputs.dtype:
            cos, sin = cos.to(inputs.dtype), sin.to(inputs.dtype)
        even, odd = inputs[..., ::2], inputs[..., 1::2]
        return torch.stack((even * cos - odd * sin, even * sin + odd * cos), dim=-1).flatten(-2)


class KVCache:
    """Per-layer key/value store for incremental decoding: ``[layers][B, kv_heads, max_len, head_dim]``.

    Two modes.  Dynamic (default): ``length`` is a Python int, a call appends ``seq`` positions and
    attends over the first ``length + seq``.  Static (``static = True``, one token per call): the
    write position is the device tensor ``position``, the new key/value row is scattered there and
    attention runs over all ``max_len`` rows under a mask, so every shape is fixed and the step can
    be recorded into a HIP graph; the caller advances ``position``."""

    def __init__(self, num_layers: int, batch: int, kv_heads: int, max_len: int, head_dim: int,
                 device, dtype) -> None:
        self.keys = [torch.zeros(batch, kv_heads, max_len, head_dim, device=device, dtype=dtype) for _ in range(num_layers)]
        self.values = [torch.zeros_like(k) for k in self.keys]
        self.length = 0
        self.max_len = max_len
        self.static = False
        self.position = torch.zeros(1, dtype=torch.long, device=device)
        self.slots = torch.arange(max_len, device=device)

    def rows(self, start: int, stop: int) -> "KVCache":
        """A cache over sequences ``start .. stop - 1`` of this one, sharing its storage (dynamic
        mode, empty): what a prompt that is processed a few sequences at a time writes into."""
        view = object.__new__(KVCache)
        view.keys = [k[start:stop] for k in self.keys]
        view.values = [v[start:stop] for v in self.values]
        view.length = 0
        view.max_len = self.max_len
        view.static = False
        view.position = self.position
        view.slots = self.slots
        return view


class MultiHeadSelfAttention(nn.Module):
    """Causal self-attention.  ``num_kv_heads < num_heads`` gives grouped-query attention (the
    reference has multi-head only; with ``num_kv_heads == num_heads`` this is the reference layer)."""

    def __init__(self, d_model: int, num_heads: int, context_length: int, position_encoding: str,
                 rope_theta: float, num_kv_heads: int | None = None) -> None:
        super().__init__()
        if d_model % num_heads != 0:
            raise ValueError("d_model must be divisible by num_heads")
        self.d_model = d_model
        self.num_heads = num_heads
        self.num_kv_heads = num_kv_heads or num_heads
        if num_heads % self.num_kv_heads != 0:
            raise ValueError("num_heads must be divisible by num_kv_heads")
        self.head_dimension = d_model // num_heads
        kv_dim = self.num_kv_heads * self.head_dimension
        self.q_proj = Linear(d_model, d_model)
        self.k_proj = Linear(d_model, kv_dim)
        self.v_proj = Linear(d_model, kv_dim)
        self.output_proj = Linear(d_model, d_model)
        self.rope = (RotaryPositionalEmbedding(rope_theta, self.head_dimension, context_length)
                     if position_encoding == "rope" else None)
        # as the reference's flag (attention.py:106-117): on a GPU, multi-token calls go to the
        # library's flash-attention kernel instead of the masked softmax below (head_dim 128, 64 or 32)
        self.use_flash_attention = False

    def forward(self, inputs: torch.Tensor, positions: torch.Tensor, cache: KVCache | None = None,
                layer_index: int = 0) -> torch.Tensor:
        batch, seq, _ = inputs.shape
        hd = self.head_dimension
        q = self.q_proj(inputs).view(batch, seq, self.num_heads, hd).transpose(1, 2)
        k = self.k_proj(inputs).view(batch, seq, self.num_kv_heads, hd).transpose(1, 2)
        v = self.v_proj(inputs).view(batch, seq, self.num_kv_heads, hd).transpose(1, 2)
        if self.rope is not None:
            q = self.rope(q, positions[:, None, :].expand(batch, self.num_heads, seq))
            k = self.rope(k, positions[:, None, :].expand(batch, self.num_kv_heads, seq))
        if cache is not None and cache.static:
            # fixed-shape step: scatter the new row at the device-side position, attend over the
            # whole cache with the rows beyond that position masked out
            cache.keys[layer_index].index_copy_(2, cache.position, k.to(cache.keys[layer_index].dtype))
            cache.values[layer_index].index_copy_(2, cache.position, v.to(cache.values[layer_index].dtype))
            k, v = cache.keys[layer_index], cache.values[layer_index]
            if k.dtype != q.dtype:  # a cache kept in a narrower type: attention itself stays in q's
                k, v = k.to(q.dtype), v.to(q.dtype)
            if self.num_kv_heads != self.num_heads:
                rep = self.num_heads // self.num_kv_heads
                k = k.repeat_interleave(rep, dim=1)
                v = v.repeat_interleave(rep, dim=1)
            mask = (cache.slots <= cache.position).view(1, cache.max_len)
            attended = scaled_dot_product_attention(q, k, v, mask)
            joined = attended.transpose(1, 2).contiguous().view(batch, seq, self.d_model)
            return self.output_proj(joined)
        start = 0
        if cache is not None:
            start = cache.length
            cache.keys[layer_index][:, :, start:start + seq] = k
            cache.values[layer_index][:, :, start:start + seq] = v
        if self.use_flash_attention and inputs.is_cuda and hd in (128, 64, 32) and seq > 1:
            from .attention import flash_prefill  # the library binding; model code stays importable without it
            if cache is not None and cache.keys[layer_index].is_contiguous():
                joined = flash_prefill(q, cache.keys[layer_index], cache.values[layer_index], start)
            else:
                if cache is not None:  # a view over some sequences of a larger cache: gather the rows
                    k = cache.keys[layer_index][:, :, :start + seq]
                    v = cache.values[layer_index][:, :, :start + seq]
                joined = flash_prefill(q, k.contiguous(), v.contiguous(), start)
            return self.output_proj(joined)
        if cache is not None:
            k = cache.keys[layer_index][:, :, :start + seq]
            v = cache.values[layer_index][:, :, :start + seq]
            if k.dtype != q.dtype:
                k, v = k.to(q.dtype), v.to(q.dtype)
        total = start + seq
        if self.num_kv_heads != self.num_heads:
            rep = self.num_heads // self.num_kv_heads
            k = k.repeat_interleave(rep, dim=1)
            v = v.repeat_interleave(rep, dim=1)
        # query i (absolute position start + i) sees keys 0 .. start + i
        mask = torch.ones(seq, total, dtype=torch.bool, device=inputs.device).tril_(diagonal=start)
        attended = scaled_dot_product_attention(q, k, v, mask)
        joined = attended.transpose(1, 2).contiguous().view(batch, seq, self.d_model)
        return self.output_proj(joined)


class TransformerBlock(nn.Module):
    def __init__(self, d_model: int, num_heads: int, d_ff: int, context_length: int, position_encoding: str,
                 rope_theta: float, normalization: str, norm_placement: str, feed_forward: str,
                 num_kv_heads: int | None = None) -> None:
        super().__init__()
        if norm_placement not in {"pre", "post"}:
            raise ValueError("normalization.placement must be 'pre' or 'post'")
        self.norm_placement = norm_placement
        self.norm1 = build_norm(normalization, d_model)
        self.norm2 = build_norm(normalization, d_model)
        self.attention = MultiHeadSelfAttention(d_model, num_heads, context_length, position_encoding,
                                                rope_theta, num_kv_heads)
        self.feed_forward = build_feed_forward(feed_forward, d_model, d_ff)

    def forward(self, inputs: torch.Tensor, positions: torch.Tensor, cache: KVCache | None = None,
                layer_index: int = 0) -> torch.Tensor:
        if self.norm_placement == "pre":
            hidden = inputs + self.attention(self.norm1(inputs), positions, cache, layer_index)
            return hidden + self.feed_forward(self.norm2(hidden))
        hidden = self.norm1(inputs + self.attention(inputs, positions, cache, layer_index))
        return self.norm2(hidden + self.feed_forward(hidden))


class TransformerLM(nn.Module):
    """Decoder-only LM.  ``forward(token_ids)`` is the reference call; passing a ``KVCache``
    makes the call incremental: ``token_ids`` are the new tokens, positions continue at ``cache.length``."""

    def __init__(self, vocab_size: int, context_length: int, d_model: int, num_layers: int, num_heads: int,
                 d_ff: int, position_encoding: str = "rope", rope_theta: float = 10_000.0,
                 normalization: str = "rmsnorm", norm_placement: str = "pre", feed_forward: str = "swiglu",
                 tie_embeddings: bool = False, num_kv_heads: int | None = None) -> None:
        super().__init__()
        if position_encoding not in {"rope", "none", "learned"}:
            raise ValueError("position encoding must be rope, none, or learned")
        self.vocab_size = vocab_size
        self.context_length = context_length
        self.d_model = d_model
        self.num_layers = num_layers
        self.num_heads = num_heads
        self.num_kv_heads = num_kv_heads or num_heads
        self.d_ff = d_ff
        self.position_encoding = position_encoding
        self.tie_embeddings = tie_embeddings
        self.token_embeddings = Embedding(vocab_size, d_model)
        self.position_embeddings = Embedding(context_length, d_model) if position_encoding == "learned" else None
        self.layers = nn.ModuleList([
            TransformerBlock(d_model, num_heads, d_ff, context_length, position_encoding, rope_theta,
                             normalization, norm_placement, feed_forward, num_kv_heads)
            for _ in range(num_layers)
        ])
        self.final_norm = build_norm(normalization if norm_placement == "pre" else "none", d_model)
        self.lm_head = None if tie_embeddings else Linear(d_model, vocab_size)

    def new_cache(self, batch: int, max_len: int | None = None, dtype: torch.dtype | None = None) -> KVCache:
        weight = self.token_embeddings.weight
        return KVCache(self.num_layers, batch, self.num_kv_heads, max_len or self.context_length,
                       self.d_model // self.num_heads, weight.device, dtype or weight.dtype)

    def forward(self, token_ids: torch.Tensor, cache: KVCache | None = None,
                last_token_only: bool = False) -> torch.Tensor:
        batch, seq = token_ids.shape
        if cache is not None and cache.static:
            if seq != 1:
                raise ValueError("a static KV cache takes one token per call")
            positions = cache.position.view(1, 1).expand(batch, 1)
            hidden = self.token_embeddings(token_ids)
            if self.position_embeddings is not None:
                hidden = hidden + self.position_embeddings(positions)
            for index, layer in enumerate(self.layers):
                hidden = layer(hidden, positions, cache, index)
            hidden = self.final_norm(hidden)
            if self.tie_embeddings:
                return hidden @ self.token_embeddings.weight.transpose(0, 1)
            return self.lm_head(hidden)
        start = cache.length if cache is not None else 0
        if start + seq > self.context_length:
            raise ValueError(f"Input length {start + seq} exceeds context length {self.context_length}")
        if cache is not None and start + seq > cache.max_len:
            raise ValueError(f"KV cache holds {cache.max_len} positions, {start + seq} needed")
        positions = torch.arange(start, start + seq, device=token_ids.device).unsqueeze(0).expand(batch, -1)
        hidden = self.token_embeddings(token_ids)
        if self.position_embeddings is not None:
            hidden = hidden + self.position_embeddings(positions)
        for index, layer in enumerate(self.layers):
            hidden = layer(hidden, positions, cache, index)
        if cache is not None:
            cache.length = start + seq
        if last_token_only:
            hidden = hidden[:, -1:, :]
        hidden = self.final_norm(hidden)
        if self.tie_embeddings:
            return hidden @ self.token_embeddings.weight.transpose(0, 1)
        return self.lm_head(hidden)


def build_model(config: dict[str, Any], vocab_size: int) -> TransformerLM:
    """Model from a reference-style config dict (keys as in the reference's model YAML)."""
    position = config.get("position_encoding", {})
    normalization = config.get("normalization", {})
    feed_forward = config.get("feed_forward", {})
    d_model = int(config["d_model"])
    ff_type = str(feed_forward.get("type", "swiglu"))
    default_d_ff = ((int(8 * d_model / 3) + 63) // 64) * 64 if ff_type == "swiglu" else 4 * d_model
    return TransformerLM(
        vocab_size=vocab_size,
        context_length=int(config["context_length"]),
        d_model=d_model,
        num_layers=int(config["num_layers"]),
        num_heads=int(config["num_heads"]),
        d_ff=int(config.get("d_ff", default_d_ff)),
        position_encoding=str(position.get("type", "rope")),
        rope_theta=float(position.get("theta", 10_000.0)),
        normalization=str(normalization.get("type", "rmsnorm")),
        norm_placement=str(normalization.get("placement", "pre")),
        feed_forward=ff_type,
        tie_embeddings=bool(config.get("tie_embeddings", False)),
        num_kv_heads=(int(config["num_kv_heads"]) if "num_kv_heads" in config else None),
    )


@torch.no_grad()
def greedy_decode(model: TransformerLM, prompt_tokens: torch.Tensor, max_new_tokens: int,
                  eos_token_id: int | None = None, return_margins: bool = False,
                  kv_dtype: torch.dtype | None = None):
    """Batched greedy decoding with a KV cache.

    Same token rule as the reference's ``generate`` at temperature <= 0
    (src/ajllm/generation/generator.py:10-28, sampling.py:9-10): next = argmax(logits[:, -1]),
    ties to the lowest index; the reference recomputes the whole sequence every step and
    handles one prompt, this keeps a KV cache and takes ``[B, T]`` prompts.  With
    ``eos_token_id`` decoding stops once every row has produced it.  Returns ``[B, T + new]``
    (and, with ``return_margins``, the fp32 top-1 minus top-2 logit of every step, ``[B, new]``)."""
    model.eval()
    tokens = prompt_tokens if prompt_tokens.dim() == 2 else prompt_tokens.reshape(1, -1)
    batch, prompt_len = tokens.shape
    cache = model.new_cache(batch, prompt_len + max_new_tokens, dtype=kv_dtype)
    out = [tokens]
    margins = []
    done = torch.zeros(batch, dtype=torch.bool, device=tokens.device)
    step_input = tokens
    for _ in range(max_new_tokens):
        logits = model(step_input, cache, last_token_only=True)[:, -1, :]
        next_token = torch.argmax(logits, dim=-1, keepdim=True)
        if return_margins:
            top2 = torch.topk(logits.float(), 2, dim=-1).values
            margins.append(top2[:, 0] - top2[:, 1])
        out.append(next_token)
        step_input = next_token
        if eos_token_id is not None:
            done |= next_token.squeeze(1) == eos_token_id
            if bool(done.all()):
                break
    result = torch.cat(out, dim=1)
    if return_margins:
        return result, torch.stack(margins, dim=1)
    return result
