"""End-to-end greedy decoding of the 12-layer benchmark model with every linear quantized.

The model is the reference architecture (src/ajllm/modeling/transformer.py:13-126) at the size the
benchmark names: 12 layers, d_model 2048, 16 heads (head_dim 128), SwiGLU d_ff 5632, vocab 32000,
RMSNorm, RoPE, untied lm_head, reference init under a fixed seed; all linears W4A16 group-128.
Prompts are seeded random token ids ``[B, 512]``; 256 tokens are decoded greedily with a KV cache.
The headline figure replays the one-token step from a HIP graph (``decoding.FusedDecoder``: the
linears, norms, RoPE, cache write, attention and SwiGLU gate all run in this library's kernels); the
eager PyTorch loop around the same linears is timed beside it, and so are the quantized linears of
one step on their own.
"""

from __future__ import annotations

import time

import torch

from . import decoding, modeling
from .quant import QuantLinear, quantize_model_

CONFIG = dict(vocab_size=32000, context_length=1024, d_model=2048, num_layers=12, num_heads=16, d_ff=5632)
PROMPT_LEN = 512
NEW_TOKENS = 256


def build_quantized_model(device, scheme: str = "w4a16_g128", seed: int = 1234, config: dict | None = None):
    torch.manual_seed(seed)
    with torch.device(device):
        model = modeling.TransformerLM(**(config or CONFIG)).eval()
    quantize_model_(model, scheme)
    torch.cuda.empty_cache()
    return model


def _linear_seconds_per_step(dec: "decoding.FusedDecoder", batch: int, device) -> float:
    """Time of the quantized linears of one decode step on their own, as the decoder launches them
    (fused q|k|v and w1|w3, output projection, w2, lm_head; plain GEMVs on ``[batch, in_features]``
    inputs), replayed from a HIP graph."""
    linears = [w[name] for w in dec.layers for name in ("qkv", "o", "w13", "w2")] + [dec.head]
    inputs = [torch.randn((batch, m.in_features), device=device).to(torch.bfloat16) for m in linears]
    stream = torch.cuda.Stream()
    torch.cuda.synchronize()  # the inputs above are complete before ``stream`` reads them
    with torch.cuda.stream(stream), torch.no_grad():
        for m, x in zip(linears, inputs):
            m(x)
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            for m, x in zip(linears, inputs):
                m(x)
        graph.replay()
        stream.synchronize()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record(stream)
        for _ in range(20):
            graph.replay()
        stop.record(stream)
        stop.synchronize()
    return start.elapsed_time(stop) / 1e3 / 20


@torch.no_grad()
def bench_decode_short(device, log=print, batches=(1, 8), scheme: str = "w4a16_g128") -> list[dict]:
    """The graph-replayed greedy decode of :func:`bench_decode` alone (prompt 512, 256 new tokens, batch 1
    and 8), without the eager-loop comparison: a few seconds, for the default benchmark line."""
    t0 = time.perf_counter()
    model = build_quantized_model(device, scheme)
    torch.cuda.synchronize()
    build_s = time.perf_counter() - t0
    packed = sum(m.wq.numel() * 4 + m.meta.numel() * m.meta.element_size()
                 for m in model.modules() if isinstance(m, QuantLinear))
    results = []
    for batch in batches:
        g = torch.Generator().manual_seed(100 + batch)
        prompt = torch.randint(0, CONFIG["vocab_size"], (batch, PROMPT_LEN), generator=g).to(device)
        dec = decoding.FusedDecoder(model, batch, PROMPT_LEN + NEW_TOKENS)
        dec.prefill(prompt, fused=True)
        dec.generate(8)  # eager step + capture + first replays
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        tokens = dec.generate(NEW_TOKENS)
        torch.cuda.synchronize()
        t_graph = time.perf_counter() - t0
        steps = NEW_TOKENS - 8
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        dec.prefill(prompt, fused=True)
        torch.cuda.synchronize()
        t_prefill = time.perf_counter() - t0
        t_linear = _linear_seconds_per_step(dec, batch, device)
        step = t_graph / steps
        r = {"scheme": scheme, "batch": batch, "prompt": PROMPT_LEN, "new_tokens": NEW_TOKENS,
             "decode_tok/s": batch * steps / t_graph, "ms_per_step": step * 1e3,
             "prefill_library_kernels_s": t_prefill, "prefill_library_kernels_tok/s": batch * PROMPT_LEN / t_prefill,
             "quant_linear_ms_per_step": t_linear * 1e3, "quant_linear_share_of_step": t_linear / step,
             "quant_linear_GB/s": packed / t_linear / 1e9, "packed_weight_bytes": packed,
             "launches_per_step": dec.launches_per_step(), "model_build_s": build_s,
             "tokens_in_vocab": bool(int(tokens.min()) >= 0 and int(tokens.max()) < CONFIG["vocab_size"])}
        # the same decode with keys and values stored as bf16 (the decoder's kv_dtype option; not the
        # reference's arithmetic: its cache has the model's dtype)
        del dec
        dec = decoding.FusedDecoder(model, batch, PROMPT_LEN + NEW_TOKENS, torch.bfloat16)
        dec.prefill(prompt, fused=True)
        dec.generate(8)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        dec.generate(NEW_TOKENS)
        torch.cuda.synchronize()
        t_bf16 = time.perf_counter() - t0
        r["bf16_kv_cache"] = {"decode_tok/s": batch * steps / t_bf16, "ms_per_step": t_bf16 / steps * 1e3}
        # the decoder's faster folding: normed activations rounded to bf16 BEFORE the norm's row scale, which is then
        # applied to the matmul outputs (fp32 cache; not the reference's rounding point)
        del dec
        dec = decoding.FusedDecoder(model, batch, PROMPT_LEN + NEW_TOKENS, activation_rounding="before_scale")
        dec.prefill(prompt, fused=True)
        dec.generate(8)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        dec.generate(NEW_TOKENS)
        torch.cuda.synchronize()
        t_fold = time.perf_counter() - t0
        r["activations_rounded_before_norm_scale"] = {"decode_tok/s": batch * steps / t_fold,
                                                      "ms_per_step": t_fold / steps * 1e3,
                                                      "launches_per_step": dec.launches_per_step()}
        log("decode", r)
        results.append(r)
        del dec
    del model
    torch.cuda.empty_cache()
    return results


def cache2_for(model, prompt):
    """A dynamic KV cache holding the prompt (for a one-step logits comparison)."""
    cache = model.new_cache(prompt.shape[0], prompt.shape[1] + 8)
    model(prompt, cache, last_token_only=True)
    return cache


@torch.no_grad()
def bench_decode(device, log=print, batches=(1, 8), scheme: str = "w4a16_g128") -> list[dict]:
    model = build_quantized_model(device, scheme)
    packed = sum(m.wq.numel() * 4 + m.meta.numel() * m.meta.element_size()
                 for m in model.modules() if isinstance(m, QuantLinear))
    results = []
    for batch in batches:
        g = torch.Generator().manual_seed(100 + batch)
        prompt = torch.randint(0, CONFIG["vocab_size"], (batch, PROMPT_LEN), generator=g).to(device)
        modeling.greedy_decode(model, prompt[:, :32], 4)  # warm-up: library load, allocator
        torch.cuda.synchronize()
        cache = model.new_cache(batch, PROMPT_LEN + NEW_TOKENS)
        t0 = time.perf_counter()
        logits = model(prompt, cache, last_token_only=True)[:, -1, :]
        torch.cuda.synchronize()
        t_prefill = time.perf_counter() - t0
        tokens = [torch.argmax(logits, dim=-1, keepdim=True)]
        top2 = [torch.topk(logits.float(), 2, dim=-1).values]
        t0 = time.perf_counter()
        for _ in range(NEW_TOKENS - 1):
            logits = model(tokens[-1], cache, last_token_only=True)[:, -1, :]
            tokens.append(torch.argmax(logits, dim=-1, keepdim=True))
            top2.append(torch.topk(logits.float(), 2, dim=-1).values)
        torch.cuda.synchronize()
        t_decode = time.perf_counter() - t0
        eager_tokens = torch.cat(tokens, dim=1)
        margins = torch.stack([t[:, 0] - t[:, 1] for t in top2], dim=1)  # [B, new]: eager top-1 minus top-2
        del cache
        # the same decode with the step replayed from a HIP graph
        dec = decoding.FusedDecoder(model, batch, PROMPT_LEN + NEW_TOKENS)
        dec.prefill(prompt)
        dec.generate(8)  # eager step + capture + first replays
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        graph_tokens = dec.generate(NEW_TOKENS)
        torch.cuda.synchronize()
        t_graph = time.perf_counter() - t0
        graph_steps = NEW_TOKENS - 8
        # where a row first differs from the eager loop, and the eager margin at that step: the two
        # runs sum in different orders, so a choice can flip where the margin is below their noise
        dec.prefill(prompt)
        noise = float((dec._logits().float() - model(dec.token, cache2_for(model, prompt))[:, -1].float()).abs().max())
        diverged = []
        for row in range(batch):
            diff = (graph_tokens[row] != eager_tokens[row]).nonzero()
            if len(diff):
                step_i = int(diff[0])
                diverged.append({"row": row, "step": step_i, "eager_margin": float(margins[row, step_i])})
        same = min([d["step"] for d in diverged], default=NEW_TOKENS)
        t_linear = _linear_seconds_per_step(dec, batch, device)
        # the prompt through this library's kernels only (GEMMs, add + RMSNorm, RoPE + cache write,
        # flash attention, the gate in the w1|w3 GEMM): flash-attention arithmetic, so not the path
        # the token comparison above uses
        dec.prefill(prompt, fused=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        dec.prefill(prompt, fused=True)
        torch.cuda.synchronize()
        t_prefill_fused = time.perf_counter() - t0
        step = t_graph / graph_steps
        r = {
            "scheme": scheme, "batch": batch, "prompt": PROMPT_LEN, "new_tokens": NEW_TOKENS,
            "prefill_s": t_prefill, "prefill_tok/s": batch * PROMPT_LEN / t_prefill,
            "prefill_library_kernels_s": t_prefill_fused,
            "prefill_library_kernels_tok/s": batch * PROMPT_LEN / t_prefill_fused,
            "decode_tok/s": batch * graph_steps / t_graph,
            "ms_per_step": step * 1e3,
            "eager_decode_tok/s": batch * (NEW_TOKENS - 1) / t_decode,
            "eager_ms_per_step": t_decode / (NEW_TOKENS - 1) * 1e3,
            "tokens_identical_to_eager_up_to_step": same,
            "first_divergences": diverged,
            "logit_noise_between_the_two_loops": noise,
            "quant_linear_ms_per_step": t_linear * 1e3,
            "quant_linear_share_of_step": t_linear / step,
            "quant_linear_GB/s": packed / t_linear / 1e9,
            "packed_weight_bytes": packed,
            "launches_per_step": dec.launches_per_step(),
            "loop": "one-token step replayed from a HIP graph (eight steps per graph launch), token fed back on the device; the step is this "
                    "library's kernels only (fused q|k|v and w1|w3 GEMVs, the residual adds and the SwiGLU gate in "
                    "the matmuls' epilogues, the RMSNorms formed on the consumers' way in up to batch 4 and as "
                    "launches of their own above, RoPE + cache write + single-query attention in one kernel, its "
                    "row chunks merged by a launch of its own, greedy pick + embedding row + step counters in one "
                    "launch)",
        }
        log("decode", r)
        results.append(r)
        del dec
    return results
