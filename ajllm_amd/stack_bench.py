"""Llama-3-8B-shaped layer stack with W8A16 per-channel linears: prefill of 4 x 2048 tokens and
batch-32 decoding at context 2048, with the quantized linears' share of each.

The stack is the reference architecture (src/ajllm/modeling/transformer.py:13-126) at that shape:
32 pre-norm RMSNorm blocks, d_model 4096, 32 query heads over 8 key/value heads (grouped-query
attention, which the reference's multi-head layer cannot express: ``modeling`` adds
``num_kv_heads``), head_dim 128, RoPE, SwiGLU d_ff 14336, vocab 128256, untied lm_head, reference
init under a fixed seed.  Every linear is a ``QuantLinear`` ("w8a16"); about 7.5 GB of int8
weights are read per decode step.  Prompts are seeded random token ids.
"""

from __future__ import annotations

import time

import torch

from . import decoding
from .e2e_bench import build_quantized_model
from .quant import QuantLinear

CONFIG = dict(vocab_size=128256, context_length=2048 + 128, d_model=4096, num_layers=32, num_heads=32,
              num_kv_heads=8, d_ff=14336)
BATCH = 32
CONTEXT = 2048
PREFILL_ROWS = 4


def _graph_seconds(fn, stream, reps: int = 10) -> float:
    """Seconds per call of ``fn`` replayed from a HIP graph on ``stream``."""
    torch.cuda.synchronize()  # inputs made on the default stream are complete before ``stream`` reads them
    with torch.cuda.stream(stream), torch.no_grad():
        fn()
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            fn()
        graph.replay()
        stream.synchronize()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record(stream)
        for _ in range(reps):
            graph.replay()
        stop.record(stream)
        stop.synchronize()
    return start.elapsed_time(stop) / 1e3 / reps


def _eager_linear_seconds(model, rows: int, device) -> float:
    """The model's QuantLinears, each once on ``[rows, in_features]`` inputs (lm_head on
    ``PREFILL_ROWS`` rows: the prefill asks for the last position's logits only)."""
    layers = [m for m in model.modules() if isinstance(m, QuantLinear)]
    inputs = [torch.randn((PREFILL_ROWS if m is model.lm_head else rows, m.in_features), device=device).to(torch.bfloat16)
              for m in layers]
    for m, x in zip(layers, inputs):
        m(x)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for m, x in zip(layers, inputs):
        m(x)
    torch.cuda.synchronize()
    return time.perf_counter() - t0


@torch.no_grad()
def bench_stack(device, log=print, config: dict | None = None, batch: int = BATCH, context: int = CONTEXT,
                decode_steps: int = 32, scheme: str = "w8a16", kv_dtype: torch.dtype | None = None,
                short: bool = False) -> dict:
    """``short`` (the default bench line's leg) leaves out the pass through the model's own PyTorch code and the
    two decoder options (bf16 cache, activations rounded before the norm's row scale)."""
    config = dict(config or CONFIG)
    t0 = time.perf_counter()
    model = build_quantized_model(device, scheme, seed=4321, config=config)
    torch.cuda.synchronize()
    build_s = time.perf_counter() - t0
    for layer in model.layers:  # prefill attention through the library's flash-attention kernel
        layer.attention.use_flash_attention = True
    quant = [m for m in model.modules() if isinstance(m, QuantLinear)]
    packed = sum(m.wq.numel() * 4 + m.meta.numel() * m.meta.element_size() for m in quant)
    g = torch.Generator().manual_seed(77)
    prompt = torch.randint(0, config["vocab_size"], (batch, context), generator=g).to(device)

    # ---- prefill, PREFILL_ROWS sequences (PREFILL_ROWS * context tokens) per pass, into the decoder's cache
    dec = decoding.FusedDecoder(model, batch, context + decode_steps + 8, kv_dtype)
    dec.prefill(prompt[:, :64], rows_per_pass=PREFILL_ROWS, fused=True)  # warm-up: library load, allocator
    dec.prefill(prompt[:, :64], rows_per_pass=PREFILL_ROWS)
    torch.cuda.synchronize()
    # (a) the model's own PyTorch code around the library's GEMMs and flash attention, one pass
    dec.cache.static = False
    eager_logits, t_pass_eager = None, None
    if not short:
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        eager_logits = model(prompt[:PREFILL_ROWS], dec.cache.rows(0, PREFILL_ROWS), last_token_only=True)[:, -1, :]
        torch.cuda.synchronize()
        t_pass_eager = time.perf_counter() - t0
    # (b) library kernels only, every pass (this is what fills the cache the decode below starts from)
    pass_times = []
    logits = []
    for start in range(0, batch, PREFILL_ROWS):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        logits.append(dec._prefill_rows(prompt[start:start + PREFILL_ROWS], start))
        torch.cuda.synchronize()
        pass_times.append(time.perf_counter() - t0)
    pass_times.sort()
    t_pass = pass_times[len(pass_times) // 2]
    t_pass_linear = _eager_linear_seconds(model, PREFILL_ROWS * context, device)
    logits_rel, first_match = None, None
    if eager_logits is not None:
        logits_rel = float((eager_logits.double() - logits[0].double()).norm() / eager_logits.double().norm())
        top2 = torch.topk(eager_logits.float(), 2, dim=-1).values
        first_match = {"rows_with_equal_argmax": int((torch.argmax(eager_logits, -1) == torch.argmax(logits[0], -1)).sum()),
                       "rows": PREFILL_ROWS, "smallest_top2_margin": float((top2[:, 0] - top2[:, 1]).min()),
                       "largest_logit_difference": float((eager_logits.float() - logits[0].float()).abs().max())}
    # hand the prefilled cache to the decoder (what FusedDecoder.prefill does after its passes)
    dec.cache.length = context
    dec.cache.static = True
    dec.cache.position.fill_(context)
    dec.step_index.zero_()
    first = torch.argmax(torch.cat(logits, dim=0), dim=-1, keepdim=True)
    dec.out.index_copy_(1, dec.step_index, first)
    dec.token.copy_(first)
    torch.index_select(dec.embedding, 0, first.view(-1), out=dec.embedded)
    dec.step_index.add_(1)
    dec.produced, dec.prompt_len = 1, context

    # ---- decode: the fused step replayed from a graph
    dec.generate(4)  # eager step + capture + replay
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    tokens = dec.generate(4 + decode_steps)
    torch.cuda.synchronize()
    t_step = (time.perf_counter() - t0) / decode_steps

    # ---- the step's parts on their own, each replayed from a graph
    stream = torch.cuda.Stream()
    xs = {name: torch.randn((batch, w.wq.shape[1] * 64 if scheme == "w8a16" else w.wq.shape[1] * 128), device=device)
          .to(torch.bfloat16) for name, w in (("qkv", dec.layers[0]["qkv"]), ("o", dec.layers[0]["o"]),
                                              ("w13", dec.layers[0]["w13"]), ("w2", dec.layers[0]["w2"]))}

    from . import _lib
    lib = _lib.load()

    def linears():
        # (with the decoder's buffer for split-K partial sums lent, as during its steps)
        _lib.check(lib.ajq_matmul_workspace_set(dec.matmul_ws.data_ptr(), dec.matmul_ws.numel()), "matmul_workspace_set")
        try:
            for w in dec.layers:
                for name in ("qkv", "o", "w13", "w2"):
                    w[name](xs[name])
            dec.head(xs["qkv"])
        finally:
            lib.ajq_matmul_workspace_set(None, 0)

    t_linear = _graph_seconds(linears, stream)

    qkv = torch.randn((batch, (dec.heads + 2 * dec.kv_heads) * 128), device=device)

    def attention():
        st = torch.cuda.current_stream().cuda_stream
        for index, w in enumerate(dec.layers):
            _lib.check(lib.ajq_attn_step(qkv.data_ptr(), w["cos"].data_ptr(), w["sin"].data_ptr(),
                                         dec.cache.position.data_ptr(), dec.cache.keys[index].data_ptr(),
                                         dec.cache.values[index].data_ptr(), dec.kv_flag, batch, dec.heads,
                                         dec.kv_heads, 128, dec.max_len, dec.attended.data_ptr(),
                                         dec.attn_ws.data_ptr(), dec.attn_ws_bytes, st), "attn_step")

    t_attention = _graph_seconds(attention, stream)
    kv_bytes = 2 * len(dec.layers) * batch * dec.kv_heads * (context + decode_steps // 2) * 128 * dec.cache.keys[0].element_size()
    result = {
        "scheme": scheme, "config": config, "batch": batch, "context": context, "build_s": build_s,
        "packed_weight_bytes": packed,
        "prefill": {"tokens_per_pass": PREFILL_ROWS * context, "s_per_pass": t_pass,
                    "path": "library kernels only: GEMMs, add + RMSNorm, RoPE + cache write, flash attention, gate",
                    "s_per_pass_model_code_with_library_gemm_and_attention": t_pass_eager,
                    "last_position_logits_relative_difference_between_the_two": logits_rel,
                    "first_token_choice_between_the_two": first_match,
                    "tok/s": PREFILL_ROWS * context / t_pass,
                    "quant_linear_s_per_pass": t_pass_linear, "quant_linear_share": t_pass_linear / t_pass,
                    "quant_linear_TFLOP/s": 2 * PREFILL_ROWS * context * sum(
                        m.in_features * m.out_features for m in quant if m is not model.lm_head) / t_pass_linear / 1e12},
        "decode": {"steps": decode_steps, "ms_per_step": t_step * 1e3, "tok/s": batch / t_step,
                   "quant_linear_ms_per_step": t_linear * 1e3, "quant_linear_share_of_step": t_linear / t_step,
                   "quant_linear_GB/s": packed / t_linear / 1e9,
                   "attention_ms_per_step": t_attention * 1e3, "attention_share_of_step": t_attention / t_step,
                   "kv_cache_GB/s": kv_bytes / t_attention / 1e9,
                   "kv_cache_dtype": str(dec.cache.keys[0].dtype).replace("torch.", ""),
                   "first_tokens_row0": tokens[0, :8].tolist()},
    }
    result["decode"]["launches_per_step"] = dec.launches_per_step()
    if short:
        result["prefill"] = {k: v for k, v in result["prefill"].items() if v is not None}
    if kv_dtype is None and not short:
        # the same decode with a bf16 KV cache (keys and values rounded on write; arithmetic fp32):
        # the attention's bytes halve
        del dec
        torch.cuda.empty_cache()
        dec16 = decoding.FusedDecoder(model, batch, context + decode_steps + 8, torch.bfloat16)
        dec16.prefill(prompt, rows_per_pass=PREFILL_ROWS, fused=True)
        dec16.generate(4)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        dec16.generate(4 + decode_steps)
        torch.cuda.synchronize()
        t16 = (time.perf_counter() - t0) / decode_steps
        result["decode_bf16_kv_cache"] = {"ms_per_step": t16 * 1e3, "tok/s": batch / t16}
        # the decoder's folded step (norms, residual adds and the gate in the matmuls' epilogues, six launches per
        # layer; the normed activations are rounded to bf16 before the norm's row scale), fp32 cache
        del dec16
        torch.cuda.empty_cache()
        decf = decoding.FusedDecoder(model, batch, context + decode_steps + 8, activation_rounding="before_scale")
        decf.prefill(prompt, rows_per_pass=PREFILL_ROWS, fused=True)
        decf.generate(4)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        decf.generate(4 + decode_steps)
        torch.cuda.synchronize()
        tf = (time.perf_counter() - t0) / decode_steps
        result["decode_activations_rounded_before_norm_scale"] = {"ms_per_step": tf * 1e3, "tok/s": batch / tf,
                                                                  "launches_per_step": decf.launches_per_step()}
    log("stack", result)
    return result
