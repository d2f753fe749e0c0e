#!/usr/bin/env python3
"""Benchmark of the quantized-linear hot path on one MI355X.

Default run (what the driver calls: ``python bench.py --gpus 1 --steps K --warmup W``):

* timed region: the W4A16-g128 decode GEMV at the headline shape K = N = 4096, M = 1.
  One *step* is one pass over ``--copies`` distinct weight matrices (default 64, 559 MB of
  packed weights, larger than the 256 MB Infinity Cache plus the L2s, so every launch
  streams its weights from HBM).  The launches of a step are recorded once into a HIP
  graph and replayed, so the host's launch cost is not part of the measurement.  Timing is
  by HIP events on the launch stream around exactly K steps.
* after it (not part of ``value``): the M = 2048 prefill GEMMs (W4 and W8, K = N = 4096) in
  TFLOP/s against the bf16 dense MFMA peak, and the CPU baseline: the oracle's quantized
  linear timed on this box's host cores for the same GEMV shape.

* also after it: the end-to-end greedy decode of the 12-layer W4A16 model (prompt 512 + 256 tokens,
  batch 1 and 8) in tokens/s, short form, and the Llama-3-8B-shaped W8A16 stack (4 x 2048 prefill passes,
  batch-32 decode at context 2048 with the quantized linears' share of the step), short form.

``--sweep`` adds the rest of the decode sweep (three shapes x M in {1, 4, 16}, W4 and W8)
and all prefill shapes; ``--decode`` replaces the short decode leg by the long one (eager PyTorch loop
beside it, token comparison between the two loops).  One JSON line is printed on stdout; everything else goes to stderr.
"""

from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

import torch

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, vendor peak
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16 MFMA, vendor peak
GEMV_W4_4096_M1_HBM_BYTES = 9.03e6  # measured: 4407.6 KiB x 1.9993 fetched + 8 KiB x 1.0 written per launch
GEMV_W4_4096_M1_HBM_BYTES_SOURCE = ("constant from profiles/gemv_w4_m1_4096_hbm_traffic.md (separate rocprofv3 --pmc "
                                    "FETCH_SIZE and WRITE_SIZE runs of this command), not measured by this run")


def log(*args) -> None:
    print(*args, file=sys.stderr, flush=True)


# ------------------------------------------------------------------ algorithmic work
def w4_gemv_bytes(m: int, n: int, k: int) -> float:
    """packed nibbles + fp16 scales + 4-bit zero-points + bf16 activations in and out"""
    return n * k / 2 + 2 * n * k / 128 + 0.5 * n * k / 128 + 2 * m * k + 2 * m * n


def w8_gemv_bytes(m: int, n: int, k: int) -> float:
    return n * k + 2 * n + 2 * m * k + 2 * m * n


def gemm_flops(m: int, n: int, k: int) -> float:
    return 2.0 * m * n * k


# ------------------------------------------------------------------ synthetic inputs
def make_w4(n: int, k: int, copies: int, device, seed: int):
    """``copies`` distinct private W4 weights.  Weights ~ N(0, 0.02) are quantized on the GPU."""
    from ajllm_amd import quantize_w4_g128, repack_w4

    out = []
    g = torch.Generator(device=device).manual_seed(seed)
    for _ in range(copies):
        w = torch.randn((n, k), generator=g, device=device, dtype=torch.float32) * 0.02
        out.append(repack_w4(*quantize_w4_g128(w)))
    return out


def make_w8(n: int, k: int, copies: int, device, seed: int):
    from ajllm_amd import quantize_w8, repack_w8

    out = []
    g = torch.Generator(device=device).manual_seed(seed)
    for _ in range(copies):
        w = torch.randn((n, k), generator=g, device=device, dtype=torch.float32) * 0.02
        q, s = quantize_w8(w)
        out.append((repack_w8(q), s))
    return out


def make_x(m: int, k: int, device, seed: int, outliers: bool = False) -> torch.Tensor:
    g = torch.Generator(device=device).manual_seed(seed)
    x = torch.randn((m, k), generator=g, device=device, dtype=torch.float32)
    if outliers:
        mask = torch.rand((m, k), generator=g, device=device) < 0.001
        x = torch.where(mask, x * 20.0, x)
    return x.to(torch.bfloat16)


# ------------------------------------------------------------------ timing
def time_graph_steps(step_fn, steps: int, warmup: int) -> float:
    """Record ``step_fn`` (kernel launches on the current stream) into a HIP graph, replay it
    ``warmup`` times untimed, then time exactly ``steps`` replays with HIP events on the same
    stream.  Returns seconds for the ``steps`` replays."""
    stream = torch.cuda.Stream()
    torch.cuda.synchronize()  # inputs made on the default stream are complete before ``stream`` reads them
    with torch.cuda.stream(stream):
        step_fn()  # eager once: sets function attributes, fills caches
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            step_fn()
        for _ in range(warmup):
            graph.replay()
        stream.synchronize()
        start = torch.cuda.Event(enable_timing=True)
        stop = torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        start.record(stream)
        for _ in range(steps):
            graph.replay()
        stop.record(stream)
        stop.synchronize()
        torch.cuda.synchronize()
    return start.elapsed_time(stop) / 1e3


def bench_gemv(scheme: str, m: int, n: int, k: int, copies: int, steps: int, warmup: int, device,
               lend_workspace: bool = False) -> dict:
    """One launch per matrix through the C ABI, `copies` distinct matrices per step.  lend_workspace: with the
    caller-lent buffer of ajq_matmul_workspace_set in place (as the decoders run), which lets shapes with a long K
    split K over workgroups."""
    from ajllm_amd import _lib, w4a16_matmul, w8a16_matmul

    weights = make_w4(n, k, copies, device, 1234) if scheme == "w4" else make_w8(n, k, copies, device, 1234)
    x = make_x(m, k, device, 99)
    fn = w4a16_matmul if scheme == "w4" else w8a16_matmul
    nbytes = w4_gemv_bytes(m, n, k) if scheme == "w4" else w8_gemv_bytes(m, n, k)
    outs = []

    def step():
        outs.clear()
        for a, b in weights:
            outs.append(fn(x, a, b, torch.bfloat16, kernel="gemv"))

    lib = _lib.load()
    lent = torch.zeros(int(lib.ajq_matmul_workspace_bytes()), dtype=torch.uint8, device=device) if lend_workspace else None
    if lent is not None:
        _lib.check(lib.ajq_matmul_workspace_set(lent.data_ptr(), lent.numel()), "matmul_workspace_set")
    try:
        seconds = time_graph_steps(step, steps, warmup)
    finally:
        if lent is not None:
            lib.ajq_matmul_workspace_set(None, 0)
    launches = steps * copies
    us = seconds / launches * 1e6
    gbs = nbytes / (seconds / launches) / 1e9
    row = {"scheme": scheme, "M": m, "N": n, "K": k, "launches": launches, "us_per_launch": us,
           "bytes_per_launch": nbytes, "GB/s": gbs, "frac_hbm_peak": gbs / HBM_PEAK_GBS,
           "ms_per_step": seconds / steps * 1e3}
    if lend_workspace:
        row["matmul_workspace"] = "lent (ajq_matmul_workspace_set)"
    return row


def bench_gemm(scheme: str, m: int, n: int, k: int, steps: int, warmup: int, device, copies: int = 4) -> dict:
    from ajllm_amd import w4a16_matmul, w8a16_matmul

    weights = make_w4(n, k, copies, device, 4321) if scheme == "w4" else make_w8(n, k, copies, device, 4321)
    x = make_x(m, k, device, 98, outliers=True)
    fn = w4a16_matmul if scheme == "w4" else w8a16_matmul
    outs = []

    def step():
        outs.clear()
        for a, b in weights:
            outs.append(fn(x, a, b, torch.bfloat16, kernel="gemm"))

    seconds = time_graph_steps(step, steps, warmup)
    launches = steps * copies
    us = seconds / launches * 1e6
    tflops = gemm_flops(m, n, k) / (seconds / launches) / 1e12
    return {"scheme": scheme, "M": m, "N": n, "K": k, "launches": launches, "us_per_launch": us,
            "TFLOP/s": tflops, "frac_mfma_peak": tflops / MFMA_BF16_PEAK_TFLOPS}


# ------------------------------------------------------------------ yardsticks
def bench_dense_library_gemm(m: int, n: int, k: int, steps: int, warmup: int, device, copies: int = 4) -> dict:
    """The vendor library's plain bf16 GEMM (``torch.matmul`` on weights already expanded to bf16) on
    the same shape, launch pattern and activations: what a GEMM with no dequantization work reaches."""
    gen = torch.Generator(device=device).manual_seed(4321)
    weights = [(torch.randn((n, k), generator=gen, device=device) * 0.02).to(torch.bfloat16) for _ in range(copies)]
    x = make_x(m, k, device, 98, outliers=True)
    outs = []

    def step():
        outs.clear()
        for w in weights:
            outs.append(torch.matmul(x, w.t()))

    seconds = time_graph_steps(step, steps, warmup)
    launches = steps * copies
    tflops = gemm_flops(m, n, k) / (seconds / launches) / 1e12
    return {"M": m, "N": n, "K": k, "us_per_launch": seconds / launches * 1e6, "TFLOP/s": tflops,
            "frac_mfma_peak": tflops / MFMA_BF16_PEAK_TFLOPS}


def bench_flash_prefill(batch: int, heads: int, kv_heads: int, seq: int, cache_dtype, device, reps: int = 10,
                        head_dim: int = 128) -> dict:
    """Causal prefill attention (``ajq_attn_prefill``) on config 5's prefill shape (head_dim 128; 64 and 32 for
    the head-size sweep), fp32 queries, bf16 output; flops counted for the causal half only."""
    from ajllm_amd.attention import flash_prefill

    g = torch.Generator(device="cpu").manual_seed(11)
    q = torch.randn((batch, heads, seq, head_dim), generator=g).to(device)
    keys = torch.randn((batch, kv_heads, seq, head_dim), generator=g).to(device).to(cache_dtype)
    values = torch.randn((batch, kv_heads, seq, head_dim), generator=g).to(device).to(cache_dtype)
    for _ in range(3):
        flash_prefill(q, keys, values, 0, out_dtype=torch.bfloat16)
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(reps):
        flash_prefill(q, keys, values, 0, out_dtype=torch.bfloat16)
    end.record()
    end.synchronize()
    us = start.elapsed_time(end) * 1e3 / reps
    flops = 4.0 * batch * heads * seq * seq * 0.5 * head_dim
    return {"B": batch, "H": heads, "Hkv": kv_heads, "T": seq, "head_dim": head_dim,
            "kv_cache": str(cache_dtype).replace("torch.", ""),
            "us_per_call": us, "causal_TFLOP/s": flops / us * 1e-6, "frac_mfma_peak": flops / us * 1e-6 / MFMA_BF16_PEAK_TFLOPS}


def bench_mfma_rate(device, workgroups: int = 256, iters: int = 100_000, launches: int = 4) -> dict:
    """bf16 MFMA rate the GPU sustains from registers alone (no memory traffic): with constant
    operands and with random mantissas, where the power limit lowers the shader clock."""
    from ajllm_amd import _lib

    lib = _lib.load_bench()
    sink = torch.empty(workgroups * 512, dtype=torch.float32, device=device)
    clocks = torch.zeros(2, dtype=torch.int64, device=device)
    flops = ctypes.c_double(0.0)
    stream = torch.cuda.current_stream()
    out = {}
    for name, rnd in (("constant_operands", 0), ("random_operands", 1)):
        def launch():
            status = lib.ajqb_mfma_rate(rnd, iters, workgroups, sink.data_ptr(), clocks.data_ptr(),
                                        ctypes.addressof(flops), stream.cuda_stream)
            if status:
                raise RuntimeError(f"ajqb_mfma_rate: {lib.ajqb_last_error().decode()}")
        launch()
        torch.cuda.synchronize()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record(stream)
        for _ in range(launches):
            launch()
        stop.record(stream)
        stop.synchronize()
        seconds = start.elapsed_time(stop) / 1e3 / launches
        cycles, ticks = (int(v) for v in clocks.tolist())
        out[name] = {"TFLOP/s": flops.value / seconds / 1e12, "ms_per_launch": seconds * 1e3,
                     "shader_clock_GHz": cycles / max(ticks, 1) * 0.1}
    return out


def cpu_baseline(m: int, n: int, k: int, budget_s: float = 15.0) -> dict:
    """The oracle's quantized linear (dequantize -> matmul, fp32) on the host cores, same shape
    and seeded inputs as the timed GEMV.  The reference project has no quantized CPU path (its
    only linear is the dense ``x @ W.T`` of src/ajllm/modeling/layers.py:32-33, also timed here),
    so ``kind`` is "port"."""
    from oracle import qspec

    threads = min(16, os.cpu_count() or 1)
    torch.set_num_threads(threads)
    g = torch.Generator().manual_seed(1234)
    w = torch.randn((n, k), generator=g, dtype=torch.float32) * 0.02
    layer = qspec.QuantLinearRef.from_weight(w, "w4a16_g128", cache_dequant=False)
    x = torch.randn((m, k), generator=torch.Generator().manual_seed(99)).to(torch.bfloat16)
    nbytes = w4_gemv_bytes(m, n, k)

    def timed(fn, reps_cap=20):
        fn()
        times = []
        t_end = time.perf_counter() + budget_s / 3
        while len(times) < reps_cap and (time.perf_counter() < t_end or len(times) < 3):
            t0 = time.perf_counter()
            fn()
            times.append(time.perf_counter() - t0)
        times.sort()
        return times[len(times) // 2], len(times)

    t0 = time.perf_counter()
    t_deq, n_deq = timed(lambda: layer(x), reps_cap=1000)  # the baseline itself: as many calls as a third of the budget holds
    spent = time.perf_counter() - t0
    layer.cache_dequant = True
    layer.dequantized()
    t_pre, n_pre = timed(lambda: layer(x))
    w_bf16 = w.to(torch.bfloat16)
    t_dense, n_dense = timed(lambda: x @ w_bf16.t())
    return {
        "value": nbytes / t_deq / 1e9, "unit": "GB/s", "cores": threads, "kind": "port",
        "sample": f"oracle QuantLinearRef (dequantize every call, fp32 matmul), W4A16-g128 M={m} N={n} K={k}, "
                  f"median of {n_deq} calls ({spent:.1f} s of host time); same algorithmic bytes as the GPU figure",
        "predequantized_GB/s": nbytes / t_pre / 1e9,
        "dense_bf16_x_at_wT_GB/s": nbytes / t_dense / 1e9,
        "ms_per_call": t_deq * 1e3, "host_cpu_count": os.cpu_count(),
    }


def bench_gemv_forms(device, batches=(1, 4, 8), reps: int = 30) -> list[dict]:
    """Microseconds per launch, in a graph chain over six distinct W4 weight sets, of the decode GEMV in its
    plain form and with work folded in: the norm / gate PROLOGUE forms (every workgroup forms the
    activations from the fp32 sources; "from sums": the norm's sums of squares come from the producer) against
    the row-scale / residual / gate EPILOGUE forms (a workgroup touches its own 16 columns), on the 12-layer
    benchmark model's four projection shapes."""
    from ajllm_amd import _lib, quantize_w4_g128, repack_w4

    lib = _lib.load()
    rows = []
    for name, n, k in (("q|k|v", 6144, 2048), ("output", 2048, 2048), ("w1|w3", 11264, 2048), ("w2", 2048, 5632)):
        weights = []
        for _ in range(6):
            q, s, z = quantize_w4_g128(torch.randn(n, k, device=device) * 0.02)
            weights.append(repack_w4(q, s, z))
        for m in batches:
            x = torch.randn(m, k, device=device).to(torch.bfloat16)
            y = torch.empty(m, n, device=device)
            yg = torch.empty(m, n // 2, device=device, dtype=torch.bfloat16)
            h, gain = torch.randn(m, n, device=device), torch.ones(n, device=device)
            h2, xt = torch.empty_like(h), torch.empty(m, n, device=device, dtype=torch.bfloat16)
            ssq_out, ssq_in = torch.zeros(16, n // 16, device=device), torch.rand(16, k // 16, device=device) + 1
            hk, dk, gk = torch.randn(m, k, device=device), torch.randn(m, k, device=device), torch.ones(k, device=device)
            hk2, ab = torch.empty_like(hk), torch.randn(m, 2 * k, device=device)
            forms = {
                "plain": lambda wq, meta, st: lib.ajq_w4a16_gemv(
                    x.data_ptr(), m, k, wq.data_ptr(), meta.data_ptr(), n, y.data_ptr(), _lib.AJQ_OUT_F32, st),
                "row_scale_epilogue": lambda wq, meta, st: lib.ajq_w4a16_gemv_rowscale(
                    x.data_ptr(), ssq_in.data_ptr(), k // 16, 1e-5, m, k, wq.data_ptr(), meta.data_ptr(), n, y.data_ptr(),
                    _lib.AJQ_OUT_F32, 0, st),
                "row_scale_and_gate_epilogue": lambda wq, meta, st: lib.ajq_w4a16_gemv_rowscale(
                    x.data_ptr(), ssq_in.data_ptr(), k // 16, 1e-5, m, k, wq.data_ptr(), meta.data_ptr(), n, yg.data_ptr(),
                    _lib.AJQ_OUT_BF16, 1, st),
                "residual_epilogue": lambda wq, meta, st: lib.ajq_w4a16_gemv_residual(
                    x.data_ptr(), m, k, wq.data_ptr(), meta.data_ptr(), n, h.data_ptr(), gain.data_ptr(), h2.data_ptr(),
                    xt.data_ptr(), ssq_out.data_ptr(), st),
            }
            if lib.ajq_gemv_fused_supported(m, k):
                forms["norm_prologue"] = lambda wq, meta, st: lib.ajq_w4a16_gemv_norm(
                    hk.data_ptr(), dk.data_ptr(), gk.data_ptr(), 1e-5, hk2.data_ptr(), m, k, wq.data_ptr(), meta.data_ptr(),
                    n, y.data_ptr(), _lib.AJQ_OUT_F32, st)
                forms["gate_prologue"] = lambda wq, meta, st: lib.ajq_w4a16_gemv_gate(
                    ab.data_ptr(), m, k, wq.data_ptr(), meta.data_ptr(), n, y.data_ptr(), _lib.AJQ_OUT_F32, st)
            if lib.ajq_gemv_fused_supported(m, k) and k // 16 <= 256:
                forms["norm_from_sums_prologue"] = lambda wq, meta, st: lib.ajq_w4a16_gemv_norm_sums(
                    hk.data_ptr(), ssq_in.data_ptr(), k // 16, gk.data_ptr(), 1e-5, m, k, wq.data_ptr(), meta.data_ptr(),
                    n, y.data_ptr(), _lib.AJQ_OUT_F32, 0, st)
            launches = 8 * len(weights)
            row = {"projection": name, "M": m, "N": n, "K": k}
            for form, call in forms.items():
                stream = torch.cuda.Stream()
                torch.cuda.synchronize()
                with torch.cuda.stream(stream):
                    def chain():
                        for i in range(launches):
                            status = call(*weights[i % len(weights)], stream.cuda_stream)
                            if status != 0:
                                raise RuntimeError(f"{form}: status {status}")
                    chain()
                    stream.synchronize()
                    graph = torch.cuda.CUDAGraph()
                    with torch.cuda.graph(graph, stream=stream):
                        chain()
                    graph.replay()
                    stream.synchronize()
                    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    start.record(stream)
                    for _ in range(reps):
                        graph.replay()
                    stop.record(stream)
                    stop.synchronize()
                row[form + "_us"] = round(start.elapsed_time(stop) * 1e3 / reps / launches, 2)
            rows.append(row)
    return rows


# ------------------------------------------------------------------ main
def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--copies", type=int, default=64, help="distinct weight matrices per step")
    ap.add_argument("--sweep", action="store_true", help="also time the full decode and prefill sweeps")
    ap.add_argument("--decode", action="store_true", help="also time end-to-end greedy decode")
    ap.add_argument("--stack", action="store_true",
                    help="also time the Llama-3-8B-shaped W8A16 stack (4 x 2048 prefill, batch-32 decode at context 2048)")
    ap.add_argument("--forms", action="store_true",
                    help="also time the decode GEMV's prologue forms against its epilogue forms (norm, gate, residual)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extras", action="store_true", help="timed region only")
    ap.add_argument("--no-decode", action="store_true",
                    help="skip the short end-to-end decode leg of the default line (counter-collection runs: "
                         "the profiler does not survive the leg's graph replays)")
    args = ap.parse_args()
    if args.gpus != 1:
        log("bench.py: this build runs on exactly one GPU (the quantized linear is a single-GPU "
            f"path; no collectives exist). --gpus {args.gpus} is not supported.")
        return 2
    if not torch.cuda.is_available():
        log("bench.py: no GPU visible")
        return 2
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    from ajllm_amd import _lib

    _lib.load()
    m, n, k = 1, 4096, 4096
    head = bench_gemv("w4", m, n, k, args.copies, args.steps, args.warmup, device)
    log("headline", json.dumps(head))
    extras: dict = {}
    if not args.no_extras:
        gemm = []
        for gn in (4096, 14336):  # the prefill configuration's two output widths at the target M = 2048
            for scheme in ("w4", "w8"):
                r = bench_gemm(scheme, 2048, gn, 4096, steps=10 if gn == 4096 else 5, warmup=3, device=device)
                log("gemm", json.dumps(r))
                gemm.append(r)
        extras["prefill_gemm"] = gemm
        # the headline kernel with 64 times the rows per launch: what it streams once the cost of
        # launching is spread over 559 MB instead of 8.7 MB
        tall = bench_gemv("w4", 1, 64 * 4096, 4096, 2, 10, 3, device)
        log("tall gemv", json.dumps(tall))
        extras["gemv_same_kernel_64x_rows_per_launch"] = tall
        dense = bench_dense_library_gemm(2048, 4096, 4096, steps=10, warmup=3, device=device)
        log("dense library gemm", json.dumps(dense))
        dense_wide = bench_dense_library_gemm(2048, 14336, 4096, steps=5, warmup=3, device=device)
        log("dense library gemm", json.dumps(dense_wide))
        rate = bench_mfma_rate(device)
        log("mfma rate", json.dumps(rate))
        extras["yardsticks"] = {
            "dense_bf16_library_gemm": [dense, dense_wide],
            "mfma_from_registers": rate,
            "note": "not part of the product path: the vendor library's plain bf16 GEMM on weights already "
                    "expanded to bf16, and the MFMA rate sustained with no memory traffic (random operands "
                    "reach the power limit and the shader clock drops)",
        }
    if not args.no_extras:
        flash = [bench_flash_prefill(4, 32, 8, 2048, dt, device) for dt in (torch.bfloat16, torch.float32)]
        for r in flash:
            log("prefill attention", json.dumps(r))
        extras["prefill_attention"] = flash
    if not args.no_extras and not args.decode and not args.no_decode:
        # config 4 end to end, short form: the 12-layer W4A16 model, prompt 512 + 256 greedy tokens,
        # batch 1 and 8, decode step replayed from a HIP graph (tokens/s is the third headline metric)
        from ajllm_amd.e2e_bench import bench_decode_short

        extras["decode"] = bench_decode_short(device, log)
    if args.sweep:
        heads_sweep = [bench_flash_prefill(b, 32, 8, t, dt, device, head_dim=hd)
                       for hd in (128, 64, 32) for (b, t) in ((4, 2048), (1, 8192))
                       for dt in (torch.bfloat16, torch.float32)]
        for r in heads_sweep:
            log("prefill attention by head size", json.dumps(r))
        extras["prefill_attention_head_sizes"] = heads_sweep
        sweep = []
        for scheme in ("w4", "w8"):
            for (sn, sk) in ((4096, 4096), (14336, 4096), (4096, 14336)):
                copies = args.copies if sn * sk < 2**25 else max(12, args.copies // 3)
                for sm in (1, 4, 16):
                    r = bench_gemv(scheme, sm, sn, sk, copies, max(5, args.steps // 5), 2, device)
                    log("sweep", json.dumps(r))
                    sweep.append(r)
        extras["decode_sweep"] = sweep
        # the rows that change when the caller lends the matmul workspace (K = 14336 at 9 to 16 rows)
        lent_rows = []
        for scheme in ("w4", "w8"):
            r = bench_gemv(scheme, 16, 4096, 14336, 10, max(5, args.steps // 5), 2, device, lend_workspace=True)
            log("sweep, workspace lent", json.dumps(r))
            lent_rows.append(r)
        extras["decode_sweep_workspace_lent"] = lent_rows
        gemm = []
        for scheme in ("w4", "w8"):
            for sm in (256, 2048, 8192):
                for sn in (4096, 14336):
                    r = bench_gemm(scheme, sm, sn, 4096, steps=5, warmup=2, device=device, copies=2)
                    log("gemm", json.dumps(r))
                    gemm.append(r)
        extras["prefill_sweep"] = gemm
        dense = []
        for sm in (256, 2048, 8192):
            for sn in (4096, 14336):
                r = bench_dense_library_gemm(sm, sn, 4096, steps=5, warmup=2, device=device, copies=2)
                log("dense library gemm", json.dumps(r))
                dense.append(r)
        extras.setdefault("yardsticks", {})["dense_bf16_library_gemm_sweep"] = dense
    if args.decode:
        from ajllm_amd.e2e_bench import bench_decode  # heavy import kept off the default path

        extras["decode"] = bench_decode(device, log)
    if args.forms:
        extras["decode_gemv_forms"] = bench_gemv_forms(device)
        for row in extras["decode_gemv_forms"]:
            log("forms", json.dumps(row))
    if args.stack or not (args.no_extras or args.no_decode):
        # the Llama-3-8B-shaped W8A16 stack: one 4 x 2048 prefill pass per four sequences, then batch-32 decode at
        # context 2048 with the quantized linears' and the attention's share of the step; the default line carries
        # the short form (fp32 cache, reference rounding only), --stack adds the decoder's two options
        from ajllm_amd.stack_bench import bench_stack

        torch.cuda.empty_cache()
        extras["stack_8b_w8a16"] = bench_stack(device, log, short=not args.stack)
        torch.cuda.empty_cache()
    # a plain device-to-device copy of known size: the yardstick the FETCH_SIZE / WRITE_SIZE
    # counters of a profiling run are scaled by (64 MiB read + 64 MiB written per launch)
    calib_src = torch.empty(64 * 2**20, dtype=torch.uint8, device=device)
    calib_dst = torch.empty_like(calib_src)
    for _ in range(3):
        calib_dst.copy_(calib_src)
    torch.cuda.synchronize()
    cpu = None if args.no_cpu else cpu_baseline(m, n, k)
    if cpu:
        log("cpu_baseline", json.dumps(cpu))

    line = {
        "metric": "W4A16 dequant-GEMV GB/s",
        "value": head["GB/s"],
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": head["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic (seeded N(0,0.02) weights quantized on the GPU, N(0,1) bf16 activations)",
        "config": {
            "workload": "W4A16-g128 decode GEMV, K=N=4096, M=1 (decode sweep headline shape)",
            "arithmetic": "bf16 activations x uint4 weights (exact integers in bf16) on MFMA, fp32 accumulate, fp16 scales applied in fp32",
            "launches_per_step": args.copies,
            "distinct_weight_bytes": args.copies * (n * k // 2 + n * k // 128 * 4),
            "launch": "HIP graph replay of one step",
        },
        "roofline": {
            "bound": "hbm",
            "achieved": head["GB/s"],
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": head["frac_hbm_peak"],
            # HBM bytes per launch from separate rocprofv3 --pmc runs of this command
            # (FETCH_SIZE, WRITE_SIZE, each scaled by what a 64 MiB copy reads on the same counter)
            "traffic": GEMV_W4_4096_M1_HBM_BYTES,
            "traffic_source": GEMV_W4_4096_M1_HBM_BYTES_SOURCE,
            "kernel": "ajq::dequant_gemv_kernel<8, 4, 1, true, true, true>",
            "algorithmic_bytes_per_launch": head["bytes_per_launch"],
            "avg_launch_us": head["us_per_launch"],
        },
        "cpu_baseline": cpu,
        "peaks": {"hbm_GB/s": HBM_PEAK_GBS, "mfma_bf16_TFLOP/s": MFMA_BF16_PEAK_TFLOPS},
    }
    line.update(extras)
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
