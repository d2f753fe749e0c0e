"""Greedy decoding with the decode step replayed from a HIP graph.

Same token rule as the reference's ``generate`` at temperature <= 0
(src/ajllm/generation/generator.py:10-28, sampling.py:9-10) and as
``modeling.greedy_decode``: next = argmax(logits[:, -1]).  The prompt is processed eagerly; the
one-token step (embedding, 12 x block, norm, lm_head, argmax, KV-cache scatter, position + 1) has
fixed shapes (``modeling.KVCache`` in static mode), is recorded once and replayed per token, with
the chosen token fed back on the device: no host round trip between steps.
"""

from __future__ import annotations

import ctypes

import torch

from . import _lib, modeling
from .quant import QuantLinear, repack_w4, repack_w8, w4a16_matmul, w8a16_matmul


class GraphDecoder:
    def __init__(self, model: modeling.TransformerLM, batch: int, max_len: int,
                 kv_dtype: torch.dtype | None = None) -> None:
        if max_len > model.context_length:
            raise ValueError(f"max_len {max_len} exceeds the model's context length {model.context_length}")
        self.model = model.eval()
        self.batch = batch
        self.max_len = max_len
        device = model.token_embeddings.weight.device
        if device.type != "cuda":
            raise ValueError("GraphDecoder needs the model on a ROCm device")
        self.device = device
        self.cache = model.new_cache(batch, max_len, dtype=kv_dtype)
        self.token = torch.zeros((batch, 1), dtype=torch.long, device=device)
        self.out = torch.zeros((batch, max_len), dtype=torch.long, device=device)
        self.step_index = torch.zeros(1, dtype=torch.long, device=device)
        self.graph: torch.cuda.CUDAGraph | None = None
        # a second graph of ``steps_per_graph`` consecutive steps, replayed while that many tokens are still
        # wanted (1: none; the step's state lives on the device, so steps chain inside one graph as they do
        # across replays)
        self.steps_per_graph = 1   # read when the graphs are captured (the first ``generate``)
        self.graph_many: torch.cuda.CUDAGraph | None = None
        self.graph_many_steps = 0
        self.stream = torch.cuda.Stream(device=device)
        # greedy unless ``set_sampling`` says otherwise
        self.temperature = 0.0
        self.top_p: float | None = None
        self.uniforms: torch.Tensor | None = None

    def set_sampling(self, temperature: float, top_p: float | None = None, seed: int = 0) -> None:
        """Choose tokens as the reference's ``sample_next_token`` does (src/ajllm/generation/sampling.py:8-22):
        ``temperature <= 0`` is the greedy choice (the default), otherwise a draw from
        ``softmax(logits / temperature)``, restricted by ``top_p`` to the most probable tokens whose mass reaches it.
        Call it before ``prefill``; graphs recorded so far are dropped.  The random numbers are ``max_len x batch``
        uniforms made once from ``seed`` on the device (one row per output column), so a recorded step replays with
        fresh ones and equal seeds give equal tokens; the draw itself is the library's ``ajq_sample_pick``."""
        if top_p is not None and not 0 < top_p <= 1:
            raise ValueError("top_p must be in (0, 1]")
        self.temperature, self.top_p = float(temperature), top_p
        self.uniforms = None
        if self.temperature > 0:
            generator = torch.Generator(device=self.device).manual_seed(int(seed))
            self.uniforms = torch.rand((self.max_len, self.batch), generator=generator, device=self.device)
        self.graph = self.graph_many = None
        self.graph_many_steps = 0

    def _sample(self, logits: torch.Tensor, embedding: torch.Tensor | None = None, hidden: torch.Tensor | None = None,
                counters: torch.Tensor | None = None, ticket: torch.Tensor | None = None, vocab: int | None = None) -> None:
        """A draw per row of fp32 ``logits`` (row stride = its width; the first ``vocab`` columns count) into
        ``self.token`` and ``self.out[:, step_index]``; with ``embedding`` the chosen rows go to ``hidden``, with
        ``counters`` the step's two counters advance."""
        _lib.check(_lib.load().ajq_sample_pick(
            logits.data_ptr(), self.batch, vocab or logits.shape[1], logits.shape[1], self.temperature,
            1.0 if self.top_p is None else float(self.top_p), self.uniforms.data_ptr(), self.uniforms.shape[0],
            embedding.data_ptr() if embedding is not None else None, embedding.shape[1] if embedding is not None else 0,
            hidden.data_ptr() if hidden is not None else None, self.token.data_ptr(), self.out.data_ptr(),
            self.out.shape[1], self.step_index.data_ptr(), counters.data_ptr() if counters is not None else None,
            ticket.data_ptr() if ticket is not None else None, None, _stream()), "sample_pick")

    def _choose(self, logits: torch.Tensor) -> None:
        """The next token of every row from ``logits`` ``[B, V]`` into ``self.token`` and ``self.out[:, step_index]``
        (greedy: the first maximum; otherwise ``_sample``)."""
        if self.temperature > 0:
            self._sample(logits.float().contiguous())
            return
        nxt = torch.argmax(logits, dim=-1, keepdim=True)
        self.out.index_copy_(1, self.step_index, nxt)
        self.token.copy_(nxt)

    def _logits(self) -> torch.Tensor:
        """Logits ``[B, V]`` of the token in ``self.token`` at cache row ``cache.position``."""
        return self.model(self.token, self.cache)[:, -1, :]

    @torch.no_grad()
    def _step(self) -> None:
        self._choose(self._logits())
        self.cache.position.add_(1)
        self.step_index.add_(1)

    @torch.no_grad()
    def prefill(self, prompt: torch.Tensor, rows_per_pass: int | None = None) -> None:
        """Run the prompt ``[B, T]`` through the model (eagerly) and choose the first new token.
        ``rows_per_pass`` sequences go through the model at a time (default: all of them)."""
        if prompt.shape[0] != self.batch or prompt.shape[1] >= self.max_len:
            raise ValueError("prompt must be [batch, T] with T < max_len")
        self.cache.static = False
        prompt = prompt.to(self.device)
        step = rows_per_pass or self.batch
        parts = []
        for start in range(0, self.batch, step):
            rows = self.cache.rows(start, min(start + step, self.batch))
            parts.append(self.model(prompt[start:start + step], rows, last_token_only=True)[:, -1, :])
        logits = torch.cat(parts, dim=0)
        self.cache.length = prompt.shape[1]
        self.cache.static = True
        self.cache.position.fill_(prompt.shape[1])
        self.step_index.zero_()
        self._choose(logits)
        self.step_index.add_(1)
        self.produced = 1
        self.prompt_len = prompt.shape[1]

    def _all_rows_done(self, eos_token_id: int) -> int | None:
        """Number of tokens after which every row has produced ``eos_token_id`` (None: not yet)."""
        seen = (self.out[:, : self.produced] == eos_token_id)
        if not bool(seen.any(dim=1).all()):
            return None
        first = seen.int().argmax(dim=1)  # index of each row's first eos
        return int(first.max()) + 1

    @torch.no_grad()
    def generate(self, new_tokens: int, eos_token_id: int | None = None, eos_check_every: int = 16) -> torch.Tensor:
        """Decode until ``new_tokens`` tokens exist since ``prefill`` and return them ``[B, new_tokens]``.

        With ``eos_token_id`` decoding stops once every row has produced it, as the reference's
        ``generate`` does for its one row (src/ajllm/generation/generator.py:26-27) and
        ``modeling.greedy_decode`` for a batch: the returned tensor ends with the step at which the
        last row produced it.  The host looks at the tokens every ``eos_check_every`` steps only (a
        look is a synchronisation); steps replayed past the stopping point are cut off the result."""
        if self.prompt_len + new_tokens > self.max_len:
            raise ValueError("the KV cache is too short for this many tokens")
        if eos_token_id is not None:
            if eos_check_every < 1:
                raise ValueError("eos_check_every must be positive")
            target = self.produced
            while True:
                done_at = self._all_rows_done(eos_token_id)
                if done_at is not None or target >= new_tokens:
                    break
                target = min(new_tokens, target + eos_check_every)
                self.generate(target)
            return self.out[:, : (done_at if done_at is not None else new_tokens)].clone()
        current = torch.cuda.current_stream(self.device)
        self.stream.wait_stream(current)
        with torch.cuda.stream(self.stream):
            if self.graph is None:
                # one eager step first (loads the library, sizes the allocator), then capture;
                # both advance the decoding state like any other step
                if self.produced < new_tokens:
                    self._step()
                    self.produced += 1
                if self.produced < new_tokens:
                    self.stream.synchronize()
                    graph = torch.cuda.CUDAGraph()
                    with torch.cuda.graph(graph, stream=self.stream):
                        self._step()
                    self.graph = graph
                    # capture does not execute: replay now for this step's effect
                    self.graph.replay()
                    self.produced += 1
                    if self.steps_per_graph > 1:
                        self.stream.synchronize()
                        many = torch.cuda.CUDAGraph()
                        with torch.cuda.graph(many, stream=self.stream):
                            for _ in range(self.steps_per_graph):
                                self._step()
                        self.graph_many, self.graph_many_steps = many, self.steps_per_graph
            while self.produced < new_tokens:
                if self.graph_many is not None and new_tokens - self.produced >= self.graph_many_steps:
                    self.graph_many.replay()
                    self.produced += self.graph_many_steps
                else:
                    self.graph.replay()
                    self.produced += 1
        # The host waits for the decode stream here instead of making the caller's stream wait for it on the device
        # (``current.wait_stream``): a stream waiting on an event of another hardware queue keeps the command processor
        # polling for it while the replays run, which costs about a microsecond per launch of the graph (0.59 -> 0.50
        # ms per step at batch 8 of the 12-layer model, measured; no cost when both streams share a hardware queue,
        # one case in four).  The tokens are host-visible results anyway.
        self.stream.synchronize()
        return self.out[:, :new_tokens].clone()


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


class _FusedLinear:
    """Several QuantLinears that share their input, as one matmul over their concatenated rows
    (the private tiles are 16-row blocks, so concatenating along N is concatenating tensors)."""

    def __init__(self, layers: list[QuantLinear]) -> None:
        scheme = layers[0].scheme
        if any(m.scheme != scheme or m.in_features != layers[0].in_features for m in layers):
            raise ValueError("fused linears must share scheme and input width")
        if any(m.out_features % 16 != 0 for m in layers[:-1]):
            raise ValueError("only the last of several fused linears may have a ragged row count")
        self.scheme = scheme
        self.out_features = sum(m.out_features for m in layers)
        self.wq = torch.cat([m.wq for m in layers], dim=0).contiguous()
        self.meta = torch.cat([m.meta for m in layers], dim=0).contiguous()

        self.in_features = layers[0].in_features
        self.rows16 = self.wq.shape[0] * 16

    def __call__(self, x_bf16: torch.Tensor) -> torch.Tensor:
        fn = w8a16_matmul if self.scheme == "w8a16" else w4a16_matmul
        return fn(x_bf16, self.wq, self.meta, torch.float32)

    def gate_fusable(self, rows: int) -> bool:
        """Whether the tile GEMM with the SwiGLU gate in its epilogue takes ``rows`` rows of this
        (w1 | w3) pair."""
        return bool(_lib.load().ajq_gemm_gate_supported(rows, self.rows16, self.in_features,
                                                        0 if self.scheme == "w8a16" else 1))

    def gated(self, x_bf16: torch.Tensor) -> torch.Tensor:
        """``bf16(silu(x w1^T) * (x w3^T))`` for this (w1 | w3) pair, one matmul launch (plus the W4
        group-sum kernel): the fp32 ``[rows, 2 F]`` intermediate is never written."""
        lib = _lib.load()
        rows = x_bf16.shape[0]
        y = torch.empty((rows, self.rows16 // 2), dtype=torch.bfloat16, device=x_bf16.device)
        if self.scheme == "w8a16":
            status = lib.ajq_w8a16_gemm_gate(x_bf16.data_ptr(), rows, self.in_features, self.wq.data_ptr(),
                                             self.meta.data_ptr(), self.rows16, y.data_ptr(), _stream())
        else:
            nbytes = lib.ajq_w4a16_gemm_workspace_bytes(rows, self.in_features)
            workspace = torch.empty((nbytes,), dtype=torch.uint8, device=x_bf16.device)
            status = lib.ajq_w4a16_gemm_gate(x_bf16.data_ptr(), rows, self.in_features, self.wq.data_ptr(),
                                             self.meta.data_ptr(), self.rows16, y.data_ptr(), workspace.data_ptr(),
                                             nbytes, _stream())
        _lib.check(status, "gemm_gate")
        return y

    @classmethod
    def interleaved_gate(cls, w1: QuantLinear, w3: QuantLinear) -> "_FusedLinear":
        """(w1 | w3) with the rows interleaved in blocks of 8, so that every 16-row tile of the private
        layout holds 8 gate-projection rows and the 8 matching up-projection rows: a GEMV workgroup
        then has both factors of ``silu(a) * u`` for its 8 outputs (``rowscaled(..., gated=True)``).
        Quantization is per row, so the canonical tensors are permuted, not requantized."""
        if w1.scheme != w3.scheme or w1.in_features != w3.in_features or w1.out_features != w3.out_features:
            raise ValueError("w1 and w3 must share scheme and shape")
        if w1.out_features % 8 != 0:
            raise ValueError("d_ff must be a multiple of 8")

        def mix(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
            blocks = torch.stack((a.reshape(a.shape[0] // 8, 8, *a.shape[1:]), b.reshape(b.shape[0] // 8, 8, *b.shape[1:])), dim=1)
            return blocks.reshape(2 * a.shape[0], *a.shape[1:]).contiguous()

        self = cls.__new__(cls)
        self.scheme = w1.scheme
        self.in_features = w1.in_features
        self.out_features = 2 * w1.out_features
        if self.scheme == "w8a16":
            self.wq = repack_w8(mix(w1.qweight, w3.qweight))
            self.meta = mix(w1.scales, w3.scales)
        else:
            self.wq, self.meta = repack_w4(mix(w1.qweight, w3.qweight), mix(w1.scales, w3.scales), mix(w1.zeros, w3.zeros))
        self.rows16 = self.wq.shape[0] * 16
        return self

    def epilogue_fusable(self, batch: int) -> bool:
        """Whether the GEMVs with a residual / row-scale / gate epilogue are built for this batch and
        input width."""
        return bool(_lib.load().ajq_gemv_epilogue_supported(batch, self.in_features))

    def rowscale_fusable(self, batch: int) -> bool:
        """Whether ``rowscaled`` is built for this batch and input width (it adds ``in_features / 16`` tile sums)."""
        return bool(_lib.load().ajq_gemv_rowscale_supported(batch, self.in_features))

    def residual(self, x_bf16: torch.Tensor, h_in: torch.Tensor, gain: torch.Tensor, h_out: torch.Tensor,
                 xt: torch.Tensor | None, ssq: torch.Tensor) -> None:
        """``h_out = h_in + self(x)``, ``xt = bf16(h_out * gain)`` (skipped if None) and the per-tile sums of squares
        of ``h_out`` in ``ssq`` (what the next ``normed_from_sums`` / ``rowscaled`` needs in place of a norm), one launch."""
        lib = _lib.load()
        fn = lib.ajq_w8a16_gemv_residual if self.scheme == "w8a16" else lib.ajq_w4a16_gemv_residual
        _lib.check(fn(x_bf16.data_ptr(), x_bf16.shape[0], self.in_features, self.wq.data_ptr(), self.meta.data_ptr(),
                      self.rows16, h_in.data_ptr(), gain.data_ptr(), h_out.data_ptr(),
                      xt.data_ptr() if xt is not None else None, ssq.data_ptr(), _stream()), "gemv_residual")

    def merge_residual(self, partial: torch.Tensor, splits: int, rows: int, h_in: torch.Tensor, gain: torch.Tensor,
                       h_out: torch.Tensor, xt: torch.Tensor | None, ssq: torch.Tensor) -> None:
        """``residual`` whose input is the attention output merged from ``splits`` partial results per (row, head) on
        the way in (as ``after_merge``), one launch."""
        lib = _lib.load()
        fn = lib.ajq_w8a16_gemv_merge_residual if self.scheme == "w8a16" else lib.ajq_w4a16_gemv_merge_residual
        _lib.check(fn(partial.data_ptr(), splits, rows, self.in_features, self.wq.data_ptr(), self.meta.data_ptr(),
                      self.rows16, h_in.data_ptr(), gain.data_ptr(), h_out.data_ptr(),
                      xt.data_ptr() if xt is not None else None, ssq.data_ptr(), _stream()), "gemv_merge_residual")

    def gated_interleaved(self, x_bf16: torch.Tensor, gated: torch.Tensor) -> torch.Tensor:
        """``bf16(silu(a) * u)`` into ``gated`` for an ``interleaved_gate`` pair and plain bf16 activations, one launch."""
        lib = _lib.load()
        fn = lib.ajq_w8a16_gemv_gated if self.scheme == "w8a16" else lib.ajq_w4a16_gemv_gated
        _lib.check(fn(x_bf16.data_ptr(), x_bf16.shape[0], self.in_features, self.wq.data_ptr(), self.meta.data_ptr(),
                      self.rows16, gated.data_ptr(), _stream()), "gemv_gated")
        return gated

    def normed_from_sums(self, h: torch.Tensor, ssq: torch.Tensor, gain: torch.Tensor, eps: float,
                         gated: torch.Tensor | None = None) -> torch.Tensor:
        """``self(bf16(RMSNorm(h) * gain))`` with the norm's sums of squares taken from what ``residual`` left in
        ``ssq``: the activations are rounded exactly where a separate norm kernel rounds them.  One launch; ``gated``
        as in ``rowscaled``."""
        lib = _lib.load()
        rows = h.shape[0]
        fn = lib.ajq_w8a16_gemv_norm_sums if self.scheme == "w8a16" else lib.ajq_w4a16_gemv_norm_sums
        if gated is None:
            y = torch.empty((rows, self.rows16), dtype=torch.float32, device=h.device)
            dtype, gate = _lib.AJQ_OUT_F32, 0
        else:
            y, dtype, gate = gated, _lib.AJQ_OUT_BF16, 1
        _lib.check(fn(h.data_ptr(), ssq.data_ptr(), ssq.shape[1], gain.data_ptr(), eps, rows, self.in_features,
                      self.wq.data_ptr(), self.meta.data_ptr(), self.rows16, y.data_ptr(), dtype, gate, _stream()),
                   "gemv_norm_sums")
        return y

    def rowscaled(self, xt: torch.Tensor, ssq: torch.Tensor, eps: float, gated: torch.Tensor | None = None) -> torch.Tensor:
        """``self(RMSNorm(h) * gain)`` from ``xt = bf16(h * gain)`` and the sums of squares ``residual`` left,
        one launch; with ``gated`` (bf16 ``[rows, out / 2]``, for an ``interleaved_gate`` pair) the SwiGLU
        product of the outputs is written there instead."""
        lib = _lib.load()
        rows = xt.shape[0]
        fn = lib.ajq_w8a16_gemv_rowscale if self.scheme == "w8a16" else lib.ajq_w4a16_gemv_rowscale
        if gated is None:
            y = torch.empty((rows, self.rows16), dtype=torch.float32, device=xt.device)
            dtype, gate = _lib.AJQ_OUT_F32, 0
        else:
            y, dtype, gate = gated, _lib.AJQ_OUT_BF16, 1
        _lib.check(fn(xt.data_ptr(), ssq.data_ptr(), ssq.shape[1], eps, rows, self.in_features, self.wq.data_ptr(),
                      self.meta.data_ptr(), self.rows16, y.data_ptr(), dtype, gate, _stream()), "gemv_rowscale")
        return y

    def fusable(self, batch: int) -> bool:
        """Whether the GEMV with a norm / gate prologue is built for this batch and input width."""
        return bool(_lib.load().ajq_gemv_fused_supported(batch, self.in_features))

    def after_norm(self, h_in: torch.Tensor, delta: torch.Tensor | None, gain: torch.Tensor, eps: float,
                   h_out: torch.Tensor) -> torch.Tensor:
        """``self(bf16(RMSNorm(h_in + delta) * gain))`` with ``h_out = h_in + delta``, one launch."""
        lib = _lib.load()
        y = torch.empty((h_in.shape[0], self.rows16), dtype=torch.float32, device=h_in.device)
        fn = lib.ajq_w8a16_gemv_norm if self.scheme == "w8a16" else lib.ajq_w4a16_gemv_norm
        _lib.check(fn(h_in.data_ptr(), delta.data_ptr() if delta is not None else None, gain.data_ptr(), eps,
                      h_out.data_ptr(), h_in.shape[0], self.in_features, self.wq.data_ptr(), self.meta.data_ptr(),
                      self.rows16, y.data_ptr(), _lib.AJQ_OUT_F32, _stream()), "gemv_norm")
        return y

    def merge_splits(self, batch: int) -> int:
        """Largest number of attention row chunks the GEMV that merges them on its way in takes
        for ``batch`` rows of this layer's input width (0: not built)."""
        return int(_lib.load().ajq_gemv_merge_max_splits(batch, self.in_features))

    def after_merge(self, partial: torch.Tensor, splits: int, rows: int) -> torch.Tensor:
        """``self(attention output)`` with the output merged from ``splits`` partial results per
        (row, head) on the way in (``ajq_attn_step_partial`` left them in ``partial``), one launch."""
        lib = _lib.load()
        y = torch.empty((rows, self.rows16), dtype=torch.float32, device=partial.device)
        fn = lib.ajq_w8a16_gemv_merge if self.scheme == "w8a16" else lib.ajq_w4a16_gemv_merge
        _lib.check(fn(partial.data_ptr(), splits, rows, self.in_features, self.wq.data_ptr(), self.meta.data_ptr(),
                      self.rows16, y.data_ptr(), _lib.AJQ_OUT_F32, _stream()), "gemv_merge")
        return y

    def after_gate(self, ab: torch.Tensor) -> torch.Tensor:
        """``self(bf16(silu(a) * u))`` for ``ab = (a | u)``, one launch."""
        lib = _lib.load()
        y = torch.empty((ab.shape[0], self.rows16), dtype=torch.float32, device=ab.device)
        fn = lib.ajq_w8a16_gemv_gate if self.scheme == "w8a16" else lib.ajq_w4a16_gemv_gate
        _lib.check(fn(ab.data_ptr(), ab.shape[0], self.in_features, self.wq.data_ptr(), self.meta.data_ptr(),
                      self.rows16, y.data_ptr(), _lib.AJQ_OUT_F32, _stream()), "gemv_gate")
        return y


class FusedDecoder(GraphDecoder):
    """GraphDecoder whose step runs on this library's kernels only: fused q|k|v and w1|w3
    matmuls, residual add + RMSNorm, RoPE + cache write + single-query attention in one launch
    and the SwiGLU gate (``ajq_add_rmsnorm`` / ``ajq_attn_step`` / ``ajq_swiglu``), the greedy pick
    with the embedding lookup and the step counters (``ajq_greedy_pick``).  Six launches per layer
    (q|k|v with the norm, attention, the merge of the attention's row chunks, output projection, w1|w3 with the
    gate, w2: ``launches_per_step``); five where the attention has one chunk per head or where ``fuse_merge`` is set
    and the output projection merges the chunks on its way in (an option: measured slower than the launch at every
    batch).  The norm's row scale, the residual add and the gate ride in the matmuls' epilogues (GEMV kernel
    up to 16 rows, weight-streaming kernel up to 255); nine launches per layer where those forms are not built.

    Needs the architecture the benchmark model has: pre-norm RMSNorm blocks, RoPE, SwiGLU,
    head_dim 128, 64 or 32 (64: the geometry of the reference's configs/models/transformer_medium.yaml; the attention's
    merge is then always a launch of its own), 1, 2 or 4 query heads per
    cache head, a quantized ``lm_head`` of its own (``quantize_model_(..., untie_head=True)`` for tied embeddings),
    every linear a QuantLinear.  ``kv_dtype``: torch.float32 (default, the model's own dtype) or
    torch.bfloat16 (keys and values rounded to nearest even on write, half the cache traffic)."""

    def __init__(self, model: modeling.TransformerLM, batch: int, max_len: int,
                 kv_dtype: torch.dtype | None = None, activation_rounding: str = "reference") -> None:
        super().__init__(model, batch, max_len, kv_dtype)
        # eight steps per graph launch: the gap between two graph launches is paid once per eight tokens
        # (measured on the 12-layer model: 0.525 -> 0.518 ms per step at batch 8)
        self.steps_per_graph = 8
        if activation_rounding not in ("reference", "before_scale"):
            raise ValueError('activation_rounding must be "reference" or "before_scale"')
        cache_dtype = self.cache.keys[0].dtype
        if cache_dtype not in (torch.float32, torch.bfloat16):
            raise ValueError("the KV cache must be float32 or bfloat16")
        self.kv_flag = _lib.AJQ_KV_F32 if cache_dtype == torch.float32 else _lib.AJQ_KV_BF16
        first = model.layers[0]
        ok = (
            model.position_encoding == "rope" and first.norm_placement == "pre"
            and isinstance(first.norm1, modeling.RMSNorm) and isinstance(first.feed_forward, modeling.SwiGLU)
            and isinstance(model.final_norm, modeling.RMSNorm) and isinstance(model.lm_head, QuantLinear)
            and model.d_model // model.num_heads in (128, 64, 32) and model.num_heads // model.num_kv_heads in (1, 2, 4)
            and all(isinstance(m, QuantLinear) and m.padded_in_features == m.in_features for layer in model.layers
                    for m in (layer.attention.q_proj, layer.attention.k_proj, layer.attention.v_proj,
                              layer.attention.output_proj, layer.feed_forward.w1, layer.feed_forward.w2,
                              layer.feed_forward.w3))
        )
        if not ok:
            raise ValueError("FusedDecoder needs pre-norm RMSNorm + RoPE + SwiGLU blocks with head_dim 128, 64 or 32 and "
                             "quantized linears everywhere with input widths that are multiples of 128 (an lm_head of its "
                             "own included: quantize_model_(..., untie_head=True) gives a model with tied embeddings one)")
        dev, d = self.device, model.d_model
        self.heads, self.kv_heads, self.head_dim = model.num_heads, model.num_kv_heads, d // model.num_heads
        self.d_ff = first.feed_forward.w1.out_features
        self.layers = []
        for layer in model.layers:
            att, ff = layer.attention, layer.feed_forward
            self.layers.append({
                "g1": layer.norm1.weight.detach().float().contiguous(), "eps1": layer.norm1.epsilon,
                "g2": layer.norm2.weight.detach().float().contiguous(), "eps2": layer.norm2.epsilon,
                "qkv": _FusedLinear([att.q_proj, att.k_proj, att.v_proj]),
                "o": _FusedLinear([att.output_proj]),
                "w13": _FusedLinear([ff.w1, ff.w3]),
                "w2": _FusedLinear([ff.w2]),
                "cos": att.rope.cosine.float().contiguous(), "sin": att.rope.sine.float().contiguous(),
            })
        self.final_gain = model.final_norm.weight.detach().float().contiguous()
        self.final_eps = model.final_norm.epsilon
        self.head = _FusedLinear([model.lm_head])
        self.vocab = model.lm_head.out_features
        self.embedding = model.token_embeddings.weight.detach().float().contiguous()
        self.embedded = torch.zeros((batch, d), dtype=torch.float32, device=dev)  # embedding row of self.token
        self.hidden = torch.zeros((batch, d), dtype=torch.float32, device=dev)
        self.hidden2 = torch.zeros((batch, d), dtype=torch.float32, device=dev)
        # write position and output column advance together: one tensor, incremented by the greedy
        # pick at the end of a step (its last workgroup to finish; ``ticket`` is its scratch word)
        self.counters = torch.zeros(2, dtype=torch.long, device=dev)
        self.ticket = torch.zeros(1, dtype=torch.int32, device=dev)
        self.cache.position = self.counters[0:1]
        self.step_index = self.counters[1:2]
        self.logits_full: torch.Tensor | None = None
        # GEMVs that form their own input (residual add + RMSNorm, SwiGLU gate) where they are built
        # (the gate reads w1|w3's output as rows of 2 * d_ff: no padding rows between the halves)
        # Every workgroup of such a GEMV re-reads the fp32 sources of all batch rows, so the saved
        # launch only pays for small batches (measured on the 12-layer model: the norm up to batch
        # 4, the gate at batch 1).
        self.fuse_norm = batch <= 4 and self.head.fusable(batch)
        self.fuse_gate = (batch == 1 and self.layers[0]["w2"].fusable(batch)
                          and self.layers[0]["w13"].rows16 == 2 * self.d_ff)
        # The output projection can merge the attention's row chunks on its way in where that is built (small
        # batches; one launch less per layer): ``fuse_merge``, off by default.  Every workgroup of that GEMV re-reads
        # every chunk of every head, and a dependent launch costs little more than its kernel in a replayed graph:
        # measured on the 12-layer model, the merge as a launch of its own is faster at every batch (0.309 against
        # 0.314 ms per step at batch 1, 0.364 against 0.398 at batch 2, 0.386 against 0.469 at batch 3).  Set it to
        # True (where ``merge_splits`` > 0) before the first ``generate`` to have the merging projection.
        self.merge_splits = (self.layers[0]["o"].merge_splits(batch)
                             if self.layers[0]["o"].in_features == d and self.head_dim == 128 else 0)
        self.fuse_merge = False
        # Larger batches (every workgroup would re-read the fp32 sources of all rows): the norm's row scale
        # is applied to the OUTPUTS of q|k|v, w1|w3 and the head instead, the output projection and w2 add
        # the residual and prepare the next norm on their way out, and w1|w3 (rows interleaved in blocks
        # of 8) applies the gate: six launches per layer instead of nine.
        # At small batch as well: the epilogue forms cost less than the prologue forms (3.3 against 4.8 us for
        # q|k|v at batch 1, 4.2 against 6.7 at batch 4).
        # Where the normed activations are rounded to bf16.  "reference": exactly where the model code rounds them,
        # bf16((h / rms) * gain) (the consumer is the GEMV with a norm prologue, fed with the producer's sums of
        # squares; built for the batches and widths ``fusable`` reports).  "before_scale": bf16(h * gain), the row
        # scale applied to the matmul's outputs (one rounding of the same quantity at a different point: the
        # logits move by about as much again as bf16 activations move them at all); built for every batch.
        # The reference-order consumer reads the fp32 stream of all batch rows in every workgroup, like any prologue
        # form: measured on the 12-layer model it beats the unfolded step up to batch 4 (0.37 / 0.46 / 0.45 / 0.53 ms
        # against 0.38 / 0.51 / 0.60 / 0.62 at batch 1 - 4) and loses from batch 5 (0.63 against 0.53), so above
        # batch 4 "reference" means the unfolded step; "before_scale" folds at every batch (0.34 / 0.42 / 0.60 ms at
        # batch 1 / 4 / 8).
        self.exact_norm = activation_rounding == "reference"
        # reference rounding above batch 4 (or where that consumer is not built): the norm is a launch of its own
        # again, the residual adds and the gate stay in the epilogues (they move no rounding point): eight
        # launches per layer instead of nine
        self.norm_launch = self.exact_norm and not (batch <= 4 and self.head.fusable(batch))
        self.fuse_epilogue = (
            self.d_ff % 8 == 0 and d // 16 <= 256  # the norm-from-sums consumer takes at most 256 tile sums
            and self.layers[0]["o"].in_features == d
            and all(self.layers[0][name].epilogue_fusable(batch) for name in ("qkv", "o", "w13", "w2"))
            and all(self.layers[0][name].rowscale_fusable(batch) for name in ("qkv", "w13"))
            and self.head.epilogue_fusable(batch) and self.head.rowscale_fusable(batch)
        )
        if self.fuse_epilogue:
            # the step's very first norm rides in layer 0's q|k|v where built
            self.first_norm_fused = self.fuse_norm and not self.norm_launch
            self.fuse_norm = self.fuse_gate = False
            for w, layer in zip(self.layers, model.layers):
                w["w13i"] = _FusedLinear.interleaved_gate(layer.feed_forward.w1, layer.feed_forward.w3)
            self.xt = torch.zeros((batch, d), dtype=torch.bfloat16, device=dev)
            self.ssq = torch.zeros((max(16, batch), d // 16), dtype=torch.float32, device=dev)
        self.normed = torch.zeros((batch, d), dtype=torch.bfloat16, device=dev)
        self.attended = torch.zeros((batch, d), dtype=torch.bfloat16, device=dev)
        self.gated = torch.zeros((batch, self.d_ff), dtype=torch.bfloat16, device=dev)
        lib = _lib.load()
        self.attn_ws_bytes = int(lib.ajq_attn_step_workspace_bytes(batch, self.heads))
        self.attn_ws = torch.zeros(max(self.attn_ws_bytes, 16), dtype=torch.uint8, device=dev)
        # lent to the library for the duration of each step (zeroed: its first 4 KiB are ticket words)
        self.matmul_ws = torch.zeros(int(lib.ajq_matmul_workspace_bytes()), dtype=torch.uint8, device=dev)

    @torch.no_grad()
    def prefill(self, prompt: torch.Tensor, rows_per_pass: int | None = None, fused: bool = False) -> None:
        """``fused``: the prompt goes through this library's kernels as well (GEMMs, add + RMSNorm,
        RoPE + cache write, flash attention, SwiGLU gate) instead of the model's PyTorch code; the
        attention then has flash-attention arithmetic, as with the model's ``use_flash_attention``."""
        if not fused:
            super().prefill(prompt, rows_per_pass)
        else:
            if prompt.shape[0] != self.batch or prompt.shape[1] >= self.max_len:
                raise ValueError("prompt must be [batch, T] with T < max_len")
            prompt = prompt.to(self.device)
            step = rows_per_pass or self.batch
            logits = torch.cat([self._prefill_rows(prompt[i:i + step], i) for i in range(0, self.batch, step)], dim=0)
            self.cache.length = prompt.shape[1]
            self.cache.static = True
            self.cache.position.fill_(prompt.shape[1])
            self.step_index.zero_()
            self._choose(logits)
            self.step_index.add_(1)
            self.produced = 1
            self.prompt_len = prompt.shape[1]
        torch.index_select(self.embedding, 0, self.token.view(-1), out=self.embedded)

    def _prefill_rows(self, prompt: torch.Tensor, first: int) -> torch.Tensor:
        """Sequences ``first .. first + rows - 1`` of the batch through the layer stack on library
        kernels, from an empty cache; returns the last position's logits ``[rows, V]``."""
        lib, st = _lib.load(), _stream()
        rows, seq = prompt.shape
        d, m = self.model.d_model, rows * seq
        hidden = self.embedding[prompt.reshape(-1)]  # [rows * seq, d] fp32, row b * seq + t
        normed = torch.empty((m, d), dtype=torch.bfloat16, device=self.device)
        q_rot = torch.empty((rows, self.heads, seq, self.head_dim), dtype=torch.float32, device=self.device)
        w13 = self.layers[0]["w13"]
        gate_in_gemm = w13.rows16 == 2 * self.d_ff and w13.gate_fusable(m)
        gated = None if gate_in_gemm else torch.empty((m, self.d_ff), dtype=torch.bfloat16, device=self.device)
        delta = None
        for index, w in enumerate(self.layers):
            _lib.check(lib.ajq_add_rmsnorm(hidden.data_ptr(), delta.data_ptr() if delta is not None else None,
                                           w["g1"].data_ptr(), w["eps1"], normed.data_ptr(), m, d, st), "add_rmsnorm")
            qkv = w["qkv"](normed)
            keys, values = self.cache.keys[index][first:first + rows], self.cache.values[index][first:first + rows]
            _lib.check(lib.ajq_rope_prefill(qkv.data_ptr(), w["cos"].data_ptr(), w["sin"].data_ptr(), q_rot.data_ptr(),
                                            keys.data_ptr(), values.data_ptr(), self.kv_flag, rows, seq, self.heads,
                                            self.kv_heads, self.head_dim, 0, self.max_len, st), "rope_prefill")
            del qkv
            attended = torch.empty((m, d), dtype=torch.bfloat16, device=self.device)
            _lib.check(lib.ajq_attn_prefill(q_rot.data_ptr(), keys.data_ptr(), values.data_ptr(), self.kv_flag, rows,
                                            self.heads, self.kv_heads, seq, 0, self.max_len, self.head_dim, attended.data_ptr(),
                                            _lib.AJQ_OUT_BF16, st), "attn_prefill")
            delta = w["o"](attended)
            del attended
            _lib.check(lib.ajq_add_rmsnorm(hidden.data_ptr(), delta.data_ptr(), w["g2"].data_ptr(), w["eps2"],
                                           normed.data_ptr(), m, d, st), "add_rmsnorm")
            if gate_in_gemm:
                gated = w["w13"].gated(normed)
            else:
                ab = w["w13"](normed)
                _lib.check(lib.ajq_swiglu(ab.data_ptr(), gated.data_ptr(), m, self.d_ff, st), "swiglu")
                del ab
            delta = w["w2"](gated)
        last = hidden.view(rows, seq, d)[:, -1, :].contiguous()
        last_delta = delta.view(rows, seq, -1)[:, -1, :d].contiguous()
        last_normed = torch.empty((rows, d), dtype=torch.bfloat16, device=self.device)
        _lib.check(lib.ajq_add_rmsnorm(last.data_ptr(), last_delta.data_ptr(), self.final_gain.data_ptr(), self.final_eps,
                                       last_normed.data_ptr(), rows, d, st), "add_rmsnorm")
        return self.head(last_normed)[:, : self.vocab]

    @torch.no_grad()
    def _step(self) -> None:
        """One token: the layer stack, then the greedy choice, its embedding row (the next step's
        input) and the two counters in one launch."""
        self._logits()
        full = self.logits_full
        if self.temperature > 0:
            self._sample(full, self.embedding, self.embedded, self.counters, self.ticket, self.vocab)
            return
        _lib.check(_lib.load().ajq_greedy_pick(full.data_ptr(), self.batch, self.vocab, full.shape[1],
                                               self.embedding.data_ptr(), self.model.d_model, self.embedded.data_ptr(),
                                               self.token.data_ptr(), self.out.data_ptr(), self.out.shape[1],
                                               self.step_index.data_ptr(), self.counters.data_ptr(),
                                               self.ticket.data_ptr(), _stream()), "greedy_pick")

    @property
    def merge_launch(self) -> bool:
        """Whether the attention's row chunks are merged by a launch of their own (not by the output projection's
        prologue, and there are several chunks)."""
        chunks = _lib.load().ajq_attn_row_chunks(self.batch, self.kv_heads, self.max_len)
        return not self.fuse_merge and chunks > 1

    def launches_per_step(self) -> int:
        """Kernel launches of one decode step as this decoder is configured."""
        lib = _lib.load()
        if self.fuse_epilogue:
            # q|k|v, attention (+ merge), output projection, w1|w3 with the gate, w2; the first norm, head, pick
            per_layer = 6 if self.merge_launch else 5
            if self.norm_launch:  # both norms of a layer and the final one as launches
                return (per_layer + 2) * len(self.layers) + 3
            return per_layer * len(self.layers) + (2 if self.first_norm_fused else 3)
        per_layer = 2 if self.fuse_norm else 4           # q|k|v and w1|w3, each with or without its norm launch
        per_layer += 1                                   # attention
        if self.merge_launch:                            # merge of its row chunks (none if there is one chunk)
            per_layer += 1
        per_layer += 1                                   # output projection
        per_layer += 1 if self.fuse_gate else 2          # w2 with or without the gate launch
        head = 1 if self.fuse_norm else 2
        first_copy = 0 if self.fuse_norm else 1          # embedding row copied into the residual stream
        return per_layer * len(self.layers) + head + first_copy + 1  # + greedy pick (token, embedding row, counters)

    def _logits(self) -> torch.Tensor:
        """Logits ``[B, V]`` of the token whose embedding row is in ``self.embedded`` (``prefill`` and
        every step leave it there), at cache row ``cache.position``; the decoding state is untouched."""
        lib = _lib.load()
        # the step's matmuls may exchange split-K partial sums through this decoder's buffer (batched steps: w2)
        _lib.check(lib.ajq_matmul_workspace_set(self.matmul_ws.data_ptr(), self.matmul_ws.numel()), "matmul_workspace_set")
        try:
            return self._logits_epilogue() if self.fuse_epilogue else self._logits_prologue()
        finally:
            lib.ajq_matmul_workspace_set(None, 0)

    def _logits_prologue(self) -> torch.Tensor:
        """``_logits`` with the norms and the gate in front of the GEMVs (small batches) or as launches of their own."""
        lib, st = _lib.load(), _stream()
        b, d = self.batch, self.model.d_model
        pos = self.cache.position
        if self.fuse_norm:
            # the first norm reads the embedding row where it is; the updated stream goes to `other`
            cur, other = self.embedded, self.hidden
        else:
            cur, other = self.hidden, self.hidden2
            cur.copy_(self.embedded)
        delta = None

        def normed_linear(linear, gain, eps):
            """linear(RMSNorm(cur + delta) * gain); afterwards ``cur`` holds cur + delta."""
            nonlocal cur, other
            if self.fuse_norm:
                out = linear.after_norm(cur, delta, gain, eps, other)
                cur, other = other, (self.hidden2 if cur is self.embedded else cur)
                return out
            _lib.check(lib.ajq_add_rmsnorm(cur.data_ptr(), delta.data_ptr() if delta is not None else None,
                                           gain.data_ptr(), eps, self.normed.data_ptr(), b, d, st), "add_rmsnorm")
            return linear(self.normed)

        for index, w in enumerate(self.layers):
            qkv = normed_linear(w["qkv"], w["g1"], w["eps1"])
            if self.fuse_merge:
                splits = ctypes.c_int(0)
                _lib.check(lib.ajq_attn_step_partial(qkv.data_ptr(), w["cos"].data_ptr(), w["sin"].data_ptr(),
                                                     pos.data_ptr(), self.cache.keys[index].data_ptr(),
                                                     self.cache.values[index].data_ptr(), self.kv_flag, b, self.heads,
                                                     self.kv_heads, self.head_dim, self.max_len, self.merge_splits,
                                                     ctypes.addressof(splits), self.attn_ws.data_ptr(),
                                                     self.attn_ws_bytes, st), "attn_step_partial")
                delta = w["o"].after_merge(self.attn_ws, splits.value, b)
            else:
                _lib.check(lib.ajq_attn_step(qkv.data_ptr(), w["cos"].data_ptr(), w["sin"].data_ptr(), pos.data_ptr(),
                                             self.cache.keys[index].data_ptr(), self.cache.values[index].data_ptr(),
                                             self.kv_flag, b, self.heads, self.kv_heads, self.head_dim, self.max_len,
                                             self.attended.data_ptr(), self.attn_ws.data_ptr(), self.attn_ws_bytes, st),
                           "attn_step")
                delta = w["o"](self.attended)
            ab = normed_linear(w["w13"], w["g2"], w["eps2"])
            if self.fuse_gate:
                delta = w["w2"].after_gate(ab)
            else:
                _lib.check(lib.ajq_swiglu(ab.data_ptr(), self.gated.data_ptr(), b, self.d_ff, st), "swiglu")
                delta = w["w2"](self.gated)
        self.logits_full = normed_linear(self.head, self.final_gain, self.final_eps)
        return self.logits_full[:, : self.vocab]


    def _attention(self, index: int, w: dict, qkv: torch.Tensor) -> None:
        """RoPE, cache write and single-query attention of layer ``index`` into ``self.attended``."""
        _lib.check(_lib.load().ajq_attn_step(qkv.data_ptr(), w["cos"].data_ptr(), w["sin"].data_ptr(),
                                             self.cache.position.data_ptr(), self.cache.keys[index].data_ptr(),
                                             self.cache.values[index].data_ptr(), self.kv_flag, self.batch, self.heads,
                                             self.kv_heads, self.head_dim, self.max_len, self.attended.data_ptr(),
                                             self.attn_ws.data_ptr(), self.attn_ws_bytes, _stream()), "attn_step")

    def _logits_epilogue(self) -> torch.Tensor:
        """``_logits`` for batches too large for the norm / gate prologues: no norm, gate or residual launch
        between the matmuls of a layer (only the very first norm of a step is a launch of its own)."""
        lib, st = _lib.load(), _stream()
        b, d = self.batch, self.model.d_model
        first = self.layers[0]
        cur = self.embedded

        def other() -> torch.Tensor:
            return self.hidden2 if cur is self.hidden else self.hidden

        xt = None if self.exact_norm else self.xt   # the producers' bf16 image is only read by the row-scale form

        def normed(linear: _FusedLinear, gain: torch.Tensor, eps: float, gated: torch.Tensor | None = None) -> torch.Tensor:
            """linear(RMSNorm(cur) * gain), the norm taken from the sums of squares cur's producer left."""
            if self.norm_launch:
                _lib.check(lib.ajq_add_rmsnorm(cur.data_ptr(), None, gain.data_ptr(), eps, self.normed.data_ptr(), b, d, st),
                           "add_rmsnorm")
                return linear(self.normed) if gated is None else linear.gated_interleaved(self.normed, gated)
            if self.exact_norm:
                return linear.normed_from_sums(cur, self.ssq, gain, eps, gated)
            return linear.rowscaled(self.xt, self.ssq, eps, gated)

        for index, w in enumerate(self.layers):
            if index > 0 or self.norm_launch:
                qkv = normed(w["qkv"], w["g1"], w["eps1"])
            elif self.first_norm_fused:
                qkv = w["qkv"].after_norm(self.embedded, None, first["g1"], first["eps1"], self.hidden)
                cur = self.hidden  # (a copy of the embedding row)
            else:
                _lib.check(lib.ajq_add_rmsnorm(self.embedded.data_ptr(), None, first["g1"].data_ptr(), first["eps1"],
                                               self.normed.data_ptr(), b, d, st), "add_rmsnorm")
                qkv = w["qkv"](self.normed)
            nxt = other()
            if self.fuse_merge:
                splits = ctypes.c_int(0)
                _lib.check(lib.ajq_attn_step_partial(qkv.data_ptr(), w["cos"].data_ptr(), w["sin"].data_ptr(),
                                                     self.cache.position.data_ptr(), self.cache.keys[index].data_ptr(),
                                                     self.cache.values[index].data_ptr(), self.kv_flag, b, self.heads,
                                                     self.kv_heads, self.head_dim, self.max_len, self.merge_splits,
                                                     ctypes.addressof(splits), self.attn_ws.data_ptr(),
                                                     self.attn_ws_bytes, st), "attn_step_partial")
                w["o"].merge_residual(self.attn_ws, splits.value, b, cur, w["g2"], nxt, xt, self.ssq)
            else:
                self._attention(index, w, qkv)
                w["o"].residual(self.attended, cur, w["g2"], nxt, xt, self.ssq)
            cur = nxt
            normed(w["w13i"], w["g2"], w["eps2"], gated=self.gated)
            nxt = other()
            gain = self.layers[index + 1]["g1"] if index + 1 < len(self.layers) else self.final_gain
            w["w2"].residual(self.gated, cur, gain, nxt, xt, self.ssq)
            cur = nxt
        self.logits_full = normed(self.head, self.final_gain, self.final_eps)
        return self.logits_full[:, : self.vocab]


@torch.no_grad()
def greedy_decode_graph(model: modeling.TransformerLM, prompt: torch.Tensor, max_new_tokens: int,
                        fused: bool = False, kv_dtype: torch.dtype | None = None) -> torch.Tensor:
    """``[B, T + new]`` like ``modeling.greedy_decode``, with the per-token step replayed from a graph."""
    cls = FusedDecoder if fused else GraphDecoder
    decoder = cls(model, prompt.shape[0], prompt.shape[1] + max_new_tokens, kv_dtype)
    decoder.prefill(prompt)
    new = decoder.generate(max_new_tokens)
    return torch.cat((prompt.to(new.device), new), dim=1)
