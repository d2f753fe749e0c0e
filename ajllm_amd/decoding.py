"""Greedy decoding with the decode step replayed from a HIP graph.

Same token rule as the reference's ``generate`` at temperature <= 0
(src/ajllm/generation/generator.py:10-28, sampling.py:9-10) and as
``modeling.greedy_decode``: next = argmax(logits[:, -1]).  The prompt is processed eagerly; the
one-token step (embedding, 12 x block, norm, lm_head, argmax, KV-cache scatter, position + 1) has
fixed shapes (``modeling.KVCache`` in static mode), is recorded once and replayed per token, with
the chosen token fed back on the device: no host round trip between steps.
"""

from __future__ import annotations

import torch

from . import modeling


class GraphDecoder:
    def __init__(self, model: modeling.TransformerLM, batch: int, max_len: int) -> None:
        if max_len > model.context_length:
            raise ValueError(f"max_len {max_len} exceeds the model's context length {model.context_length}")
        self.model = model.eval()
        self.batch = batch
        self.max_len = max_len
        device = model.token_embeddings.weight.device
        if device.type != "cuda":
            raise ValueError("GraphDecoder needs the model on a ROCm device")
        self.device = device
        self.cache = model.new_cache(batch, max_len)
        self.token = torch.zeros((batch, 1), dtype=torch.long, device=device)
        self.out = torch.zeros((batch, max_len), dtype=torch.long, device=device)
        self.step_index = torch.zeros(1, dtype=torch.long, device=device)
        self.graph: torch.cuda.CUDAGraph | None = None
        self.stream = torch.cuda.Stream(device=device)

    @torch.no_grad()
    def _step(self) -> None:
        logits = self.model(self.token, self.cache)[:, -1, :]
        nxt = torch.argmax(logits, dim=-1, keepdim=True)
        self.out.index_copy_(1, self.step_index, nxt)
        self.token.copy_(nxt)
        self.cache.position.add_(1)
        self.step_index.add_(1)

    @torch.no_grad()
    def prefill(self, prompt: torch.Tensor) -> None:
        """Run the prompt ``[B, T]`` through the model (eagerly) and choose the first new token."""
        if prompt.shape[0] != self.batch or prompt.shape[1] >= self.max_len:
            raise ValueError("prompt must be [batch, T] with T < max_len")
        self.cache.static = False
        self.cache.length = 0
        logits = self.model(prompt.to(self.device), self.cache, last_token_only=True)[:, -1, :]
        self.cache.static = True
        self.cache.position.fill_(prompt.shape[1])
        self.step_index.zero_()
        nxt = torch.argmax(logits, dim=-1, keepdim=True)
        self.out.index_copy_(1, self.step_index, nxt)
        self.token.copy_(nxt)
        self.step_index.add_(1)
        self.produced = 1
        self.prompt_len = prompt.shape[1]

    @torch.no_grad()
    def generate(self, new_tokens: int) -> torch.Tensor:
        """Decode until ``new_tokens`` tokens exist since ``prefill`` and return them ``[B, new_tokens]``."""
        if self.prompt_len + new_tokens > self.max_len:
            raise ValueError("the KV cache is too short for this many tokens")
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
            while self.produced < new_tokens:
                self.graph.replay()
                self.produced += 1
        current.wait_stream(self.stream)
        return self.out[:, :new_tokens].clone()


@torch.no_grad()
def greedy_decode_graph(model: modeling.TransformerLM, prompt: torch.Tensor, max_new_tokens: int) -> torch.Tensor:
    """``[B, T + new]`` like ``modeling.greedy_decode``, with the per-token step replayed from a graph."""
    decoder = GraphDecoder(model, prompt.shape[0], prompt.shape[1] + max_new_tokens)
    decoder.prefill(prompt)
    new = decoder.generate(max_new_tokens)
    return torch.cat((prompt.to(new.device), new), dim=1)
