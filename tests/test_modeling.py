"""The restated Transformer (CPU, dense linears): same behaviour as the reference's model tests
ask for (tests/unit/modeling/test_transformer.py: finite [B, T, V] logits for every variant,
over-length input rejected) plus what pins the restated glue: library equivalents, RoPE closed
forms, and KV-cache decoding equal to full recomputation."""

import itertools
import math

import pytest
import torch
import torch.nn.functional as F

from ajllm_amd import modeling as M


def _model(**kw):
    torch.manual_seed(0)
    args = dict(vocab_size=37, context_length=16, d_model=32, num_layers=2, num_heads=4, d_ff=64)
    args.update(kw)
    return M.TransformerLM(**args).eval()


@pytest.mark.parametrize("pos,norm,place,ff,tie", [
    c for c in itertools.product(["rope", "none", "learned"], ["rmsnorm", "none"], ["pre", "post"],
                                 ["swiglu", "silu"], [False, True])
][::3])
def test_variants_give_finite_logits(pos, norm, place, ff, tie):
    model = _model(position_encoding=pos, normalization=norm, norm_placement=place, feed_forward=ff,
                   tie_embeddings=tie)
    logits = model(torch.randint(0, 37, (3, 8)))
    assert logits.shape == (3, 8, 37) and torch.isfinite(logits).all()


def test_over_length_input_is_rejected():
    with pytest.raises(ValueError):
        _model()(torch.zeros((1, 17), dtype=torch.long))


def test_state_dict_keys_follow_the_reference_names():
    keys = set(_model().state_dict())
    for name in ("token_embeddings.weight", "layers.0.norm1.weight", "layers.1.attention.q_proj.weight",
                 "layers.0.attention.output_proj.weight", "layers.0.feed_forward.w3.weight",
                 "final_norm.weight", "lm_head.weight"):
        assert name in keys
    assert not any("rope" in k for k in keys)  # RoPE tables are non-persistent buffers


def test_linear_init_statistics():
    torch.manual_seed(1)
    lin = M.Linear(512, 256)
    std = math.sqrt(2.0 / 768)
    assert lin.weight.shape == (256, 512)
    assert abs(float(lin.weight.std()) - std) < 0.05 * std  # truncation at 3 std barely shrinks it
    assert float(lin.weight.abs().max()) <= 3 * std + 1e-7


def test_rmsnorm_matches_library():
    x = torch.randn(4, 7, 32)
    norm = M.RMSNorm(32)
    with torch.no_grad():
        norm.weight.copy_(torch.rand(32) + 0.5)
    assert torch.allclose(norm(x), F.rms_norm(x, (32,), norm.weight, eps=1e-5), atol=1e-6)
    assert norm(x.to(torch.bfloat16)).dtype == torch.bfloat16


def test_attention_matches_library_sdpa():
    q, k, v = (torch.randn(2, 4, 9, 8) for _ in range(3))
    mask = torch.tril(torch.ones(9, 9, dtype=torch.bool))
    ours = M.scaled_dot_product_attention(q, k, v, mask)
    assert torch.allclose(ours, F.scaled_dot_product_attention(q, k, v, is_causal=True), atol=1e-5)
    x = torch.randn(3, 11)
    assert torch.allclose(M.softmax(x, -1), torch.softmax(x, -1), atol=1e-6)
    assert torch.allclose(M.silu(x), F.silu(x), atol=1e-6)


def test_rope_closed_forms():
    rope = M.RotaryPositionalEmbedding(10_000.0, 8, 64)
    x = torch.randn(2, 3, 5, 8)
    pos0 = torch.zeros(2, 3, 5, dtype=torch.long)
    assert torch.equal(rope(x, pos0), x)  # position 0 is the identity
    pos = torch.arange(5).expand(2, 3, 5)
    y = rope(x, pos)
    assert torch.allclose(y.norm(dim=-1), x.norm(dim=-1), atol=1e-5)  # rotations keep the norm
    # first pair rotates by exactly pos radians (frequency theta^0 = 1)
    angle = torch.atan2(y[..., 1], y[..., 0]) - torch.atan2(x[..., 1], x[..., 0])
    assert torch.allclose(torch.remainder(angle - pos + math.pi, 2 * math.pi) - math.pi,
                          torch.zeros_like(angle), atol=1e-4)
    # relative-position property: <rope(q, m), rope(k, n)> depends on m - n only
    q, k = torch.randn(8), torch.randn(8)
    def dot(m, n):
        return float(rope(q[None], torch.tensor([m])) @ rope(k[None], torch.tensor([n])).t())
    assert abs(dot(5, 2) - dot(13, 10)) < 1e-4 and abs(dot(7, 7) - float(q @ k)) < 1e-4


@pytest.mark.parametrize("kv_heads", [4, 2, 1])
def test_kv_cache_decoding_equals_full_recomputation(kv_heads):
    model = _model(num_kv_heads=kv_heads)
    tokens = torch.randint(0, 37, (2, 12))
    full = model(tokens)
    cache = model.new_cache(2, 12)
    first = model(tokens[:, :7], cache)
    assert torch.allclose(first, full[:, :7], atol=1e-5) and cache.length == 7
    for t in range(7, 12):
        step = model(tokens[:, t:t + 1], cache)
        assert torch.allclose(step[:, 0], full[:, t], atol=1e-5)
    last = model(tokens[:, :12], model.new_cache(2), last_token_only=True)
    assert last.shape == (2, 1, 37) and torch.allclose(last[:, 0], full[:, -1], atol=1e-5)


def test_gqa_with_all_heads_is_the_reference_layer():
    torch.manual_seed(3)
    a = M.MultiHeadSelfAttention(32, 4, 16, "rope", 10_000.0)
    torch.manual_seed(3)
    b = M.MultiHeadSelfAttention(32, 4, 16, "rope", 10_000.0, num_kv_heads=4)
    x = torch.randn(2, 6, 32)
    pos = torch.arange(6).expand(2, 6)
    assert torch.equal(a(x, pos), b(x, pos))
    assert M.MultiHeadSelfAttention(32, 4, 16, "rope", 1e4, num_kv_heads=2).k_proj.out_features == 16


def test_greedy_decode_follows_the_reference_token_rule():
    """Reference generate() at temperature 0: append argmax of the last position's logits, stop at eos."""
    model = _model()
    prompt = torch.randint(0, 37, (2, 5))
    out, margins = M.greedy_decode(model, prompt, 6, return_margins=True)
    assert out.shape == (2, 11) and torch.equal(out[:, :5], prompt) and margins.shape == (2, 6)
    seq = prompt.clone()
    for _ in range(6):  # the reference loop: full recomputation, no cache
        nxt = torch.argmax(model(seq)[:, -1, :], dim=-1, keepdim=True)
        seq = torch.cat((seq, nxt), dim=1)
    assert torch.equal(out, seq) and (margins >= 0).all()
    eos = int(out[0, 5])
    stopped = M.greedy_decode(model, prompt[:1], 6, eos_token_id=eos)
    assert stopped.shape == (1, 6) and int(stopped[0, -1]) == eos


def test_build_model_reads_reference_style_config():
    cfg = {"context_length": 32, "d_model": 48, "num_layers": 1, "num_heads": 4,
           "position_encoding": {"type": "rope", "theta": 5000.0}, "normalization": {"placement": "pre"}}
    model = M.build_model(cfg, vocab_size=50)
    assert model.d_ff == 128  # ceil(8*48/3 = 128) to a multiple of 64
    assert M.build_model({**cfg, "feed_forward": {"type": "silu"}}, 50).d_ff == 192


def test_static_cache_steps_equal_dynamic_decoding():
    """One-token steps against a static KV cache (fixed shapes, device-side position) choose the
    same tokens as the dynamic cache."""
    torch.manual_seed(11)
    model = _model(num_layers=2)
    prompt = torch.randint(0, model.vocab_size, (2, 6))
    want = M.greedy_decode(model, prompt, 7)
    cache = model.new_cache(2, 13)
    logits = model(prompt, cache, last_token_only=True)[:, -1]
    cache.static = True
    cache.position.fill_(6)
    tokens = [logits.argmax(-1, keepdim=True)]
    for _ in range(6):
        logits = model(tokens[-1], cache)[:, -1]
        cache.position.add_(1)
        tokens.append(logits.argmax(-1, keepdim=True))
    assert torch.equal(torch.cat([prompt] + tokens, dim=1), want)
    with pytest.raises(ValueError):
        model(prompt, cache)  # a static cache takes one token per call


def test_cache_rows_view_prefills_a_few_sequences_at_a_time():
    """KVCache.rows(): prompts pushed through the model two sequences at a time into views of one
    cache leave it exactly as one pass over all sequences does, and give the same logits."""
    torch.manual_seed(12)
    model = _model(num_layers=2)
    prompt = torch.randint(0, model.vocab_size, (5, 9))
    whole = model.new_cache(5, 12)
    want = model(prompt, whole, last_token_only=True)
    parts = model.new_cache(5, 12)
    got = torch.cat([model(prompt[i:i + 2], parts.rows(i, min(i + 2, 5)), last_token_only=True) for i in (0, 2, 4)])
    assert torch.allclose(got, want, atol=1e-6, rtol=1e-5)
    for a, b in zip(parts.keys + parts.values, whole.keys + whole.values):
        assert torch.allclose(a, b, atol=1e-6, rtol=1e-5)
    assert parts.length == 0  # the views keep their own length; the owner's is set by the caller


def test_narrower_kv_cache_rounds_keys_and_values_only():
    """A bf16 KV cache: keys and values are rounded on write and widened on read; decoding with it
    equals decoding where k and v are rounded by hand, and stays close to the fp32 cache."""
    torch.manual_seed(13)
    model = _model(num_layers=2)
    prompt = torch.randint(0, model.vocab_size, (2, 8))
    cache16 = model.new_cache(2, 10, dtype=torch.bfloat16)
    cache32 = model.new_cache(2, 10)
    a = model(prompt, cache16)
    b = model(prompt, cache32)
    assert cache16.keys[0].dtype == torch.bfloat16 and a.dtype == b.dtype == torch.float32
    assert torch.equal(cache16.keys[0][:, :, :8], cache32.keys[0][:, :, :8].to(torch.bfloat16))
    assert (a - b).abs().max() < 5e-2 and not torch.equal(a, b)
    step16 = model(prompt[:, :1], cache16)
    assert torch.isfinite(step16).all() and cache16.length == 9


def test_flash_attention_flag_is_off_by_default_and_ignored_on_the_host():
    """use_flash_attention mirrors the reference's flag: off by default, and a CPU call keeps the
    masked-softmax path whatever it says (the kernel is a GPU one; no CPU fallback of it exists)."""
    torch.manual_seed(14)
    model = _model(num_layers=1)
    tokens = torch.randint(0, model.vocab_size, (1, 7))
    want = model(tokens)
    assert all(not layer.attention.use_flash_attention for layer in model.layers)
    for layer in model.layers:
        layer.attention.use_flash_attention = True
    assert torch.equal(model(tokens), want)


def test_quantized_checkpoint_manifest_and_foreign_files(tmp_path):
    """The checkpoint reader refuses files that are not its own format (no GPU needed)."""
    from safetensors.torch import save_file

    from ajllm_amd import checkpoint
    save_file({"x": torch.zeros(2)}, str(tmp_path / "foreign.safetensors"))
    with pytest.raises(ValueError):
        checkpoint.read_quantized(tmp_path / "foreign.safetensors")
    model = _model()
    cfg = checkpoint.model_config(model)
    assert M.TransformerLM(**cfg).state_dict().keys() == model.state_dict().keys()
    with pytest.raises(ValueError):
        checkpoint.save_quantized(tmp_path / "dense.safetensors", model, "w4a16_g128")  # nothing quantized


def _token_file(tmp_path, tokens):
    import numpy as np
    path = tmp_path / "tokens.bin"
    np.asarray(tokens, dtype=np.uint32).tofile(path)
    return path


def test_cross_entropy_matches_library_and_closed_forms():
    from ajllm_amd import evaluation
    logits = torch.randn(3, 5, 37) * 4
    targets = torch.randint(0, 37, (3, 5))
    want = F.cross_entropy(logits.reshape(-1, 37), targets.reshape(-1))
    assert torch.allclose(evaluation.cross_entropy(logits, targets), want, atol=1e-6)
    assert abs(float(evaluation.cross_entropy(torch.zeros(4, 37), targets[0, :4])) - math.log(37)) < 1e-6
    big = torch.full((2, 37), -1e4)
    big[0, 3] = big[1, 9] = 1e4  # no overflow, certain prediction -> zero loss
    assert float(evaluation.cross_entropy(big, torch.tensor([3, 9]))) == 0.0


def test_token_file_windows_and_evaluation(tmp_path):
    """Reference evaluate_model (evaluator.py:14-31): windows at generator.integers starts, targets one
    token on, mean of per-batch losses, perplexity = exp(min(loss, 50))."""
    import numpy as np

    from ajllm_amd import evaluation
    stream = np.arange(100) % 37
    data = evaluation.TokenFile(_token_file(tmp_path, stream))
    assert len(data) == 100
    inputs, targets = data.batch(4, 8, "cpu", np.random.default_rng(5))
    starts = np.random.default_rng(5).integers(0, 100 - 8 - 1 + 1, size=4)
    assert inputs.dtype == torch.int64 and inputs.shape == targets.shape == (4, 8)
    for row, s in enumerate(starts):
        assert inputs[row].tolist() == stream[s:s + 8].tolist()
        assert targets[row].tolist() == stream[s + 1:s + 9].tolist()
    with pytest.raises(ValueError):
        data.batch(1, 100, "cpu", np.random.default_rng(0))
    (tmp_path / "odd.bin").write_bytes(b"\0" * 6)
    with pytest.raises(ValueError):
        evaluation.TokenFile(tmp_path / "odd.bin")

    model = _model()
    got = evaluation.evaluate_model(model, data, batches=3, batch_size=2, context_length=8, device="cpu", seed=9)
    rng = np.random.default_rng(9)
    losses = []
    for _ in range(3):
        x, y = data.batch(2, 8, "cpu", rng)
        losses.append(float(F.cross_entropy(model(x).reshape(-1, 37), y.reshape(-1))))
    assert abs(got["loss"] - sum(losses) / 3) < 1e-6 and got["batches"] == 3
    assert abs(got["perplexity"] - math.exp(got["loss"])) < 1e-9
    with pytest.raises(ValueError):
        evaluation.evaluate_model(model, data, 0, 2, 8, "cpu", 9)
