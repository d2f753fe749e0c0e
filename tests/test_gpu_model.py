"""QuantLinear as a drop-in for the model's Linear, and end-to-end greedy decoding against the
oracle model (the same restated Transformer with the oracle's CPU QuantLinearRef in every
linear slot)."""

import copy

import pytest
import torch

from ajllm_amd import QuantLinear, decoding, modeling, quantize_model_
from oracle import qspec
from tests.helpers import MAX_ABS_TOL, REL_FRO_TOL, compare_greedy, errors, make_activations, make_weight

pytestmark = pytest.mark.gpu


def _oracle_model(model: modeling.TransformerLM, scheme: str) -> modeling.TransformerLM:
    ref = copy.deepcopy(model).cpu()
    for parent in list(ref.modules()):
        for name, child in list(parent.named_children()):
            if isinstance(child, modeling.Linear):
                setattr(parent, name, qspec.QuantLinearRef.from_linear(child, scheme))
    return ref.eval()


@pytest.mark.parametrize("scheme", ["w4a16_g128", "w8a16"])
def test_quant_linear_is_a_drop_in(cuda, scheme):
    torch.manual_seed(0)
    dense = modeling.Linear(256, 200)  # 200 rows: not a multiple of the 16-row tile
    ref = qspec.QuantLinearRef.from_linear(dense, scheme)
    layer = QuantLinear.from_linear(dense.to(cuda), scheme)
    assert (layer.in_features, layer.out_features) == (256, 200)
    x = make_activations(15, 256, 3).reshape(3, 5, 256)
    y = layer(x.to(cuda))
    assert y.shape == (3, 5, 200) and y.dtype == torch.bfloat16
    want = ref(x)
    assert errors(y, want)[1] <= REL_FRO_TOL
    y32 = layer(x.float().to(cuda))  # fp32 activations in -> rounded to bf16 -> fp32 out
    assert y32.dtype == torch.float32
    max_abs, rel = errors(y32, ref(x.float()))
    assert max_abs <= 1e-4 and rel <= 1e-5
    big = layer(make_activations(300, 256, 4).to(cuda))  # GEMM path, same layer
    assert big.shape == (300, 200)
    assert errors(big, ref(make_activations(300, 256, 4)))[1] <= REL_FRO_TOL
    # canonical buffers are what a checkpoint holds and they equal the oracle's bit for bit
    state = layer.state_dict()
    assert set(state) == {"qweight", "scales", "zeros"}
    assert torch.equal(state["qweight"].cpu(), ref.qweight)
    assert torch.equal(state["scales"].cpu().view(torch.int16), ref.scales.view(torch.int16))
    fresh = QuantLinear(256, 200, scheme)
    fresh.load_state_dict({k: v.clone() for k, v in state.items()})
    assert torch.equal(fresh(x.to(cuda)), y)


def test_quant_linear_rejects_bias_and_bad_k(cuda):
    with pytest.raises(ValueError):
        QuantLinear.from_linear(torch.nn.Linear(128, 16, bias=True).to(cuda))
    with pytest.raises(ValueError):
        QuantLinear.from_weight(torch.zeros(16, 100, device=cuda))


def test_w8_layer_with_an_input_width_off_the_128_grid(cuda):
    """Per-channel W8 puts no condition on K (the reference's configs/models/transformer_baseline.yaml has d_ff
    1344 = 10.5 groups of 128): the canonical tensors are the oracle's, the kernel-private copy is padded with zero
    codes to 1408 columns and the activations with zeros, which adds exact zeros to every product."""
    torch.manual_seed(5)
    dense = modeling.Linear(1344, 520)
    ref = qspec.QuantLinearRef.from_linear(dense, "w8a16")
    layer = QuantLinear.from_linear(dense.to(cuda), "w8a16")
    assert (layer.in_features, layer.padded_in_features, layer.out_features) == (1344, 1408, 520)
    state = layer.state_dict()
    assert tuple(state["qweight"].shape) == (520, 1344) and torch.equal(state["qweight"].cpu(), ref.qweight)
    assert torch.equal(state["scales"].cpu().view(torch.int16), ref.scales.view(torch.int16))
    for m in (1, 15, 40, 300):   # GEMV, weight-streaming and tile kernels
        x = make_activations(m, 1344, m)
        assert errors(layer(x.to(cuda)), ref(x))[1] <= REL_FRO_TOL, m
    fresh = QuantLinear(1344, 520, "w8a16")
    fresh.load_state_dict({k: v.clone() for k, v in state.items()})
    x = make_activations(7, 1344, 9)
    assert torch.equal(fresh(x.to(cuda)), layer(x.to(cuda)))
    with pytest.raises(ValueError):
        QuantLinear.from_linear(dense.to(cuda), "w4a16_g128")   # groups of 128 input channels need K on that grid


@pytest.mark.parametrize("geometry", ["baseline", "tiny"])
def test_reference_baseline_and_tiny_geometries_decode_with_w8(cuda, geometry):
    """configs/models/transformer_baseline.yaml (d_model 512, 16 heads of 32, d_ff 1344, 4 layers, context 256) and
    transformer_tiny.yaml (d_model 64, 4 heads of 16, d_ff 128, 2 layers, vocabulary 300, context 32) under W8A16:
    every linear is swapped (input widths 1344 and 64 are padded to the kernels' 128-column grid), the greedy
    tokens follow the oracle model's up to its own margin noise, and the graph-replayed loop (with the library's
    prefill attention where the head size is built: 32) gives the eager loop's tokens.  The all-kernel decoder
    does not take such a model."""
    torch.manual_seed(24)
    if geometry == "baseline":
        model = modeling.TransformerLM(vocab_size=1024, context_length=256, d_model=512, num_layers=4, num_heads=16,
                                       d_ff=1344).eval()
        layers, new, vocab = 4, 32, 1024
    else:
        model = modeling.TransformerLM(vocab_size=300, context_length=32, d_model=64, num_layers=2, num_heads=4,
                                       d_ff=128).eval()
        layers, new, vocab = 2, 8, 300
    ref = _oracle_model(model, "w8a16")
    fast = quantize_model_(copy.deepcopy(model).to(cuda), "w8a16")
    assert len([m for m in fast.modules() if isinstance(m, QuantLinear)]) == layers * 7 + 1
    prompt = torch.randint(0, vocab, (2, 24), generator=torch.Generator().manual_seed(8))
    ref_tokens, margins = modeling.greedy_decode(ref, prompt, new, return_margins=True)
    noise = errors(fast(ref_tokens.to(cuda)), ref(ref_tokens))[0]
    assert noise <= 5e-2
    eager = modeling.greedy_decode(fast, prompt.to(cuda), new)
    report = compare_greedy(eager.cpu(), ref_tokens, margins, 24, noise=noise)
    assert not report["unexplained"], report
    for layer in fast.layers:
        layer.attention.use_flash_attention = True   # (head_dim 16 of the tiny model: the model's own attention)
    flash, flash_margins = modeling.greedy_decode(fast, prompt.to(cuda), new, return_margins=True)
    report = compare_greedy(flash.cpu(), eager.cpu(), flash_margins.cpu(), 24, noise=2e-2)   # flash-attention arithmetic
    assert not report["unexplained"], report
    dec = decoding.GraphDecoder(fast, 2, 24 + new)
    dec.prefill(prompt.to(cuda))
    got = dec.generate(new)
    report = compare_greedy(torch.cat((prompt.to(cuda), got), 1).cpu(), flash.cpu(), flash_margins.cpu(), 24, noise=1e-3)
    assert not report["unexplained"], report
    with pytest.raises(ValueError, match="multiples of 128"):
        decoding.FusedDecoder(fast, 2, 24 + new)


def test_quantize_model_swaps_every_linear(cuda):
    torch.manual_seed(1)
    model = modeling.TransformerLM(vocab_size=512, context_length=64, d_model=256, num_layers=2, num_heads=2,
                                   d_ff=512).to(cuda)
    quantize_model_(model, "w4a16_g128")
    swapped = [n for n, m in model.named_modules() if isinstance(m, QuantLinear)]
    assert len(swapped) == 2 * 7 + 1 and "lm_head" in swapped and "layers.1.feed_forward.w3" in swapped
    assert not any(isinstance(m, modeling.Linear) for m in model.modules())
    assert isinstance(model.token_embeddings, modeling.Embedding)
    logits = model(torch.randint(0, 512, (2, 9), device=cuda))
    assert logits.shape == (2, 9, 512) and torch.isfinite(logits).all()
    tied = modeling.TransformerLM(vocab_size=512, context_length=64, d_model=256, num_layers=1, num_heads=2,
                                  d_ff=512, tie_embeddings=True).to(cuda)
    quantize_model_(tied, "w8a16")  # tied models have no lm_head module: the logits matmul stays dense
    assert tied.lm_head is None and tied(torch.randint(0, 512, (1, 4), device=cuda)).shape == (1, 4, 512)


@pytest.mark.parametrize("scheme,batch", [("w4a16_g128", 1), ("w4a16_g128", 4), ("w8a16", 2)])
def test_greedy_tokens_match_the_oracle_model(cuda, scheme, batch):
    """fp32 residual stream, norms and attention in both runs; only the linears differ (HIP kernels
    with bf16-rounded inputs and fp32 outputs vs the oracle's CPU dequantize-and-matmul).

    Two runs whose fp32 sums differ in the last bits round a few activations to different bf16
    values, and a network amplifies that: logits of the two runs differ by about 1e-2 here even
    when BOTH runs use the oracle's own arithmetic on two devices.  So the token sequences are
    required to be identical up to the first step whose top-1/top-2 margin in the oracle run is
    below that measured noise; a difference at a larger margin fails the test."""
    torch.manual_seed(2)
    model = modeling.TransformerLM(vocab_size=512, context_length=96, d_model=256, num_layers=3, num_heads=2,
                                   d_ff=640).eval()
    ref = _oracle_model(model, scheme)
    fast = quantize_model_(copy.deepcopy(model).to(cuda), scheme)
    prompt = torch.randint(0, 512, (batch, 24), generator=torch.Generator().manual_seed(5))
    ref_tokens, margins = modeling.greedy_decode(ref, prompt, 32, return_margins=True)
    got_tokens = modeling.greedy_decode(fast, prompt.to(cuda), 32)
    # noise level: logits of the two runs on the SAME tokens (the oracle's whole sequence)
    logits_ref = ref(ref_tokens)
    logits_got = fast(ref_tokens.to(cuda))
    max_abs, rel = errors(logits_got, logits_ref)
    assert rel <= 2e-2, (max_abs, rel)
    noise = 3 * max_abs
    report = compare_greedy(got_tokens, ref_tokens, margins, 24, noise=noise)
    print(scheme, batch, "logit noise", max_abs, report)
    assert not report["unexplained"], report
    # teacher-forced: with the oracle's tokens as context, every next-token choice agrees
    # wherever the oracle's margin exceeds the noise
    pred_ref = logits_ref[:, 23:-1].argmax(-1)
    pred_got = logits_got[:, 23:-1].argmax(-1).cpu()
    assert torch.equal(pred_ref, ref_tokens[:, 24:])
    disagree = (pred_got != pred_ref)
    assert (margins[disagree] < noise).all(), margins[disagree]
    assert int(disagree.sum()) <= max(1, disagree.numel() // 10)


@pytest.mark.parametrize("scheme", ["w4a16_g128", "w8a16"])
def test_reference_medium_geometry_decodes_through_the_graph_decoder(cuda, scheme):
    """The geometry of the reference's own configs/models/transformer_medium.yaml (d_model 768, 12 heads of
    head_dim 64, d_ff 2048, RoPE, pre-norm RMSNorm, SwiGLU, tied embeddings; fewer layers and a smaller
    vocabulary here): every Linear is swapped, and the graph-replayed decode over the model's own code gives
    the eager loop's tokens.  The all-kernel FusedDecoder is built for head_dim 128 and an untied head and
    says so instead of running something else."""
    torch.manual_seed(21)
    model = modeling.TransformerLM(vocab_size=1024, context_length=128, d_model=768, num_layers=3, num_heads=12,
                                   d_ff=2048, tie_embeddings=True).eval()
    fast = quantize_model_(copy.deepcopy(model).to(cuda), scheme)
    swapped = [m for m in fast.modules() if isinstance(m, QuantLinear)]
    assert len(swapped) == 3 * 7 and fast.lm_head is None
    prompt = torch.randint(0, 1024, (2, 24), generator=torch.Generator().manual_seed(5)).to(cuda)
    eager, margins = modeling.greedy_decode(fast, prompt, 32, return_margins=True)
    dec = decoding.GraphDecoder(fast, 2, 64)
    dec.prefill(prompt)
    got = dec.generate(32)
    report = compare_greedy(torch.cat((prompt, got), 1).cpu(), eager.cpu(), margins.cpu(), 24, noise=1e-3)
    assert not report["unexplained"], report
    with torch.no_grad():
        dense = model.to(cuda)(prompt).float()
        quant = fast(prompt).float()
    assert errors(quant.cpu(), dense.cpu())[1] <= (0.3 if scheme == "w4a16_g128" else 0.05)  # the quantization error itself
    with pytest.raises(ValueError, match="lm_head of its own"):
        decoding.FusedDecoder(fast, 2, 64)   # tied embeddings: the head is a dense product of the model code


@pytest.mark.parametrize("scheme,batch,kv_dtype", [("w4a16_g128", 1, None), ("w8a16", 3, None), ("w4a16_g128", 8, torch.bfloat16)])
def test_reference_medium_geometry_decodes_through_the_fused_decoder(cuda, scheme, batch, kv_dtype):
    """The same geometry (head_dim 64, d_model 768, tied embeddings) with the head untied into a quantized
    linear of its own (``untie_head``): the all-kernel decoder gives the eager loop's tokens, and the untied
    quantized head's logits differ from the tied dense head's by the quantization error only."""
    torch.manual_seed(22)
    model = modeling.TransformerLM(vocab_size=1024, context_length=128, d_model=768, num_layers=3, num_heads=12,
                                   d_ff=2048, tie_embeddings=True).eval()
    fast = quantize_model_(copy.deepcopy(model).to(cuda), scheme, untie_head=True)
    assert isinstance(fast.lm_head, QuantLinear) and not fast.tie_embeddings
    assert len([m for m in fast.modules() if isinstance(m, QuantLinear)]) == 3 * 7 + 1
    prompt = torch.randint(0, 1024, (batch, 24), generator=torch.Generator().manual_seed(6)).to(cuda)
    with torch.no_grad():
        tied = quantize_model_(copy.deepcopy(model).to(cuda), scheme)(prompt).float()
        untied = fast(prompt).float()
    assert errors(untied.cpu(), tied.cpu())[1] <= (0.15 if scheme == "w4a16_g128" else 0.02)
    eager, margins = modeling.greedy_decode(fast, prompt, 40, return_margins=True, kv_dtype=kv_dtype)
    dec = decoding.FusedDecoder(fast, batch, 80, kv_dtype=kv_dtype)
    assert dec.head_dim == 64 and not dec.fuse_merge
    dec.prefill(prompt)
    got = dec.generate(40)
    report = compare_greedy(torch.cat((prompt, got), 1).cpu(), eager.cpu(), margins.cpu(), 24, noise=2e-3)
    assert not report["unexplained"], report
    assert report["identical_rows"] + len(report["attributable"]) == batch
    # logits of one fused step against the eager model on the same context: the same bf16 activations up to the few
    # that a differently ordered sum of squares in a norm moves to the neighbouring bf16 value (2^-8 relative each),
    # and different summation orders in the matmuls
    dec.prefill(prompt)
    with torch.no_grad():
        logits_fused = dec._logits()
        cache = fast.new_cache(batch, 80, dtype=kv_dtype)
        fast(prompt, cache)
        logits_eager = fast(dec.token, cache)[:, -1, :]
    assert errors(logits_fused, logits_eager.cpu())[1] <= 3e-3
    # the prompt through the library's kernels only (flash-attention arithmetic at head_dim 64): the same caches up
    # to bf16-level noise, the first layer's keys up to the rotation's rounding, the step's logits within that noise
    keys_model = [k.clone() for k in dec.cache.keys]
    dec.prefill(prompt, fused=True)
    assert int(dec.cache.position) == 24
    assert errors(dec.cache.keys[0][:, :, :24].float(), keys_model[0][:, :, :24].float().cpu())[1] <= 4e-3
    for mine, theirs in zip(dec.cache.keys, keys_model):
        assert errors(mine[:, :, :24].float(), theirs[:, :, :24].float().cpu())[1] <= 1e-2
    assert errors(dec._logits(), logits_eager.cpu())[1] <= 2e-2


@pytest.mark.parametrize("scheme,batch,kv_dtype", [("w8a16", 2, None), ("w4a16_g128", 5, torch.bfloat16)])
def test_head_dim_32_model_decodes_through_the_fused_decoder(cuda, scheme, batch, kv_dtype):
    """The head size of the reference's configs/models/transformer_baseline.yaml (d_model 512, 16 heads of 32;
    its d_ff 1344 is no multiple of 128 and cannot be quantized in groups, so 1408 here): decode attention, its
    merge and the prefill attention at head_dim 32 inside the all-kernel decoder, against the eager loop."""
    torch.manual_seed(23)
    model = modeling.TransformerLM(vocab_size=1024, context_length=128, d_model=512, num_layers=2, num_heads=16,
                                   d_ff=1408).eval()
    fast = quantize_model_(copy.deepcopy(model).to(cuda), scheme)
    prompt = torch.randint(0, 1024, (batch, 24), generator=torch.Generator().manual_seed(7)).to(cuda)
    eager, margins = modeling.greedy_decode(fast, prompt, 40, return_margins=True, kv_dtype=kv_dtype)
    dec = decoding.FusedDecoder(fast, batch, 80, kv_dtype=kv_dtype)
    assert dec.head_dim == 32
    dec.prefill(prompt)
    got = dec.generate(40)
    report = compare_greedy(torch.cat((prompt, got), 1).cpu(), eager.cpu(), margins.cpu(), 24, noise=2e-3)
    assert not report["unexplained"], report
    dec.prefill(prompt)
    with torch.no_grad():
        logits_fused = dec._logits()
        cache = fast.new_cache(batch, 80, dtype=kv_dtype)
        fast(prompt, cache)
        logits_eager = fast(dec.token, cache)[:, -1, :]
    assert errors(logits_fused, logits_eager.cpu())[1] <= 3e-3
    keys_model = [k.clone() for k in dec.cache.keys]
    dec.prefill(prompt, fused=True)    # flash-attention arithmetic at head_dim 32
    for mine, theirs in zip(dec.cache.keys, keys_model):
        assert errors(mine[:, :, :24].float(), theirs[:, :, :24].float().cpu())[1] <= 1e-2
    assert errors(dec._logits(), logits_eager.cpu())[1] <= 2e-2


@pytest.mark.parametrize("batch", [1, 3])
def test_graph_replayed_decoding_matches_eager_decoding(cuda, batch):
    """The decode step recorded into a HIP graph and replayed per token (with the program's own
    eager work in between: prefill, clones, a second generate call) yields the tokens of the eager
    loop; compared step by step, a difference is accepted only below the eager run's own margin noise."""
    torch.manual_seed(3)
    model = modeling.TransformerLM(vocab_size=512, context_length=96, d_model=256, num_layers=3, num_heads=2,
                                   d_ff=640).eval()
    fast = quantize_model_(copy.deepcopy(model).to(cuda), "w4a16_g128")
    prompt = torch.randint(0, 512, (batch, 20), generator=torch.Generator().manual_seed(8)).to(cuda)
    eager, margins = modeling.greedy_decode(fast, prompt, 40, return_margins=True)
    dec = decoding.GraphDecoder(fast, batch, 60)
    dec.prefill(prompt)
    first = dec.generate(10)          # eager step + capture + replays
    torch.cuda.synchronize()
    _ = fast(prompt)                  # unrelated eager work between replays
    got = dec.generate(40)            # replays only
    assert torch.equal(got[:, :10], first)
    report = compare_greedy(torch.cat((prompt, got), 1).cpu(), eager.cpu(), margins.cpu(), 20, noise=1e-3)
    assert not report["unexplained"], report
    # a second prompt through the same decoder (same graph, new state)
    prompt2 = torch.randint(0, 512, (batch, 20), generator=torch.Generator().manual_seed(9)).to(cuda)
    eager2, margins2 = modeling.greedy_decode(fast, prompt2, 12, return_margins=True)
    dec.prefill(prompt2)
    got2 = dec.generate(12)
    report2 = compare_greedy(torch.cat((prompt2, got2), 1).cpu(), eager2.cpu(), margins2.cpu(), 20, noise=1e-3)
    assert not report2["unexplained"], report2


def test_decode_step_operators_match_their_pytorch_statement(cuda):
    """ajq_add_rmsnorm / ajq_rope_cache / ajq_attn_decode / ajq_swiglu against the model code's own
    PyTorch operators on the same fp32 inputs (outputs are bf16: compared after the same cast)."""
    from ajllm_amd import _lib
    lib = _lib.load()
    st = torch.cuda.current_stream().cuda_stream
    g = torch.Generator().manual_seed(21)
    for b, heads, kv_heads in ((1, 4, 2), (3, 4, 4), (8, 4, 1), (32, 8, 2), (64, 4, 4)):  # the last: a workgroup per whole cache head
        d, hd, max_len, ff = heads * 128, 128, 40, 384
        # residual add + RMSNorm
        hidden = torch.randn((b, d), generator=g).to(cuda)
        delta = torch.randn((b, d), generator=g).to(cuda)
        norm = modeling.RMSNorm(d).to(cuda)
        norm.weight.data = torch.rand(d, generator=g).to(cuda) + 0.5
        want = norm(hidden + delta).to(torch.bfloat16)
        out = torch.empty((b, d), dtype=torch.bfloat16, device=cuda)
        h2 = hidden.clone()
        _lib.check(lib.ajq_add_rmsnorm(h2.data_ptr(), delta.data_ptr(), norm.weight.data_ptr(), norm.epsilon,
                                       out.data_ptr(), b, d, st), "add_rmsnorm")
        assert torch.equal(h2, hidden + delta)
        assert errors(out, want.cpu())[1] <= 3e-3 and (out.float() - want.float()).abs().max() <= 2 ** -6
        # RoPE + cache write, then attention over the cache
        att = modeling.MultiHeadSelfAttention(d, heads, 64, "rope", 10000.0, num_kv_heads=kv_heads).to(cuda)
        qkv = torch.randn((b, (heads + 2 * kv_heads) * hd), generator=g).to(cuda)
        cache_dtype = torch.bfloat16 if b in (3, 32) else torch.float32  # both cache element types
        kv_flag = _lib.AJQ_KV_BF16 if cache_dtype == torch.bfloat16 else _lib.AJQ_KV_F32
        kc = torch.randn((b, kv_heads, max_len, hd), generator=g).to(cuda).to(cache_dtype)
        vc = torch.randn((b, kv_heads, max_len, hd), generator=g).to(cuda).to(cache_dtype)
        for p in (0, 5, 39):
            pos = torch.tensor([p], device=cuda)
            q_rot = torch.empty((b, heads, hd), device=cuda)
            k2, v2 = kc.clone(), vc.clone()
            _lib.check(lib.ajq_rope_cache(qkv.data_ptr(), att.rope.cosine.data_ptr(), att.rope.sine.data_ptr(),
                                          pos.data_ptr(), q_rot.data_ptr(), k2.data_ptr(), v2.data_ptr(), kv_flag, b,
                                          heads, kv_heads, hd, max_len, st), "rope_cache")
            q_in = qkv[:, : heads * hd].view(b, heads, 1, hd)
            k_in = qkv[:, heads * hd: (heads + kv_heads) * hd].view(b, kv_heads, 1, hd)
            v_in = qkv[:, (heads + kv_heads) * hd:].view(b, kv_heads, 1, hd)
            pp = pos.view(1, 1, 1)
            q_want = att.rope(q_in, pp.expand(b, heads, 1))
            k_want = att.rope(k_in, pp.expand(b, kv_heads, 1))
            assert torch.allclose(q_rot, q_want[:, :, 0], atol=1e-6, rtol=1e-6)
            if cache_dtype == torch.float32:
                assert torch.allclose(k2[:, :, p], k_want[:, :, 0], atol=1e-6, rtol=1e-6)
            else:  # the bf16 row is the rounding of the fp32 rotation (1 ulp where that sits on a tie)
                assert (k2[:, :, p].float() - k_want[:, :, 0]).abs().max() <= 2 ** -7 * k_want.abs().max()
            assert torch.equal(v2[:, :, p], v_in[:, :, 0].to(cache_dtype))
            untouched = torch.ones(max_len, dtype=torch.bool); untouched[p] = False
            assert torch.equal(k2[:, :, untouched], kc[:, :, untouched]) and torch.equal(v2[:, :, untouched], vc[:, :, untouched])
            ws_bytes = lib.ajq_attn_decode_workspace_bytes(b, heads)
            ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=cuda)
            got = torch.empty((b, heads * hd), dtype=torch.bfloat16, device=cuda)
            _lib.check(lib.ajq_attn_decode(q_rot.data_ptr(), k2.data_ptr(), v2.data_ptr(), kv_flag, pos.data_ptr(), b,
                                           heads, kv_heads, hd, max_len, got.data_ptr(), ws.data_ptr(), ws_bytes, st),
                       "attn")
            rep = heads // kv_heads
            keys = k2[:, :, : p + 1].float().repeat_interleave(rep, dim=1)
            vals = v2[:, :, : p + 1].float().repeat_interleave(rep, dim=1)
            want_att = modeling.scaled_dot_product_attention(q_rot.unsqueeze(2), keys, vals)[:, :, 0].reshape(b, heads * hd)
            assert (got.float() - want_att).abs().max() <= 2e-2 and errors(got, want_att.cpu())[1] <= 3e-3
            # the same step as one launch: same cache rows, same attention output (the step's own
            # row enters the running softmax first instead of last: rounding differs, nothing else)
            k3, v3 = kc.clone(), vc.clone()
            ws3_bytes = lib.ajq_attn_step_workspace_bytes(b, heads)
            ws3 = torch.zeros(max(ws3_bytes, 16), dtype=torch.uint8, device=cuda)
            for _ in range(2):
                got3 = torch.zeros((b, heads * hd), dtype=torch.bfloat16, device=cuda)
                _lib.check(lib.ajq_attn_step(qkv.data_ptr(), att.rope.cosine.data_ptr(), att.rope.sine.data_ptr(),
                                             pos.data_ptr(), k3.data_ptr(), v3.data_ptr(), kv_flag, b, heads, kv_heads,
                                             hd, max_len, got3.data_ptr(), ws3.data_ptr(), ws3_bytes, st), "attn_step")
                assert torch.equal(v3, v2)
                if cache_dtype == torch.float32:  # the two kernels may contract the rotation's FMAs differently
                    assert torch.allclose(k3, k2, atol=1e-6, rtol=1e-6)
                else:
                    assert (k3.float() - k2.float()).abs().max() <= 2 ** -7 * k2.float().abs().max()
                assert (got3.float() - want_att).abs().max() <= 2e-2 and errors(got3, want_att.cpu())[1] <= 3e-3
                assert (got3.float() - got.float()).abs().max() <= 2 ** -6
        # SwiGLU gate
        ab = torch.randn((b, 2 * ff), generator=g).to(cuda) * 3
        want_g = (modeling.silu(ab[:, :ff]) * ab[:, ff:]).to(torch.bfloat16)
        got_g = torch.empty((b, ff), dtype=torch.bfloat16, device=cuda)
        _lib.check(lib.ajq_swiglu(ab.data_ptr(), got_g.data_ptr(), b, ff, st), "swiglu")
        assert errors(got_g, want_g.cpu())[1] <= 3e-3


@pytest.mark.parametrize("d", [4, 132, 1024, 2048, 4096, 4100, 5632, 12292])
def test_add_rmsnorm_over_widths(cuda, d):
    """ajq_add_rmsnorm at widths on both sides of what a workgroup keeps in registers between its two passes
    (4096 elements), with and without the residual add, against the model code's RMSNorm (layers.py:70-74)."""
    from ajllm_amd import _lib
    lib = _lib.load()
    st = torch.cuda.current_stream().cuda_stream
    g = torch.Generator().manual_seed(d)
    for b in (1, 5):
        hidden = (torch.randn((b, d), generator=g) * 2).to(cuda)
        delta = torch.randn((b, d), generator=g).to(cuda)
        norm = modeling.RMSNorm(d).to(cuda)
        norm.weight.data = torch.rand(d, generator=g).to(cuda) + 0.5
        for with_delta in (True, False):
            h2 = hidden.clone()
            out = torch.zeros((b, d), dtype=torch.bfloat16, device=cuda)
            _lib.check(lib.ajq_add_rmsnorm(h2.data_ptr(), delta.data_ptr() if with_delta else None, norm.weight.data_ptr(),
                                           norm.epsilon, out.data_ptr(), b, d, st), "add_rmsnorm")
            summed = hidden + delta if with_delta else hidden
            assert torch.equal(h2, summed)
            want = norm(summed).to(torch.bfloat16)
            assert errors(out, want.cpu())[1] <= 3e-3 and (out.float() - want.float()).abs().max() <= 2 ** -5


@pytest.mark.parametrize("b,heads,kv_heads,max_len,cache_dtype,hd", [
    (4, 8, 8, 1100, torch.float32, 128), (8, 8, 4, 2100, torch.bfloat16, 128), (16, 8, 2, 1500, torch.float32, 128),
    (6, 16, 4, 1400, torch.bfloat16, 128), (32, 8, 8, 300, torch.float32, 128), (64, 16, 4, 520, torch.bfloat16, 128),
    (128, 4, 2, 200, torch.float32, 128), (16, 8, 8, 1100, torch.float32, 64), (64, 16, 4, 600, torch.bfloat16, 64),
    (12, 12, 12, 900, torch.bfloat16, 64), (32, 16, 16, 1100, torch.float32, 32), (16, 16, 8, 2100, torch.bfloat16, 32),
    (1, 16, 16, 256, torch.float32, 32), (3, 16, 4, 200, torch.bfloat16, 32), (2, 12, 12, 512, torch.float32, 64)])
def test_decode_attention_over_caches_that_are_streamed(cuda, b, heads, kv_heads, max_len, cache_dtype, hd):
    """Caches above 16 MB per launch take the kernel's streaming form (non-temporal loads, rows dealt to the row
    chunks in blocks of 32), and from 256 (sequence, cache head) pairs on one 1024-thread workgroup reads a whole
    head (256 pairs and more); head_dim 128, 64 and 32 (the last three cases: the small caches of the reference's own
    configurations, read with ordinary loads): ajq_attn_decode and ajq_attn_step against the model code's attention, at positions
    on both sides of block and chunk boundaries, with scores spread widely enough that the running reference
    exponent of the grouped-head form has to move many times."""
    from ajllm_amd import _lib
    lib = _lib.load()
    st = torch.cuda.current_stream().cuda_stream
    assert 2 * b * kv_heads * max_len * hd * (4 if cache_dtype == torch.float32 else 2) > 16 << 20 or max_len <= 512
    g = torch.Generator().manual_seed(b * 1000 + max_len)
    att = modeling.MultiHeadSelfAttention(heads * hd, heads, max_len, "rope", 10000.0, num_kv_heads=kv_heads).to(cuda)
    kv_flag = _lib.AJQ_KV_BF16 if cache_dtype == torch.bfloat16 else _lib.AJQ_KV_F32
    kc = torch.randn((b, kv_heads, max_len, hd), generator=g).to(cuda).to(cache_dtype)
    vc = torch.randn((b, kv_heads, max_len, hd), generator=g).to(cuda).to(cache_dtype)
    qkv = torch.randn((b, (heads + 2 * kv_heads) * hd), generator=g).to(cuda)
    qkv[:, : heads * hd] *= 4.0     # scores with a standard deviation of 4: exponents 17 apart are common
    ws_bytes = lib.ajq_attn_step_workspace_bytes(b, heads)
    ws = torch.zeros(max(ws_bytes, 16), dtype=torch.uint8, device=cuda)
    rep = heads // kv_heads
    for p in (0, 31, 32, 63, 64, 127, 128, max_len // 2, max_len - 33, max_len - 1):
        pos = torch.tensor([p], device=cuda)
        k2, v2 = kc.clone(), vc.clone()
        got = torch.zeros((b, heads * hd), dtype=torch.bfloat16, device=cuda)
        _lib.check(lib.ajq_attn_step(qkv.data_ptr(), att.rope.cosine.data_ptr(), att.rope.sine.data_ptr(), pos.data_ptr(),
                                     k2.data_ptr(), v2.data_ptr(), kv_flag, b, heads, kv_heads, hd, max_len,
                                     got.data_ptr(), ws.data_ptr(), ws_bytes, st), "attn_step")
        pp = pos.view(1, 1, 1)
        q_rot = att.rope(qkv[:, : heads * hd].view(b, heads, 1, hd), pp.expand(b, heads, 1))[:, :, 0].contiguous()
        k_new = att.rope(qkv[:, heads * hd: (heads + kv_heads) * hd].view(b, kv_heads, 1, hd), pp.expand(b, kv_heads, 1))
        v_new = qkv[:, (heads + kv_heads) * hd:].view(b, kv_heads, hd)
        untouched = torch.ones(max_len, dtype=torch.bool); untouched[p] = False
        assert torch.equal(k2[:, :, untouched], kc[:, :, untouched]) and torch.equal(v2[:, :, untouched], vc[:, :, untouched])
        assert torch.equal(v2[:, :, p], v_new.to(cache_dtype))
        assert (k2[:, :, p].float() - k_new[:, :, 0]).abs().max() <= 2 ** -7 * k_new.abs().max()
        keys = k2[:, :, : p + 1].float().repeat_interleave(rep, dim=1)
        vals = v2[:, :, : p + 1].float().repeat_interleave(rep, dim=1)
        want = modeling.scaled_dot_product_attention(q_rot.unsqueeze(2), keys, vals)[:, :, 0].reshape(b, heads * hd)
        assert (got.float() - want).abs().max() <= 2e-2 and errors(got, want.cpu())[1] <= 3e-3, p
        # the attention alone over the cache the step left (ajq_attn_decode: every row comes from memory)
        got2 = torch.zeros((b, heads * hd), dtype=torch.bfloat16, device=cuda)
        _lib.check(lib.ajq_attn_decode(q_rot.data_ptr(), k2.data_ptr(), v2.data_ptr(), kv_flag, pos.data_ptr(), b, heads,
                                       kv_heads, hd, max_len, got2.data_ptr(), ws.data_ptr(), ws_bytes, st), "attn")
        assert (got2.float() - want).abs().max() <= 2e-2 and errors(got2, want.cpu())[1] <= 3e-3, p
        assert (got2.float() - got.float()).abs().max() <= 2 ** -6


@pytest.mark.parametrize("batch", [1, 5])
def test_several_steps_per_graph_give_the_tokens_of_one_step_per_graph(cuda, batch):
    """FusedDecoder replays a graph of eight consecutive steps while eight tokens are still wanted and the
    one-step graph for the rest: the same kernels in the same order, so the tokens equal those of a decoder
    that replays one step at a time bit for bit, across calls, with eager work between the replays, and with
    an end-of-sequence stop."""
    torch.manual_seed(14)
    model = modeling.TransformerLM(vocab_size=512, context_length=128, d_model=256, num_layers=2, num_heads=2,
                                   d_ff=640).eval()
    fast = quantize_model_(copy.deepcopy(model).to(cuda), "w4a16_g128")
    prompt = torch.randint(0, 512, (batch, 20), generator=torch.Generator().manual_seed(12)).to(cuda)
    one = decoding.FusedDecoder(fast, batch, 100)
    one.steps_per_graph = 1
    many = decoding.FusedDecoder(fast, batch, 100)
    assert many.steps_per_graph == 8
    for dec in (one, many):
        dec.prefill(prompt)
    a1, b1 = one.generate(5), many.generate(5)          # eager step, both captures, a few single replays
    assert one.graph_many is None and many.graph_many is not None
    torch.cuda.synchronize()
    _ = fast(prompt)                                       # unrelated eager work between replays
    a2, b2 = one.generate(31), many.generate(31)        # 26 more: three graphs of eight and two single steps
    a3, b3 = one.generate(70), many.generate(70)
    assert torch.equal(a1, b1) and torch.equal(a2, b2) and torch.equal(a3, b3) and torch.equal(a3[:, :31], a2)
    assert int(many.cache.position) == int(one.cache.position) == 20 + 70 - 1
    eos = int(a3[0, 40])
    for dec in (one, many):
        dec.prefill(prompt)
    assert torch.equal(one.generate(70, eos_token_id=eos, eos_check_every=5),
                       many.generate(70, eos_token_id=eos, eos_check_every=5))


@pytest.mark.parametrize("scheme,batch,kv_heads,kv_dtype,folded", [
    ("w4a16_g128", 1, 2, None, True), ("w4a16_g128", 5, 2, None, True), ("w8a16", 2, 2, None, True),
    ("w8a16", 32, 1, None, True), ("w4a16_g128", 20, 1, None, True), ("w4a16_g128", 3, 2, torch.bfloat16, True),
    ("w8a16", 24, 1, torch.bfloat16, True), ("w4a16_g128", 5, 2, None, False), ("w8a16", 32, 1, None, False),
    ("w4a16_g128", 1, 1, None, False)])
def test_fused_decoder_matches_eager_decoding(cuda, scheme, batch, kv_heads, kv_dtype, folded):
    """The all-kernel decode step (FusedDecoder) against the eager model loop, replayed from a
    graph; differences only below the eager run's own logit-margin noise.  Batches above 16 take
    the batched-decode matmul; one key/value head under two query heads is grouped-query attention.
    ``folded`` True: norms, gates and residual adds in the matmuls' epilogues with the activations rounded before the
    norm's row scale (the only folded form built for this model's d_model 256); False: every norm, gate, merge and
    residual add as a launch of its own."""
    torch.manual_seed(4)
    model = modeling.TransformerLM(vocab_size=512, context_length=96, d_model=256, num_layers=3, num_heads=2,
                                   d_ff=640, num_kv_heads=kv_heads).eval()
    fast = quantize_model_(copy.deepcopy(model).to(cuda), scheme)
    prompt = torch.randint(0, 512, (batch, 20), generator=torch.Generator().manual_seed(10)).to(cuda)
    eager, margins = modeling.greedy_decode(fast, prompt, 40, return_margins=True, kv_dtype=kv_dtype)
    dec = decoding.FusedDecoder(fast, batch, 60, kv_dtype, activation_rounding="before_scale" if folded else "reference")
    if folded:
        assert dec.fuse_epilogue and not dec.exact_norm   # (d_model 256: the reference-order consumer is not built)
    else:
        dec.fuse_epilogue = dec.fuse_norm = dec.fuse_gate = dec.fuse_merge = False
        # nine per layer, eight where the attention has a single row chunk and so no merge launch (60 rows here)
        from ajllm_amd import _lib
        chunks = _lib.load().ajq_attn_row_chunks(batch, kv_heads, 60)
        assert dec.launches_per_step() == (9 if chunks > 1 else 8) * 3 + 4
    dec.prefill(prompt, rows_per_pass=8 if batch > 16 else None)
    first = dec.generate(10)
    torch.cuda.synchronize()
    _ = fast(prompt)  # unrelated eager work between replays
    got = dec.generate(40)
    assert torch.equal(got[:, :10], first)
    report = compare_greedy(torch.cat((prompt, got), 1).cpu(), eager.cpu(), margins.cpu(), 20, noise=2e-3)
    print(scheme, batch, report)
    # a first difference at a larger margin must be explained by the two loops' logits at that very
    # step: the fused step's logits (its own cache, same tokens so far) against the eager model's
    for row, step, margin in report["unexplained"]:
        assert step >= 1
        dec.prefill(prompt)
        dec.generate(step)
        with torch.no_grad():
            fused_logits = dec._logits()[row].float()
            eager_logits = fast(eager[row:row + 1, : 20 + step], fast.new_cache(1, 60, dtype=kv_dtype))[0, -1].float()
        gap = float((fused_logits - eager_logits).abs().max())
        print("row", row, "step", step, "eager margin", margin, "logit difference", gap)
        assert gap <= (2e-2 if folded else 1e-2) and margin <= 2 * gap, (row, step, margin, gap)
    # logits of one fused step against the eager model on the same context
    dec.prefill(prompt)
    with torch.no_grad():
        logits_fused = dec._logits()
        cache = fast.new_cache(batch, 60, dtype=kv_dtype)
        fast(prompt, cache)
        logits_eager = fast(dec.token, cache)[:, -1, :]
    max_abs, rel = errors(logits_fused, logits_eager.cpu())
    # unfolded, both loops round the same bf16 activations and differ by summation order only; folded, the norm's
    # row scale is applied after the matmul, so every normed activation is rounded at a different point (2^-9
    # relative each, independent of the eager loop's rounding): a few 1e-3 on this 3-layer model
    assert rel <= (6e-3 if folded else 1e-3), (max_abs, rel)


@pytest.mark.parametrize("batch", [1, 3])
def test_graph_decoders_stop_at_eos(cuda, batch):
    """generate(eos_token_id=...): the result is the plain run cut after the step at which the last
    row has produced the token (generator.py:26-27 for one row; every row, as modeling.greedy_decode),
    whatever the spacing of the host's looks."""
    torch.manual_seed(4)
    model = modeling.TransformerLM(vocab_size=512, context_length=96, d_model=256, num_layers=2, num_heads=2,
                                   d_ff=640, num_kv_heads=2).eval()
    fast = quantize_model_(copy.deepcopy(model).to(cuda), "w8a16")
    prompt = torch.randint(0, 512, (batch, 12), generator=torch.Generator().manual_seed(3)).to(cuda)
    for cls in (decoding.GraphDecoder, decoding.FusedDecoder):
        dec = cls(fast, batch, 60)
        dec.prefill(prompt)
        full = dec.generate(40).cpu()
        # a token every row produces if there is one (else row 0's sixth: the run then goes to the end)
        common = set(full[0].tolist())
        for row in full[1:]:
            common &= set(row.tolist())
        eos = min(common) if common else int(full[0, 5])
        seen = full == eos
        stop = int(seen.int().argmax(dim=1).max()) + 1 if bool(seen.any(dim=1).all()) else 40
        for every in (1, 7, 16):
            dec = cls(fast, batch, 60)
            dec.prefill(prompt)
            got = dec.generate(40, eos_token_id=eos, eos_check_every=every).cpu()
            assert got.shape[1] == stop and torch.equal(got, full[:, :stop]), (cls.__name__, every, stop, got.shape)
    if batch == 1:
        assert stop < 40  # (one row always has a common token: the stop is exercised)


@pytest.mark.parametrize("hd", [128, 64, 32])
@pytest.mark.parametrize("b,heads,kv_heads,t,start,cache_dtype", [
    (2, 4, 2, 100, 0, torch.float32), (1, 2, 2, 64, 0, torch.float32), (1, 4, 1, 130, 37, torch.float32),
    (3, 2, 1, 257, 5, torch.bfloat16), (1, 1, 1, 1, 9, torch.float32), (1, 8, 2, 512, 0, torch.bfloat16),
    (1, 32, 8, 2048, 0, torch.bfloat16), (2, 8, 8, 300, 131, torch.bfloat16), (1, 3, 1, 200, 70, torch.float32),
    (1, 12, 12, 511, 0, torch.float32)])
def test_flash_prefill_attention(cuda, b, heads, kv_heads, t, start, cache_dtype, hd):
    """ajq_attn_prefill against the model code's masked softmax attention.  The kernel rounds q, k, v
    and the probabilities to bf16 (flash-attention arithmetic): compared with the fp32 statement on the
    same bf16-rounded inputs within 4e-3 relative Frobenius, and with the unrounded one within 1e-2.
    head_dim 128 (the benchmark models), 64 (the reference's configs/models/transformer_medium.yaml, whose
    shape 12 heads x 511 positions is the last case) and 32 (transformer_baseline.yaml)."""
    from ajllm_amd.attention import flash_prefill
    g = torch.Generator().manual_seed(b * 1000 + t)
    max_len = start + t + 3
    q = torch.randn((b, heads, t, hd), generator=g).to(cuda)
    keys = torch.randn((b, kv_heads, max_len, hd), generator=g).to(cuda).to(cache_dtype)
    values = torch.randn((b, kv_heads, max_len, hd), generator=g).to(cuda).to(cache_dtype)
    got = flash_prefill(q, keys, values, start)
    assert got.shape == (b, t, heads * hd) and bool(torch.isfinite(got).all())
    got16 = flash_prefill(q, keys, values, start, out_dtype=torch.bfloat16)  # the rounding of the fp32 result
    assert got16.dtype == torch.bfloat16 and torch.equal(got16, got.to(torch.bfloat16))
    total = start + t
    rep = heads // kv_heads
    k32 = keys[:, :, :total].float().repeat_interleave(rep, dim=1)
    v32 = values[:, :, :total].float().repeat_interleave(rep, dim=1)
    mask = torch.ones(t, total, dtype=torch.bool, device=cuda).tril_(diagonal=start)
    def statement(qq, kk, vv):
        return modeling.scaled_dot_product_attention(qq, kk, vv, mask).transpose(1, 2).reshape(b, t, heads * hd)
    rounded = lambda x: x.to(torch.bfloat16).float()
    want_rounded = statement(rounded(q), rounded(k32), rounded(v32))
    want = statement(q, k32, v32)
    assert errors(got, want_rounded.cpu())[1] <= 4e-3, errors(got, want_rounded.cpu())
    assert errors(got, want.cpu())[1] <= 1e-2, errors(got, want.cpu())


def test_model_with_flash_attention_flag(cuda):
    """use_flash_attention on every attention layer: prefill logits stay within flash-attention noise of
    the eager model, with and without a KV cache, and a following cached step agrees as well."""
    torch.manual_seed(2)
    model = modeling.TransformerLM(vocab_size=512, context_length=160, d_model=512, num_layers=2, num_heads=4,
                                   d_ff=1408, num_kv_heads=2).eval()
    fast = quantize_model_(copy.deepcopy(model).to(cuda), "w8a16")
    tokens = torch.randint(0, 512, (2, 150), generator=torch.Generator().manual_seed(4)).to(cuda)
    with torch.no_grad():
        eager = fast(tokens)
        cache_e = fast.new_cache(2, 160)
        fast(tokens[:, :149], cache_e)
        step_e = fast(tokens[:, 149:], cache_e)
        for layer in fast.layers:
            layer.attention.use_flash_attention = True
        flash = fast(tokens)
        cache_f = fast.new_cache(2, 160)
        first = fast(tokens[:, :100], cache_f)      # two chunks: the second starts at row 100
        second = fast(tokens[:, 100:149], cache_f)
        step_f = fast(tokens[:, 149:], cache_f)
    assert errors(flash, eager.cpu())[1] <= 1e-2
    assert errors(torch.cat((first, second), 1), eager[:, :149].cpu())[1] <= 1e-2
    assert errors(step_f, step_e.cpu())[1] <= 1e-2


@pytest.mark.parametrize("scheme,kv_dtype", [("w4a16_g128", None), ("w8a16", torch.bfloat16)])
def test_fused_prefill_matches_the_model_with_flash_attention(cuda, scheme, kv_dtype):
    """FusedDecoder.prefill(fused=True): the prompt on library kernels only (GEMMs, add + RMSNorm, RoPE +
    cache write, flash attention, gate), sequences a few at a time, against the model's own PyTorch
    prefill with use_flash_attention: same caches, same first tokens, logits within flash-attention noise;
    decoding continues from either state alike."""
    torch.manual_seed(21)
    model = modeling.TransformerLM(vocab_size=512, context_length=200, d_model=512, num_layers=2, num_heads=4,
                                   d_ff=1408, num_kv_heads=2).eval()
    fast = quantize_model_(copy.deepcopy(model).to(cuda), scheme)
    for layer in fast.layers:
        layer.attention.use_flash_attention = True
    prompt = torch.randint(0, 512, (5, 150), generator=torch.Generator().manual_seed(3)).to(cuda)
    a = decoding.FusedDecoder(fast, 5, 180, kv_dtype)
    b = decoding.FusedDecoder(fast, 5, 180, kv_dtype)
    a.prefill(prompt)
    b.prefill(prompt, rows_per_pass=2, fused=True)
    for x, y in zip(a.cache.keys + a.cache.values, b.cache.keys + b.cache.values):
        # later layers see the earlier layers' flash-attention noise: bf16-level agreement
        assert errors(y[:, :, :150].float(), x[:, :, :150].float().cpu())[1] <= 1e-2
    # the first layer's keys see no attention at all: equal up to the rotation's fp32 rounding
    assert errors(b.cache.keys[0][:, :, :150].float(), a.cache.keys[0][:, :, :150].float().cpu())[1] <= 2e-3
    la, lb = a._logits(), b._logits()
    assert errors(lb, la.cpu())[1] <= 2e-2
    assert int(a.cache.position) == int(b.cache.position) == 150
    ta, tb = a.generate(12), b.generate(12)
    assert ta.shape == tb.shape == (5, 12) and (ta == tb).float().mean() >= 0.8


def test_greedy_pick(cuda):
    """ajq_greedy_pick against torch.argmax (first maximum wins), the output column and the embedding row."""
    from ajllm_amd import _lib
    lib = _lib.load()
    st = torch.cuda.current_stream().cuda_stream
    g = torch.Generator().manual_seed(3)
    for b, v, ld, d in ((1, 32000, 32000, 2048), (5, 1000, 1008, 256), (32, 128256, 128256, 64)):
        logits = torch.randn((b, ld), generator=g).to(cuda)
        logits[:, v:] = 100.0                      # padding columns must not be looked at
        logits[0, 7] = logits[0, 900] = 50.0       # equal maxima: the lower index
        if b > 1:
            logits[1, v - 1] = 60.0                # the last valid column
        emb = torch.randn((v, d), generator=g).to(cuda)
        hidden = torch.zeros((b, d), device=cuda)
        token = torch.zeros((b, 1), dtype=torch.long, device=cuda)
        out = torch.full((b, 9), -1, dtype=torch.long, device=cuda)
        step = torch.tensor([4], device=cuda)
        _lib.check(lib.ajq_greedy_pick(logits.data_ptr(), b, v, ld, emb.data_ptr(), d, hidden.data_ptr(), token.data_ptr(),
                                       out.data_ptr(), 9, step.data_ptr(), None, None, st), "greedy_pick")
        want = torch.argmax(logits[:, :v], dim=-1)
        assert want[0] == 7 and torch.equal(token.view(-1), want) and torch.equal(out[:, 4], want)
        assert (out[:, :4] == -1).all() and (out[:, 5:] == -1).all() and torch.equal(hidden, emb[want])
        assert int(step) == 4
        # with the step's counters advanced by the kernel itself: every workgroup still writes column 4,
        # both counters end one higher, the ticket word is left at zero; twice in a row
        counters = torch.tensor([100, 4], dtype=torch.long, device=cuda)
        ticket = torch.zeros(1, dtype=torch.int32, device=cuda)
        for rep in range(2):
            out.fill_(-1)
            _lib.check(lib.ajq_greedy_pick(logits.data_ptr(), b, v, ld, emb.data_ptr(), d, hidden.data_ptr(),
                                           token.data_ptr(), out.data_ptr(), 9, counters[1:].data_ptr(),
                                           counters.data_ptr(), ticket.data_ptr(), st), "greedy_pick")
            assert torch.equal(out[:, 4 + rep], want) and int((out != -1).sum()) == b
            assert counters.tolist() == [101 + rep, 5 + rep] and int(ticket) == 0
        with pytest.raises(ValueError):
            _lib.check(lib.ajq_greedy_pick(logits.data_ptr(), b, v, ld, emb.data_ptr(), d, hidden.data_ptr(),
                                           token.data_ptr(), out.data_ptr(), 9, step.data_ptr(), counters.data_ptr(), None,
                                           st), "greedy_pick")


@pytest.mark.parametrize("scheme", ["w4a16_g128", "w8a16"])
@pytest.mark.parametrize("b,h,hkv,pos,max_len", [(1, 16, 16, 700, 768), (2, 16, 4, 300, 2048), (4, 16, 8, 90, 128),
                                                 (1, 32, 8, 2000, 2100), (2, 32, 32, 40, 64), (1, 16, 16, 0, 768)])
def test_output_projection_that_merges_the_attention_chunks(cuda, scheme, b, h, hkv, pos, max_len):
    """ajq_attn_step_partial + ajq_w*a16_gemv_merge against ajq_attn_step (which merges the chunks in a
    launch of its own and rounds to bf16) followed by the plain GEMV: the same activations up to a
    differently ordered sum, so the outputs agree to a bf16 rounding of a few activations; also
    against the masked-softmax statement of the model code times the oracle's dequantized weight."""
    import ctypes

    from ajllm_amd import _lib
    lib = _lib.load()
    st = torch.cuda.current_stream().cuda_stream
    g = torch.Generator().manual_seed(1000 * b + h + pos)
    d = h * 128
    cap = lib.ajq_gemv_merge_max_splits(b, d)
    assert cap >= 4
    layer = QuantLinear.from_weight((torch.randn((272, d), generator=g) * 0.02).to(cuda), scheme)
    fused = decoding._FusedLinear([layer])
    qkv = torch.randn((b, (h + 2 * hkv) * 128), generator=g).to(cuda)
    keys = torch.randn((b, hkv, max_len, 128), generator=g).to(cuda)
    values = torch.randn((b, hkv, max_len, 128), generator=g).to(cuda)
    half = torch.arange(64, dtype=torch.float32)
    angles = torch.arange(max_len, dtype=torch.float32)[:, None] / (10000.0 ** (2 * half / 128))[None, :]
    cos, sin = torch.cos(angles).to(cuda).contiguous(), torch.sin(angles).to(cuda).contiguous()
    position = torch.tensor([pos], device=cuda)
    ws_bytes = lib.ajq_attn_step_workspace_bytes(b, h)
    ws = torch.zeros(max(ws_bytes, 16), dtype=torch.uint8, device=cuda)
    k1, v1, k2, v2 = keys.clone(), values.clone(), keys.clone(), values.clone()
    attended = torch.empty((b, d), dtype=torch.bfloat16, device=cuda)
    _lib.check(lib.ajq_attn_step(qkv.data_ptr(), cos.data_ptr(), sin.data_ptr(), position.data_ptr(), k1.data_ptr(),
                                 v1.data_ptr(), _lib.AJQ_KV_F32, b, h, hkv, 128, max_len, attended.data_ptr(),
                                 ws.data_ptr(), ws_bytes, st), "attn_step")
    want = fused(attended)
    ws2 = torch.zeros_like(ws).view(torch.float32)
    splits = ctypes.c_int(0)
    _lib.check(lib.ajq_attn_step_partial(qkv.data_ptr(), cos.data_ptr(), sin.data_ptr(), position.data_ptr(),
                                         k2.data_ptr(), v2.data_ptr(), _lib.AJQ_KV_F32, b, h, hkv, 128, max_len, cap,
                                         ctypes.addressof(splits), ws2.data_ptr(), ws_bytes, st), "attn_step_partial")
    assert 1 <= splits.value <= cap
    got = fused.after_merge(ws2, splits.value, b)
    torch.cuda.synchronize()
    assert torch.equal(k1, k2) and torch.equal(v1, v2)           # the step's cache row, written by both
    max_abs, rel = errors(got, want)
    assert rel <= 2e-3 and max_abs <= 2e-2, (max_abs, rel)
    # against the statement: softmax(q k^T / sqrt(128)) v per head with the step's row included, in fp64
    qk = qkv.double().cpu()
    rot = lambda x, p: torch.stack((x[..., 0::2] * torch.cos(angles[p]).double() - x[..., 1::2] * torch.sin(angles[p]).double(),
                                    x[..., 0::2] * torch.sin(angles[p]).double() + x[..., 1::2] * torch.cos(angles[p]).double()),
                                   dim=-1).flatten(-2)
    q = rot(qk[:, : h * 128].view(b, h, 128), pos)
    kk, vv = k2[:, :, : pos + 1].double().cpu(), v2[:, :, : pos + 1].double().cpu()
    rep = h // hkv
    scores = torch.einsum("bhd,bhtd->bht", q, kk.repeat_interleave(rep, dim=1)) / 128 ** 0.5
    att = torch.einsum("bht,bhtd->bhd", torch.softmax(scores, -1), vv.repeat_interleave(rep, dim=1)).reshape(b, d)
    w_hat = (qspec.dequantize_w8(layer.qweight.cpu().numpy(), layer.scales.cpu().numpy()) if scheme == "w8a16" else
             qspec.dequantize_w4(layer.qweight.cpu().numpy(), layer.scales.cpu().numpy(), layer.zeros.cpu().numpy()))
    ref = qspec.quant_linear(att.to(torch.bfloat16), torch.from_numpy(w_hat), accumulate=torch.float64,
                             out_dtype=torch.float64)
    max_abs, rel = errors(got[:, :272], ref)
    assert rel <= 2e-3 and max_abs <= MAX_ABS_TOL, (max_abs, rel)
    # the same launch with the residual epilogue: bit for bit h_in + (the merged product), its bf16 image
    # times the next norm's gain, and the per-tile sums of squares
    n16 = fused.rows16
    h_in = torch.randn((b, n16), generator=g).to(cuda)
    gain = (torch.rand(n16, generator=g) + 0.5).to(cuda)
    h_out = torch.zeros_like(h_in)
    xt = torch.zeros((b, n16), dtype=torch.bfloat16, device=cuda)
    ssq = torch.zeros((16, n16 // 16), dtype=torch.float32, device=cuda)
    fused.merge_residual(ws2, splits.value, b, h_in, gain, h_out, xt, ssq)
    torch.cuda.synchronize()
    assert torch.equal(h_out, h_in + got)
    assert torch.equal(xt, (h_out * gain).to(torch.bfloat16))
    tiles = h_out.double().square().reshape(b, n16 // 16, 16).sum(-1)
    assert float((ssq[:b].double() - tiles).abs().max() / tiles.max()) <= 1e-6 and not ssq[b:].any()


@pytest.mark.parametrize("scheme", ["w4a16_g128", "w8a16"])
@pytest.mark.parametrize("m,k", [(1, 1024), (3, 2048), (16, 2048), (1, 4096), (8, 4096), (2, 5632), (8, 5632)])
def test_gemv_with_norm_or_gate_prologue(cuda, scheme, m, k):
    """ajq_w*a16_gemv_norm / _gate against the separate operators (add + RMSNorm, SwiGLU gate) followed by
    the plain GEMV: same bf16 activations up to the rounding of a differently ordered sum of squares."""
    from ajllm_amd import _lib
    lib = _lib.load()
    st = torch.cuda.current_stream().cuda_stream
    g = torch.Generator().manual_seed(5 + m + k)
    n = 272
    layer = QuantLinear.from_weight((torch.randn((n, k), generator=g) * 0.02).to(cuda), scheme)
    fused = decoding._FusedLinear([layer])
    assert fused.fusable(m) and not fused.fusable(17)
    h = torch.randn((m, k), generator=g).to(cuda)
    d = torch.randn((m, k), generator=g).to(cuda)
    gain = (torch.rand(k, generator=g) + 0.5).to(cuda)
    for delta in (d, None):
        h_out = torch.zeros_like(h)
        y = fused.after_norm(h, delta, gain, 1e-5, h_out)
        h_ref = h.clone()
        normed = torch.empty((m, k), dtype=torch.bfloat16, device=cuda)
        _lib.check(lib.ajq_add_rmsnorm(h_ref.data_ptr(), delta.data_ptr() if delta is not None else None, gain.data_ptr(),
                                       1e-5, normed.data_ptr(), m, k, st), "add_rmsnorm")
        assert torch.equal(h_out, h_ref)
        want = fused(normed)
        assert errors(y, want.cpu())[1] <= 1e-3 and (y - want).abs().max() <= 2e-2
    ab = (torch.randn((m, 2 * k), generator=g) * 2).to(cuda)
    y = fused.after_gate(ab)
    gated = torch.empty((m, k), dtype=torch.bfloat16, device=cuda)
    _lib.check(lib.ajq_swiglu(ab.data_ptr(), gated.data_ptr(), m, k, st), "swiglu")
    want = fused(gated)
    assert torch.equal(y, want)  # same expression per element: identical activations, identical GEMV order


@pytest.mark.parametrize("scheme,batch", [("w4a16_g128", 1), ("w8a16", 4), ("w4a16_g128", 16)])
def test_fused_decoder_with_gemv_prologues(cuda, scheme, batch):
    """A model whose widths the prologue GEMVs are built for (d_model 1024, d_ff 2048): the decoder
    folds both norms and the gate into the following GEMVs; tokens against the eager loop."""
    torch.manual_seed(14)
    model = modeling.TransformerLM(vocab_size=512, context_length=96, d_model=1024, num_layers=2, num_heads=8,
                                   d_ff=2048, num_kv_heads=4).eval()
    fast = quantize_model_(copy.deepcopy(model).to(cuda), scheme)
    prompt = torch.randint(0, 512, (batch, 20), generator=torch.Generator().manual_seed(11)).to(cuda)
    eager, margins = modeling.greedy_decode(fast, prompt, 30, return_margins=True)
    dec = decoding.FusedDecoder(fast, batch, 60)
    assert dec.head.fusable(batch) and dec.layers[0]["w2"].fusable(batch)
    dec.fuse_norm = dec.fuse_gate = True  # also at the batches where the decoder would not choose them
    dec.fuse_epilogue, dec.fuse_merge = False, dec.merge_splits > 0   # (it prefers the epilogue forms where both are built)
    dec.prefill(prompt)
    got = dec.generate(30)
    report = compare_greedy(torch.cat((prompt, got), 1).cpu(), eager.cpu(), margins.cpu(), 20, noise=2e-3)
    print(scheme, batch, report)
    for row, step, margin in report["unexplained"]:
        dec.prefill(prompt)
        dec.generate(step)
        with torch.no_grad():
            fused_logits = dec._logits()[row].float()
            eager_logits = fast(eager[row:row + 1, : 20 + step], fast.new_cache(1, 60))[0, -1].float()
        gap = float((fused_logits - eager_logits).abs().max())
        assert gap <= 1e-2 and margin <= 2 * gap, (row, step, margin, gap)
    dec.prefill(prompt)
    with torch.no_grad():
        logits_fused = dec._logits()
        cache = fast.new_cache(batch, 60)
        fast(prompt, cache)
        logits_eager = fast(dec.token, cache)[:, -1, :]
    assert errors(logits_fused, logits_eager.cpu())[1] <= REL_FRO_TOL


def test_fused_decoder_tokens_match_the_oracle_model(cuda):
    """The all-kernel, graph-replayed decode against the CPU oracle model (the restated Transformer
    with the oracle's QuantLinearRef in every linear slot), batch 4, head_dim 128, GQA off: the
    end-to-end statement of "identical greedy tokens", up to the oracle's own margin noise."""
    torch.manual_seed(6)
    model = modeling.TransformerLM(vocab_size=2048, context_length=128, d_model=512, num_layers=4, num_heads=4,
                                   d_ff=1408).eval()
    ref = _oracle_model(model, "w4a16_g128")
    fast = quantize_model_(copy.deepcopy(model).to(cuda), "w4a16_g128")
    prompt = torch.randint(0, 2048, (4, 64), generator=torch.Generator().manual_seed(12))
    ref_tokens, margins = modeling.greedy_decode(ref, prompt, 48, return_margins=True)
    dec = decoding.FusedDecoder(fast, 4, 112)
    dec.prefill(prompt.to(cuda))
    got = torch.cat((prompt, dec.generate(48).cpu()), dim=1)
    with torch.no_grad():
        noise = 3 * errors(fast(ref_tokens.to(cuda)), ref(ref_tokens))[0]
    report = compare_greedy(got, ref_tokens, margins, 64, noise=noise)
    print("fused vs oracle", noise, report)
    assert not report["unexplained"], report
    assert report["identical_rows"] + len(report["attributable"]) == 4


def _fused_decoder_against_the_oracle_model(cuda, scheme, batch, model, configure, rounding="reference"):
    """The graph-replayed tokens of a FusedDecoder (set up by ``configure``) against the CPU oracle model,
    and the decode-step logits of every step along the oracle's tokens against the oracle's logits."""
    ref = _oracle_model(model, scheme)
    fast = quantize_model_(copy.deepcopy(model).to(cuda), scheme)
    prompt = torch.randint(0, 2048, (batch, 48), generator=torch.Generator().manual_seed(13))
    new = 48
    with torch.no_grad():
        cache = ref.new_cache(batch, 48 + new)
        step_input, ref_new, ref_logits = prompt, [], []
        for _ in range(new):
            logits = ref(step_input, cache, last_token_only=True)[:, -1, :].float()
            step_input = logits.argmax(-1, keepdim=True)
            ref_new.append(step_input)
            ref_logits.append(logits)
    ref_new, ref_logits = torch.cat(ref_new, 1), torch.stack(ref_logits, 1)
    top2 = torch.topk(ref_logits, 2, dim=-1).values
    margins = top2[..., 0] - top2[..., 1]
    dec = decoding.FusedDecoder(fast, batch, 48 + new, activation_rounding=rounding)
    configure(dec)
    dec.prefill(prompt.to(cuda))
    got = dec.generate(new).cpu()
    dec.prefill(prompt.to(cuda))
    assert torch.equal(dec.generate(new).cpu(), got)            # sums run in a fixed order: run-to-run identical
    # teacher-forced: decode-step logits along the oracle's tokens
    dec.prefill(prompt.to(cuda))
    forced = []
    with torch.no_grad():
        for t in range(1, new):
            torch.index_select(dec.embedding, 0, ref_new[:, t - 1].to(cuda), out=dec.embedded)
            forced.append(dec._logits().float().cpu())
            dec.counters.add_(1)
    forced = torch.stack(forced, 1)                              # rows t = 1 .. new - 1
    diff = forced.double() - ref_logits[:, 1:].double()
    step_err = torch.cat((torch.zeros(batch, 1, dtype=torch.float64), diff.abs().amax(-1)), 1)
    rel = float(diff.norm() / ref_logits[:, 1:].double().norm())
    print(scheme, batch, "teacher-forced logits rel", rel, "max-abs", float(step_err.max()))
    assert rel <= 1e-2, rel
    pred = forced.argmax(-1)
    disagree = pred != ref_new[:, 1:]
    assert bool((margins[:, 1:][disagree] <= 2 * step_err[:, 1:][disagree] + 1e-6).all())
    for b in range(batch):
        d = (got[b] != ref_new[b]).nonzero()
        if len(d) and int(d[0]) > 0:
            first = int(d[0])
            assert float(margins[b, first]) <= 2 * float(step_err[b, first]) + 1e-6, (b, first)


@pytest.mark.parametrize("scheme,batch", [("w4a16_g128", 1), ("w8a16", 4)])
def test_fused_decoder_with_gemv_prologues_matches_the_oracle_model(cuda, scheme, batch):
    """Widths the prologue GEMVs are built for (d_model 1024, d_ff 2048, grouped-query heads), with the
    norm and gate prologues forced on."""
    torch.manual_seed(16)
    model = modeling.TransformerLM(vocab_size=2048, context_length=128, d_model=1024, num_layers=3, num_heads=8,
                                   d_ff=2048, num_kv_heads=4).eval()

    def configure(dec):
        assert dec.head.fusable(batch) and dec.layers[0]["w2"].fusable(batch)
        dec.fuse_norm = dec.fuse_gate = True
        dec.fuse_epilogue, dec.fuse_merge = False, dec.merge_splits > 0   # (it prefers the epilogue forms where both are built)

    _fused_decoder_against_the_oracle_model(cuda, scheme, batch, model, configure)


@pytest.mark.parametrize("scheme,batch,d_ff,rounding", [
    ("w4a16_g128", 1, 5632, "reference"), ("w8a16", 4, 2048, "reference"), ("w4a16_g128", 2, 4096, "reference"),
    ("w8a16", 3, 5632, "reference"), ("w4a16_g128", 8, 5632, "reference"), ("w8a16", 13, 2048, "reference"),
    ("w4a16_g128", 8, 5632, "before_scale"), ("w8a16", 13, 2048, "before_scale"),
    ("w4a16_g128", 5, 4096, "before_scale"), ("w8a16", 1, 2048, "before_scale"), ("w4a16_g128", 12, 5632, "before_scale"),
    ("w8a16", 20, 2048, "before_scale"), ("w4a16_g128", 33, 5632, "before_scale")])
def test_fused_decoder_with_gemv_epilogues_matches_the_oracle_model(cuda, scheme, batch, d_ff, rounding):
    """Widths the epilogue GEMVs are built for (d_model 2048): no norm, gate or residual launch inside a layer
    (the norm's row scale is applied to the matmul outputs, the residual add and the next norm's preparation
    ride in the output projection and w2, w1|w3 applies the gate on interleaved rows): six launches per
    layer, five at batch 1, where the output projection also merges the attention's row chunks on its way in; up
    to batch 4 the step's first norm rides in layer 0's q|k|v.  With the reference's rounding point above batch 4 the
    norms are launches of their own (eight per layer), the residual adds and the gate stay folded.  Above 16 rows, and for shapes the GEMV kernel's
    straight-line configurations do not cover (12 rows on K = 5632), the weight-streaming kernel carries the epilogues."""
    torch.manual_seed(18)
    model = modeling.TransformerLM(vocab_size=2048, context_length=128, d_model=2048, num_layers=2, num_heads=16,
                                   d_ff=d_ff, num_kv_heads=4).eval()

    def configure(dec):
        assert dec.fuse_epilogue and not dec.fuse_norm and not dec.fuse_gate
        assert dec.exact_norm == (rounding == "reference")
        # reference rounding above batch 4: the norms are launches of their own again (eight per layer)
        assert dec.norm_launch == (rounding == "reference" and batch > 4)
        assert not dec.fuse_merge and dec.first_norm_fused == (batch <= 4)
        if batch == 1 and rounding == "before_scale":
            dec.fuse_merge = True   # the output projection that merges the attention's row chunks (an option)
        if dec.norm_launch:
            assert dec.launches_per_step() == 8 * 2 + 3
        else:
            assert dec.launches_per_step() == (5 if dec.fuse_merge else 6) * 2 + (2 if batch <= 4 else 3)

    _fused_decoder_against_the_oracle_model(cuda, scheme, batch, model, configure, rounding)


def test_quantized_checkpoint_round_trip(cuda, tmp_path):
    """save_quantized -> load_quantized gives a model with the same canonical tensors and the same
    logits; a dense reference-style checkpoint converts to the same file contents; a flipped byte is
    caught by the manifest's digest."""
    from ajllm_amd import checkpoint
    torch.manual_seed(7)
    cfg = dict(vocab_size=512, context_length=64, d_model=256, num_layers=2, num_heads=2, d_ff=640)
    dense = modeling.TransformerLM(**cfg).eval()
    torch.save({"model_state_dict": dense.state_dict(), "optimizer_state_dict": {}, "step": 5, "metadata": {}},
               tmp_path / "dense.pt")
    fast = quantize_model_(copy.deepcopy(dense).to(cuda), "w4a16_g128")
    path = checkpoint.save_quantized(tmp_path / "q.safetensors", fast, "w4a16_g128",
                                     config=checkpoint.model_config(fast), metadata={"note": "test"})
    loaded, manifest = checkpoint.load_quantized(path, cuda)
    assert manifest["scheme"] == "w4a16_g128" and manifest["group_size"] == 128 and manifest["metadata"]["note"] == "test"
    a, b = fast.state_dict(), loaded.state_dict()
    assert set(a) == set(b) and all(torch.equal(a[k], b[k]) for k in a)
    tokens = torch.randint(0, 512, (2, 9), device=cuda)
    assert torch.equal(fast(tokens), loaded(tokens))
    converted = checkpoint.convert_dense_checkpoint(tmp_path / "dense.pt", tmp_path / "c.safetensors", cfg,
                                                    "w4a16_g128", cuda)
    t1, m1 = checkpoint.read_quantized(path)
    t2, m2 = checkpoint.read_quantized(converted)
    assert m1["sha256"] == m2["sha256"] and m2["metadata"]["step"] == 5
    raw = bytearray(path.read_bytes())
    raw[-10] ^= 0xFF
    (tmp_path / "bad.safetensors").write_bytes(bytes(raw))
    with pytest.raises(ValueError):
        checkpoint.read_quantized(tmp_path / "bad.safetensors")


def test_quantization_report_against_the_oracle_model(cuda, tmp_path):
    """Held-out loss of the quantized model (reference evaluate_model, evaluator.py:14-31) equals the
    loss of the oracle model on the same windows, both schemes cost little, and the
    caller's dense model is left untouched."""
    import numpy as np

    from ajllm_amd import evaluation
    torch.manual_seed(21)
    cfg = dict(vocab_size=512, context_length=64, d_model=256, num_layers=2, num_heads=2, d_ff=640)
    dense = modeling.TransformerLM(**cfg).eval()
    with torch.no_grad():  # sharpen the random-init model so its own samples are predictable to it
        dense.lm_head.weight.mul_(6.0)
        sample = torch.randint(0, 512, (1, 1))
        gen = torch.Generator().manual_seed(3)
        stream = [int(sample)]
        cache = dense.new_cache(1, 64)
        for _ in range(63):
            probs = torch.softmax(dense(sample, cache)[0, -1], -1)
            sample = torch.multinomial(probs, 1, generator=gen).view(1, 1)
            stream.append(int(sample))
    path = tmp_path / "heldout.bin"
    np.asarray(stream * 8, dtype=np.uint32).tofile(path)
    data = evaluation.TokenFile(path)
    args = dict(batches=2, batch_size=4, context_length=32, seed=17)
    deltas = {}
    for scheme in ("w8a16", "w4a16_g128"):
        report = evaluation.quantization_report(dense, data, scheme, device=cuda, **args)
        oracle = evaluation.evaluate_model(_oracle_model(dense, scheme), data, device="cpu", **args)
        print(scheme, report, oracle)
        assert abs(report["quantized"]["loss"] - oracle["loss"]) < 2e-3
        assert report["dense"]["loss"] < 6.0  # below ln(512) = 6.24: the stream is the model's own
        deltas[scheme] = abs(report["loss_delta"])
        assert abs(report["perplexity_ratio"] - np.exp(report["loss_delta"])) < 1e-6
    # W8's delta is mostly the bf16 rounding of the activations at every linear, not the weights
    assert deltas["w8a16"] < 0.05 and deltas["w4a16_g128"] < 0.25
    assert all(isinstance(m, modeling.Linear) for m in (dense.lm_head, dense.layers[0].attention.q_proj))
    dense.cpu()
