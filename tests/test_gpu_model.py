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
