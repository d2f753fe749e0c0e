"""ajq_sample_pick and the decoders' sampling mode against the reference's sample_next_token
(src/ajllm/generation/sampling.py:8-22), restated here with torch on the CPU in float64.

The reference draws with torch.multinomial; the library draws by inverse CDF over the kept tokens in index order from
uniforms the caller supplies.  The two share the DISTRIBUTION, not the random bits, so what is checked is: the set of
tokens the top-p filter keeps (against the reference's own formula), that every draw lies in it, that the draw is the
inverse CDF it says it is (monotone in u; the CDF's jumps sit where the kept probabilities put them), the frequencies
over many draws, the limits (top_p -> 0 and temperature -> 0 are argmax; top_p = 1 keeps everything), determinism, the
outputs it shares with ajq_greedy_pick, and the two decoders end to end (equal seeds give equal tokens, a replayed graph
equals eager steps).  Parity of the random stream itself with torch.multinomial is unpinned by construction.
"""

import copy

import pytest
import torch

from ajllm_amd import decoding, modeling, quantize_model_

pytestmark = pytest.mark.gpu


def _reference_kept(logits: torch.Tensor, temperature: float, top_p: float):
    """(probabilities, kept mask, mass strictly above every token) as sample_next_token forms them, in float64."""
    p = torch.softmax(logits.double() / temperature, dim=-1)
    sp, si = torch.sort(p, descending=True, dim=-1)
    above = torch.cumsum(sp, dim=-1) - sp
    keep_sorted = ~(above >= top_p)
    keep = torch.zeros_like(keep_sorted)
    keep.scatter_(-1, si, keep_sorted)
    above_by_token = torch.zeros_like(above)
    above_by_token.scatter_(-1, si, above)
    return p, keep, above_by_token


def _pick(cuda, logits, temperature, top_p, uniforms, step=0, v=None, with_embedding=False):
    from ajllm_amd import _lib
    lib = _lib.load()
    b, ld = logits.shape
    v = v or ld
    lg, un = logits.to(cuda).contiguous(), uniforms.to(cuda).contiguous()
    token = torch.full((b, 1), -1, dtype=torch.long, device=cuda)
    out = torch.full((b, 7), -1, dtype=torch.long, device=cuda)
    kept = torch.full((b,), -1, dtype=torch.int32, device=cuda)
    st = torch.tensor([step], device=cuda)
    emb = hidden = None
    if with_embedding:
        emb = torch.arange(v * 8, dtype=torch.float32, device=cuda).reshape(v, 8)
        hidden = torch.zeros((b, 8), device=cuda)
    _lib.check(lib.ajq_sample_pick(lg.data_ptr(), b, v, ld, temperature, top_p, un.data_ptr(), un.shape[0],
                                   emb.data_ptr() if emb is not None else None, 8 if emb is not None else 0,
                                   hidden.data_ptr() if hidden is not None else None, token.data_ptr(), out.data_ptr(), 7,
                                   st.data_ptr(), None, None, kept.data_ptr(), torch.cuda.current_stream().cuda_stream),
               "sample_pick")
    torch.cuda.synchronize()
    return token.view(-1).cpu(), out.cpu(), kept.cpu(), (hidden.cpu() if hidden is not None else None, emb)


@pytest.mark.parametrize("v,ld", [(1000, 1000), (32000, 32000), (128256, 128256), (50, 64)])
@pytest.mark.parametrize("temperature,top_p", [(1.0, 0.9), (0.7, 0.3), (1.5, 0.95)])
def test_top_p_keeps_what_the_reference_keeps_and_draws_inside_it(cuda, v, ld, temperature, top_p):
    g = torch.Generator().manual_seed(v + int(100 * top_p))
    b = 24
    logits = torch.randn((b, ld), generator=g) * 3.0
    logits[:, v:] = 50.0  # padding columns must not be looked at
    u = torch.rand((3, b), generator=g)
    token, out, kept, _ = _pick(cuda, logits, temperature, top_p, u, step=1, v=v)
    p, keep, above = _reference_kept(logits[:, :v], temperature, top_p)
    want = keep.sum(-1)
    # the boundary token's "mass above" is compared with top_p in 40-bit fixed point here and in float32 in the
    # reference: the counts may differ by a token whose mass above lies within rounding of top_p
    assert int((kept - want).abs().max()) <= 1 and int((kept == want).sum()) >= b - 2, (kept, want)
    rows = torch.arange(b)
    assert bool(((token >= 0) & (token < v)).all())
    inside = keep[rows, token] | ((above[rows, token] - top_p).abs() < 1e-5)
    assert bool(inside.all())
    assert torch.equal(out[:, 1], token) and int((out != -1).sum()) == b


def test_the_draw_is_the_inverse_cdf_over_the_kept_tokens_in_index_order(cuda):
    """One row of logits for 4096 sorted uniforms: the chosen index never decreases with u, every kept token with a
    probability above the grid's spacing is drawn, and the share of uniforms that land on a token is its renormalised
    probability (within two grid cells)."""
    g = torch.Generator().manual_seed(5)
    v, b, top_p, temperature = 300, 4096, 0.8, 0.9
    row = torch.randn((1, v), generator=g) * 2.0
    logits = row.expand(b, v).contiguous()
    u = ((torch.arange(b, dtype=torch.float64) + 0.5) / b).float().reshape(1, b)
    token, _, kept, _ = _pick(cuda, logits, temperature, top_p, u)
    p, keep, _ = _reference_kept(row, temperature, top_p)
    assert int(kept[0]) == int(keep.sum()) and bool((kept == kept[0]).all())
    assert bool((token[1:] >= token[:-1]).all())
    q = (p * keep)[0] / (p * keep)[0].sum()
    share = torch.bincount(token, minlength=v).double() / b
    assert float((share - q).abs().max()) <= 2.0 / b + 1e-6
    assert bool((share[~keep[0]] == 0).all()) and bool((share[q > 2.0 / b] > 0).all())


def test_sampling_frequencies_over_many_random_draws(cuda):
    g = torch.Generator().manual_seed(9)
    v, b, steps = 40, 2048, 16
    row = torch.randn((1, v), generator=g)
    logits = row.expand(b, v).contiguous()
    u = torch.rand((steps, b), generator=g)
    counts = torch.zeros(v, dtype=torch.double)
    for s in range(steps):
        token, out, _, _ = _pick(cuda, logits, 1.0, 1.0, u, step=s)
        assert torch.equal(out[:, min(s, 6)], token)  # the output column follows the step (held inside the row)
        counts += torch.bincount(token, minlength=v).double()
    p = torch.softmax(row.double(), -1)[0]
    n = b * steps
    # every frequency within five standard deviations of its binomial
    assert bool(((counts / n - p).abs() <= 5 * torch.sqrt(p * (1 - p) / n) + 1e-9).all())


def test_limits_determinism_and_shared_outputs(cuda):
    g = torch.Generator().manual_seed(11)
    b, v = 8, 5000
    logits = torch.randn((b, v), generator=g) * 2.0
    u = torch.rand((2, b), generator=g)
    best = torch.argmax(logits, -1)
    # a vanishing top_p keeps the most probable token alone; so does a vanishing temperature
    token, _, kept, (hidden, emb) = _pick(cuda, logits, 1.0, 1e-6, u, with_embedding=True)
    assert torch.equal(token, best) and bool((kept == 1).all()) and torch.equal(hidden, emb.cpu()[best])
    token, _, _, _ = _pick(cuda, logits, 1e-3, 1.0, u)
    assert torch.equal(token, best)
    # top_p = 1 keeps every token; equal inputs give equal tokens; u = 0 and u -> 1 are the ends of the CDF
    a = _pick(cuda, logits, 0.8, 1.0, u, step=1)
    c = _pick(cuda, logits, 0.8, 1.0, u, step=1)
    assert bool((a[2] == v).all()) and torch.equal(a[0], c[0])
    ends = torch.tensor([[0.0] * b, [0.99999994] * b])
    p = torch.softmax(logits.double() / 0.8, -1)
    first, _, _, _ = _pick(cuda, logits, 0.8, 1.0, ends, step=0)
    last, _, _, _ = _pick(cuda, logits, 0.8, 1.0, ends, step=1)
    assert bool((first == 0).all() | (p[torch.arange(b), 0] < 2.0 ** -40).any()) and bool((last >= v - 200).all())
    # argument errors are refused before any launch
    from ajllm_amd import _lib
    lib = _lib.load()
    x = logits.to(cuda)
    tok = torch.zeros((b, 1), dtype=torch.long, device=cuda)
    out = torch.zeros((b, 4), dtype=torch.long, device=cuda)
    st = torch.zeros(1, dtype=torch.long, device=cuda)
    un = u.to(cuda)
    args = lambda t, pp, unp: (x.data_ptr(), b, v, v, t, pp, unp, 2, None, 0, None, tok.data_ptr(), out.data_ptr(), 4,
                               st.data_ptr(), None, None, None, None)
    assert lib.ajq_sample_pick(*args(0.0, 0.9, un.data_ptr())) == -2
    assert lib.ajq_sample_pick(*args(1.0, 0.0, un.data_ptr())) == -2
    assert lib.ajq_sample_pick(*args(1.0, 0.9, None)) == -1


@pytest.mark.parametrize("batch", [1, 5])
def test_decoders_sample_reproducibly_and_graph_replay_equals_eager_steps(cuda, batch):
    """FusedDecoder and GraphDecoder with set_sampling: equal seeds give equal tokens, another seed gives others, a
    graph of eight steps gives the tokens of one step per graph, every token is in the vocabulary, and
    temperature <= 0 is the greedy decoder."""
    torch.manual_seed(21)
    model = modeling.TransformerLM(vocab_size=512, context_length=128, d_model=256, num_layers=2, num_heads=2,
                                   d_ff=640).eval()
    fast = quantize_model_(copy.deepcopy(model).to(cuda), "w4a16_g128")
    prompt = torch.randint(0, 512, (batch, 20), generator=torch.Generator().manual_seed(2)).to(cuda)

    def run(kind, seed, temperature=0.9, top_p=0.9, steps_per_graph=None, fused_prefill=False):
        dec = kind(fast, batch, 100)
        if steps_per_graph is not None:
            dec.steps_per_graph = steps_per_graph
        dec.set_sampling(temperature, top_p, seed=seed)
        if fused_prefill:
            dec.prefill(prompt, fused=True)
        else:
            dec.prefill(prompt)
        first = dec.generate(6)
        torch.cuda.synchronize()
        _ = fast(prompt)  # unrelated eager work between replays
        return first, dec.generate(60)

    a1, a2 = run(decoding.FusedDecoder, 7)
    b1, b2 = run(decoding.FusedDecoder, 7, steps_per_graph=1)
    c1, c2 = run(decoding.FusedDecoder, 8)
    assert torch.equal(a2, b2) and torch.equal(a2[:, :6], a1) and torch.equal(a1, b1) and not torch.equal(a2, c2)
    assert bool(((a2 >= 0) & (a2 < 512)).all())
    greedy = decoding.FusedDecoder(fast, batch, 100)
    greedy.prefill(prompt)
    want = greedy.generate(60)
    assert not torch.equal(a2, want)
    assert torch.equal(run(decoding.FusedDecoder, 7, temperature=0.0)[1], want)
    # a vanishing top_p follows the greedy path token for token (the same logits, the most probable token alone)
    assert torch.equal(run(decoding.FusedDecoder, 7, temperature=1.0, top_p=1e-6)[1], want)
    g1, g2 = run(decoding.GraphDecoder, 7)
    h1, h2 = run(decoding.GraphDecoder, 7)
    assert torch.equal(g2, h2) and bool(((g2 >= 0) & (g2 < 512)).all())
    with pytest.raises(ValueError):
        decoding.GraphDecoder(fast, batch, 100).set_sampling(1.0, 1.5)
