"""GPU parity of the fused vocabulary projection + confidence reduction (mdx_lm_head_confidence) against
the oracle's confidence_argmax on the fp32 product x @ W.T rounded to bf16 (the projection's output type in the
reference, embed_head.py:61-67), and against the two-step path (library GEMM + mdx_confidence_argmax)."""
import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu


def _reference(x, w, temps=None, rows_per_temp=1, row_ids=None):
    """fp64 softmax confidence and first argmax of bf16(x @ w.T) / T on the host."""
    logits = (x.float() @ w.float().T).bfloat16().to(torch.float64).numpy()
    T = None
    if temps is not None:
        ids = np.arange(x.shape[0]) if row_ids is None else np.asarray(row_ids)
        T = np.asarray(temps, dtype=np.float64)[ids // rows_per_temp]
    ex0, ep = oracle.confidence_argmax(logits[None] if T is None else logits[:, None, :], T)
    return ex0.reshape(-1), ep.reshape(-1), logits


def _check(x0, p, ex0, ep, logits, T=None):
    """The device sums the products in another order than the host, so a logit can land on the neighbouring bf16
    value where the exact sum sits on a rounding boundary.  A pick other than the host's is therefore accepted
    only if its logit is within one bf16 step of the host's maximum (a near-tie), and must stay rare; and a
    confidence may be off by what one such step does to a probability: exp(step / T) - 1 of itself.
    `logits` are the unscaled bf16 logits, T the rows' temperatures (default 1)."""
    x0, p = x0.cpu().numpy().reshape(-1), p.cpu().numpy().reshape(-1)
    rows = np.arange(len(x0))
    top = logits[rows, logits.argmax(-1)]
    step = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(top), 2.0 ** -100))) - 7)
    same = x0 == ex0
    assert np.all(same | (logits[rows, x0] >= top - step)), "a pick that is not a near-tie of the maximum"
    if len(x0) >= 64:
        assert same.mean() > 0.97
    T = np.ones(len(x0)) if T is None else np.asarray(T, dtype=np.float64)
    tol = np.expm1(step / T) * 1.1 + 1e-4
    rel = np.abs(p - ep) / ep
    assert np.all(rel[same] <= tol[same]), f"confidence off by {rel[same].max()}"
    return same


@pytest.mark.parametrize("rows,vocab,hidden", [(1, 128, 128), (7, 300, 256), (256, 256, 128), (257, 1000, 384), (300, 5000, 2048),
                                               (33, 151936, 2048), (1024, 2049, 256)])
def test_lm_head_confidence_matches_the_oracle(dev, rows, vocab, hidden):
    import mdx
    g = torch.Generator().manual_seed(rows + vocab)
    x = torch.randn(rows, hidden, generator=g).bfloat16()
    w = (torch.randn(vocab, hidden, generator=g) * (3.0 / hidden ** 0.5)).bfloat16()       # logits ~ N(0, 3^2)
    x0, p = mdx.lm_head_confidence(x.to(dev), w.to(dev))
    torch.cuda.synchronize()
    ex0, ep, logits = _reference(x, w)
    _check(x0, p, ex0, ep, logits)
    # and against the two-step path on the device (library GEMM output in bf16, then the vocabulary pass)
    two = torch.nn.functional.linear(x.to(dev), w.to(dev))
    tx0, tp = mdx.confidence_argmax(two.unsqueeze(0))
    same = (tx0.view(-1) == x0).float().mean().item()
    assert same > 0.9


def test_lm_head_confidence_temperatures_and_row_ids(dev):
    import mdx
    g = torch.Generator().manual_seed(5)
    bs, S, hidden, vocab = 6, 32, 256, 3000
    x_all = torch.randn(bs * S, hidden, generator=g).bfloat16()
    w = (torch.randn(vocab, hidden, generator=g) * (3.0 / hidden ** 0.5)).bfloat16()
    temps = torch.linspace(0.5, 1.6, bs)
    ids = torch.sort(torch.randperm(bs * S, generator=g)[:77]).values                  # compacted rows
    x0, p = mdx.lm_head_confidence(x_all[ids].to(dev), w.to(dev), temps.to(dev), rows_per_temp=S, row_ids=ids.to(dev))
    torch.cuda.synchronize()
    ex0, ep, logits = _reference(x_all[ids], w, temps.numpy(), S, ids.numpy())
    _check(x0, p, ex0, ep, logits, T=temps.numpy()[ids.numpy() // S])
    # all rows, no ids
    x0b, pb = mdx.lm_head_confidence(x_all.view(bs, S, hidden).to(dev), w.to(dev), temps.to(dev))
    assert x0b.shape == (bs, S) and torch.equal(x0b.view(-1)[ids.to(dev)], x0)


def test_lm_head_confidence_exact_logits(dev):
    """Inputs whose products are exact in fp32 whatever the order of the sums (small integers): the logits are the
    same numbers on both sides, so token and confidence must agree to the vocabulary pass's own tolerance, ties at
    the maximum included (first index wins)."""
    import mdx
    g = torch.Generator().manual_seed(9)
    rows, vocab, hidden = 200, 1500, 128
    x = torch.randint(-2, 3, (rows, hidden), generator=g).float().bfloat16()
    w = torch.randint(-2, 3, (vocab, hidden), generator=g).float().bfloat16()
    w[700] = w[20]                                                                       # a guaranteed tie between two columns
    x0, p = mdx.lm_head_confidence(x.to(dev), w.to(dev))
    torch.cuda.synchronize()
    ex0, ep, logits = _reference(x, w)
    assert np.abs(logits).max() < 256                                                    # exact in bf16 too
    assert np.array_equal(x0.cpu().numpy(), ex0)
    np.testing.assert_allclose(p.cpu().numpy(), ep, rtol=2e-5)
    assert (np.sort(logits, -1)[:, -1] == np.sort(logits, -1)[:, -2]).any()              # ties at the top do occur


@pytest.mark.parametrize("vocab", [1, 129, 257, 4097])
@pytest.mark.parametrize("T", [0.5, 0.77, 1.0, 1.9])
def test_lm_head_confidence_when_the_last_vocab_tile_holds_one_entry(dev, vocab, T):
    """A vocabulary that ends one entry into a 128-entry slice: every lane of that slice but one sees only entries
    beyond the end (-inf).  Their sums must be 0 whatever the temperature (the correction factor of the stand-in
    maximum overflows for some of them: 0 x inf is not 0), or the slice's record poisons the row."""
    import mdx
    g = torch.Generator().manual_seed(vocab)
    rows, hidden = 70, 256
    x = torch.randn(rows, hidden, generator=g).bfloat16()
    w = (torch.randn(vocab, hidden, generator=g) * (3.0 / hidden ** 0.5)).bfloat16()
    w[vocab - 1] = w[vocab - 1] * 2.5                                          # the lone entry of the last slice often wins
    temps = torch.full((1,), T)
    x0, p = mdx.lm_head_confidence(x.to(dev), w.to(dev), temps.to(dev))
    torch.cuda.synchronize()
    assert torch.isfinite(p).all()
    ex0, ep, logits = _reference(x, w, temps.numpy(), rows, None)
    _check(x0, p, ex0, ep, logits, T=np.full(rows, T))
    assert vocab == 1 or (x0 == vocab - 1).any()
