"""GPU parity: top-k / top-p logit filtering through the C ABI vs the oracle.

The kept set is compared exactly.  The top-p cut-off compares a cumulative probability with p; the
kernel sums it in fp32, the oracle in fp64, so a row is only compared when no cumulative probability
of its distinct values lies within 2e-5 of p (almost every row: the tests assert how many)."""
import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu


def _f64(t):
    return t.detach().cpu().to(torch.float64).numpy()


def _decided_rows(x, keep_k, p, T):
    """Rows of x (fp64 [rows, V]; keep_k = what top-k left) whose top-p cut-off does not hinge on rounding."""
    ok = np.ones(x.shape[0], dtype=bool)
    if p >= 1.0:
        return ok
    for r in range(x.shape[0]):
        v = x[r][keep_k[r]] / T[r]
        if v.size == 0 or not np.isfinite(v.max()):       # nothing finite in the row: no softmax, left alone
            continue
        vals, counts = np.unique(v, return_counts=True)
        mass = counts * np.exp(vals - vals[-1])
        cum = np.cumsum(mass[::-1]) / mass.sum()
        ok[r] = np.abs(cum - p).min() > 2e-5
    return ok


def _check(dev, logits, k, p, temps=None, out=None, min_decided=0.9):
    import mdx
    rows = logits.reshape(-1, logits.shape[-1]).shape[0]
    got = mdx.filter_logits(logits.to(dev) if out is None else out, top_k=k, top_p=p,
                            temperatures=None if temps is None else temps.to(dev), out=out)
    torch.cuda.synchronize()
    x = _f64(logits).reshape(rows, -1)
    T = np.ones(rows) if temps is None else np.repeat(temps.numpy().astype(np.float64), rows // temps.numel())
    want = oracle.filter_logits(x, top_k=k, top_p=p, temperatures=T)
    g = _f64(got).reshape(rows, -1)
    decided = _decided_rows(x, np.isfinite(oracle.filter_logits(x, top_k=k)), p, T)
    assert decided.mean() >= min_decided, f"only {decided.mean():.2f} of the rows are clear of a rounding boundary"
    assert np.array_equal(g[decided], want[decided])            # -inf where dropped, the same bits elsewhere
    return got, decided


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("V", [1, 9, 257, 4096 + 5, 151936])
@pytest.mark.parametrize("k,p", [(50, 1.0), (0, 0.9), (20, 0.8), (1, 1.0), (0, 0.0), (0, 0.2)])
def test_filter_shapes(dev, dtype, V, k, p):
    g = torch.Generator().manual_seed(V + k)
    logits = (torch.randn(3, 4, V, generator=g) * 3).to(dtype)
    _check(dev, logits, k, p)


def test_filter_temperatures_per_sequence(dev):
    g = torch.Generator().manual_seed(2)
    logits = (torch.randn(4, 8, 30011, generator=g) * 2.5).bfloat16()
    temps = torch.tensor([0.5, 1.0, 1.7, 0.9])
    _, decided = _check(dev, logits, 0, 0.85, temps)
    _check(dev, logits, 100, 0.6, temps)
    # colder sequences keep fewer elements
    import mdx
    kept = torch.isfinite(mdx.filter_logits(logits.to(dev), top_p=0.85, temperatures=temps.to(dev)).float()).sum(-1).float().mean(-1).cpu()
    assert kept[0] < kept[1] < kept[2]


def test_filter_in_place_unaligned_rows_and_existing_minus_inf(dev):
    """Rows that start off a 16-byte boundary, input and output aligned differently, out == logits, and
    rows that already hold -inf (kept at -inf; an all -inf row is left alone)."""
    import mdx
    g = torch.Generator().manual_seed(5)
    V, stride = 3001, 3003
    buf = (torch.randn(10, stride, generator=g) * 3).bfloat16()
    buf[2, :V:3] = float("-inf")
    buf[7, :] = float("-inf")
    logits = buf[:, :V]                                           # row stride 3003: every row starts elsewhere mod 16
    x = _f64(logits)
    want = oracle.filter_logits(x, top_k=64, top_p=0.95)
    decided = _decided_rows(x, np.isfinite(oracle.filter_logits(x, top_k=64)), 0.95, np.ones(10))
    assert decided.sum() >= 9
    d = buf.to(dev)
    out_other = torch.empty(10, V + 1, dtype=torch.bfloat16, device=dev)[:, 1:]     # another alignment than the input's
    got = mdx.filter_logits(d[:, :V], top_k=64, top_p=0.95, out=out_other)
    torch.cuda.synchronize()
    assert np.array_equal(_f64(got)[decided], want[decided])
    got2 = mdx.filter_logits(d[:, :V], top_k=64, top_p=0.95, out=d[:, :V])         # in place
    torch.cuda.synchronize()
    assert got2.data_ptr() == d.data_ptr()
    assert np.array_equal(_f64(d[:, :V])[decided], want[decided])
    assert np.array_equal(_f64(d[:, V:]), _f64(buf[:, V:]))                          # the padding is not touched
    assert not torch.isfinite(d[7, :V].float()).any()


def test_filter_heavy_ties_and_large_logits(dev):
    """Rows of few distinct values (ties at both cut-offs are all kept) and logits far from zero, where
    a softmax term taken relative to anything but the row maximum would underflow."""
    g = torch.Generator().manual_seed(8)
    few = torch.randint(-3, 4, (6, 5000), generator=g).to(torch.bfloat16)
    _check(dev, few, 10, 1.0)
    _check(dev, few, 0, 0.5, min_decided=0.5)
    big = (torch.randn(6, 20000, generator=g) * 2 + 150).bfloat16()
    _check(dev, big, 0, 0.9, min_decided=0.5)
    neg = (torch.randn(6, 20000, generator=g) * 2 - 300).to(torch.float16)
    _check(dev, neg, 30, 0.7, min_decided=0.5)


def test_filtered_sampling_matches_oracle_end_to_end(dev):
    """filter -> confidence_argmax with Gumbel noise == the oracle's confidence on the oracle's filtered
    logits: the picked token is always one that survived, its probability is the filtered softmax's."""
    import mdx
    g = torch.Generator().manual_seed(13)
    V = 151936
    logits = (torch.randn(2, 8, V, generator=g) * 3).bfloat16()
    u = torch.rand(2, 8, V, generator=g).clamp_(1e-10, 1 - 1e-10)
    noise = -torch.log(-torch.log(u))
    temps = torch.tensor([0.8, 1.2])
    f, decided = _check(dev, logits, 50, 0.9, temps)
    x0, p = mdx.confidence_argmax(f, temps.to(dev), noise.to(dev))
    torch.cuda.synchronize()
    want = oracle.filter_logits(_f64(logits).reshape(16, V), top_k=50, top_p=0.9, temperatures=np.repeat(temps.numpy().astype(np.float64), 8))
    ex0, ep = oracle.confidence_argmax(want.reshape(2, 8, V), temps.numpy(), noise.numpy())
    d = decided.reshape(2, 8)
    assert np.array_equal(x0.cpu().numpy()[d], ex0[d])
    np.testing.assert_allclose(p.cpu().numpy()[d], ep[d], rtol=2e-5)
    assert np.all(np.isfinite(want.reshape(2, 8, V)[np.arange(2)[:, None], np.arange(8)[None], ex0]))


def test_filter_rejects_fp32_and_bad_arguments(dev):
    import mdx
    x = torch.randn(2, 100, device=dev)
    with pytest.raises(mdx.MdxError):
        mdx.filter_logits(x, top_k=5)
    with pytest.raises(mdx.MdxError):
        mdx.filter_logits(x.bfloat16(), top_k=-1)
    with pytest.raises(mdx.MdxError):
        mdx.filter_logits(x.bfloat16(), top_p=float("nan"))
    same = mdx.filter_logits(x.bfloat16())                                            # both filters off: a copy
    assert torch.equal(same, x.bfloat16())


def test_unmask_step_with_filters(dev):
    """The whole step with the HF variant's sampling arguments (temperature, top-k, top-p, Gumbel noise)."""
    import mdx
    g = torch.Generator().manual_seed(21)
    V, MASK = 50021, 50000
    logits = (torch.randn(3, 16, V, generator=g) * 3).bfloat16()
    noise = -torch.log(-torch.log(torch.rand(3, 16, V, generator=g).clamp_(1e-10, 1 - 1e-10)))
    temps = torch.tensor([0.7, 1.0, 1.4])
    tokens = torch.where(torch.rand(3, 16, generator=g) < 0.7, torch.tensor(MASK), torch.randint(0, V, (3, 16), generator=g))
    T = np.repeat(temps.numpy().astype(np.float64), 16)
    x = _f64(logits).reshape(48, V)
    decided = _decided_rows(x, np.isfinite(oracle.filter_logits(x, top_k=40)), 0.9, T)
    assert decided.all()
    want = oracle.filter_logits(x, top_k=40, top_p=0.9, temperatures=T).reshape(3, 16, V)
    ex0, ep, etr, etok = oracle.unmask_step(want, tokens.numpy(), MASK, 0.5, 2, temps.numpy(), noise.numpy())
    d_tokens = tokens.clone().to(dev)
    x0, p, tr, cnt = mdx.unmask_step(logits.to(dev), d_tokens, MASK, 0.5, 2, temps.to(dev), noise.to(dev), top_k=40, top_p=0.9)
    torch.cuda.synchronize()
    assert np.array_equal(x0.cpu().numpy(), ex0)
    np.testing.assert_allclose(p.cpu().numpy(), ep, rtol=2e-5)
    assert np.array_equal(tr.cpu().numpy(), etr) and np.array_equal(d_tokens.cpu().numpy(), etok)
