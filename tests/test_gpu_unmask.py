"""GPU parity: the unmask step through the C ABI vs the oracle.
x0 / transfer / tokens / count are compared bit-exactly, x0_p to 1e-5 relative."""
import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu
MASK_ID = 151669


def _f64(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().to(torch.float64).numpy()


def _check_conf(dev, logits, temps=None, noise=None, rtol=2e-5):
    import mdx
    x0, p = mdx.confidence_argmax(logits.to(dev), None if temps is None else temps.to(dev),
                                  None if noise is None else noise.to(dev))
    torch.cuda.synchronize()
    ex0, ep = oracle.confidence_argmax(_f64(logits), None if temps is None else temps.numpy(),
                                       None if noise is None else noise.numpy())
    assert np.array_equal(x0.cpu().numpy(), ex0)
    np.testing.assert_allclose(p.cpu().numpy(), ep, rtol=rtol, atol=1e-30)
    return x0, p


@pytest.mark.parametrize("V", [1, 7, 8, 64, 1000, 2048 + 3, 151936])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_confidence_argmax_shapes(dev, V, dtype):
    g = torch.Generator().manual_seed(V)
    logits = (torch.randn(2, 5, V, generator=g) * 3).to(dtype)
    _check_conf(dev, logits)


def test_confidence_many_rows_single_split(dev):
    g = torch.Generator().manual_seed(9)
    logits = (torch.randn(64, 32, 4096, generator=g) * 3).bfloat16()   # 2048 rows -> one split per row
    _check_conf(dev, logits)


def test_confidence_ties_pick_first_index(dev):
    g = torch.Generator().manual_seed(3)
    logits = (torch.randn(4, 32, 151936, generator=g) * 3).bfloat16()
    tied = int((logits == logits.amax(-1, keepdim=True)).sum(-1).gt(1).sum())
    assert tied > 0, "bf16 N(0,9) rows of this length are expected to contain tied maxima"
    _check_conf(dev, logits)
    flat = torch.zeros(1, 3, 5000).bfloat16()              # everything tied
    x0, p = _check_conf(dev, flat)
    assert x0.abs().sum().item() == 0


def test_confidence_unaligned_rows(dev):
    """Rows that start off a 16-byte boundary (row stride not a multiple of 8 elements)."""
    import mdx
    g = torch.Generator().manual_seed(11)
    V, stride = 3001, 3003
    buf = (torch.randn(12, stride, generator=g) * 3).bfloat16()
    dbuf = buf.to(dev)
    view = dbuf[:, 1:1 + V]
    assert view.stride(0) == stride and view.data_ptr() % 16 != 0
    L = mdx.lib()
    x0 = torch.empty(12, dtype=torch.int64, device=dev)
    p = torch.empty(12, dtype=torch.float32, device=dev)
    ws_bytes = L.mdx_confidence_argmax_workspace_bytes(12, V)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
    rc = L.mdx_confidence_argmax(view.data_ptr(), stride, 0, None, 1, None, 0, x0.data_ptr(), p.data_ptr(),
                                 12, V, ws.data_ptr(), ws_bytes, torch.cuda.current_stream().cuda_stream)
    assert rc == 0, L.mdx_last_error()
    torch.cuda.synchronize()
    ex0, ep = oracle.confidence_argmax(_f64(buf[:, 1:1 + V]).reshape(12, 1, V))
    assert np.array_equal(x0.cpu().numpy(), ex0[:, 0])
    np.testing.assert_allclose(p.cpu().numpy(), ep[:, 0], rtol=2e-5)


def test_confidence_temperature_and_noise(dev):
    g = torch.Generator().manual_seed(21)
    logits = (torch.randn(3, 4, 5003, generator=g) * 3).bfloat16()
    temps = torch.tensor([0.5, 1.0, 2.5])
    _check_conf(dev, logits, temps)
    gumbel = -torch.empty(3, 4, 5003).exponential_(generator=g).log()
    x0, _ = _check_conf(dev, logits, temps, gumbel)
    assert not np.array_equal(x0.cpu().numpy(), logits.float().argmax(-1).numpy())   # noise moved some picks


def _tokens(g, bs, S, lo=0.5):
    tok = torch.randint(0, 1000, (bs, S), generator=g, dtype=torch.int64)
    for b in range(bs):
        n = int(torch.randint(int(lo * S), S + 1, (1,), generator=g))
        tok[b, torch.randperm(S, generator=g)[:n]] = MASK_ID
    return tok


def _check_step(dev, logits, tokens, thr, k, temps=None):
    import mdx
    dtok = tokens.clone().to(dev)
    x0, p, transfer, count = mdx.unmask_step(logits.to(dev), dtok, MASK_ID, thr, k,
                                             temperatures=None if temps is None else temps.to(dev))
    torch.cuda.synchronize()
    ex0, ep, etr, etok = oracle.unmask_step(_f64(logits), tokens.numpy(), MASK_ID, thr, k,
                                            None if temps is None else temps.numpy())
    # the fixture must not sit on a decision boundary the fp32/fp64 difference could flip
    conf = np.where(tokens.numpy() == MASK_ID, ep, -np.inf)
    assert np.abs(conf[np.isfinite(conf)] - thr).min() > 1e-4
    for b in range(conf.shape[0]):
        c = np.sort(conf[b][np.isfinite(conf[b])])[::-1]
        if (c > thr).sum() < k < len(c):
            assert c[k - 1] - c[k] > 1e-6 * c[k - 1]
    assert np.array_equal(x0.cpu().numpy(), ex0)
    assert np.array_equal(transfer.cpu().numpy(), etr)
    assert np.array_equal(dtok.cpu().numpy(), etok)
    assert np.array_equal(count.cpu().numpy(), etr.sum(-1))
    return etr


@pytest.mark.parametrize("k", [1, 4])
def test_unmask_topk_branch(dev, k):
    g = torch.Generator().manual_seed(100 + k)
    logits = (torch.randn(6, 32, 20011, generator=g) * 3).bfloat16()     # flat rows: confidence << 0.9
    etr = _check_step(dev, logits, _tokens(g, 6, 32), 0.9, k)
    assert (etr.sum(-1) == k).all()


@pytest.mark.parametrize("k", [1, 4])
def test_unmask_threshold_branch(dev, k):
    g = torch.Generator().manual_seed(200 + k)
    logits = (torch.randn(6, 32, 20011, generator=g) * 3).bfloat16()
    hot = torch.randint(0, 20011, (6, 32), generator=g)
    n_hot = [0, 1, 3, 4, 9, 32]                       # rows with fewer than k peaked positions fall back to top-k
    for b in range(6):
        for p_ in torch.randperm(32, generator=g)[:n_hot[b]].tolist():
            logits[b, p_, hot[b, p_]] += 40.0
    tokens = torch.full((6, 32), MASK_ID, dtype=torch.int64)
    etr = _check_step(dev, logits, tokens, 0.9, k)
    for b in range(6):
        assert etr[b].sum() == (n_hot[b] if n_hot[b] >= k else k)


def test_unmask_fewer_masked_than_k_and_none(dev):
    g = torch.Generator().manual_seed(7)
    logits = (torch.randn(3, 32, 4099, generator=g) * 3).bfloat16()
    tokens = torch.randint(0, 1000, (3, 32), generator=g, dtype=torch.int64)
    tokens[0, 5] = MASK_ID                            # 1 masked, k = 4 -> commits exactly that one
    tokens[1, [2, 30]] = MASK_ID                      # 2 masked
    etr = _check_step(dev, logits, tokens, 0.9, 4)    # row 2: nothing masked -> nothing committed
    assert etr.sum(-1).tolist() == [1, 2, 0]


@pytest.mark.parametrize("S", [32, 100])
def test_select_never_commits_a_position_without_a_confidence(dev, S):
    """A masked position whose confidence is -inf (a caller's mark for "no fresh logits") stays masked and does
    not use up one of the k places: wavefront kernel (S <= 64) and workgroup kernel."""
    import mdx
    g = torch.Generator().manual_seed(S)
    bs = 5
    conf = torch.rand(bs, S, generator=g)
    conf[torch.rand(bs, S, generator=g) < 0.4] = float("-inf")
    conf[4] = float("-inf")                                                       # a sequence with no confidence at all
    x0 = torch.randint(0, 1000, (bs, S), generator=g)
    tokens = torch.where(torch.rand(bs, S, generator=g) < 0.7, torch.tensor(MASK_ID), torch.randint(0, 1000, (bs, S), generator=g))
    for thr, k in ((0.5, 3), (2.0, 6), (2.0, S)):
        dtok = tokens.clone().to(dev)
        tr, cnt = mdx.select_transfer(x0.to(dev), conf.to(dev), dtok, MASK_ID, thr, k)
        torch.cuda.synchronize()
        want = oracle.select_transfer(conf.numpy(), tokens.numpy() == MASK_ID, thr, k)
        assert np.array_equal(tr.cpu().numpy(), want)
        assert not (tr.cpu() & torch.isinf(conf)).any() and int(cnt[4]) == 0
        assert np.array_equal(dtok.cpu().numpy(), np.where(want, x0.numpy(), tokens.numpy()))


def test_k_zero_commits_the_positions_above_the_threshold_only(dev):
    """The HF schedule gives k = 0 to the late steps of a block with fewer positions than steps: hi.sum() >= 0 always
    holds, so exactly the positions above the threshold are committed (modeling_mineru_diffusion.py:526-529)."""
    import mdx
    g = torch.Generator().manual_seed(12)
    conf = torch.rand(4, 32, generator=g)
    x0 = torch.randint(0, 1000, (4, 32), generator=g)
    tokens = torch.where(torch.rand(4, 32, generator=g) < 0.6, torch.tensor(MASK_ID), torch.randint(0, 1000, (4, 32), generator=g))
    dtok = tokens.clone().to(dev)
    tr, cnt = mdx.select_transfer(x0.to(dev), conf.to(dev), dtok, MASK_ID, 0.7, 0)
    torch.cuda.synchronize()
    want = oracle.select_transfer(conf.numpy(), tokens.numpy() == MASK_ID, 0.7, 0)
    assert np.array_equal(want, (tokens.numpy() == MASK_ID) & (conf.numpy() > 0.7))
    assert np.array_equal(tr.cpu().numpy(), want) and cnt.cpu().tolist() == want.sum(1).tolist()
    tr2, cnt2 = mdx.select_transfer(x0.to(dev), conf.to(dev), tokens.clone().to(dev), MASK_ID, 2.0, 0)
    assert not tr2.any() and int(cnt2.sum()) == 0


def test_unmask_block_lengths(dev):
    g = torch.Generator().manual_seed(8)
    for S in (1, 4, 33, 64, 128):
        logits = (torch.randn(2, S, 1031, generator=g) * 3).bfloat16()
        tokens = torch.full((2, S), MASK_ID, dtype=torch.int64)
        _check_step(dev, logits, tokens, 0.9, min(4, S), temps=torch.tensor([0.7, 1.3]))


def test_unmask_full_size(dev):
    """benchmark config 4: [32 x 32 x 151936] bf16 N(0, 3^2), 50-100 % masked, k = 4, thr 0.9.
    The oracle runs on every 8th row's softmax in fp64; argmax is checked on all rows."""
    import mdx
    g = torch.Generator().manual_seed(4)
    logits = torch.empty(32, 32, 151936, dtype=torch.bfloat16)
    for b in range(32):
        logits[b] = (torch.randn(32, 151936, generator=g) * 3).bfloat16()
    tokens = _tokens(g, 32, 32)
    dtok = tokens.clone().to(dev)
    x0, p, transfer, count = mdx.unmask_step(logits.to(dev), dtok, MASK_ID, 0.9, 4)
    torch.cuda.synchronize()
    ex0 = logits.float().argmax(-1)                   # torch.argmax: first index on ties
    assert torch.equal(x0.cpu(), ex0)
    rows = logits[::8].to(torch.float64)
    ep = torch.softmax(rows, -1).gather(-1, ex0[::8].unsqueeze(-1)).squeeze(-1)
    np.testing.assert_allclose(p.cpu()[::8].numpy(), ep.numpy(), rtol=2e-5)
    etr = oracle.select_transfer(p.cpu().numpy(), (tokens == MASK_ID).numpy(), 0.9, 4)
    assert np.array_equal(transfer.cpu().numpy(), etr)
    assert np.array_equal(dtok.cpu().numpy(), np.where(etr, ex0.numpy(), tokens.numpy()))
    assert (count.cpu().numpy() == 4).all()


def test_confidence_extreme_logits(dev):
    """Large magnitudes (the bf16 range allows them), -inf entries (a masked-out vocabulary slice)
    and a row whose maximum sits in the last, unaligned elements."""
    g = torch.Generator().manual_seed(41)
    logits = (torch.randn(3, 4, 5003, generator=g) * 3)
    logits[0] *= 1000.0                                     # differences of thousands: one-hot softmax
    logits[1, :, 100:2000] = float("-inf")
    logits[2, 0, -1] = 50.0
    logits[2, 1, 0] = 50.0
    logits[2, 2, 5001] = 50.0
    x0, p = _check_conf(dev, logits.bfloat16())
    assert x0[2, 0].item() == 5002 and x0[2, 1].item() == 0 and x0[2, 2].item() == 5001
    assert torch.isfinite(p).all() and (p > 0).all() and (p <= 1).all()
    # With a temperature the reference rounds logits / T to fp32 before the softmax (sampler.py:13) and
    # so does the oracle; at |logits / T| of 10^4..10^5 that rounding alone moves a probability by up
    # to a percent, while the kernel scales the exact difference to the maximum: the argmax must
    # still agree exactly, the probability within that rounding.
    _check_conf(dev, logits.bfloat16(), temps=torch.tensor([0.05, 1.0, 7.0]), rtol=3e-2)


def test_rows_without_a_finite_logit_are_never_committed(dev):
    """A row of -inf logits has no softmax: token 0 with confidence 0, with and without noise and
    through the split-row path, so neither selection rule can pick it over a real candidate."""
    import mdx
    g = torch.Generator().manual_seed(17)
    logits = (torch.randn(1, 4, 151936, generator=g) * 3).bfloat16()
    logits[0, 1] = float("-inf")
    logits[0, 3, 5:] = float("-inf")                      # a row with a few finite entries is an ordinary row
    x0, p = mdx.confidence_argmax(logits.to(dev))
    ex0, ep = oracle.confidence_argmax(_f64(logits[:, [0, 2, 3]]))
    assert np.array_equal(x0.cpu().numpy()[:, [0, 2, 3]], ex0)
    np.testing.assert_allclose(p.cpu().numpy()[:, [0, 2, 3]], ep, rtol=2e-5)
    assert x0[0, 1].item() == 0 and p[0, 1].item() == 0.0
    noise = torch.zeros(1, 4, 151936)
    x0n, pn = mdx.confidence_argmax(logits.to(dev), None, noise.to(dev))
    assert x0n[0, 1].item() == 0 and pn[0, 1].item() == 0.0
    tokens = torch.full((1, 4), MASK_ID, dtype=torch.int64, device=dev)
    _, _, transfer, count = mdx.unmask_step(logits.to(dev), tokens, MASK_ID, 0.9, 3)
    assert transfer.cpu().tolist() == [[True, False, True, True]] and int(count[0]) == 3
