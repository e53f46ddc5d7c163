"""Pins the KV-store, unmask and slot oracles against library routines and brute force."""
import itertools

import numpy as np
import pytest
import torch

import oracle


def test_store_matches_index_copy_and_leaves_the_rest():
    g = torch.Generator().manual_seed(0)
    N, hkv, d, pages, page = 50, 2, 8, 4, 32
    key = torch.randn(N, hkv, d, generator=g)
    val = torch.randn(N, hkv, d, generator=g)
    kc0, vc0 = torch.randn(pages, page, hkv, d, generator=g), torch.randn(pages, page, hkv, d, generator=g)
    slots = torch.randperm(pages * page, generator=g)[:N].to(torch.int32)
    slots[::7] = -1
    kc, vc = kc0.clone().numpy(), vc0.clone().numpy()
    oracle.store_kvcache(key.numpy(), val.numpy(), kc, vc, slots.numpy())
    keep = slots >= 0
    want_k = kc0.clone().view(-1, hkv * d).index_copy_(0, slots[keep].long(), key.view(N, -1)[keep])
    want_v = vc0.clone().view(-1, hkv * d).index_copy_(0, slots[keep].long(), val.view(N, -1)[keep])
    assert np.array_equal(kc.reshape(-1, hkv * d), want_k.numpy())
    assert np.array_equal(vc.reshape(-1, hkv * d), want_v.numpy())
    untouched = np.setdiff1d(np.arange(pages * page), slots[keep].numpy())
    assert np.array_equal(kc.reshape(-1, hkv * d)[untouched], kc0.view(-1, hkv * d).numpy()[untouched])


def test_store_then_gather_round_trips_through_the_page_table():
    g = torch.Generator().manual_seed(1)
    L, hkv, d, page = 70, 2, 4, 16
    table = [9, 3, 0, 5, 7]
    k = torch.randn(L, hkv, d, generator=g)
    kc, vc = np.zeros((12, page, hkv, d), np.float32), np.zeros((12, page, hkv, d), np.float32)
    oracle.store_kvcache(k.numpy(), k.numpy(), kc, vc, np.array(oracle.get_slots(table, 0, L, page)))
    assert torch.equal(oracle.paged_gather(torch.from_numpy(kc), table, L), k)


def test_slots_brute_force_and_warmup():
    table = [4, 1, 6]
    for lo, hi in [(0, 0), (0, 5), (250, 262), (0, 768), (255, 257), (256, 512), (300, 301)]:
        got = oracle.get_slots(table, lo, hi)
        want = [table[t // 256] * 256 + t % 256 for t in range(lo, hi)]
        assert got == want
    assert oracle.get_slots([], 3, 8) == [-1] * 5


def test_confidence_matches_torch_softmax_and_argmax():
    g = torch.Generator().manual_seed(2)
    logits = (torch.randn(3, 5, 777, generator=g) * 3).bfloat16()
    temps = torch.tensor([0.5, 1.0, 3.0])
    x0, p = oracle.confidence_argmax(logits.float().numpy(), temps.numpy())
    l = logits.float() / temps.view(-1, 1, 1)
    assert np.array_equal(x0, l.argmax(-1).numpy())
    want = torch.softmax(l.double(), -1).gather(-1, l.argmax(-1, keepdim=True)).squeeze(-1)
    np.testing.assert_allclose(p, want.numpy(), rtol=1e-12)
    # conf of the argmax without noise is 1 / sum exp(l - max)
    np.testing.assert_allclose(p, 1 / torch.exp(l.double() - l.double().amax(-1, keepdim=True)).sum(-1).numpy(), rtol=1e-12)


def test_confidence_ties_take_the_first_index_and_noise_moves_the_pick():
    logits = np.zeros((1, 2, 10), np.float32)
    logits[0, 0, [3, 7]] = 5.0
    x0, p = oracle.confidence_argmax(logits)
    assert x0.tolist() == [[3, 0]]
    assert torch.argmax(torch.from_numpy(logits), -1).tolist() == [[3, 0]]
    noise = np.zeros_like(logits)
    noise[0, 0, 8] = 100.0
    x0n, pn = oracle.confidence_argmax(logits, None, noise)
    assert x0n[0, 0] == 8
    want = np.exp(0.0 - 5.0) / (2 + 8 * np.exp(-5.0))          # softmax WITHOUT the noise, at the noisy pick
    np.testing.assert_allclose(pn[0, 0], want, rtol=1e-12)


def test_num_transfer_tokens():
    assert oracle.num_transfer_tokens(32, 8) == [4] * 8
    assert oracle.num_transfer_tokens(32, 32) == [1] * 32
    assert oracle.num_transfer_tokens(10, 4) == [3, 3, 2, 2]


def _select_by_library(conf, masked, thr, k):
    """The reference rule spelled with torch.topk (valid when there are no ties and >= k masked)."""
    c = torch.where(torch.from_numpy(masked), torch.from_numpy(conf), torch.tensor(-torch.inf))
    out = torch.zeros_like(c, dtype=torch.bool)
    for b in range(c.shape[0]):
        hi = c[b] > thr
        if hi.sum() >= k:
            out[b] = hi
        else:
            out[b, torch.topk(c[b], k).indices] = True
    return out.numpy()


@pytest.mark.parametrize("k", [1, 2, 4])
def test_select_matches_topk_rule_on_tie_free_inputs(k):
    rng = np.random.default_rng(k)
    for trial in range(50):
        conf = rng.random((4, 32)).astype(np.float32)          # distinct with probability 1
        conf[0] *= 0.5                                         # row 0: nothing above 0.9
        conf[1, :6] = 0.95 + 0.001 * np.arange(6)              # row 1: 6 above
        masked = rng.random((4, 32)) < 0.7
        masked[:, :8] = True                                   # at least 8 masked: topk never reaches -inf
        got = oracle.select_transfer(conf, masked, 0.9, k)
        assert np.array_equal(got, _select_by_library(conf, masked, 0.9, k))
        assert not (got & ~masked).any()


def test_select_brute_force_over_all_masks_on_six_positions():
    conf = np.array([[0.95, 0.2, 0.91, 0.5, 0.7, 0.1]], np.float32)
    for bits in itertools.product([False, True], repeat=6):
        masked = np.array([bits])
        for k in (1, 2, 3):
            got = oracle.select_transfer(conf, masked, 0.9, k)[0]
            idx = [i for i in range(6) if bits[i]]
            hi = [i for i in idx if conf[0, i] > 0.9]
            want = set(hi) if len(hi) >= k else set(sorted(idx, key=lambda i: -conf[0, i])[:k])
            assert set(np.flatnonzero(got)) == want


def test_select_strict_threshold_ties_and_engine_rule():
    conf = np.array([[0.9, 0.9, 0.3, 0.3]], np.float32)
    masked = np.ones((1, 4), bool)
    # strict '>' : 0.9 is not above the 0.9 threshold -> top-k; equal values: lower position first
    assert oracle.select_transfer(conf, masked, np.float32(0.9), 1).tolist() == [[True, False, False, False]]
    assert oracle.select_transfer(conf, masked, np.float32(0.9), 3).tolist() == [[True, True, True, False]]
    # engine rule = k 1: any above threshold -> all of them
    assert oracle.select_transfer(conf, masked, 0.5, 1).tolist() == [[True, True, False, False]]
    # rows without masked positions commit nothing (sampler.py:42-43)
    assert not oracle.select_transfer(conf, np.zeros((1, 4), bool), 0.5, 1).any()
    # a masked position without a confidence (-inf) is never committed, and does not use up one of the k places
    gaps = np.array([[-np.inf, 0.2, -np.inf, 0.1]], np.float32)
    assert oracle.select_transfer(gaps, masked, 0.5, 3).tolist() == [[False, True, False, True]]
    assert not oracle.select_transfer(np.full((1, 4), -np.inf, np.float32), masked, 0.5, 2).any()


def test_unmask_step_end_to_end_small():
    g = torch.Generator().manual_seed(5)
    logits = (torch.randn(2, 8, 50, generator=g) * 3).numpy()
    tokens = np.full((2, 8), 99, np.int64)
    tokens[0, :3] = [1, 2, 3]
    x0, p, tr, new = oracle.unmask_step(logits, tokens, 99, 0.9, 2)
    assert (new[0, :3] == [1, 2, 3]).all() and not tr[0, :3].any()
    assert (new[tr] == x0[tr]).all() and (new[~tr] == tokens[~tr]).all()
    assert tr.sum(-1).tolist() == [2, 2] or (p > 0.9).any()


# ---- filter_logits (top-k / top-p before sampling) ----------------------------------------------

def _torch_topk_topp(logits, k, p, T=1.0):
    """The filters written with the library routines the reference composes them from (topk / where;
    sort / softmax / cumsum / scatter), in fp64."""
    x = torch.from_numpy(np.asarray(logits, dtype=np.float64)) / T
    if k > 0:
        kth = torch.topk(x, k).values[..., -1, None]
        x = torch.where(x < kth, torch.full_like(x, float("-inf")), x)
    if p < 1.0:
        srt, order = torch.sort(x, descending=True)
        drop = torch.cumsum(torch.softmax(srt, dim=-1), dim=-1) > p
        drop = torch.cat([torch.zeros_like(drop[..., :1]), drop[..., :-1]], dim=-1)
        x = x.masked_fill(torch.zeros_like(drop).scatter(-1, order, drop), float("-inf"))
    return torch.isfinite(x).numpy()


@pytest.mark.parametrize("k,p,T", [(5, 1.0, 1.0), (0, 0.9, 1.0), (0, 0.3, 0.7), (40, 0.8, 1.3), (1, 1.0, 1.0), (0, 0.0, 1.0), (200, 0.999, 1.0)])
def test_filter_matches_library_formulation_on_tie_free_rows(k, p, T):
    rng = np.random.default_rng(k * 7 + int(p * 100))
    x = rng.permutation(np.linspace(-6, 9, 6 * 257)).reshape(6, 257)          # all values distinct
    got = np.isfinite(oracle.filter_logits(x, top_k=k, top_p=p, temperatures=T))
    assert np.array_equal(got, _torch_topk_topp(x, k, p, T))
    kept = oracle.filter_logits(x, top_k=k, top_p=p, temperatures=T)
    assert np.array_equal(kept[got], x[got])                                   # survivors keep their value


def test_filter_counting_and_mass_invariants():
    rng = np.random.default_rng(4)
    x = rng.normal(0, 3, (16, 500))
    for k in (1, 7, 499):
        assert np.all(np.isfinite(oracle.filter_logits(x, top_k=k)).sum(1) == k)
    assert np.array_equal(oracle.filter_logits(x, top_k=0, top_p=1.0), x)
    assert np.array_equal(oracle.filter_logits(x, top_k=500), x)              # k >= V: nothing goes
    for p in (0.1, 0.5, 0.95):
        keep = np.isfinite(oracle.filter_logits(x, top_p=p))
        pr = np.exp(x - x.max(1, keepdims=True))
        pr /= pr.sum(1, keepdims=True)
        for r in range(16):
            mass = pr[r][keep[r]].sum()
            assert mass > p and mass - pr[r][keep[r]].min() <= p               # minimal prefix that exceeds p
            assert pr[r][keep[r]].min() > pr[r][~keep[r]].max()                # and it is a prefix


def test_filter_brute_force_and_ties():
    x = np.array([[2.0, -1.0, 0.5, 3.0, 0.0, 1.5, -2.0, 2.5]])
    pr = np.exp(x[0]) / np.exp(x[0]).sum()
    order = np.argsort(-x[0])
    for p in np.linspace(0.01, 0.99, 50):
        n = 1
        while pr[order[:n]].sum() <= p:
            n += 1
        want = np.zeros(8, dtype=bool)
        want[order[:n]] = True
        assert np.array_equal(np.isfinite(oracle.filter_logits(x, top_p=float(p)))[0], want)
    # top-k keeps every element equal to the k-th largest (`logits < min_values` drops none of them)
    t = np.array([[1.0, 3.0, 2.0, 2.0, 2.0, 0.0]])
    assert np.isfinite(oracle.filter_logits(t, top_k=2)).sum() == 4
    assert np.array_equal(np.isfinite(oracle.filter_logits(t, top_k=2)), _torch_topk_topp(t, 2, 1.0))
    # top-p: all elements equal to the crossing value stay (the reference's sort order would pick among them)
    assert np.isfinite(oracle.filter_logits(t, top_p=0.6)).sum() == 4
    # temperature enters the top-p probabilities: a colder row needs fewer elements
    x2 = np.linspace(0, 5, 50)[None]
    assert np.isfinite(oracle.filter_logits(x2, top_p=0.9, temperatures=0.5)).sum() < np.isfinite(oracle.filter_logits(x2, top_p=0.9, temperatures=2.0)).sum()
    # rows already holding -inf: those never come back, and an all -inf row is left alone
    y = np.array([[0.0, -np.inf, 1.0, -np.inf], [-np.inf] * 4])
    f = oracle.filter_logits(y, top_k=3, top_p=0.99)
    assert np.array_equal(np.isfinite(f), [[True, False, True, False], [False] * 4])


# ---- the counter-based generator behind the in-kernel Gumbel noise ------------------------------

def test_philox_known_answers():
    """The three known-answer vectors that the Random123 distribution ships for philox4x32 with 10 rounds
    (kat_vectors: counter words, key words -> output words)."""
    kat = [((0, 0, 0, 0), (0, 0), (0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8)),
           ((0xffffffff,) * 4, (0xffffffff,) * 2, (0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd)),
           ((0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344), (0xa4093822, 0x299f31d0), (0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1))]
    for ctr, key, want in kat:
        got = oracle.philox4x32_10([np.array([w]) for w in ctr], key)
        assert tuple(int(g[0]) for g in got) == want
    # vectorised over counters = one at a time; neighbouring counters and keys give unrelated words
    c = [np.arange(5), np.zeros(5), np.full(5, 7), np.zeros(5)]
    many = oracle.philox4x32_10(c, (1, 2))
    for i in range(5):
        one = oracle.philox4x32_10([np.array([x[i]]) for x in c], (1, 2))
        assert all(int(one[j][0]) == int(many[j][i]) for j in range(4))
    assert len({int(w) for out in many for w in out}) == 20
    assert int(oracle.philox4x32_10(c, (1, 3))[0][0]) != int(many[0][0])


def test_gumbel_noise_law_and_coordinates():
    g = oracle.gumbel_noise(64, 4099, seed=11, offset=5)
    assert g.shape == (64, 4099) and np.isfinite(g).all()
    assert -2.82 < g.min() and g.max() < 16.65                     # -ln(-ln u) for u on the 2^-23 grid inside (0, 1)
    assert abs(g.mean() - 0.5772156649) < 0.01 and abs(g.var() - np.pi ** 2 / 6) < 0.03
    # a pure function of (seed, offset, row, column): rows and offsets are separate streams, row_ids relabel rows
    assert np.array_equal(oracle.gumbel_noise(3, 50, 11, 5), g[:3, :50])
    assert not np.array_equal(oracle.gumbel_noise(3, 50, 11, 6), g[:3, :50])
    assert not np.array_equal(oracle.gumbel_noise(3, 50, 12, 5), g[:3, :50])
    assert np.array_equal(oracle.gumbel_noise(2, 50, 11, 5, row_ids=[40, 7]), g[[40, 7], :50])
    big = oracle.gumbel_noise(1, 8, seed=2 ** 40 + 3, offset=2 ** 35 + 1)            # high words of seed and offset matter
    assert not np.array_equal(big, oracle.gumbel_noise(1, 8, seed=3, offset=1))
    # Gumbel-max: argmax(l + g) is a draw from softmax(l)
    l = np.array([0.0, 1.0, 2.0, -1.0, 0.5])
    draws = (l[None, :] + oracle.gumbel_noise(40000, 5, seed=1)).argmax(1)
    freq = np.bincount(draws, minlength=5) / 40000
    want = np.exp(l) / np.exp(l).sum()
    assert np.abs(freq - want).max() < 0.01
