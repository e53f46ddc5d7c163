"""Pins the attention oracle by closed forms, a second independent formula, library
routines and brute force (the reference ships no fixtures for this path)."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle


def test_mask_hand_written_case():
    # L = 7, S = 3: padded length 9, pad 2 -> blocks {0}, {1,2,3}, {4,5,6}
    expect = np.array([
        [1, 0, 0, 0, 0, 0, 0],
        [1, 1, 1, 1, 0, 0, 0],
        [1, 1, 1, 1, 0, 0, 0],
        [1, 1, 1, 1, 0, 0, 0],
        [1, 1, 1, 1, 1, 1, 1],
        [1, 1, 1, 1, 1, 1, 1],
        [1, 1, 1, 1, 1, 1, 1]], dtype=bool)
    assert np.array_equal(oracle.staircase_mask(7, 3), expect)
    assert np.array_equal(oracle.staircase_mask_tril(7, 3), expect)


@pytest.mark.parametrize("S", [1, 2, 4, 8, 16, 32, 64, 128])
def test_mask_two_formulas_agree_for_every_length(S):
    for L in range(1, 200):
        a, b = oracle.staircase_mask(L, S), oracle.staircase_mask_tril(L, S)
        assert np.array_equal(a, b), (L, S)
        assert a.sum() == oracle.staircase_pairs(L, S)


def test_mask_limits_and_right_alignment():
    for L in (1, 5, 33, 100):
        assert np.array_equal(oracle.staircase_mask(L, 1), np.tril(np.ones((L, L), bool)))     # S=1: causal
        assert oracle.staircase_mask(L, 128).all() == (L <= 128)                                # S>=L: full
    m = oracle.staircase_mask(70, 32)            # blocks of 6, 32, 32: the SHORT block comes first
    assert m[0, :6].all() and not m[0, 6:].any()
    assert m[6, :38].all() and not m[6, 38:].any()
    assert m[-1].all()
    left_aligned = (np.arange(70)[:, None] // 32) >= (np.arange(70)[None, :] // 32)
    assert not np.array_equal(m, left_aligned)   # the tempting left-aligned formula is a different mask


def test_pairs_closed_form_on_multiples():
    for S in (4, 32):
        for nb in (1, 2, 7, 256):
            L = nb * S
            assert oracle.staircase_pairs(L, S) == L * (L + S) // 2
    assert oracle.staircase_pairs(0, 32) == 0


def test_sdpa_matches_explicit_fp64_loops():
    g = torch.Generator().manual_seed(0)
    q = torch.randn(9, 4, 16, generator=g)
    k = torch.randn(9, 2, 16, generator=g)
    v = torch.randn(9, 2, 16, generator=g)
    mask = oracle.staircase_mask(9, 4)
    got = oracle.masked_attention_f32(q, k, v, mask, 0.25).numpy()
    want = oracle.attention_f64_explicit(q.numpy(), k.numpy(), v.numpy(), mask, 0.25)
    np.testing.assert_allclose(got, want, atol=2e-6)
    # a transposed mask or a dropped scale must fail this check
    bad = oracle.masked_attention_f32(q, k, v, mask.T | np.eye(9, dtype=bool), 0.25).numpy()
    assert np.abs(bad - want).max() > 1e-3
    assert np.abs(oracle.masked_attention_f32(q, k, v, mask, 1.0).numpy() - want).max() > 1e-3


def test_gqa_equals_mha_with_duplicated_kv_heads():
    g = torch.Generator().manual_seed(1)
    q = torch.randn(40, 6, 32, generator=g)
    k = torch.randn(40, 2, 32, generator=g)
    v = torch.randn(40, 2, 32, generator=g)
    mask = oracle.staircase_mask(40, 8)
    a = oracle.masked_attention_f32(q, k, v, mask, 0.2)
    b = oracle.masked_attention_f32(q, k.repeat_interleave(3, 1), v.repeat_interleave(3, 1), mask, 0.2)
    assert torch.allclose(a, b, atol=1e-6)            # kv head = q head // (Hq/Hkv)


def test_varlen_special_cases_reduce_to_library_attention():
    g = torch.Generator().manual_seed(2)
    lens = [37, 5, 64]
    N = sum(lens)
    q, k, v = (torch.randn(N, 4, 32, generator=g) for _ in range(3))
    cu = np.concatenate([[0], np.cumsum(lens)])
    causal = oracle.staircase_attn_varlen(q, k, v, cu, 1)
    full = oracle.staircase_attn_varlen(q, k, v, cu, 128)
    for b in range(3):
        s, e = cu[b], cu[b + 1]
        qq, kk, vv = (t[s:e].permute(1, 0, 2)[None] for t in (q, k, v))
        assert torch.allclose(causal[s:e], F.scaled_dot_product_attention(qq, kk, vv, is_causal=True)[0].permute(1, 0, 2), atol=1e-5)
        assert torch.allclose(full[s:e], F.scaled_dot_product_attention(qq, kk, vv)[0].permute(1, 0, 2), atol=1e-5)


def test_block_outputs_do_not_depend_on_later_blocks():
    g = torch.Generator().manual_seed(3)
    L, S = 75, 16                                  # blocks 11, 16, 16, 16, 16
    q, k, v = (torch.randn(L, 2, 16, generator=g) for _ in range(3))
    o1 = oracle.staircase_attn_varlen(q, k, v, [0, L], S)
    k2, v2 = k.clone(), v.clone()
    k2[43:] += 1.0
    v2[43:] -= 2.0
    o2 = oracle.staircase_attn_varlen(q, k2, v2, [0, L], S)
    assert torch.equal(o1[:43], o2[:43]) and not torch.allclose(o1[43:], o2[43:])


def test_paged_equals_contiguous_and_ignores_placement():
    g = torch.Generator().manual_seed(4)
    page, hkv, d = 16, 2, 8
    ctxs = [40, 0, 16, 17]
    kcont = [torch.randn(c, hkv, d, generator=g) for c in ctxs]
    vcont = [torch.randn(c, hkv, d, generator=g) for c in ctxs]
    pool = 12
    kc, vc = torch.randn(pool, page, hkv, d, generator=g), torch.randn(pool, page, hkv, d, generator=g)
    perm = torch.randperm(pool, generator=g).tolist()
    bt = torch.full((4, 3), -1, dtype=torch.int32)
    for b, c in enumerate(ctxs):
        for i in range((c + page - 1) // page):
            pg = perm.pop()
            bt[b, i] = pg
            n = min(page, c - i * page)
            kc[pg, :n] = kcont[b][i * page:i * page + n]
            vc[pg, :n] = vcont[b][i * page:i * page + n]
    q = torch.randn(4, 5, 4, d, generator=g)
    got = oracle.paged_block_attn(q, kc, vc, bt, ctxs, 0.3)
    for b, c in enumerate(ctxs):
        if c == 0:
            assert got[b].abs().sum() == 0
            continue
        assert torch.equal(oracle.paged_gather(kc, bt[b], c), kcont[b])
        want = oracle.masked_attention_f32(q[b], kcont[b], vcont[b], None, 0.3)
        assert torch.allclose(got[b], want, atol=1e-6)


def test_config1_anchor():
    """benchmark config 1: B=1, prefix 1024 + block 32, Hq 16, Hkv 8, d 128, fp32; the block's
    rows of the staircase mask are all True and the op equals unmasked SDPA; 276.8 MFLOP."""
    g = torch.Generator().manual_seed(1)
    L = 1056
    q = torch.randn(32, 16, 128, generator=g)
    k, v = torch.randn(L, 8, 128, generator=g), torch.randn(L, 8, 128, generator=g)
    band = oracle.staircase_mask(L, 32)[-32:]
    assert band.all()
    o = oracle.masked_attention_f32(q, k, v, band, 1 / math.sqrt(128))
    p_rows = torch.softmax(torch.einsum("qhd,khd->hqk", q, k.repeat_interleave(2, 1)) / math.sqrt(128), -1)
    assert torch.allclose(p_rows.sum(-1), torch.ones(16, 32), atol=1e-5)
    want = torch.einsum("hqk,khd->qhd", p_rows, v.repeat_interleave(2, 1))
    assert torch.allclose(o, want, atol=1e-5)
    assert 4 * 32 * L * 128 * 16 == 276_824_064
