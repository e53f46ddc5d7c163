"""GPU parity at the benchmark configurations' REAL sizes (the other GPU tests use sizes the oracle
covers whole): the oracle is evaluated on sampled 32-row bands, whose visible keys are known in
closed form, and the bandwidth ops are compared whole.

  config 1  one block of 32 queries over a 1024-token prefix + itself (the CPU anchor's exact shape)
  config 3  8 packed sequences, 38 690 tokens, store_kvcache + staircase attention through mdx.Attention
  config 4  1024 rows x 151 936 logits: how often a selection decision sits on a rounding boundary
"""
import math

import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu
HQ, HKV, D, S, PAGE = 16, 8, 128, 32, 256


def _i16(t):
    return t.contiguous().view(torch.int16).cpu().numpy()


def _band_reference(q, k, v, L, r0, r1, scale):
    """fp32 SDPA of query rows [r0, r1) of one sequence of length L against the keys they can see, with
    the rows' slice of the explicit staircase mask (block_prefill_attention_v2.py:98-102,137-139)."""
    nb = (L + S - 1) // S
    pad = nb * S - L
    rows = np.arange(r0, r1)
    limit = np.minimum(((rows + pad) // S + 1) * S - 1 - pad, L - 1)          # last visible key per row
    n_keys = int(limit.max()) + 1
    mask = np.arange(n_keys)[None, :] <= limit[:, None]
    return oracle.masked_attention_f32(q[r0:r1], k[:n_keys], v[:n_keys], mask, scale)


def test_config3_full_size_through_attention_layer(dev):
    """bench.py's config-3 input, whole, through mdx.Attention (store + staircase attention): the KV
    cache bit for bit against the oracle's store, and 64 sampled 32-row bands per sequence (always
    including the first rows, the rows around the short first block and the last block) against
    banded fp32 SDPA, max-abs < 2e-2."""
    import bench
    import mdx
    host, g3 = bench.make_cfg3(dev)
    lens, cu = host["lens"], host["cu"]
    assert len(lens) == 8 and sum(lens) == 38690 and any(L % S for L in lens)
    N = sum(lens)
    attn = mdx.Attention(HQ, D, 1 / math.sqrt(D), HKV)
    attn.k_cache, attn.v_cache = g3["k_cache"], g3["v_cache"]
    mdx.set_context(True, g3["cu"], g3["cu"], max(lens), max(lens), g3["slots"], None, None, block_size=S)
    try:
        o = attn(g3["q"], g3["k"], g3["v"]).view(N, HQ, D)
    finally:
        mdx.reset_context()
    torch.cuda.synchronize()

    fused = host["fused"]
    hq = fused[:, :HQ * D].view(N, HQ, D)
    hk = fused[:, HQ * D:(HQ + HKV) * D].view(N, HKV, D)
    hv = fused[:, (HQ + HKV) * D:].view(N, HKV, D)
    ek = np.zeros((host["n_pages"], PAGE, HKV, D), dtype=np.int16)
    ev = np.zeros_like(ek)
    oracle.store_kvcache(_i16(hk), _i16(hv), ek, ev, host["slots"].numpy())
    assert np.array_equal(_i16(attn.k_cache), ek), "K cache differs"
    assert np.array_equal(_i16(attn.v_cache), ev), "V cache differs"
    stored = int((host["slots"] >= 0).sum())
    assert stored == N - 8 * S

    o_host = o.float().cpu()
    rng = np.random.default_rng(33)
    worst = 0.0
    for b, L in enumerate(lens):
        s0 = int(cu[b])
        first = L - (L - 1) // S * S                                  # rows of the short first block
        starts = {0, max(0, first - 16), min(first, L - S), L - S, L - 2 * S, (L // 2) // S * S}
        while len(starts) < 64:
            starts.add(int(rng.integers(0, L - S + 1)))               # bands that straddle block boundaries too
        for r0 in sorted(starts):
            ref = _band_reference(hq[s0:s0 + L], hk[s0:s0 + L], hv[s0:s0 + L], L, r0, r0 + S, 1 / math.sqrt(D))
            worst = max(worst, (o_host[s0 + r0:s0 + r0 + S] - ref).abs().max().item())
    assert worst < 2e-2, f"config 3 attention max-abs {worst}"


def test_config1_shape_bf16_against_fp32_anchor(dev):
    """Config 1's exact shape (B = 1, 1024 cached tokens + a 32-token block, Hq 16 / Hkv 8 / d 128, N(0,1)
    inputs, scale 1/sqrt(128)): the fp32 SDPA anchor with its explicit all-True [32, 1056] mask against
    (a) the paged single-block attention and (b) the last block of the staircase prefill, both bf16."""
    import mdx
    g = torch.Generator().manual_seed(1)
    L, prefix = 1056, 1024
    scale = 1 / math.sqrt(D)
    q = torch.randn(L, HQ, D, generator=g).bfloat16()
    k = torch.randn(L, HKV, D, generator=g).bfloat16()
    v = torch.randn(L, HKV, D, generator=g).bfloat16()
    anchor = oracle.masked_attention_f32(q[prefix:], k, v, np.ones((S, L), dtype=bool), scale)
    # (a) decode form: K/V in pages 3, 0, 4, 1, 2 of a 6-page pool
    table = [3, 0, 4, 1, 2]
    kc = torch.zeros(6, PAGE, HKV, D, dtype=torch.bfloat16)
    vc = torch.zeros_like(kc)
    slots = torch.tensor(oracle.get_slots(table, 0, L))
    kc.view(-1, HKV, D)[slots] = k
    vc.view(-1, HKV, D)[slots] = v
    o = mdx.flash_attn_with_kvcache(q[prefix:].unsqueeze(0).to(dev), kc.to(dev), vc.to(dev),
                                    cache_seqlens=torch.tensor([L], dtype=torch.int32, device=dev),
                                    block_table=torch.tensor([table], dtype=torch.int32, device=dev), softmax_scale=scale)
    assert (o[0].float().cpu() - anchor).abs().max().item() < 2e-2
    # (b) prefill form: the last 32 rows of the staircase attention see exactly the same keys
    cu = torch.tensor([0, L], dtype=torch.int32, device=dev)
    o2 = mdx.sparse_attn_varlen(q.to(dev), k.to(dev), v.to(dev), cu, cu, S, softmax_scale=scale)
    assert (o2[prefix:].float().cpu() - anchor).abs().max().item() < 2e-2


def test_config4_decisions_on_rounding_boundaries(dev):
    """The selection is bit-exact GIVEN the confidences; the confidences themselves are fp32 sums taken in
    another order than the oracle's fp64 ones (relative difference < 2e-5), so a decision can differ
    only where a confidence sits within that distance of the threshold, or two confidences of one
    block within it of each other.  Counted here on config-4-sized data (1024 rows x 151 936, N(0, 3^2),
    50-100 % masked): thresholds are placed INSIDE the data's confidence range (at its quartiles; the
    configured 0.9 is far above every confidence of such data), and every differing decision must be
    explained by such a near-tie.  The count for this seed is 0."""
    import bench
    import mdx
    c4 = bench.make_cfg4(dev, n_sets=1)
    logits, tokens = c4["logits"][0], c4["tokens"]
    x0, p = mdx.confidence_argmax(logits)
    torch.cuda.synchronize()
    x0, p = x0.cpu().numpy(), p.cpu().numpy()
    ep = np.empty((32, S))
    ex0 = np.empty((32, S), dtype=np.int64)
    for b in range(0, 32, 4):                                          # fp64 oracle, 128 rows at a time
        ex0[b:b + 4], ep[b:b + 4] = oracle.confidence_argmax(logits[b:b + 4].cpu().to(torch.float64).numpy())
    assert np.array_equal(x0, ex0)
    np.testing.assert_allclose(p, ep, rtol=2e-5)
    masked = tokens.numpy() == bench.MASK_ID
    ep32 = ep.astype(np.float32)
    flips = near = 0
    for thr in np.quantile(ep32[masked], [0.25, 0.5, 0.75]).tolist() + [0.9]:
        for k in (1, 4):
            got, _ = mdx.select_transfer(torch.from_numpy(x0).to(dev), torch.from_numpy(p).to(dev),
                                         tokens.clone().to(dev), bench.MASK_ID, float(thr), k)
            want = oracle.select_transfer(ep32, masked, float(thr), k)
            diff = got.cpu().numpy() != want
            flips += int(diff.sum())
            for b in np.nonzero(diff.any(1))[0]:                       # every flip needs a near-tie in its block
                c = np.where(masked[b], ep[b], -np.inf)
                srt = np.sort(c[np.isfinite(c)])[::-1]
                tie = np.any(np.abs(srt[:-1] - srt[1:]) <= 4e-5 * srt[:-1]) or np.any(np.abs(c - thr) <= 4e-5 * thr)
                assert tie, f"decision of block {b} differs without a near-tie (threshold {thr}, k {k})"
                near += 1
    print(f"config-4 boundary flips: {flips} positions in {near} blocks over 8 (threshold, k) settings")
    assert flips == 0


def test_config2_real_pool(dev):
    """bench.py's config-2 input as it is timed: 16 sequences over a 65 536-page pool (2 x 32 GiB; page ids up to
    65 535, byte offsets up to 32 GiB, far beyond 32-bit element indices), both launch forms of the paged attention.
    Only the referenced pages (at most 272 per cache) come back to the host, where the oracle runs on a compacted
    copy of the pool with a renumbered page table; max-abs < 2e-2.  Then store_kvcache into slots whose element
    offsets lie above 2^31, checked bit for bit with their neighbouring slots."""
    import bench
    import mdx
    c2 = bench.make_cfg2(dev, n_sets=1)
    bt, lens, q = c2["tables"][0], c2["lens"], c2["q"]
    kc, vc = c2["k_cache"], c2["v_cache"]
    assert kc.shape == (65536, PAGE, HKV, D) and bt.shape[0] == 16
    ids = bt[bt >= 0].long()
    assert int(ids.max()) > 60000 and ids.numel() <= 272
    assert int(ids.max()) * PAGE * HKV * D > 2 ** 33                        # element offsets need 64 bits
    scale = 1 / math.sqrt(D)
    o_two = mdx.flash_attn_with_kvcache(q, kc, vc, cache_seqlens=lens, block_table=bt, softmax_scale=scale, counters=False)
    o_one = mdx.flash_attn_with_kvcache(q, kc, vc, cache_seqlens=lens, block_table=bt, softmax_scale=scale)
    torch.cuda.synchronize()
    # compacted pool on the host: page i of the copy = page ids[i] of the real pool
    remap = {int(p): i for i, p in enumerate(ids.tolist())}
    hk, hv = kc[ids].cpu(), vc[ids].cpu()
    hbt = torch.tensor([[remap.get(int(p), -1) for p in row] for row in bt.cpu().tolist()], dtype=torch.int32)
    ref = oracle.paged_block_attn(q.cpu(), hk, hv, hbt, lens.cpu(), scale)
    for o in (o_two, o_one):
        err = (o.float().cpu() - ref).abs().max().item()
        assert err < 2e-2, err
    assert torch.equal(o_two, o_one)

    # store into the last pages of the pool: slot * 1024 elements > 2^31 from page 8192 on
    g = torch.Generator().manual_seed(22)
    free = sorted(set(range(65000, 65536)) - set(ids.tolist()))[:6]
    n = 700
    slots = torch.tensor(oracle.get_slots(free, 100, 100 + n), dtype=torch.int32)
    slots[::7] = -1
    assert int(slots.max()) * HKV * D > 2 ** 31
    key = torch.randn(n, HKV, D, generator=g).bfloat16()
    fused = torch.randn(n, 4096, generator=g).bfloat16()
    val = fused[:, 3072:].view(n, HKV, D)                                    # strided rows, as in the engine
    pages = torch.tensor(free, device=dev)
    kc[pages] = 0
    vc[pages] = 0
    mdx.store_kvcache(key.to(dev), fused.to(dev)[:, 3072:].view(n, HKV, D), kc, vc, slots.to(dev))
    torch.cuda.synchronize()
    ek = np.zeros((len(free) * PAGE, HKV * D), dtype=np.int16)
    ev = np.zeros_like(ek)
    local = {p: i for i, p in enumerate(free)}
    lslots = np.array([-1 if s < 0 else local[s // PAGE] * PAGE + s % PAGE for s in slots.tolist()], dtype=np.int32)
    oracle.store_kvcache(_i16(key), _i16(val), ek, ev, lslots)
    assert np.array_equal(_i16(kc[pages]).reshape(-1, HKV * D), ek)
    assert np.array_equal(_i16(vc[pages]).reshape(-1, HKV * D), ev)
    del c2, kc, vc
    torch.cuda.empty_cache()


def test_config5_full_size_properties(dev):
    """Config 5 at full size (28 layers, hidden 2048, batch 32, 1088-token prompts, 2048 new tokens in 32-token blocks,
    8 denoising passes per block) through the engine's device loop, as bench.py times it.  No oracle covers a
    2-billion-parameter run; what must hold whatever the weights is asserted inside run_cfg5: every sequence
    complete, no mask token in the output, one step-map entry per token, and exactly 64 x 9 - 1 decode passes (no
    confidence of a random-init model reaches the threshold, so every denoising pass commits k = 4 positions)."""
    import bench
    out = bench.run_cfg5(dev)
    assert out["committed_tokens"] == 32 * 2048 and out["layers"] == 28 and out["batch"] == 32
    assert out["decode_passes"] == 64 * 9 - 1 and out["prefill_passes"] >= 1
    print(f"config 5: {out['tokens_per_s']} tokens/s, {out['ms_per_decode_pass']} ms per decode pass")
    torch.cuda.empty_cache()
