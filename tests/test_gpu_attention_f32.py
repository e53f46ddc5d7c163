"""GPU parity of the two attention calls' fp32-arithmetic kernels (fp32 tensors, and heads that the 16-bit kernels do
not take: wider than 128 columns or not a multiple of 16) through the C ABI vs the fp32 oracle.

The reference's prefill kernel takes any q.dtype and BLOCK_DMODEL = head_dim (block_prefill_attention_v2.py:179-197),
flash_attn_with_kvcache (sdar_attention.py:48-56) heads of up to 256 columns.
Tolerances: fp32 tensors 3e-5 max-abs (both sides compute in fp32; only the order of the sums differs), 16-bit
tensors 1e-2 (the output's own rounding: the arithmetic in between is fp32)."""
import math

import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu
TOL_F32 = 3e-5
TOL_16 = 1e-2


def _packed(g, lens, hq, hkv, d, dtype):
    N = sum(lens)
    q = torch.randn(N, hq, d, generator=g).to(dtype)
    k = torch.randn(N, hkv, d, generator=g).to(dtype)
    v = torch.randn(N, hkv, d, generator=g).to(dtype)
    cu = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32)
    return q, k, v, cu


def _check(dev, lens, S, hq, hkv, d, dtype, seed, max_seqlen=None):
    import mdx
    g = torch.Generator().manual_seed(seed)
    q, k, v, cu = _packed(g, lens, hq, hkv, d, dtype)
    o = mdx.sparse_attn_varlen(q.to(dev), k.to(dev), v.to(dev), cu.to(dev), cu.to(dev), S, max_seqlen=max_seqlen)
    torch.cuda.synchronize()
    assert o.dtype == dtype and o.shape == q.shape
    ref = oracle.staircase_attn_varlen(q, k, v, cu, S)
    err = (o.float().cpu() - ref).abs().max().item()
    tol = TOL_F32 if dtype == torch.float32 else TOL_16
    assert err < tol, f"max-abs {err} for lens={lens} S={S} d={d} {dtype}"
    assert bool(torch.isfinite(o).all())
    return err


@pytest.mark.parametrize("L", [1, 31, 32, 33, 100, 128, 129, 257, 700])
def test_fp32_single_sequence_block32(dev, L):
    _check(dev, [L], 32, 16, 8, 128, torch.float32, seed=L)


@pytest.mark.parametrize("S", [1, 2, 4, 8, 16, 32, 64, 128])
def test_fp32_all_staircase_sizes(dev, S):
    _check(dev, [203, 77, 1, 160], S, 4, 2, 128, torch.float32, seed=100 + S)


@pytest.mark.parametrize("hq,hkv", [(16, 8), (8, 8), (4, 1), (3, 1)])
def test_fp32_head_ratios_and_empty_sequences(dev, hq, hkv):
    _check(dev, [150, 0, 97, 0], 32, hq, hkv, 128, torch.float32, seed=hq * 10 + hkv, max_seqlen=150)


@pytest.mark.parametrize("d", [4, 20, 64, 100, 128, 132, 192, 256])
def test_fp32_head_widths(dev, d):
    _check(dev, [261, 40], 32, 4, 2, d, torch.float32, seed=d)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("d", [8, 72, 136, 192, 256])
def test_16bit_heads_outside_the_16bit_kernels(dev, d, dtype):
    """Heads wider than 128 columns, or not a multiple of 16: 16-bit tensors through the fp32 arithmetic."""
    _check(dev, [333, 64, 31], 32, 4, 2, d, dtype, seed=7000 + d)
    _check(dev, [200], 4, 3, 1, d, dtype, seed=7100 + d)


def test_fp32_config1_shape_as_a_prefill(dev):
    """The fp32 anchor of the benchmark's first configuration (32 queries on a prefix of 1024 keys plus their own
    block, 16 query heads on 8 KV heads, d = 128) is the last block of a staircase prefill of 1056 tokens: those 32
    rows see every key."""
    import mdx
    g = torch.Generator().manual_seed(1)
    L, hq, hkv, d = 1056, 16, 8, 128
    q, k, v, cu = _packed(g, [L], hq, hkv, d, torch.float32)
    o = mdx.sparse_attn_varlen(q.to(dev), k.to(dev), v.to(dev), cu.to(dev), cu.to(dev), 32)
    torch.cuda.synchronize()
    qh = q[-32:].permute(1, 0, 2)[None]                                  # [1, 16, 32, 128]
    kh, vh = k.permute(1, 0, 2)[None], v.permute(1, 0, 2)[None]          # [1, 8, 1056, 128]
    mask = torch.ones(32, L, dtype=torch.bool)
    ref = torch.nn.functional.scaled_dot_product_attention(qh, kh, vh, attn_mask=mask, scale=1 / math.sqrt(d), enable_gqa=True)
    err = (o[-32:].cpu() - ref[0].permute(1, 0, 2)).abs().max().item()
    assert err < TOL_F32, err


def test_fp32_reads_fused_projection_views_and_honours_the_strides_of_o(dev):
    import mdx
    g = torch.Generator().manual_seed(77)
    N, hq, hkv, d = 333, 8, 4, 64
    fused = torch.randn(N, (hq + 2 * hkv) * d, generator=g)
    q = fused[:, :hq * d].view(N, hq, d)
    k = fused[:, hq * d:(hq + hkv) * d].view(N, hkv, d)
    v = fused[:, (hq + hkv) * d:].view(N, hkv, d)
    cu = torch.tensor([0, 200, N], dtype=torch.int32)
    fd = fused.to(dev)
    dq, dk, dv = fd[:, :hq * d].view(N, hq, d), fd[:, hq * d:(hq + hkv) * d].view(N, hkv, d), fd[:, (hq + hkv) * d:].view(N, hkv, d)
    ref = oracle.staircase_attn_varlen(q, k, v, cu, 32)
    o = mdx.sparse_attn_varlen(dq, dk, dv, cu.to(dev), cu.to(dev), 32)
    assert (o.cpu() - ref).abs().max().item() < TOL_F32
    # o inside a wider buffer: columns beyond the head's width stay as they were
    wide = torch.full((N, hq, 68), 7.0, dtype=torch.float32, device=dev)
    cud = cu.to(dev)
    rc = mdx._lib.lib().mdx_staircase_attn_varlen(
        dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), wide.data_ptr(), dq.stride(0), dq.stride(1), dk.stride(0), dk.stride(1),
        dv.stride(0), dv.stride(1), wide.stride(0), wide.stride(1), cud.data_ptr(), cud.data_ptr(), 2, 200, N, hq, hkv, d, 32,
        1 / math.sqrt(d), 2, torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert bool((wide[..., d:] == 7.0).all())
    assert torch.equal(wide[..., :d], o)


def test_fp32_peaked_scores_and_large_magnitudes(dev):
    """Scores of hundreds (a softmax that is one-hot in fp32) and a dominant key placed anywhere in a tile."""
    import mdx
    g = torch.Generator().manual_seed(5)
    L, hq, hkv, d = 160, 2, 1, 128
    q, k, v, cu = _packed(g, [L], hq, hkv, d, torch.float32)
    q = q * 6.0
    k = k * 6.0
    o = mdx.sparse_attn_varlen(q.to(dev), k.to(dev), v.to(dev), cu.to(dev), cu.to(dev), 32)
    ref = oracle.staircase_attn_varlen(q, k, v, cu, 32)
    assert bool(torch.isfinite(o).all())
    assert (o.cpu() - ref).abs().max().item() < 2e-4


def test_fp32_arguments_are_validated(dev):
    import mdx
    x = torch.zeros(10, 2, 130, device=dev)                              # head_dim not a multiple of 4
    cu = torch.tensor([0, 10], dtype=torch.int32, device=dev)
    with pytest.raises(mdx.MdxError):
        mdx.sparse_attn_varlen(x, x, x, cu, cu, 32)
    y = torch.zeros(10, 2, 260, device=dev)                              # wider than 256
    with pytest.raises(mdx.MdxError):
        mdx.sparse_attn_varlen(y, y, y, cu, cu, 32)


# --------------------------------------------------------------------------- paged single-block attention
def _paged_inputs(g, ctxs, sq, hq, hkv, d, dtype, page=64, pool=80):
    bs = len(ctxs)
    maxp = max(1, max((c + page - 1) // page for c in ctxs))
    q = torch.randn(bs, sq, hq, d, generator=g).to(dtype)
    kc = torch.randn(pool, page, hkv, d, generator=g).to(dtype)
    vc = torch.randn(pool, page, hkv, d, generator=g).to(dtype)
    perm = torch.randperm(pool, generator=g)
    bt = torch.full((bs, maxp), -1, dtype=torch.int32)
    at = 0
    for b, c in enumerate(ctxs):
        n = (c + page - 1) // page
        bt[b, :n] = perm[at:at + n].to(torch.int32)
        at += n
    return q, kc, vc, bt, torch.tensor(ctxs, dtype=torch.int32)


def _check_paged(dev, ctxs, sq, hq, hkv, d, dtype, seed, page=64):
    import mdx
    g = torch.Generator().manual_seed(seed)
    q, kc, vc, bt, lens = _paged_inputs(g, ctxs, sq, hq, hkv, d, dtype, page=page)
    scale = 1 / math.sqrt(d)
    o = mdx.flash_attn_with_kvcache(q.to(dev), kc.to(dev), vc.to(dev), cache_seqlens=lens.to(dev), block_table=bt.to(dev),
                                    softmax_scale=scale, causal=False)
    torch.cuda.synchronize()
    assert o.dtype == dtype and o.shape == q.shape
    ref = oracle.paged_block_attn(q, kc, vc, bt, lens, scale)
    err = (o.float().cpu() - ref).abs().max().item()
    tol = TOL_F32 if dtype == torch.float32 else TOL_16
    assert err < tol, f"max-abs {err} for ctxs={ctxs} sq={sq} d={d} {dtype}"
    return o


@pytest.mark.parametrize("ctx", [1, 31, 32, 33, 64, 65, 257, 1000])
def test_paged_fp32_single_sequence(dev, ctx):
    _check_paged(dev, [ctx], 32, 16, 8, 128, torch.float32, seed=ctx)


@pytest.mark.parametrize("hq,hkv,sq", [(16, 8, 32), (8, 8, 7), (4, 1, 32), (3, 1, 20), (10, 2, 64), (6, 1, 100)])
def test_paged_fp32_head_layouts_block_lengths_and_padding_rows(dev, hq, hkv, sq):
    """One to six query heads per KV head (more than a workgroup's four wavefronts: a second round over the keys),
    blocks shorter and longer than a query tile, a graph-padding row (context 0) that must come out as zeros."""
    o = _check_paged(dev, [700, 0, 33, 1234], sq, hq, hkv, 128, torch.float32, seed=hq * 100 + sq)
    assert o[1].abs().max().item() == 0


@pytest.mark.parametrize("d,dtype", [(d, t) for d in (8, 72, 128, 160, 256) for t in (torch.float32, torch.bfloat16, torch.float16)
                                     if d != 128 or t == torch.float32])       # 16-bit at d = 128 is the 16-bit kernel's own shape
def test_paged_head_widths_outside_the_16bit_kernel(dev, d, dtype):
    _check_paged(dev, [300, 2100, 64], 32, 4, 2, d, dtype, seed=8000 + d, page=256 if d >= 128 else 32)


def test_paged_fp32_invalid_pages_are_left_out(dev):
    """Keys on a page id outside the pool are excluded; a sequence without any valid page yields zeros."""
    import mdx
    g = torch.Generator().manual_seed(91)
    q, kc, vc, bt, lens = _paged_inputs(g, [200, 300], 32, 4, 2, 128, torch.float32)
    scale = 1 / math.sqrt(128)
    bad = bt.clone()
    bad[0] = -1
    bad[0, 0] = kc.shape[0] + 5
    bad[1, 1] = -1                                  # keys 64 .. 127 of sequence 1 drop out
    o = mdx.flash_attn_with_kvcache(q.to(dev), kc.to(dev), vc.to(dev), cache_seqlens=lens.to(dev), block_table=bad.to(dev),
                                    softmax_scale=scale, causal=False).cpu()
    assert o[0].abs().max().item() == 0 and not torch.isnan(o).any()
    keep = torch.cat([torch.arange(0, 64), torch.arange(128, 300)])
    kk = oracle.paged_gather(kc, bt[1], 300)[keep]
    vv = oracle.paged_gather(vc, bt[1], 300)[keep]
    ref = oracle.masked_attention_f32(q[1], kk, vv, None, scale)
    assert (o[1] - ref).abs().max().item() < TOL_F32


def test_paged_fp32_length_beyond_the_page_table_is_clipped(dev):
    import mdx
    g = torch.Generator().manual_seed(17)
    q, kc, vc, bt, lens = _paged_inputs(g, [128], 32, 4, 2, 64, torch.float32)
    scale = 1 / math.sqrt(64)
    o = mdx.flash_attn_with_kvcache(q.to(dev), kc.to(dev), vc.to(dev), cache_seqlens=torch.tensor([5000], dtype=torch.int32, device=dev),
                                    block_table=bt.to(dev), softmax_scale=scale, causal=False).cpu()
    ref = oracle.paged_block_attn(q, kc, vc, bt, lens, scale)          # the table holds 2 pages of 64 keys
    assert (o - ref).abs().max().item() < TOL_F32


def test_decode_matches_prefill_last_block_in_fp32(dev):
    """The last block of a staircase prefill and the paged call over the same keys are the same attention."""
    import mdx
    g = torch.Generator().manual_seed(3)
    L, hq, hkv, d, page = 200, 4, 2, 192, 64
    q, k, v, cu = _packed(g, [L], hq, hkv, d, torch.float32)
    o1 = mdx.sparse_attn_varlen(q.to(dev), k.to(dev), v.to(dev), cu.to(dev), cu.to(dev), 8)
    n_pages = (L + page - 1) // page
    kc = torch.zeros(n_pages + 2, page, hkv, d)
    vc = torch.zeros(n_pages + 2, page, hkv, d)
    table = torch.tensor([[2, 0, 5, 1][:n_pages]], dtype=torch.int32)
    for t in range(L):
        kc[table[0, t // page], t % page] = k[t]
        vc[table[0, t // page], t % page] = v[t]
    o2 = mdx.flash_attn_with_kvcache(q[-8:][None].to(dev), kc.to(dev), vc.to(dev), cache_seqlens=torch.tensor([L], dtype=torch.int32, device=dev),
                                     block_table=table.to(dev), softmax_scale=1 / math.sqrt(d), causal=False)
    assert (o1[-8:] - o2[0]).abs().max().item() < TOL_F32


def test_fp32_sequence_bounds_are_clipped_to_the_tensors(dev):
    """cu_seqlens that run past the packed tensors (or backwards) are clipped to them: no row outside q/k/v/o is touched."""
    import mdx
    g = torch.Generator().manual_seed(81)
    q, k, v, cu = _packed(g, [200], 4, 2, 64, torch.float32)
    good = mdx.sparse_attn_varlen(q.to(dev), k.to(dev), v.to(dev), cu.to(dev), cu.to(dev), 32)
    long = torch.tensor([0, 250], dtype=torch.int32)
    o = mdx.sparse_attn_varlen(q.to(dev), k.to(dev), v.to(dev), long.to(dev), long.to(dev), 32)
    assert torch.equal(o, good)
    back = torch.tensor([0, 120, 60, 200], dtype=torch.int32)           # the second sequence runs backwards: empty
    o = mdx.sparse_attn_varlen(q.to(dev), k.to(dev), v.to(dev), back.to(dev), back.to(dev), 32)
    torch.cuda.synchronize()
    ref = oracle.staircase_attn_varlen(q[:120], k[:120], v[:120], torch.tensor([0, 120], dtype=torch.int32), 32)
    assert (o[:60].cpu() - ref[:60]).abs().max().item() < TOL_F32
