"""The entry point that allocates nothing, mdx_paged_block_attn_static, through the C ABI: its output
must equal mdx_paged_block_attn's bit for bit, on two calls in a row that share the static scratch
array, the second with a smaller input (fewer, shorter sequences: stale partials of the first call
stay in the array and must not be read)."""
import ctypes
import math

import pytest
import torch

pytestmark = pytest.mark.gpu
HQ, HKV, D, S, PAGE = 16, 8, 128, 32, 256


def _case(dev, seed, bs, lo, hi, max_pages):
    g = torch.Generator().manual_seed(seed)
    ctx = torch.randint(lo, hi + 1, (bs,), generator=g).to(torch.int32)
    n_pages = 2 * bs * max_pages
    kc = torch.randn(n_pages, PAGE, HKV, D, generator=g).bfloat16().to(dev)
    vc = torch.randn(n_pages, PAGE, HKV, D, generator=g).bfloat16().to(dev)
    perm = torch.randperm(n_pages, generator=g).to(torch.int32)
    bt = torch.full((bs, max_pages), -1, dtype=torch.int32)
    at = 0
    for b in range(bs):
        n = (int(ctx[b]) + PAGE - 1) // PAGE
        bt[b, :n] = perm[at:at + n]
        at += n
    q = torch.randn(bs, S, HQ, D, generator=g).bfloat16().to(dev)
    return q, kc, vc, bt.to(dev), ctx.to(dev)


def _both(dev, q, kc, vc, bt, ctx):
    import mdx
    L = mdx.lib()
    bs, max_pages = bt.shape
    stream = torch.cuda.current_stream().cuda_stream
    common = (kc.data_ptr(), vc.data_ptr(), q.stride(0), q.stride(1), q.stride(2), q.stride(0), q.stride(1), q.stride(2),
              kc.stride(0), kc.stride(1), kc.stride(2), bt.data_ptr(), bt.stride(0), ctx.data_ptr(),
              bs, S, HQ, HKV, D, max_pages, PAGE, kc.shape[0], 1 / math.sqrt(D), 0)
    ws_bytes = L.mdx_paged_block_attn_workspace_bytes(bs, S, HQ, HKV, D, max_pages, PAGE)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
    o_ref = torch.full_like(q, float("nan"))
    o_new = torch.full_like(q, float("nan"))
    torch.cuda.synchronize()
    rc = L.mdx_paged_block_attn(q.data_ptr(), o_ref.data_ptr(), *common, ws.data_ptr(), ws_bytes, stream)
    assert rc == 0, L.mdx_last_error()
    rc = L.mdx_paged_block_attn_static(q.data_ptr(), o_new.data_ptr(), *common, stream)
    assert rc == 0, L.mdx_last_error()
    torch.cuda.synchronize()
    return o_ref, o_new, ws_bytes


def test_static_scratch_entry_point_matches_workspace_entry_point(dev):
    import oracle
    # first call: 16 sequences of up to 4128 keys, every one split (about 25 MB of partials)
    first = _case(dev, 71, 16, 544, 4128, 17)
    o_ref, o_new, ws_bytes = _both(dev, *first)
    assert ws_bytes > (16 << 20), "the first call is meant to use most of the scratch array"
    assert torch.equal(o_ref.view(torch.int16), o_new.view(torch.int16))
    ref = oracle.paged_block_attn(first[0].cpu(), first[1].cpu(), first[2].cpu(), first[3].cpu(), first[4].cpu(), 1 / math.sqrt(D))
    assert (o_new.float().cpu() - ref).abs().max().item() < 2e-2
    # second call right after it: smaller input, same array
    second = _case(dev, 72, 5, 40, 1500, 6)
    o_ref2, o_new2, ws2 = _both(dev, *second)
    assert 0 < ws2 < ws_bytes
    assert torch.equal(o_ref2.view(torch.int16), o_new2.view(torch.int16))
    ref2 = oracle.paged_block_attn(second[0].cpu(), second[1].cpu(), second[2].cpu(), second[3].cpu(), second[4].cpu(), 1 / math.sqrt(D))
    assert (o_new2.float().cpu() - ref2).abs().max().item() < 2e-2


def test_static_scratch_entry_point_refuses_what_does_not_fit(dev):
    import mdx
    L = mdx.lib()
    one = ctypes.c_void_p(256)
    # 64 sequences x 16 heads with 17-page tables: 65 MiB of partials; refused before anything is touched
    need = L.mdx_paged_block_attn_workspace_bytes(64, S, HQ, HKV, D, 17, PAGE)
    assert need > (40 << 20)
    rc = L.mdx_paged_block_attn_static(one, one, one, one, 65536, 2048, 128, 65536, 2048, 128, 262144, 1024, 128, one, 17, one,
                                       64, S, HQ, HKV, D, 17, PAGE, 100, 0.1, 0, None)
    assert rc == -3 and b"static array" in L.mdx_last_error()
