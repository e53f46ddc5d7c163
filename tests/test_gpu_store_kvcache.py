"""GPU parity: store_kvcache through the C ABI vs the oracle, bit-exact."""
import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu


def _bits(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def _case(dev, N, hkv, d, pages, page, seed, frac_skip=0.2, v_strided=True, dtype=torch.bfloat16):
    import mdx
    g = torch.Generator().manual_seed(seed)
    D = hkv * d
    key = torch.randn(N, hkv, d, generator=g).to(dtype)
    if v_strided:   # V as a view into a fused [N, 4*D] projection output (row stride 4*D)
        fused = torch.randn(N, 4 * D, generator=g).to(dtype)
        value = fused[:, 2 * D:3 * D].view(N, hkv, d)
    else:
        value = torch.randn(N, hkv, d, generator=g).to(dtype)
    k_cache = torch.randn(pages, page, hkv, d, generator=g).to(dtype)
    v_cache = torch.randn(pages, page, hkv, d, generator=g).to(dtype)
    slots = torch.randperm(pages * page, generator=g)[:N].to(torch.int32)
    skip = torch.rand(N, generator=g) < frac_skip
    slots[skip] = -1

    ek, ev = _bits(k_cache).copy(), _bits(v_cache).copy()
    oracle.store_kvcache(_bits(key), _bits(value), ek, ev, slots.numpy())

    dk, dv = k_cache.to(dev), v_cache.to(dev)
    if v_strided:
        dfused = fused.to(dev)
        dvalue = dfused[:, 2 * D:3 * D].view(N, hkv, d)
        assert N == 1 or dvalue.stride(0) == 4 * D
    else:
        dvalue = value.to(dev)
    mdx.store_kvcache(key.to(dev), dvalue, dk, dv, slots.to(dev))
    torch.cuda.synchronize()
    assert np.array_equal(_bits(dk), ek)
    assert np.array_equal(_bits(dv), ev)


@pytest.mark.parametrize("N", [1, 3, 4, 5, 257, 4099])
def test_store_bf16_engine_shape(dev, N):
    _case(dev, N, 8, 128, pages=20, page=256, seed=N)


def test_store_all_skipped(dev):
    _case(dev, 64, 8, 128, pages=2, page=256, seed=1, frac_skip=1.1)


def test_store_contiguous_value_fp16(dev):
    _case(dev, 100, 8, 128, pages=2, page=256, seed=2, v_strided=False, dtype=torch.float16)


@pytest.mark.parametrize("hkv,d", [(1, 128), (2, 64), (3, 20), (16, 128), (1, 7)])
def test_store_other_row_sizes(dev, hkv, d):
    # (3,20): 120-byte rows -> element-wise path; (16,128): 4 KiB rows -> long-row path; (1,7): odd
    _case(dev, 77, hkv, d, pages=3, page=64, seed=hkv * 100 + d, v_strided=(hkv * d) % 8 == 0)


def test_store_4d_decode_form(dev):
    import mdx
    g = torch.Generator().manual_seed(5)
    bs, S, hkv, d, pages, page = 6, 32, 8, 128, 12, 256
    k = torch.randn(bs, S, hkv, d, generator=g).bfloat16()
    v = torch.randn(bs, S, hkv, d, generator=g).bfloat16()
    kc = torch.zeros(pages, page, hkv, d).bfloat16()
    vc = torch.zeros(pages, page, hkv, d).bfloat16()
    slots = torch.randperm(pages * page, generator=g)[:bs * S].to(torch.int32).view(bs, S)
    slots[-1] = -1                                    # a graph-padding row
    ek, ev = _bits(kc).copy(), _bits(vc).copy()
    oracle.store_kvcache(_bits(k), _bits(v), ek, ev, slots.numpy())
    dk, dv = kc.to(dev), vc.to(dev)
    mdx.store_kvcache_maybe4d(k.to(dev), v.to(dev), dk, dv, slots.to(dev))
    torch.cuda.synchronize()
    assert np.array_equal(_bits(dk), ek) and np.array_equal(_bits(dv), ev)


def test_store_out_of_range_slots_are_skipped(dev):
    import mdx
    N, hkv, d = 8, 8, 128
    k = torch.ones(N, hkv, d, dtype=torch.bfloat16, device=dev)
    kc = torch.zeros(1, 256, hkv, d, dtype=torch.bfloat16, device=dev)
    vc = torch.zeros_like(kc)
    slots = torch.tensor([0, 255, 256, 100000, -1, -7, 3, 2 ** 31 - 1], dtype=torch.int32, device=dev)
    mdx.store_kvcache(k, k, kc, vc, slots)
    torch.cuda.synchronize()
    written = (kc.view(256, -1).float().abs().sum(1) > 0).nonzero().flatten().tolist()
    assert written == [0, 3, 255]


def test_store_full_size_round_trip(dev):
    """benchmark config 3 size (about 36.9k tokens): store, gather back through the slots, compare."""
    import mdx
    g = torch.Generator().manual_seed(33)
    N, hkv, d, page = 36864 + 17, 8, 128, 256
    pages = (N + page - 1) // page + 8
    fused = torch.randn(N, 4 * hkv * d, generator=g).bfloat16().to(dev)
    key = fused[:, :hkv * d].view(N, hkv, d).contiguous()
    value = fused[:, 2 * hkv * d:3 * hkv * d].view(N, hkv, d)
    kc = torch.zeros(pages, page, hkv, d, dtype=torch.bfloat16, device=dev)
    vc = torch.zeros_like(kc)
    slots = torch.randperm(pages * page, generator=g)[:N].to(torch.int32).to(dev)
    mdx.store_kvcache(key, value, kc, vc, slots)
    torch.cuda.synchronize()
    assert torch.equal(kc.view(-1, hkv, d)[slots.long()], key)
    assert torch.equal(vc.view(-1, hkv, d)[slots.long()], value)
    assert int((kc.view(-1, hkv * d).float().abs().sum(1) > 0).sum()) <= N   # nothing else touched
