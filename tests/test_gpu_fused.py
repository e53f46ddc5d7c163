"""GPU parity: fused q/k RMSNorm + RoPE + KV store through the C ABI vs the oracle.
q and k may differ from the oracle by one bf16 rounding (the reciprocal square root is not
bit-identical across devices); what is stored in the caches must equal the returned k and the
input v bit for bit."""
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu


def _tables(d=128, max_pos=512, theta=1.0e6):
    inv_freq = 1.0 / (theta ** (torch.arange(0, d, 2, dtype=torch.float) / d))
    ang = torch.arange(max_pos).float()[:, None] * inv_freq[None]
    return ang.cos().contiguous(), ang.sin().contiguous()


@pytest.mark.parametrize("N,hq,hkv", [(1, 16, 8), (37, 16, 8), (300, 4, 1), (64, 8, 8), (5, 40, 8)])
def test_fused_matches_oracle(dev, N, hq, hkv):
    import mdx
    g = torch.Generator().manual_seed(N + hq)
    d, pages, page = 128, 3, 256
    qkv = (torch.randn(N, (hq + 2 * hkv) * d, generator=g) * 2).bfloat16()
    qw = (torch.rand(d, generator=g) + 0.5).bfloat16()
    kw = (torch.rand(d, generator=g) + 0.5).bfloat16()
    cos, sin = _tables()
    pos = torch.randint(0, 512, (N,), generator=g)
    slots = torch.randperm(pages * page, generator=g)[:N].to(torch.int32)
    slots[::5] = -1
    kc = torch.zeros(pages, page, hkv, d, dtype=torch.bfloat16, device=dev)
    vc = torch.zeros_like(kc)
    q, k, v = mdx.qk_norm_rope_store(qkv.to(dev), qw.to(dev), kw.to(dev), 1e-6, cos.to(dev), sin.to(dev), pos.to(dev),
                                     hq, hkv, d, kc, vc, slots.to(dev))
    torch.cuda.synchronize()
    eq, ek, ev = oracle.qk_norm_rope(qkv, qw, kw, 1e-6, cos, sin, pos, hq, hkv, d)
    for got, want in ((q, eq), (k, ek)):
        diff = (got.float().cpu() - want.float()).abs()
        tol = want.float().abs() * 2 ** -7 + 2 ** -7          # one bf16 ulp, generous near zero
        assert (diff <= tol).all(), diff.max()
        assert (diff == 0).float().mean() > 0.9                # and almost everywhere identical
    assert torch.equal(v.cpu(), ev)
    keep = slots >= 0
    assert torch.equal(kc.view(-1, hkv, d)[slots[keep].long().to(dev)], k[keep.to(dev)])
    assert torch.equal(vc.view(-1, hkv, d)[slots[keep].long().to(dev)], v[keep.to(dev)])
    untouched = torch.ones(pages * page, dtype=torch.bool)
    untouched[slots[keep].long()] = False
    assert kc.view(pages * page, -1)[untouched.to(dev)].abs().sum().item() == 0


def test_fused_decode_shape_without_k_out_and_without_cache(dev):
    import mdx
    g = torch.Generator().manual_seed(9)
    hq, hkv, d = 16, 8, 128
    qkv = torch.randn(3, 32, (hq + 2 * hkv) * d, generator=g).bfloat16().to(dev)
    w = torch.ones(d, dtype=torch.bfloat16, device=dev)
    cos, sin = (t.to(dev) for t in _tables())
    pos = (torch.arange(32)[None] + torch.tensor([[5], [100], [300]])).to(dev)
    q, k, v = mdx.qk_norm_rope_store(qkv, w, w, 1e-6, cos, sin, pos, hq, hkv, d, want_k=False)
    assert k is None and q.shape == (3, 32, hq, d) and v.shape == (3, 32, hkv, d)
    eq, _, ev = oracle.qk_norm_rope(qkv.view(96, -1), w, w, 1e-6, cos, sin, pos.view(-1), hq, hkv, d)
    assert (q.view(96, hq, d).float().cpu() - eq.float()).abs().max().item() < 0.05
    assert torch.equal(v.reshape(96, hkv, d).cpu(), ev)


def test_engine_fused_and_unfused_paths_agree(dev):
    """The decoder scaffold with the fused launch vs the same scaffold on stock ops.  The unmask
    step is scripted (commit 16 fixed tokens per pass) so both runs feed identical tokens."""
    from mdx.engine import BlockDiffusionEngine, Decoder, DecoderConfig, SamplingParams

    def scripted_unmask(logits, x, mask_id, thr, k, temperatures=None):
        masked = x == mask_id
        first = masked & (masked.long().cumsum(-1) <= 16)
        x[first] = (torch.arange(x.shape[1], device=x.device)[None].expand_as(x) + 7)[first]
        return None, None, first, first.sum(-1).to(torch.int32)

    outs = []
    for fused in (True, False):
        cfg = DecoderConfig(num_layers=2, hidden_size=256, num_heads=4, num_kv_heads=2, head_dim=128, intermediate_size=512,
                            vocab_size=1000, max_position=1024, mask_token_id=999, fused_qk_rope_store=fused, fused_layer_ops=fused)
        model = Decoder(cfg, dev, seed=3)
        logits = []
        eng = BlockDiffusionEngine(model, num_pages=6, unmask=scripted_unmask,
                                   on_logits=lambda p, s, l: logits.append(l.float().cpu().clone()))
        eng.add_request(list(range(3, 203)), SamplingParams(max_new_tokens=64, ignore_eos=True))
        for _ in range(5):                      # prefill, denoise, caching pass, next block ...
            eng.step()
        outs.append((logits, eng.kv_cache.float().cpu().clone()))
    (la, ca), (lb, cb) = outs
    assert len(la) == 5
    for a, b in zip(la, lb):
        assert (a - b).abs().max().item() < 0.05 * a.abs().max().item()
    assert (ca - cb).abs().max().item() < 0.05 * ca.abs().max().item()


def _ulp_close(got, want, frac_equal=0.98):
    """At most one bf16 rounding apart everywhere, identical almost everywhere."""
    diff = (got.float().cpu() - want.float()).abs()
    tol = want.float().abs() * 2 ** -7 + 1e-30
    assert (diff <= tol).all(), (diff.max(), (diff > tol).sum())
    assert (diff == 0).float().mean() >= frac_equal, (diff == 0).float().mean()


@pytest.mark.parametrize("rows,hidden", [(1, 2048), (37, 2048), (1024, 2048), (5, 8), (3, 1000), (4, 4096), (2, 8192), (9, 6144)])
def test_add_rms_norm_matches_oracle(dev, rows, hidden):
    import mdx
    g = torch.Generator().manual_seed(rows * 7 + hidden)
    x = (torch.randn(rows, hidden, generator=g) * 3).bfloat16()
    r = (torch.randn(rows, hidden, generator=g) * 5).bfloat16()
    w = (torch.rand(hidden, generator=g) + 0.5).bfloat16()
    y, nr = mdx.rms_norm(x.to(dev), w.to(dev), 1e-6, r.to(dev))
    ey, er = oracle.add_rms_norm(x, r, w, 1e-6)
    assert torch.equal(nr.cpu(), er)                          # the new residual is one rounding of an exact fp32 sum
    _ulp_close(y, ey)
    y1 = mdx.rms_norm(x.to(dev), w.to(dev), 1e-6)
    _ulp_close(y1, oracle.add_rms_norm(x, None, w, 1e-6)[0])


def test_add_rms_norm_strided_rows_and_in_place(dev):
    import mdx
    g = torch.Generator().manual_seed(11)
    rows, hidden = 33, 512
    wide = (torch.randn(rows, 3 * hidden, generator=g) * 2).bfloat16().to(dev)
    x, r = wide[:, hidden:2 * hidden], wide[:, 2 * hidden:]   # row stride 3 * hidden
    w = (torch.rand(hidden, generator=g) + 0.5).bfloat16().to(dev)
    ey, er = oracle.add_rms_norm(x, r, w, 1e-5)
    y, nr = mdx.rms_norm(x, w, 1e-5, r)
    assert torch.equal(nr.cpu(), er)
    _ulp_close(y, ey)
    # through the C ABI with out aliasing x and residual_out aliasing residual_in
    xc, rc_ = x.contiguous(), r.contiguous()
    rc = mdx.lib().mdx_add_rms_norm(xc.data_ptr(), hidden, rc_.data_ptr(), hidden, rc_.data_ptr(), hidden, w.data_ptr(), 1e-5,
                                    xc.data_ptr(), hidden, rows, hidden, 0, torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.equal(rc_.cpu(), er) and torch.equal(xc, y)
    assert torch.equal(wide[:, :hidden].cpu(), wide.cpu()[:, :hidden])     # neighbours untouched


def test_add_rms_norm_rejects_bad_arguments(dev):
    import mdx
    x = torch.zeros(2, 12, dtype=torch.bfloat16, device=dev)
    w = torch.ones(12, dtype=torch.bfloat16, device=dev)
    with pytest.raises(mdx.MdxError):
        mdx.rms_norm(x, w, 1e-6)                              # hidden not a multiple of 8
    x = torch.zeros(2, 16384, dtype=torch.bfloat16, device=dev)
    with pytest.raises(mdx.MdxError):
        mdx.rms_norm(x, torch.ones(16384, dtype=torch.bfloat16, device=dev), 1e-6)
    xs = torch.zeros(2, 16, dtype=torch.bfloat16, device=dev)
    L = mdx.lib()
    s = torch.cuda.current_stream().cuda_stream
    assert L.mdx_add_rms_norm(xs.data_ptr(), 16, xs.data_ptr(), 16, None, 0, w.data_ptr(), 1e-6, xs.data_ptr(), 16, 2, 16, 0, s) < 0
    assert L.mdx_add_rms_norm(xs.data_ptr(), 16, None, 0, None, 0, w.data_ptr(), 1e-6, xs.data_ptr(), 16, 2, 16, 1, s) < 0   # fp16
    assert L.mdx_add_rms_norm(None, 16, None, 0, None, 0, None, 1e-6, None, 16, 0, 16, 0, s) == 0                          # no rows


@pytest.mark.parametrize("rows,inter", [(1, 6144), (1024, 6144), (7, 8), (33, 1000)])
def test_silu_and_mul_matches_oracle(dev, rows, inter):
    import mdx
    g = torch.Generator().manual_seed(rows + inter)
    x = (torch.randn(rows, 2 * inter, generator=g) * 4).bfloat16()
    x[0, :4] = torch.tensor([0.0, -100.0, 100.0, -0.0]).bfloat16()
    y = mdx.silu_and_mul(x.to(dev))
    _ulp_close(y, oracle.silu_and_mul(x), frac_equal=0.97)
    assert y[0, 0].item() == 0 and y[0, 1].item() == 0        # silu(0) = 0, silu(-100) = 0 times anything finite
    assert torch.equal(y[0, 2].cpu(), (torch.tensor(100.0).bfloat16() * x[0, inter + 2]))
    # rows taken out of a wider matrix
    wide = (torch.randn(rows, 2 * inter + 64, generator=g)).bfloat16().to(dev)
    _ulp_close(mdx.silu_and_mul(wide[:, 64:]), oracle.silu_and_mul(wide[:, 64:].cpu()), frac_equal=0.97)
