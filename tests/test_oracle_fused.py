"""Pins the q/k-norm + RoPE oracle by closed forms and library routines."""
import torch
import torch.nn.functional as F

import oracle


def test_rms_norm_closed_forms():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(5, 3, 128, generator=g)
    y = oracle.rms_norm_ref(x, torch.ones(128), 0.0)
    assert torch.allclose(y.pow(2).mean(-1), torch.ones(5, 3), atol=1e-5)          # unit RMS
    w = torch.rand(128, generator=g) + 0.5
    assert torch.allclose(oracle.rms_norm_ref(x, w, 1e-6), F.rms_norm(x, (128,), w, 1e-6), atol=1e-5)
    assert torch.allclose(oracle.rms_norm_ref(3 * x, w, 0.0), oracle.rms_norm_ref(x, w, 0.0), atol=1e-5)   # scale invariant


def test_rope_is_a_rotation_of_half_split_pairs():
    g = torch.Generator().manual_seed(1)
    d, theta = 128, 1.0e6
    inv_freq = 1.0 / (theta ** (torch.arange(0, d, 2, dtype=torch.float) / d))
    pos = torch.tensor([0, 1, 7, 1000])
    ang = pos[:, None].float() * inv_freq[None]
    x = torch.randn(4, 2, d, generator=g)
    y = oracle.rope_ref(x, ang.cos().unsqueeze(1), ang.sin().unsqueeze(1))
    assert torch.equal(y[0], x[0])                                                   # position 0: identity
    # pairs are (i, i + d/2), not (2i, 2i+1): as complex numbers y = x * e^{i angle}
    xc = torch.complex(x[..., :64], x[..., 64:])
    yc = xc * torch.polar(torch.ones_like(ang), ang).unsqueeze(1)
    assert torch.allclose(y[..., :64], yc.real, atol=1e-5) and torch.allclose(y[..., 64:], yc.imag, atol=1e-5)
    assert torch.allclose(y[..., :64] ** 2 + y[..., 64:] ** 2, x[..., :64] ** 2 + x[..., 64:] ** 2, atol=1e-4)
    # relative-position property: <rope(q, m), rope(k, n)> depends on m - n only
    q, k = torch.randn(1, 1, d, generator=g), torch.randn(1, 1, d, generator=g)
    def at(v, p):
        a = (torch.tensor([p]).float()[:, None] * inv_freq[None])
        return oracle.rope_ref(v, a.cos().unsqueeze(1), a.sin().unsqueeze(1))
    assert torch.allclose((at(q, 10) * at(k, 3)).sum(), (at(q, 107) * at(k, 100)).sum(), atol=1e-3)


def test_qk_norm_rope_splits_heads_q_k_v():
    g = torch.Generator().manual_seed(2)
    hq, hkv, d, N = 4, 2, 128, 6
    qkv = torch.randn(N, (hq + 2 * hkv) * d, generator=g).bfloat16()
    cos, sin = torch.ones(16, 64), torch.zeros(16, 64)                               # no rotation
    q, k, v = oracle.qk_norm_rope(qkv, torch.ones(d).bfloat16(), torch.ones(d).bfloat16(), 1e-6, cos, sin,
                                  torch.arange(N), hq, hkv, d)
    assert torch.equal(v, qkv[:, (hq + hkv) * d:].view(N, hkv, d))
    assert torch.allclose(q.float().pow(2).mean(-1), torch.ones(N, hq), atol=2e-2)
    assert torch.equal(k[2, 1], oracle.rms_norm_ref(qkv[2, (hq + 1) * d:(hq + 2) * d], torch.ones(d).bfloat16(), 1e-6))


def test_add_rms_norm_rounds_the_residual_but_not_the_variance():
    g = torch.Generator().manual_seed(3)
    x = (torch.randn(6, 256, generator=g) * 3).bfloat16()
    r = (torch.randn(6, 256, generator=g) * 3).bfloat16()
    w = (torch.rand(256, generator=g) + 0.5).bfloat16()
    y, nr = oracle.add_rms_norm(x, r, w, 1e-6)
    s = x.float() + r.float()                                   # exact in fp32 for bf16 operands of similar size
    assert torch.equal(nr, s.bfloat16())
    assert torch.allclose(y.float(), F.rms_norm(s, (256,), w.float(), 1e-6), rtol=2 ** -6, atol=1e-3)
    # a zero residual reduces it to the plain norm, bit for bit
    y0, nr0 = oracle.add_rms_norm(x, torch.zeros_like(x), w, 1e-6)
    assert torch.equal(y0, oracle.rms_norm_ref(x, w, 1e-6)) and torch.equal(nr0, x)
    assert oracle.add_rms_norm(x, None, w, 1e-6)[1] is None
    # the mean of squares is taken over the unrounded sum: 256 + 1 rounds to 256 in bf16, and the
    # row [257, 0, ...] must normalise with 257, not 256
    x1 = torch.zeros(1, 8).bfloat16(); x1[0, 0] = 256.0
    r1 = torch.zeros(1, 8).bfloat16(); r1[0, 0] = 1.0
    y1, nr1 = oracle.add_rms_norm(x1, r1, torch.ones(8).bfloat16(), 0.0)
    assert nr1[0, 0].item() == 256.0                            # the stored residual lost the 1
    assert y1[0, 0].item() == torch.tensor(257.0 / (257.0 / 8 ** 0.5)).bfloat16().item()   # = sqrt(8) either way here
    x2 = torch.tensor([[256.0, 128.0] + [0.0] * 6]).bfloat16()
    r2 = torch.tensor([[1.0, 0.0] + [0.0] * 6]).bfloat16()
    y2, _ = oracle.add_rms_norm(x2, r2, torch.ones(8).bfloat16(), 0.0)
    rms_unrounded = ((257.0 ** 2 + 128.0 ** 2) / 8) ** 0.5
    assert y2[0, 1].item() == torch.tensor(128.0 / rms_unrounded).bfloat16().item()


def test_silu_and_mul_closed_forms():
    g = torch.Generator().manual_seed(4)
    x = (torch.randn(5, 64, generator=g) * 3).bfloat16()
    y = oracle.silu_and_mul(x)
    assert y.shape == (5, 32)
    assert torch.equal(y, F.silu(x[:, :32]) * x[:, 32:])        # the library routine, same rounding points
    t = torch.tensor([[0.0, 30.0, -30.0, 1.0, 1.0, 2.0, 2.0, 2.0]]).bfloat16()
    yt = oracle.silu_and_mul(t)
    assert yt[0, 0].item() == 0.0 and yt[0, 1].item() == 60.0 and abs(yt[0, 2].item()) < 1e-10
    assert abs(yt[0, 3].item() - 2 * 0.7310585786) < 2e-2       # silu(1) = 1 / (1 + e^-1)
