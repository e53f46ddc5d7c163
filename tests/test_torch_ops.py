"""torch.ops.mdx.*: the registrations exist, say what they return without running (fake tensors, no GPU
needed), and on the GPU a traced function calling them gives the results of the direct calls."""
import math

import pytest
import torch
from torch._subclasses.fake_tensor import FakeTensorMode


def test_ops_are_registered_with_shape_only_implementations():
    import mdx.torch_ops  # noqa: F401
    with FakeTensorMode():
        bf = dict(device="cuda", dtype=torch.bfloat16)
        q = torch.empty(100, 16, 128, **bf)
        kv = torch.empty(100, 8, 128, **bf)
        cu = torch.empty(3, device="cuda", dtype=torch.int32)
        o = torch.ops.mdx.sparse_attn_varlen(q, kv, kv, cu, cu, 32, 64, 0.1)
        assert o.shape == q.shape and o.dtype == q.dtype and o.device.type == "cuda"
        cache = torch.empty(4, 256, 8, 128, **bf)
        assert torch.ops.mdx.store_kvcache(kv, kv, cache, cache, torch.empty(100, device="cuda", dtype=torch.int32)) is None
        q4 = torch.empty(2, 32, 16, 128, **bf)
        o4 = torch.ops.mdx.paged_block_attn(q4, cache, cache, torch.empty(2, device="cuda", dtype=torch.int32),
                                            torch.empty(2, 2, device="cuda", dtype=torch.int32), 0.1)
        assert o4.shape == q4.shape
        logits = torch.empty(2, 32, 1000, **bf)
        x0, p = torch.ops.mdx.confidence_argmax(logits, None)
        assert x0.shape == (2, 32) and x0.dtype == torch.int64 and p.dtype == torch.float32
        tok = torch.empty(2, 32, device="cuda", dtype=torch.int64)
        x0, p, tr, cnt = torch.ops.mdx.unmask_step(logits, tok, 999, 0.9, 4, None)
        assert tr.dtype == torch.bool and tr.shape == (2, 32) and cnt.shape == (2,) and cnt.dtype == torch.int32
        x = torch.empty(2, 32, 256, **bf)
        w = torch.empty(256, **bf)
        assert torch.ops.mdx.rms_norm(x, w, 1e-6).shape == x.shape
        y, r = torch.ops.mdx.add_rms_norm(x, x, w, 1e-6)
        assert y.shape == x.shape and r.shape == x.shape
        assert torch.ops.mdx.silu_and_mul(x).shape == (2, 32, 128)
        x0, p = torch.ops.mdx.lm_head_confidence(x, torch.empty(1000, 256, **bf), None)
        assert x0.shape == (2, 32) and x0.dtype == torch.int64 and p.shape == (2, 32) and p.dtype == torch.float32


def test_mutated_arguments_are_declared():
    import mdx.torch_ops  # noqa: F401
    writes = {name: [a.name for a in getattr(torch.ops.mdx, name).default._schema.arguments if a.is_write]
              for name in ("store_kvcache", "unmask_step", "sparse_attn_varlen", "paged_block_attn")}
    assert writes == {"store_kvcache": ["k_cache", "v_cache"], "unmask_step": ["tokens"],
                      "sparse_attn_varlen": [], "paged_block_attn": []}


@pytest.mark.gpu
def test_traced_function_matches_direct_calls(dev):
    """A function that stores K/V, runs both attentions, the layer ops and the unmask step through
    torch.ops.mdx, traced whole by torch.compile (no graph breaks allowed), against mdx.ops."""
    import mdx
    import mdx.torch_ops  # noqa: F401
    g = torch.Generator().manual_seed(5)
    L, S = 96, 32
    q = torch.randn(L, 4, 128, generator=g).bfloat16().to(dev)
    k = torch.randn(L, 2, 128, generator=g).bfloat16().to(dev)
    v = torch.randn(L, 2, 128, generator=g).bfloat16().to(dev)
    cu = torch.tensor([0, L], dtype=torch.int32, device=dev)
    slots = (torch.arange(L, dtype=torch.int32) + 256).to(dev)          # page 1
    bt = torch.tensor([[1]], dtype=torch.int32, device=dev)
    lens = torch.tensor([L], dtype=torch.int32, device=dev)
    w = (1 + 0.1 * torch.randn(512, generator=g)).bfloat16().to(dev)
    head = (torch.randn(1000, 512, generator=g) * 0.3).bfloat16().to(dev)
    scale = 1 / math.sqrt(128)

    def step(mod, q, k, v, k_cache, v_cache, tokens):
        mod.store_kvcache(k, v, k_cache, v_cache, slots)
        o = mod.sparse_attn_varlen(q, k, v, cu, cu, S, L, scale)
        od = mod.paged_block_attn(q[-S:].unsqueeze(0), k_cache, v_cache, lens, bt, scale)
        x = o[-S:].reshape(1, S, 512)
        y, r = mod.add_rms_norm(x, od.reshape(1, S, 512), w, 1e-6)
        y = mod.rms_norm(mod.silu_and_mul(torch.cat([y, r], -1)), w, 1e-6)
        logits = torch.nn.functional.linear(y, head)
        x0, p, tr, cnt = mod.unmask_step(logits, tokens, 999, 0.9, 4, None)
        hx0, hp = mod.lm_head_confidence(y, head, None)           # hidden 512: a multiple of 128
        return o, od, y, x0, p, tr, cnt, hx0, hp

    class Direct:
        store_kvcache = staticmethod(mdx.store_kvcache)
        sparse_attn_varlen = staticmethod(lambda q, k, v, a, b, s, m, sc: mdx.sparse_attn_varlen(q, k, v, a, b, s, max_seqlen=m, softmax_scale=sc))
        paged_block_attn = staticmethod(lambda q, kc, vc, ln, t, sc: mdx.flash_attn_with_kvcache(
            q, kc, vc, cache_seqlens=ln, block_table=t, softmax_scale=sc, counters=False))
        add_rms_norm = staticmethod(lambda x, r, w_, e: mdx.rms_norm(x, w_, e, r))
        rms_norm = staticmethod(mdx.rms_norm)
        silu_and_mul = staticmethod(mdx.silu_and_mul)
        unmask_step = staticmethod(lambda lg, t, m, th, k_, tm: mdx.unmask_step(lg, t, m, th, k_, temperatures=tm))
        lm_head_confidence = staticmethod(mdx.lm_head_confidence)

    def fresh():
        return (torch.zeros(2, 256, 2, 128, dtype=torch.bfloat16, device=dev), torch.zeros(2, 256, 2, 128, dtype=torch.bfloat16, device=dev),
                torch.full((1, S), 999, dtype=torch.int64, device=dev))

    kc1, vc1, t1 = fresh()
    want = step(Direct, q, k, v, kc1, vc1, t1)
    kc2, vc2, t2 = fresh()
    traced = torch.compile(lambda *a: step(torch.ops.mdx, *a), backend="aot_eager", fullgraph=True)
    got = traced(q, k, v, kc2, vc2, t2)
    torch.cuda.synchronize()
    for a, b in zip(want, got):
        assert torch.equal(a, b)
    assert torch.equal(kc1, kc2) and torch.equal(vc1, vc2) and torch.equal(t1, t2)
    assert kc2[1, :L].abs().sum().item() > 0 and (t2 != 999).sum().item() >= 4
