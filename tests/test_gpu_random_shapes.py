"""GPU parity on randomly drawn (but fixed-seed) shapes: batch sizes, lengths, head layouts, block
and page sizes that the parametrised tests do not name one by one.  Every case is checked against
the fp32 oracle (max-abs 2e-2) and, for the paged kernel, the one-launch call against the
two-launch call bit for bit."""
import math

import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu
TOL = 2e-2
HEADS = [(16, 8), (8, 8), (4, 1), (6, 3), (3, 1), (2, 1), (12, 4)]


def test_prefill_random_shapes(dev):
    import mdx
    rng = np.random.default_rng(2024)
    for case in range(36):
        dtype = torch.bfloat16 if case < 24 else torch.float16     # the reference kernel computes in q's dtype
        hq, hkv = HEADS[rng.integers(len(HEADS))]
        S = int(2 ** rng.integers(0, 8))
        B = int(rng.integers(1, 7))
        lens = [int(x) for x in rng.integers(0, 400, B)]
        if case % 4 == 0 or case >= 30:
            lens[rng.integers(B)] = int(rng.integers(400, 1500))
        if sum(lens) == 0:
            lens[0] = 5
        g = torch.Generator().manual_seed(1000 + case)
        N = sum(lens)
        q = torch.randn(N, hq, 128, generator=g).to(dtype)
        k = torch.randn(N, hkv, 128, generator=g).to(dtype)
        v = torch.randn(N, hkv, 128, generator=g).to(dtype)
        cu = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32)
        print(f"prefill case {case}: {dtype} heads {hq}/{hkv} S {S} lens {lens}", flush=True)
        o = mdx.sparse_attn_varlen(q.to(dev), k.to(dev), v.to(dev), cu.to(dev), cu.to(dev), S)
        torch.cuda.synchronize()
        ref = oracle.staircase_attn_varlen(q, k, v, cu, S)
        err = (o.float().cpu() - ref).abs().max().item()
        assert err < TOL, f"case {case}: max-abs {err} (heads {hq}/{hkv}, S {S}, lens {lens})"
        # a looser (still valid) length bound changes the launch grid and, for short batches, the kernel that runs
        o2 = mdx.sparse_attn_varlen(q.to(dev), k.to(dev), v.to(dev), cu.to(dev), cu.to(dev), S, max_seqlen=max(1024, max(lens)))
        torch.cuda.synchronize()
        err2 = (o2.float().cpu() - ref).abs().max().item()
        assert err2 < TOL, f"case {case}: max-abs {err2} with a bound of {max(1024, max(lens))}"


def test_paged_random_shapes(dev):
    import mdx
    rng = np.random.default_rng(4048)
    for case in range(40):
        hq, hkv = HEADS[rng.integers(len(HEADS))]
        page = int(rng.choice([32, 64, 128, 256, 512, 96]))
        sq = int(rng.choice([32, 32, 32, 1, 7, 16])) if case < 28 else int(rng.choice([33, 48, 64, 96, 100, 128]))    # blocks of up to 128 positions
        bs = int(rng.choice([1, 2, 3, 5, 8, 13, 24, 32, 40, 64, 70]))
        top = int(rng.choice([200, 700, 2500]))
        ctxs = [int(x) for x in rng.integers(0, top, bs)]
        if case % 3 == 0:
            ctxs[rng.integers(bs)] = int(rng.integers(top, 4 * top))
        if max(ctxs) == 0:
            ctxs[0] = 3
        extra = int(rng.integers(0, 3))                         # unused table columns (-1)
        if case % 4 == 1:
            extra += int(rng.integers(8, 48))                   # a table far wider than the contexts (the kernel then re-sizes the splits)
        pages = [(c + page - 1) // page for c in ctxs]
        pool = sum(pages) + 3
        g = torch.Generator().manual_seed(2000 + case)
        q = torch.randn(bs, sq, hq, 128, generator=g).bfloat16()
        kc = torch.randn(pool, page, hkv, 128, generator=g).bfloat16()
        vc = torch.randn(pool, page, hkv, 128, generator=g).bfloat16()
        perm = torch.randperm(pool, generator=g)
        bt = torch.full((bs, max(1, max(pages)) + extra), -1, dtype=torch.int32)
        at = 0
        for b, n in enumerate(pages):
            bt[b, :n] = perm[at:at + n].to(torch.int32)
            at += n
        lens = torch.tensor(ctxs, dtype=torch.int32)
        scale = 1 / math.sqrt(128)
        print(f"paged case {case}: heads {hq}/{hkv} page {page} sq {sq} bs {bs} max ctx {max(ctxs)} width {bt.shape[1]}", flush=True)
        args = (q.to(dev), kc.to(dev), vc.to(dev))
        kw = dict(cache_seqlens=lens.to(dev), block_table=bt.to(dev), softmax_scale=scale, causal=False)
        own = torch.zeros(8192, dtype=torch.float32, device=dev)
        one = mdx.flash_attn_with_kvcache(*args, **kw, counters=own)
        two = mdx.flash_attn_with_kvcache(*args, **kw, counters=False)
        torch.cuda.synchronize()
        ref = oracle.paged_block_attn(q, kc, vc, bt, lens, scale)
        err = (two.float().cpu() - ref).abs().max().item()
        assert err < TOL, f"case {case}: max-abs {err}"
        assert torch.equal(one, two), f"case {case}: one launch differs from two"
        assert own.abs().sum().item() == 0


def test_prefill_random_shapes_with_many_sequences(dev):
    """65 to 600 sequences per launch (the lookup of a workgroup's row group then walks them 64 at a time), lengths
    from empty to a few row groups, occasionally one long sequence; both kernels (even and odd head ratios)."""
    import mdx
    rng = np.random.default_rng(909)
    for case in range(10):
        hq, hkv = HEADS[rng.integers(len(HEADS))]
        S = int(rng.choice([4, 32, 32, 64, 128]))
        B = int(rng.choice([65, 100, 128, 129, 257, 400, 600]))
        top = int(rng.choice([40, 150, 500]))
        lens = [int(x) for x in rng.integers(0, top, B)]
        if case % 3 == 0:
            lens[rng.integers(B)] = int(rng.integers(600, 1400))
        g = torch.Generator().manual_seed(3000 + case)
        N = sum(lens)
        q = torch.randn(N, hq, 128, generator=g).bfloat16()
        k = torch.randn(N, hkv, 128, generator=g).bfloat16()
        v = torch.randn(N, hkv, 128, generator=g).bfloat16()
        cu = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32)
        print(f"many-sequence case {case}: heads {hq}/{hkv} S {S} B {B} tokens {N} longest {max(lens)}", flush=True)
        o = mdx.sparse_attn_varlen(q.to(dev), k.to(dev), v.to(dev), cu.to(dev), cu.to(dev), S, max_seqlen=max(lens))
        torch.cuda.synchronize()
        ref = oracle.staircase_attn_varlen(q, k, v, cu, S)
        err = (o.float().cpu() - ref).abs().max().item()
        assert err < TOL, f"case {case}: max-abs {err}"


def test_fused_head_random_shapes(dev):
    """Random row counts, vocabulary sizes (tile edges on both axes), hidden sizes, row strides, temperatures and
    compacted rows: tokens equal to the oracle's on bf16(x @ W.T) up to near-ties of one bf16 step at the maximum."""
    import mdx
    rng = np.random.default_rng(31337)
    for case in range(14):
        rows = int(rng.choice([1, 5, 31, 64, 130, 255, 256, 257, 300, 513, 700]))
        vocab = int(rng.choice([1, 100, 128, 129, 255, 256, 257, 1000, 4097, 20000]))
        hidden = int(rng.choice([128, 256, 384, 1024, 2048]))
        xs, ws = hidden + int(rng.choice([0, 8, 64])), hidden + int(rng.choice([0, 16]))
        g = torch.Generator().manual_seed(7000 + case)
        xbuf = torch.randn(rows, xs, generator=g).bfloat16()
        wbuf = (torch.randn(vocab, ws, generator=g) * (3.0 / hidden ** 0.5)).bfloat16()
        x, w = xbuf[:, :hidden], wbuf[:, :hidden]
        n_temp = int(rng.choice([0, 1, 3]))
        print(f"fused head case {case}: rows {rows} vocab {vocab} hidden {hidden} strides {xs}/{ws} temps {n_temp}", flush=True)
        logits = (x.float() @ w.float().T).bfloat16().to(torch.float64).numpy()
        if n_temp == 0:
            x0, p = mdx.lm_head_confidence(xbuf.to(dev)[:, :hidden], wbuf.to(dev)[:, :hidden])
            scaled = logits
        else:
            temps = torch.tensor(rng.uniform(0.5, 2.0, n_temp), dtype=torch.float32)
            ids = torch.tensor(np.sort(rng.choice(n_temp * 16, size=rows, replace=rows > n_temp * 16)), dtype=torch.int64)
            x0, p = mdx.lm_head_confidence(xbuf.to(dev)[:, :hidden], wbuf.to(dev)[:, :hidden], temps.to(dev), rows_per_temp=16, row_ids=ids.to(dev))
            scaled = (logits.astype(np.float32) / temps.numpy()[ids.numpy() // 16][:, None]).astype(np.float64)
        torch.cuda.synchronize()
        ex0 = scaled.argmax(-1)
        e = np.exp(scaled - scaled.max(-1, keepdims=True))
        ep = e[np.arange(rows), ex0] / e.sum(-1)
        got = x0.cpu().numpy()
        top = logits[np.arange(rows), logits.argmax(-1)]
        step = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(top), 2.0 ** -100))) - 7)
        same = got == ex0
        assert np.all(same | (logits[np.arange(rows), got] >= top - step)), f"case {case}: a pick that is not a near-tie of the maximum"
        if rows >= 64:
            assert same.mean() > 0.95
        # a logit one bf16 step off (another order of summation, a sum on a rounding boundary) moves a probability by up to
        # exp(step / T) - 1 of itself: the tolerance of a row follows from its own largest logit and temperature
        T_row = np.ones(rows) if n_temp == 0 else temps.numpy()[ids.numpy() // 16].astype(np.float64)
        tol = np.expm1(step / T_row) * 1.1 + 1e-4
        rel = np.abs(p.cpu().numpy() - ep) / ep
        assert np.all(rel[same] <= tol[same]), f"case {case}: confidence off by {rel[same].max()} (allowed {tol[same][rel[same].argmax()]})"


def test_filter_and_seeded_sampling_random_shapes(dev):
    """Random vocabulary sizes, row counts, alignments (rows that start off a 16-byte boundary), dtypes, temperatures
    and filter settings: the filtered logits against the oracle's (rows whose top-p cut-off hinges on rounding aside),
    and the step with noise drawn in the kernel against the step fed the same noise as a tensor (tokens bit for bit)."""
    import mdx
    rng = np.random.default_rng(777)
    checked = 0
    for case in range(20):
        V = int(rng.choice([3, 17, 100, 1000, 4097, 30000, 151936]))
        bs, S = int(rng.integers(1, 5)), int(rng.choice([1, 4, 32]))
        rows = bs * S
        dtype = torch.bfloat16 if case % 3 else torch.float16
        pad = int(rng.integers(0, 8))                                   # row stride V + pad: most rows unaligned
        g = torch.Generator().manual_seed(5000 + case)
        buf = (torch.randn(rows, V + pad, generator=g) * float(rng.uniform(0.5, 4.0))).to(dtype)
        logits = buf[:, :V]
        temps = torch.tensor(rng.uniform(0.5, 2.0, bs), dtype=torch.float32)
        k = int(rng.choice([0, 0, 1, 5, 50])) if V > 60 else int(rng.choice([0, 1, 2]))
        p = float(rng.choice([1.0, 0.95, 0.7, 0.3]))
        seed, offset = int(rng.integers(0, 2 ** 40)), int(rng.integers(0, 2 ** 34))
        print(f"case {case}: V {V} bs {bs} S {S} {dtype} pad {pad} top_k {k} top_p {p}", flush=True)
        d = buf.to(dev)[:, :V]
        f = mdx.filter_logits(d, top_k=k, top_p=p, temperatures=temps.to(dev))
        torch.cuda.synchronize()
        x = logits.to(torch.float64).numpy()
        T = np.repeat(temps.numpy().astype(np.float64), S)
        want = oracle.filter_logits(x, top_k=k, top_p=p, temperatures=T)
        got = f.to(torch.float64).cpu().numpy()
        for r in range(rows):
            if not np.array_equal(got[r], want[r]):                     # allowed only where a cumulative probability touches p
                kept = x[r][np.isfinite(oracle.filter_logits(x[r:r + 1], top_k=k)[0])] / T[r]
                vals, counts = np.unique(kept, return_counts=True)
                mass = counts * np.exp(vals - vals[-1])
                cum = np.cumsum(mass[::-1]) / mass.sum()
                assert p < 1.0 and np.abs(cum - p).min() <= 2e-5, f"case {case} row {r}: kept set differs away from a rounding boundary"
            else:
                checked += 1
        tokens = torch.where(torch.rand(bs, S, generator=g) < 0.7, torch.tensor(V + 5), torch.randint(0, V, (bs, S), generator=g))
        t1, t2 = tokens.clone().to(dev), tokens.clone().to(dev)
        a = mdx.unmask_step(f.view(bs, S, V), t1, V + 5, 0.4, 2, temps.to(dev), seed=seed, offset=offset)
        noise = mdx.gumbel_noise(rows, V, seed, offset, device=dev).view(bs, S, V)
        b = mdx.unmask_step(f.view(bs, S, V), t2, V + 5, 0.4, 2, temps.to(dev), noise=noise)
        torch.cuda.synchronize()
        assert torch.equal(a[0], b[0]) and torch.equal(a[2], b[2]) and torch.equal(t1, t2)
        torch.testing.assert_close(a[1], b[1], rtol=3e-6, atol=0)
        kept_mask = torch.isfinite(f.float()).view(bs, S, V)
        assert bool(kept_mask.gather(-1, a[0].unsqueeze(-1)).all())      # a drawn token is always one that survived the filter
    assert checked > 100


def test_fp32_arithmetic_attention_random_shapes(dev):
    """Both attention calls on element types and head widths that run in fp32 arithmetic (fp32 tensors; 16-bit tensors
    whose head is wider than 128 columns or not a multiple of 16): random batches, lengths, head layouts, staircase,
    block and page sizes.  fp32 tensors within 3e-5 of the fp32 oracle, 16-bit ones within their output rounding."""
    import mdx
    rng = np.random.default_rng(777)
    widths16 = [8, 24, 40, 72, 100, 136, 160, 200, 256]
    for case in range(30):
        if case % 3 == 0:
            dtype, d = torch.float32, int(rng.choice([4, 32, 64, 96, 128, 192, 256]))
        else:
            dtype, d = (torch.bfloat16 if case % 3 == 1 else torch.float16), int(rng.choice(widths16))
        tol = 3e-5 if dtype == torch.float32 else 1e-2
        hq, hkv = HEADS[rng.integers(len(HEADS))]
        g = torch.Generator().manual_seed(5000 + case)
        # prefill
        S = int(2 ** rng.integers(0, 8))
        B = int(rng.integers(1, 5))
        lens = [int(x) for x in rng.integers(0, 300, B)]
        if sum(lens) == 0:
            lens[0] = 7
        N = sum(lens)
        q = torch.randn(N, hq, d, generator=g).to(dtype)
        k = torch.randn(N, hkv, d, generator=g).to(dtype)
        v = torch.randn(N, hkv, d, generator=g).to(dtype)
        cu = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32)
        print(f"case {case}: {dtype} d {d} heads {hq}/{hkv} S {S} lens {lens}", flush=True)
        o = mdx.sparse_attn_varlen(q.to(dev), k.to(dev), v.to(dev), cu.to(dev), cu.to(dev), S)
        torch.cuda.synchronize()
        err = (o.float().cpu() - oracle.staircase_attn_varlen(q, k, v, cu, S)).abs().max().item()
        assert err < tol, f"prefill case {case}: max-abs {err}"
        # paged
        page = int(rng.choice([32, 64, 256]))
        sq = int(rng.integers(1, 70))
        ctxs = [int(x) for x in rng.integers(0, 700, int(rng.integers(1, 5)))]
        maxp = max(1, max((c + page - 1) // page for c in ctxs))
        pool = sum((c + page - 1) // page for c in ctxs) + 3
        qp = torch.randn(len(ctxs), sq, hq, d, generator=g).to(dtype)
        kc = torch.randn(pool, page, hkv, d, generator=g).to(dtype)
        vc = torch.randn(pool, page, hkv, d, generator=g).to(dtype)
        perm = torch.randperm(pool, generator=g)
        bt = torch.full((len(ctxs), maxp), -1, dtype=torch.int32)
        at = 0
        for b, c in enumerate(ctxs):
            n = (c + page - 1) // page
            bt[b, :n] = perm[at:at + n].to(torch.int32)
            at += n
        lens_d = torch.tensor(ctxs, dtype=torch.int32)
        print(f"case {case}: paged sq {sq} page {page} ctxs {ctxs}", flush=True)
        od = mdx.flash_attn_with_kvcache(qp.to(dev), kc.to(dev), vc.to(dev), cache_seqlens=lens_d.to(dev), block_table=bt.to(dev),
                                         softmax_scale=1 / math.sqrt(d), causal=False)
        torch.cuda.synchronize()
        err = (od.float().cpu() - oracle.paged_block_attn(qp, kc, vc, bt, lens_d, 1 / math.sqrt(d))).abs().max().item()
        assert err < tol, f"paged case {case}: max-abs {err}"
