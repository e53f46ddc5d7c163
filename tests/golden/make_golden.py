"""Writes the small fixtures of this folder (run from the repository root: python tests/golden/make_golden.py).

The reference ships no tests, fixtures or known-answer vectors for this path, and nothing of it was
imported to make these: the expected outputs come from this repository's own CPU oracle (oracle/),
whose functions are pinned by closed forms and library routines in tests/test_oracle_*.py.  The
fixtures freeze those answers as data, so that (a) a later change of the oracle that alters an
answer is caught by tests/test_golden.py on the CPU, and (b) the HIP kernels are checked against
numbers that do not depend on the oracle's code at test time.

bf16 tensors are stored as their uint16 bit patterns (numpy has no bf16)."""
import math
import pathlib
import sys

import numpy as np
import torch

ROOT = pathlib.Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))
import oracle  # noqa: E402

OUT = pathlib.Path(__file__).resolve().parent


def bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


ONLY = set(sys.argv[1:])          # python tests/golden/make_golden.py [name.npz ...]: write only these (default: all)


def save(name, **arrays):
    if not ONLY or name in ONLY:
        np.savez_compressed(OUT / name, **arrays)


def main():
    g = torch.Generator().manual_seed(20240607)
    d = 128

    # ---- staircase block-prefill attention: two packed sequences, lengths not multiples of the block
    lens, hq, hkv, S = [70, 45], 2, 1, 32
    N = sum(lens)
    q = torch.randn(N, hq, d, generator=g).bfloat16()
    k = torch.randn(N, hkv, d, generator=g).bfloat16()
    v = torch.randn(N, hkv, d, generator=g).bfloat16()
    cu = [0, lens[0], N]
    o = oracle.staircase_attn_varlen(q, k, v, cu, S)
    save("staircase_attn.npz", q=bits(q), k=bits(k), v=bits(v), cu=np.array(cu, np.int32),
                        block=np.int32(S), o=o.float().numpy().astype(np.float32))

    # ---- paged single-block attention: contexts of 1, 40 and 270 keys, pages of 32, one padding row
    page, pool, sq = 32, 12, 32
    ctxs = [40, 0, 270, 1]
    qd = torch.randn(len(ctxs), sq, hq, d, generator=g).bfloat16()
    kc = torch.randn(pool, page, hkv, d, generator=g).bfloat16()
    vc = torch.randn(pool, page, hkv, d, generator=g).bfloat16()
    perm = torch.randperm(pool, generator=g)
    maxp = max((c + page - 1) // page for c in ctxs)
    bt = torch.full((len(ctxs), maxp), -1, dtype=torch.int32)
    at = 0
    for b, c in enumerate(ctxs):
        n = (c + page - 1) // page
        bt[b, :n] = perm[at:at + n].to(torch.int32)
        at += n
    lens_t = torch.tensor(ctxs, dtype=torch.int32)
    od = oracle.paged_block_attn(qd, kc, vc, bt, lens_t, 1 / math.sqrt(d))
    save("paged_block_attn.npz", q=bits(qd), k_cache=bits(kc), v_cache=bits(vc), block_table=bt.numpy(),
                        context_lens=lens_t.numpy(), o=od.float().numpy().astype(np.float32))

    # ---- store_kvcache: 9 tokens into 3 pages of 8 slots, two skipped, V a strided view of a fused projection
    n_tok, pages, page_len = 9, 3, 8
    fused = torch.randn(n_tok, 3 * hkv * d, generator=g).bfloat16()
    key = bits(fused[:, :hkv * d]).reshape(n_tok, hkv, d)
    val = bits(fused[:, 2 * hkv * d:]).reshape(n_tok, hkv, d)
    slot = np.array([5, -1, 23, 0, 7, -1, 12, 1, 16], dtype=np.int32)
    kcache = bits(torch.randn(pages, page_len, hkv, d, generator=g).bfloat16())
    vcache = bits(torch.randn(pages, page_len, hkv, d, generator=g).bfloat16())
    k_after, v_after = kcache.copy(), vcache.copy()
    oracle.store_kvcache(key, val, k_after, v_after, slot)
    save("store_kvcache.npz", fused=bits(fused), slot_mapping=slot, k_cache=kcache, v_cache=vcache,
                        k_after=k_after, v_after=v_after, hkv=np.int32(hkv))

    # ---- unmask step: 3 sequences x 32 positions x 1000 logits; one sequence has peaked rows so that
    #      the threshold branch fires; k = 4, threshold 0.9, temperatures 1 and 0.7
    V, bs, mask_id = 1000, 3, 999
    logits = (torch.randn(bs, 32, V, generator=g) * 3).bfloat16()
    logits[1, :12, 17] += 15.0                                  # confident rows
    logits[:, :, mask_id] = -30.0                               # the mask token is never the argmax
    tokens = torch.randint(0, 900, (bs, 32), generator=g, dtype=torch.int64)
    for b, n_masked in enumerate((32, 20, 3)):
        tokens[b, torch.randperm(32, generator=g)[:n_masked]] = mask_id
    temps = np.array([1.0, 0.7, 1.0], dtype=np.float32)
    x0, x0_p, transfer, after = oracle.unmask_step(logits.float().numpy(), tokens.numpy(), mask_id, 0.9, 4, temperatures=temps)
    # the fixture must not sit on a tie: k-th and (k+1)-th confidence apart, nothing near the threshold
    conf = np.where(tokens.numpy() == mask_id, x0_p, -1.0)
    for b in range(bs):
        c = np.sort(conf[b][conf[b] >= 0])[::-1]
        assert np.all(np.abs(c - 0.9) > 1e-3) and (len(c) <= 4 or c[3] - c[4] > 1e-4), "fixture sits on a tie: change the seed"
    save("unmask_step.npz", logits=bits(logits), tokens=tokens.numpy(), temperatures=temps,
                        mask_id=np.int64(mask_id), threshold=np.float32(0.9), k=np.int32(4),
                        x0=x0.astype(np.int64), x0_p=x0_p.astype(np.float32), tokens_after=after.astype(np.int64),
                        transfer=transfer.astype(np.uint8), count=transfer.sum(-1).astype(np.int32))

    # ---- layer ops
    x = (torch.randn(5, 256, generator=g) * 3).bfloat16()
    r = (torch.randn(5, 256, generator=g) * 3).bfloat16()
    w = (torch.rand(256, generator=g) + 0.5).bfloat16()
    y, nr = oracle.add_rms_norm(x, r, w, 1e-6)
    y0, _ = oracle.add_rms_norm(x, None, w, 1e-6)
    gu = (torch.randn(5, 128, generator=g) * 4).bfloat16()
    save("layer_ops.npz", x=bits(x), residual=bits(r), weight=bits(w), eps=np.float32(1e-6),
                        normed=bits(y), new_residual=bits(nr), normed_no_residual=bits(y0),
                        gate_up=bits(gu), act=bits(oracle.silu_and_mul(gu)))
    # ---- sampling: top-k 20 then top-p 0.8 on 8 rows of 600 logits, then the step's Gumbel draw from (seed, offset);
    #      a generator of its own, so that the fixtures above keep their bytes
    g2 = torch.Generator().manual_seed(777002)
    V2 = 600
    lg = (torch.randn(2, 4, V2, generator=g2) * 2.5).bfloat16()
    t2 = np.array([0.8, 1.25], dtype=np.float32)
    seed, offset = 2 ** 33 + 12345, 2 ** 32 + 7
    x64 = lg.to(torch.float64).numpy().reshape(8, V2)
    T8 = np.repeat(t2.astype(np.float64), 4)
    kept_k = np.isfinite(oracle.filter_logits(x64, top_k=20))
    for r in range(8):                                           # no cumulative probability within 1e-3 of p: not a rounding matter
        vals = np.sort(x64[r][kept_k[r]])[::-1] / T8[r]
        pr = np.exp(vals - vals[0])
        assert np.abs(np.cumsum(pr / pr.sum()) - 0.8).min() > 1e-3, "fixture sits on the top-p boundary: change the seed"
    filt = oracle.filter_logits(x64, top_k=20, top_p=0.8, temperatures=T8)
    noise = oracle.gumbel_noise(8, V2, seed, offset)
    sx0, sp = oracle.confidence_argmax(filt.reshape(2, 4, V2), t2, noise.reshape(2, 4, V2))
    noisy = np.where(np.isfinite(filt), (filt.astype(np.float32) / T8[:, None].astype(np.float32)).astype(np.float64) + noise, -np.inf)
    top2 = np.sort(noisy, axis=-1)[:, -2:]
    assert np.all(top2[:, 1] - top2[:, 0] > 1e-3), "fixture sits on a tie of the noisy argmax: change the seed"
    save("sampling.npz", logits=bits(lg), temperatures=t2, top_k=np.int32(20), top_p=np.float32(0.8),
                        kept=np.isfinite(filt).astype(np.uint8), seed=np.uint64(seed), offset=np.uint64(offset),
                        noise=noise.astype(np.float32), x0=sx0.astype(np.int64), x0_p=sp.astype(np.float32))

    # ---- block state on the device: 5 lanes of 8 positions, pages of 16 tokens
    rng = np.random.default_rng(991)
    S8, page16, mask_id2 = 8, 16, 99
    lens5 = np.array([16, 40, 8, 0, 24], dtype=np.int32)
    phase5 = np.array([1, 2, 1, 0, 2], dtype=np.int32)          # denoising, caching, denoising, idle, caching
    bt5 = np.array([[3, 7, -1, -1], [1, 0, 5, 9], [2, 6, -1, -1], [-1, -1, -1, -1], [4, 8, 10, -1]], dtype=np.int32)
    pos5, slots5, ctx5 = oracle.block_prepare(lens5, phase5, bt5, page16, S8)
    tok5 = rng.integers(0, 90, (5, S8)).astype(np.int64)
    tok5[0, [1, 4, 6]] = mask_id2
    tok5[2, :] = mask_id2
    tok5[1, 3] = 55                                              # lane 1 (caching) holds its stop token
    rows5, n5 = oracle.masked_rows(tok5, phase5, mask_id2, 16)
    transfer5 = np.zeros((5, S8), dtype=np.uint8)
    transfer5[0, [1, 4, 6]] = 1                                  # lane 0 commits its last three positions -> caching
    transfer5[2, [0, 5]] = 1
    tok_sel = tok5.copy()
    tok_sel[0, [1, 4, 6]] = [11, 12, 13]
    tok_sel[2, [0, 5]] = [21, 22]
    step_map5 = rng.integers(0, 3, (5, S8)).astype(np.int32)
    step5 = np.array([3, 8, 0, 0, 8], dtype=np.int32)
    first5 = np.array([8, 16, 8, 0, 8], dtype=np.int32)
    maxnew5 = np.array([64, 64, 64, 64, 24], dtype=np.int32)    # lane 4 reaches its budget with this block
    stop5 = np.array([[-1, -1], [55, -1], [-1, -1], [-1, -1], [77, -1]], dtype=np.int64)
    a_tok, a_map, a_step, a_phase, a_lens, appended, status = oracle.block_advance(
        tok_sel, transfer5, step_map5, step5, phase5, lens5, first5, maxnew5, stop5, mask_id2)
    out_tok = np.full((5, 64), -1, dtype=np.int64)
    out_step = np.full((5, 64), -1, dtype=np.int32)
    for b, ap in enumerate(appended):
        if ap is not None:
            at = int(lens5[b] - first5[b])
            out_tok[b, at:at + S8], out_step[b, at:at + S8] = ap
    st = np.array([[s[0], lens5[b] if s[1] is None else s[1], s[2], s[3]] for b, s in enumerate(status)], dtype=np.int32)
    save("block_state.npz", lens=lens5, phase=phase5, block_table=bt5, page=np.int32(page16), block_len=np.int32(S8),
                        positions=pos5, slot_mapping=slots5, context_lens=ctx5, mask_id=np.int64(mask_id2),
                        tokens=tok5, rows=rows5, n_rows=np.int32(n5), tokens_selected=tok_sel, transfer=transfer5,
                        step_map=step_map5, step=step5, first_len=first5, max_new=maxnew5, stop_ids=stop5,
                        tokens_after=a_tok, step_map_after=a_map, step_after=a_step, phase_after=a_phase, lens_after=a_lens,
                        out_tokens=out_tok, out_steps=out_step, status=st)
    for f in sorted(OUT.glob("*.npz")):
        print(f.name, f.stat().st_size, "bytes")


    # ---- vocabulary projection fused with the confidence reduction: operands whose products are exact in fp32 in any
    # order of summation (small integers), so that the logits -- and their bf16 rounding -- are the same numbers for every
    # implementation; a forced tie between two columns (first index wins), temperatures per group of 8 rows
    gh = torch.Generator().manual_seed(20240608)
    rows, vocab, hidden = 40, 300, 128
    xh = torch.randint(-2, 3, (rows, hidden), generator=gh).float().bfloat16()
    wh = torch.randint(-2, 3, (vocab, hidden), generator=gh).float().bfloat16()
    wh[250] = wh[17]
    temps = np.array([0.5, 0.8, 1.0, 1.25, 2.0], dtype=np.float32)
    logits = (xh.float() @ wh.float().T).bfloat16().to(torch.float64).numpy()
    assert np.abs(logits).max() < 256
    x0, p = oracle.confidence_argmax(logits.reshape(5, 8, vocab), temps)
    save("lm_head.npz", x=bits(xh), w=bits(wh), temperatures=temps, rows_per_temp=np.int32(8),
         x0=x0.reshape(-1).astype(np.int64), x0_p=p.reshape(-1).astype(np.float64))

if __name__ == "__main__":
    main()
