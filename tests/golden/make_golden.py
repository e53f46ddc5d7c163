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
    np.savez_compressed(OUT / "staircase_attn.npz", q=bits(q), k=bits(k), v=bits(v), cu=np.array(cu, np.int32),
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
    np.savez_compressed(OUT / "paged_block_attn.npz", q=bits(qd), k_cache=bits(kc), v_cache=bits(vc), block_table=bt.numpy(),
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
    np.savez_compressed(OUT / "store_kvcache.npz", fused=bits(fused), slot_mapping=slot, k_cache=kcache, v_cache=vcache,
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
    np.savez_compressed(OUT / "unmask_step.npz", logits=bits(logits), tokens=tokens.numpy(), temperatures=temps,
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
    np.savez_compressed(OUT / "layer_ops.npz", x=bits(x), residual=bits(r), weight=bits(w), eps=np.float32(1e-6),
                        normed=bits(y), new_residual=bits(nr), normed_no_residual=bits(y0),
                        gate_up=bits(gu), act=bits(oracle.silu_and_mul(gu)))
    for f in sorted(OUT.glob("*.npz")):
        print(f.name, f.stat().st_size, "bytes")


if __name__ == "__main__":
    main()
