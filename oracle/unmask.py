"""Oracle: the per-block confidence unmask step.  Test infrastructure only.

Reference followed:
  engines/nano_dvlm/nanovllm/layers/sampler.py:11-61            (engine variant)
  mineru_diffusion/modeling_mineru_diffusion.py:518-532,602-623,702-719 (HF variant)
"""
from __future__ import annotations

import numpy as np


def num_transfer_tokens(block_length: int, steps: int) -> list[int]:
    """modeling_mineru_diffusion.py:617-623: block_length split over steps, the
    remainder given to the first steps."""
    base, rem = divmod(block_length, steps)
    return [base + (1 if i < rem else 0) for i in range(steps)]


def confidence_argmax(logits: np.ndarray, temperatures=None, noise: np.ndarray | None = None):
    """logits [bs, S, V] (any float dtype, already widened to >= fp32 by the caller),
    temperatures [bs] or None (= 1) -> (x0 int64 [bs, S], x0_p float64 [bs, S]).

    sampler.py:13  l = logits.float() / T          (fp32 division)
    sampler.py:15-18  x0 = argmax(l + noise); noise is an explicit input here,
                      None = plain argmax (first index on ties, as torch.argmax)
    sampler.py:20-21  x0_p = softmax(l)[x0]        (summed in fp64 here)
    """
    l32 = np.asarray(logits, dtype=np.float32)
    if temperatures is not None:
        t = np.asarray(temperatures, dtype=np.float32).reshape(-1, 1, 1)
        l32 = (l32 / t).astype(np.float32)
    pick = l32 if noise is None else (l32 + np.asarray(noise, dtype=np.float32)).astype(np.float32)
    x0 = pick.argmax(axis=-1).astype(np.int64)          # numpy: first occurrence
    l64 = l32.astype(np.float64)
    m = l64.max(axis=-1, keepdims=True)
    e = np.exp(l64 - m)
    chosen = np.take_along_axis(e, x0[..., None], axis=-1)[..., 0]
    return x0, chosen / e.sum(axis=-1)


_PHILOX_M0, _PHILOX_M1 = 0xD2511F53, 0xCD9E8D57
_PHILOX_W0, _PHILOX_W1 = 0x9E3779B9, 0xBB67AE85


def philox4x32_10(counter, key):
    """Philox-4x32 with 10 rounds (Salmon, Moraes, Dror, Shaw: "Parallel random numbers: as easy as 1, 2, 3",
    SC 2011; the generator of the Random123 library): counter = 4 arrays of uint32, key = 2 uint32 ->
    4 arrays of uint32.  A round maps (c0, c1, c2, c3) to (hi(M1 c2) ^ c1 ^ k0, lo(M1 c2), hi(M0 c0) ^ c3 ^ k1,
    lo(M0 c0)); the key is bumped by the Weyl constants between rounds."""
    c = [np.asarray(x, dtype=np.uint64) & 0xFFFFFFFF for x in counter]
    k0, k1 = int(key[0]) & 0xFFFFFFFF, int(key[1]) & 0xFFFFFFFF
    for _ in range(10):
        p0 = _PHILOX_M0 * c[0]
        p1 = _PHILOX_M1 * c[2]
        c = [(p1 >> 32) ^ c[1] ^ k0, p1 & 0xFFFFFFFF, (p0 >> 32) ^ c[3] ^ k1, p0 & 0xFFFFFFFF]
        k0 = (k0 + _PHILOX_W0) & 0xFFFFFFFF
        k1 = (k1 + _PHILOX_W1) & 0xFFFFFFFF
    return [x.astype(np.uint32) for x in c]


def gumbel_noise(rows: int, vocab: int, seed: int, offset: int = 0, row_ids=None) -> np.ndarray:
    """The noise that the library's in-kernel generator stands for, [rows, vocab] float64:
    sampler.py:15-16 draws gumbel = -log(Exponential(1)); here element (row, column) takes output
    column % 4 of Philox-4x32-10 with key = (seed low, seed high) and counter = (column // 4, row,
    offset low, offset high), turns its 32 bits r into u = ((r >> 9) + 1/2) / 2^23 in (0, 1),
    e = -ln u (a unit exponential) and returns -ln e."""
    rid = np.arange(rows, dtype=np.uint64) if row_ids is None else np.asarray(row_ids, dtype=np.uint64)
    groups = (vocab + 3) // 4
    g = np.arange(groups, dtype=np.uint64)
    c0 = np.broadcast_to(g[None, :], (rows, groups))
    c1 = np.broadcast_to(rid[:, None], (rows, groups))
    off = int(offset) & (2 ** 64 - 1)
    c2 = np.full((rows, groups), off & 0xFFFFFFFF, dtype=np.uint64)
    c3 = np.full((rows, groups), off >> 32, dtype=np.uint64)
    out = philox4x32_10((c0, c1, c2, c3), (int(seed) & 0xFFFFFFFF, (int(seed) >> 32) & 0xFFFFFFFF))
    bits = np.stack(out, axis=-1).reshape(rows, groups * 4)[:, :vocab]
    u = ((bits >> 9).astype(np.float64) + 0.5) / 2.0 ** 23
    return -np.log(-np.log(u))


def filter_logits(logits: np.ndarray, top_k: int = 0, top_p: float = 1.0, temperatures=None) -> np.ndarray:
    """logits [rows, V] -> float64 copy with the filtered-out elements at -inf.

    modeling_mineru_diffusion.py:608-611  top-k first (if top_k > 0), then top-p (if top_p < 1)
    :585-590  top-k: elements below the k-th largest VALUE go (elements equal to it stay)
    :593-600  top-p: sort descending, cumulative softmax; an element goes when the cumulative
              probability BEFORE it already exceeds p (the crossing element stays, the first always)
    :606      the probabilities are those of logits / T

    Defined here where the reference leaves it open: among equal values at the top-p cut-off the
    reference's (unstable) sort order decides which stay; here all of them stay, so both filters
    are "keep x >= one value of the row".  temperatures: scalar or one per row."""
    x = np.asarray(logits, dtype=np.float64)
    rows, V = x.shape
    T = np.ones(rows) if temperatures is None else np.broadcast_to(np.asarray(temperatures, dtype=np.float64).reshape(-1), (rows,))
    out = x.copy()
    for r in range(rows):
        keep = np.ones(V, dtype=bool)
        if 0 < top_k < V:
            kth = np.sort(x[r])[V - top_k]
            keep &= x[r] >= kth
        if top_p < 1.0 and np.isfinite(x[r].max()):
            kept = np.sort(x[r][keep])[::-1] / T[r]
            pr = np.exp(kept - kept[0])
            cum = np.cumsum(pr / pr.sum())
            over = np.nonzero(cum > top_p)[0]
            cut = kept[over[0]] if len(over) else kept[-1]
            keep &= x[r] / T[r] >= cut
        out[r, ~keep] = -np.inf
    return out


def select_transfer(conf: np.ndarray, masked: np.ndarray, threshold: float, k: int) -> np.ndarray:
    """conf [bs, S] float, masked [bs, S] bool -> transfer [bs, S] bool.

    confidence = where(masked, conf, -inf)            (modeling:708, sampler.py:39)
    hi = confidence > threshold (strict)              (modeling:526, sampler.py:44)
    if hi.sum() >= k: commit all of hi                (modeling:527-529)
    else: commit the k most confident masked positions (modeling:530-531)

    Defined here where the reference leaves it open: among equal confidences the
    LOWER position wins, and at most #masked positions are committed (the
    reference's topk would otherwise return already-committed -inf positions);
    a masked position whose confidence is -inf (no softmax ever gives that) is
    never committed, so a caller can mark positions it has no confidence for.
    The engine variant (sampler.py:41-50: skip rows without masked positions,
    all of hi if any else top-1) is this rule with k = 1.
    """
    conf = np.asarray(conf)
    masked = np.asarray(masked, dtype=bool)
    out = np.zeros(conf.shape, dtype=bool)
    for b in range(conf.shape[0]):
        c = np.where(masked[b], conf[b].astype(np.float64), -np.inf)
        hi = c > threshold
        if hi.sum() >= k:
            out[b] = hi
            continue
        eligible = masked[b] & (c > -np.inf)
        want = min(k, int(eligible.sum()))
        taken = np.zeros_like(hi)
        for _ in range(want):
            best = -1
            for p in range(c.shape[0]):
                if eligible[p] and not taken[p] and (best < 0 or c[p] > c[best]):
                    best = p
            taken[best] = True
        out[b] = taken
    return out


def unmask_step(logits: np.ndarray, tokens: np.ndarray, mask_token_id: int, threshold: float, k: int,
                temperatures=None, noise=None):
    """One unmask step on identical logits: returns (x0, x0_p, transfer, new_tokens).
    masked = tokens == mask_token_id (sampler.py:32); x[transfer] = x0[transfer]
    (sampler.py:54, modeling:717)."""
    x0, x0_p = confidence_argmax(logits, temperatures, noise)
    masked = np.asarray(tokens) == mask_token_id
    transfer = select_transfer(x0_p.astype(np.float32), masked, threshold, k)
    new_tokens = np.where(transfer, x0, np.asarray(tokens)).astype(np.int64)
    return x0, x0_p, transfer, new_tokens
