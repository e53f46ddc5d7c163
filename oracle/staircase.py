"""Oracle: staircase (block-causal) attention, contiguous and paged.

Test infrastructure only (see the package docstring).  Reference followed:
  engines/nano_dvlm/nanovllm/kernels/triton/attention/block_prefill_attention_v2.py:46-53,82-102,134-156
  engines/nano_dvlm/nanovllm/layers/sdar_attention.py:48-56     (paged, non-causal decode call)
  mineru_diffusion/modeling_mineru_diffusion.py:189-206,450-478  (SDPA + boolean block mask)
"""
from __future__ import annotations

import numpy as np
import torch
import torch.nn.functional as F


def staircase_mask(L: int, S: int) -> np.ndarray:
    """Boolean [L, L] visibility; row = query, column = key.

    Restates the Triton kernel's index arithmetic
    (block_prefill_attention_v2.py:52-53 ``blocks``/``pad``; :98-102
    ``row_band``/``col_limit_abs``; :137-139 the compare): blocks of S tokens are
    RIGHT-aligned, the first block is the short one.
    """
    nb = (L + S - 1) // S
    pad = nb * S - L
    i = np.arange(L)[:, None]
    j = np.arange(L)[None, :]
    row_band = (i + pad) // S
    col_limit = (row_band + 1) * S - 1 - pad
    return (j <= col_limit) & (j < L)


def staircase_mask_tril(L: int, S: int) -> np.ndarray:
    """Same mask built the way the HF twin builds it
    (modeling_mineru_diffusion.py:450-453 tril of blocks, repeat_interleave;
    :462-464 keep the LAST L rows/columns).  Independent of ``staircase_mask``.
    """
    nb = (L + S - 1) // S
    blk = np.tril(np.ones((nb, nb), dtype=bool))
    full = np.repeat(np.repeat(blk, S, axis=0), S, axis=1)
    return full[nb * S - L:, nb * S - L:]


def staircase_pairs(L: int, S: int) -> int:
    """Number of visible (query, key) pairs of one sequence: f^2 + sum_b S*(f+S*b),
    f = size of the first (short) block."""
    if L == 0:
        return 0
    nb = (L + S - 1) // S
    f = L - (nb - 1) * S
    return f * f + sum(S * (f + S * b) for b in range(1, nb))


def masked_attention_f32(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                         mask: torch.Tensor | None, scale: float) -> torch.Tensor:
    """fp32 softmax attention with an explicit boolean mask and GQA.

    q [Lq, Hq, d], k/v [Lk, Hkv, d], mask [Lq, Lk] bool or None -> [Lq, Hq, d] fp32.
    This is the call the reference's HF path makes
    (modeling_mineru_diffusion.py:197-205: SDPA, ``attn_mask=bool``,
    ``scale=``, ``enable_gqa=True``), on CPU in fp32.
    """
    qf = q.detach().to("cpu", torch.float32).permute(1, 0, 2).unsqueeze(0)
    kf = k.detach().to("cpu", torch.float32).permute(1, 0, 2).unsqueeze(0)
    vf = v.detach().to("cpu", torch.float32).permute(1, 0, 2).unsqueeze(0)
    m = None if mask is None else torch.as_tensor(mask, dtype=torch.bool)[None, None]
    o = F.scaled_dot_product_attention(qf, kf, vf, attn_mask=m, scale=scale, enable_gqa=True)
    return o[0].permute(1, 0, 2).contiguous()


def attention_f64_explicit(q, k, v, mask, scale: float) -> np.ndarray:
    """Plain-loop fp64 softmax(QK^T * scale + mask) V with kv = h // (Hq/Hkv)
    (block_prefill_attention_v2.py:34).  Only for tiny shapes; pins
    ``masked_attention_f32``."""
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    Lq, Hq, d = q.shape
    Lk, Hkv, _ = k.shape
    g = Hq // Hkv
    out = np.zeros((Lq, Hq, d))
    for h in range(Hq):
        for i in range(Lq):
            s = np.array([q[i, h] @ k[j, h // g] * scale for j in range(Lk)])
            if mask is not None:
                s = np.where(np.asarray(mask)[i], s, -np.inf)
            p = np.exp(s - s.max())
            p /= p.sum()
            out[i, h] = sum(p[j] * v[j, h // g] for j in range(Lk))
    return out


def staircase_attn_varlen(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                          cu_seqlens, staircase_size: int, scale: float | None = None) -> torch.Tensor:
    """Packed varlen staircase attention, fp32 on CPU.

    q [N, Hq, d], k/v [N, Hkv, d], cu_seqlens [B+1]; mirrors
    ``sparse_attn_varlen`` (block_prefill_attention_v2.py:168-202; q_len == k_len,
    :48-50; scale = d^-0.5, :194).
    """
    cu = [int(x) for x in cu_seqlens]
    d = q.shape[-1]
    scale = d ** -0.5 if scale is None else scale
    out = torch.zeros(q.shape, dtype=torch.float32)
    for b in range(len(cu) - 1):
        s, e = cu[b], cu[b + 1]
        if e == s:
            continue
        mask = staircase_mask(e - s, staircase_size)
        out[s:e] = masked_attention_f32(q[s:e], k[s:e], v[s:e], mask, scale)
    return out


def paged_gather(cache: torch.Tensor, block_table_row, ctx: int) -> torch.Tensor:
    """cache [pages, page, Hkv, d] -> the first ``ctx`` rows of the sequence whose
    pages are ``block_table_row`` (token t lives in page block_table[t // page] at
    row t % page; engine/sequence.py:117-141, engine/model_runner.py:121-125)."""
    page = cache.shape[1]
    n = (ctx + page - 1) // page
    idx = torch.as_tensor([int(x) for x in block_table_row[:n]], dtype=torch.long)
    return cache[idx].reshape(n * page, *cache.shape[2:])[:ctx]


def paged_block_attn(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                     block_table, context_lens, scale: float) -> torch.Tensor:
    """Non-causal attention of the Sq queries of each sequence over the first
    context_lens[b] cached keys (sdar_attention.py:50-55 with causal=False).
    q [bs, Sq, Hq, d] -> fp32 [bs, Sq, Hq, d].  Rows with context_lens == 0
    (graph padding, model_runner.py:205-208) produce zeros."""
    bs = q.shape[0]
    out = torch.zeros(q.shape, dtype=torch.float32)
    for b in range(bs):
        ctx = int(context_lens[b])
        if ctx == 0:
            continue
        kk = paged_gather(k_cache, block_table[b], ctx)
        vv = paged_gather(v_cache, block_table[b], ctx)
        out[b] = masked_attention_f32(q[b], kk, vv, None, scale)
    return out
