"""The reference's hot-path functions, same signatures, running in libmdx.so.

Tensors must live on the GPU; every kernel is enqueued on torch's current
stream, allocates nothing itself (outputs and workspaces come from torch's
caching allocator, so the calls are safe under graph capture) and never
synchronises.
"""
from __future__ import annotations

import math

import torch

from . import _lib
from ._lib import MdxError, check

_DTYPES = {torch.bfloat16: _lib.MDX_BF16, torch.float16: _lib.MDX_F16, torch.float32: _lib.MDX_F32}


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _need_gpu(*tensors: torch.Tensor) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise MdxError("mdx ops run on the GPU only: got a tensor on " + str(t.device))


def _i32(t: torch.Tensor, what: str) -> torch.Tensor:
    if t.dtype != torch.int32:
        raise MdxError(f"{what} must be int32, got {t.dtype}")
    return t if t.is_contiguous() else t.contiguous()


# --------------------------------------------------------------------------- store_kvcache
def store_kvcache(key: torch.Tensor, value: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                  slot_mapping: torch.Tensor) -> None:
    """nanovllm/layers/attention.py:33-40: key/value [N, Hkv, d] (row stride free, rows dense),
    caches [pages, page, Hkv, d], slot_mapping [N] int32 with -1 = skip.  In place."""
    _need_gpu(key, value, k_cache, v_cache, slot_mapping)
    N, num_heads, head_dim = key.shape
    D = num_heads * head_dim
    assert key.stride(-1) == 1 and value.stride(-1) == 1
    assert key.stride(1) == head_dim and value.stride(1) == head_dim
    assert k_cache.stride(1) == D and v_cache.stride(1) == D
    assert slot_mapping.numel() == N
    assert key.dtype == value.dtype == k_cache.dtype == v_cache.dtype
    assert k_cache.is_contiguous() and v_cache.is_contiguous()
    slots = _i32(slot_mapping, "slot_mapping")
    num_slots = k_cache.numel() // D
    rc = _lib.lib().mdx_store_kvcache(key.data_ptr(), value.data_ptr(), key.stride(0), value.stride(0),
                                      k_cache.data_ptr(), v_cache.data_ptr(), slots.data_ptr(),
                                      N, D, key.element_size(), num_slots, _stream(key))
    check(rc, "store_kvcache")


def store_kvcache_maybe4d(k, v, k_cache, v_cache, slot_mapping) -> None:
    """nanovllm/layers/sdar_attention.py:11-16: [b, s, h, d] inputs are flattened to [(b s), h, d]."""
    if k.dim() == 4:
        k = k.reshape(-1, k.shape[2], k.shape[3]) if k.is_contiguous() else k.flatten(0, 1)
        v = v.reshape(-1, v.shape[2], v.shape[3]) if v.is_contiguous() else v.flatten(0, 1)
        slot_mapping = slot_mapping.reshape(-1)
    store_kvcache(k, v, k_cache, v_cache, slot_mapping)


def qk_norm_rope_store(qkv: torch.Tensor, q_weight: torch.Tensor, k_weight: torch.Tensor, eps: float,
                       cos: torch.Tensor, sin: torch.Tensor, positions: torch.Tensor,
                       num_q_heads: int, num_kv_heads: int, head_dim: int,
                       k_cache: torch.Tensor | None = None, v_cache: torch.Tensor | None = None,
                       slot_mapping: torch.Tensor | None = None, want_k: bool = True):
    """One launch for nanovllm/models/sdar.py:79-83 plus the cache store: qkv [..., (Hq+2Hkv)*d]
    -> (q [..., Hq, d], k [..., Hkv, d] or None, v view [..., Hkv, d]); rotated k and raw v are
    written to the caches at slot_mapping when caches are given.  cos/sin: fp32 [max_pos, d/2]."""
    _need_gpu(qkv, q_weight, k_weight, cos, sin, positions, k_cache, v_cache, slot_mapping)
    lead = qkv.shape[:-1]
    width = (num_q_heads + 2 * num_kv_heads) * head_dim
    assert qkv.shape[-1] == width and qkv.stride(-1) == 1
    q2 = qkv.reshape(-1, width)
    n = q2.shape[0]
    pos = positions.reshape(-1)
    assert pos.numel() == n and pos.dtype == torch.int64 and cos.dtype == torch.float32 and sin.dtype == torch.float32
    pos = pos if pos.is_contiguous() else pos.contiguous()
    q = torch.empty((n, num_q_heads, head_dim), dtype=qkv.dtype, device=qkv.device)
    k = torch.empty((n, num_kv_heads, head_dim), dtype=qkv.dtype, device=qkv.device) if want_k else None
    slots = None
    num_slots = 0
    if k_cache is not None and k_cache.numel():
        assert k_cache.is_contiguous() and v_cache.is_contiguous()
        slots = _i32(slot_mapping.reshape(-1), "slot_mapping")
        assert slots.numel() == n
        num_slots = k_cache.numel() // (num_kv_heads * head_dim)
    else:
        k_cache = v_cache = None
    rc = _lib.lib().mdx_qk_norm_rope_store(
        q2.data_ptr(), q2.stride(0), q_weight.data_ptr(), k_weight.data_ptr(), float(eps),
        cos.data_ptr(), sin.data_ptr(), cos.shape[0], pos.data_ptr(),
        q.data_ptr(), q.stride(0), k.data_ptr() if k is not None else None, k.stride(0) if k is not None else 0,
        k_cache.data_ptr() if k_cache is not None else None, v_cache.data_ptr() if v_cache is not None else None,
        slots.data_ptr() if slots is not None else None, num_slots,
        n, num_q_heads, num_kv_heads, head_dim, _DTYPES[qkv.dtype], _stream(qkv))
    check(rc, "qk_norm_rope_store")
    v = qkv[..., (num_q_heads + num_kv_heads) * head_dim:].unflatten(-1, (num_kv_heads, head_dim))   # strided view
    return q.view(*lead, num_q_heads, head_dim), None if k is None else k.view(*lead, num_kv_heads, head_dim), v


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float, residual: torch.Tensor | None = None):
    """RMSNorm.forward (nanovllm/layers/layernorm.py:43-51): returns the normed x, or with a
    residual the pair (normed x + residual, x + residual), in one launch."""
    _need_gpu(x, weight, residual)
    hidden = x.shape[-1]
    assert x.stride(-1) == 1 and weight.shape == (hidden,) and weight.is_contiguous() and weight.dtype == x.dtype
    shape = x.shape
    x2 = x.reshape(-1, hidden)
    out = torch.empty((x2.shape[0], hidden), dtype=weight.dtype, device=x.device)
    r2 = r_out = None
    if residual is not None:
        assert residual.shape == shape and residual.dtype == weight.dtype and residual.stride(-1) == 1
        r2 = residual.reshape(-1, hidden)
        r_out = torch.empty_like(out)
    rc = _lib.lib().mdx_add_rms_norm(
        x2.data_ptr(), x2.stride(0),
        r2.data_ptr() if r2 is not None else None, r2.stride(0) if r2 is not None else 0,
        r_out.data_ptr() if r_out is not None else None, r_out.stride(0) if r_out is not None else 0,
        weight.data_ptr(), float(eps), out.data_ptr(), out.stride(0), x2.shape[0], hidden, _DTYPES[weight.dtype], _stream(x))
    check(rc, "rms_norm")
    if residual is None:
        return out.view(shape)
    return out.view(shape), r_out.view(shape)


def silu_and_mul(x: torch.Tensor) -> torch.Tensor:
    """SiluAndMul.forward (nanovllm/layers/activation.py:13-16): x [..., 2I] -> silu(x[..., :I]) * x[..., I:]."""
    _need_gpu(x)
    assert x.shape[-1] % 2 == 0 and x.stride(-1) == 1
    inter = x.shape[-1] // 2
    x2 = x.reshape(-1, 2 * inter)
    out = torch.empty((x2.shape[0], inter), dtype=x.dtype, device=x.device)
    rc = _lib.lib().mdx_silu_and_mul(x2.data_ptr(), x2.stride(0), out.data_ptr(), out.stride(0), x2.shape[0], inter,
                                     _DTYPES[x.dtype], _stream(x))
    check(rc, "silu_and_mul")
    return out.view(*x.shape[:-1], inter)


# --------------------------------------------------------------------------- staircase prefill
def sparse_attn_varlen(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cu_seqlens_q: torch.Tensor,
                       cu_seqlens_k: torch.Tensor, staircase_size: int = 4, *, max_seqlen: int | None = None,
                       softmax_scale: float | None = None) -> torch.Tensor:
    """block_prefill_attention_v2.py:168-202: q [N, Hq, d], k/v [N, Hkv, d] packed over
    sequences, cu_seqlens int32 [B+1], blocks of `staircase_size` right-aligned; returns o like q.
    max_seqlen (keyword, not in the reference) sizes the grid and must be >= the longest sequence:
    rows beyond it are not computed, and the lengths live on the device, so this call cannot check
    it.  None (the default) takes the total token count, which is always enough; the engine passes
    the value it computed on the host while building cu_seqlens (Context.max_seqlen_k)."""
    _need_gpu(q, k, v, cu_seqlens_q, cu_seqlens_k)
    assert q.dim() == k.dim() == v.dim() == 3
    assert q.shape[0] == k.shape[0] == v.shape[0]
    assert k.shape[1] == v.shape[1] and k.shape[2] == v.shape[2]
    assert q.shape[2] == k.shape[2]
    assert q.shape[1] % k.shape[1] == 0
    assert staircase_size in [1, 2, 4, 8, 16, 32, 64, 128]
    assert q.dtype == k.dtype == v.dtype
    total, hq, d = q.shape
    hkv = k.shape[1]
    # strided views (e.g. slices of a fused QKV projection) are read in place
    q, k, v = (t if t.stride(-1) == 1 else t.contiguous() for t in (q, k, v))
    o = torch.empty((total, hq, d), dtype=q.dtype, device=q.device)
    cu_q, cu_k = _i32(cu_seqlens_q, "cu_seqlens_q"), _i32(cu_seqlens_k, "cu_seqlens_k")
    batch = cu_k.numel() - 1
    scale = 1.0 / math.sqrt(d) if softmax_scale is None else float(softmax_scale)
    rc = _lib.lib().mdx_staircase_attn_varlen(
        q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(),
        q.stride(0), q.stride(1), k.stride(0), k.stride(1), v.stride(0), v.stride(1), o.stride(0), o.stride(1),
        cu_q.data_ptr(), cu_k.data_ptr(), batch, int(max_seqlen) if max_seqlen else total, total,
        hq, hkv, d, staircase_size, scale, _DTYPES[q.dtype], _stream(q))
    check(rc, "sparse_attn_varlen")
    return o


sparse_attn_varlen_v2 = sparse_attn_varlen


# --------------------------------------------------------------------------- paged decode
_arrival_counters: dict = {}          # (device index, stream) -> zeroed fp32 counters of the single-launch mode
_COUNTER_FLOATS = 64 * 256            # the single-launch path exists for up to 64 sequences; 256 head groups is far beyond any model


def _paged_counters(device: torch.device, n_bytes: int):
    """The arrival counters of mdx_paged_block_attn_single_launch that this module keeps: one buffer
    per device and stream, zero when created, left zero by every launch.  Launches on one stream run
    one after the other, so they can share a buffer; a HIP graph keeps using the buffer of the stream
    it was captured on wherever it is replayed, which is why a buffer, once handed out, is never
    replaced or freed: it has its full size from the start.  None when the request does not fit it,
    or while a graph is being captured and that stream has no buffer yet (it could not be zeroed
    outside the graph): the caller then takes the two-launch entry point -- run the forward once on
    the capture stream before capturing."""
    if n_bytes > _COUNTER_FLOATS * 4:
        return None
    index = device.index if device.index is not None else torch.cuda.current_device()
    key = (index, torch.cuda.current_stream(device).cuda_stream)
    buf = _arrival_counters.get(key)
    if buf is None:
        if torch.cuda.is_current_stream_capturing():
            return None
        buf = torch.zeros(_COUNTER_FLOATS, dtype=torch.float32, device=device)
        _arrival_counters[key] = buf
    return buf


def flash_attn_with_kvcache(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, *,
                            cache_seqlens: torch.Tensor, block_table: torch.Tensor,
                            softmax_scale: float | None = None, causal: bool = False,
                            counters: torch.Tensor | None | bool = None) -> torch.Tensor:
    """The subset of flash_attn.flash_attn_with_kvcache used at sdar_attention.py:50-55:
    q [bs, Sq, Hq, d], caches [pages, page, Hkv, d], block_table [bs, max_pages] int32,
    cache_seqlens [bs] int32, non-causal.  Returns o like q.

    counters (keyword, not in the reference): None = single launch with this module's arrival
    counters (one buffer per device and stream); a zeroed fp32 tensor of the caller's = single
    launch with those; False = attention launch + combine launch."""
    if causal:
        raise MdxError("flash_attn_with_kvcache: only causal=False (block-diffusion decode) is implemented")
    _need_gpu(q, k_cache, v_cache, cache_seqlens, block_table)
    assert q.dim() == 4 and k_cache.dim() == 4 and v_cache.shape == k_cache.shape
    assert q.dtype == k_cache.dtype == v_cache.dtype
    bs, sq, hq, d = q.shape
    num_pages, page, hkv, _ = k_cache.shape
    if q.stride(-1) != 1:
        q = q.contiguous()
    assert k_cache.stride(-1) == 1 and v_cache.stride() == k_cache.stride()
    bt, lens = _i32(block_table, "block_table"), _i32(cache_seqlens, "cache_seqlens")
    assert bt.dim() == 2 and bt.shape[0] == bs and lens.numel() == bs
    o = torch.empty((bs, sq, hq, d), dtype=q.dtype, device=q.device)
    L = _lib.lib()
    ws_bytes = L.mdx_paged_block_attn_workspace_bytes(bs, sq, hq, hkv, d, bt.shape[1], page)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=q.device)
    scale = 1.0 / math.sqrt(d) if softmax_scale is None else float(softmax_scale)
    args = (q.data_ptr(), o.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
            q.stride(0), q.stride(1), q.stride(2), o.stride(0), o.stride(1), o.stride(2),
            k_cache.stride(0), k_cache.stride(1), k_cache.stride(2),
            bt.data_ptr(), bt.stride(0), lens.data_ptr(),
            bs, sq, hq, hkv, d, bt.shape[1], page, num_pages, scale, _DTYPES[q.dtype],
            ws.data_ptr(), ws_bytes)
    if counters is None:               # more than 64 sequences never take the single-launch path
        counters = _paged_counters(q.device, L.mdx_paged_block_attn_counter_bytes(bs, hq, hkv)) if bs <= 64 else False
    if counters is None or counters is False:
        rc = L.mdx_paged_block_attn(*args, _stream(q))
    else:
        assert counters.dtype == torch.float32 and counters.is_contiguous() and counters.device == q.device
        rc = L.mdx_paged_block_attn_single_launch(*args, counters.data_ptr(), counters.numel() * 4, _stream(q))
    check(rc, "flash_attn_with_kvcache")
    return o


# --------------------------------------------------------------------------- unmask step
def _logits2d(logits: torch.Tensor) -> torch.Tensor:
    if logits.stride(-1) != 1:
        logits = logits.contiguous()
    v = logits.shape[-1]
    l2 = logits.reshape(-1, v) if logits.dim() != 2 else logits
    return l2


def _generator_args(seed, offset, offset_dev, row_ids, rows):
    """(seed, offset, offset_dev pointer, row_ids pointer) of the in-kernel Gumbel generator."""
    if offset_dev is not None:
        assert offset_dev.dtype == torch.int64 and offset_dev.numel() == 1 and offset_dev.is_cuda
    if row_ids is not None:
        assert row_ids.dtype == torch.int64 and row_ids.numel() == rows and row_ids.is_contiguous() and row_ids.is_cuda
    return (int(seed) & (2 ** 64 - 1), int(offset) & (2 ** 64 - 1),
            None if offset_dev is None else offset_dev.data_ptr(), None if row_ids is None else row_ids.data_ptr())


def gumbel_noise(rows: int, vocab: int, seed: int, offset: int = 0, device=None,
                 offset_dev: torch.Tensor | None = None, row_ids: torch.Tensor | None = None) -> torch.Tensor:
    """The [rows, vocab] fp32 noise tensor that `seed` / `offset` stand for in confidence_argmax and
    unmask_step: passing it as `noise` gives the same result as passing the two integers."""
    out = torch.empty((rows, vocab), dtype=torch.float32, device=device if device is not None else "cuda")
    _need_gpu(out, offset_dev, row_ids)
    rc = _lib.lib().mdx_gumbel_noise(out.data_ptr(), out.stride(0) if rows else vocab, rows, vocab,
                                     *_generator_args(seed, offset, offset_dev, row_ids, rows), _stream(out))
    check(rc, "gumbel_noise")
    return out


def confidence_argmax(logits: torch.Tensor, temperatures: torch.Tensor | None = None,
                      noise: torch.Tensor | None = None, seed: int | None = None, offset: int = 0,
                      offset_dev: torch.Tensor | None = None, row_ids: torch.Tensor | None = None):
    """Sampler.prepare (nanovllm/layers/sampler.py:11-22):
    logits [bs, S, V], temperatures [bs] or [bs, 1] fp32 -> (x0 int64 [bs, S], x0_p fp32 [bs, S]).
    The Gumbel noise that the reference adds to logits/T before the argmax is either an explicit tensor
    `noise` ([bs, S, V] fp32), or drawn inside the kernel from (`seed`, `offset`): a counter-based
    generator, so the same integers give the same tokens (give every step another offset; `offset_dev`,
    a one-element int64 device tensor, is added to it at run time; `row_ids` [rows] int64 names the
    generator row of each logits row when rows were compacted).  Neither = plain argmax."""
    _need_gpu(logits, temperatures, noise)
    assert noise is None or seed is None, "either a noise tensor or a seed"
    lead = logits.shape[:-1]
    l2 = _logits2d(logits)
    rows, vocab = l2.shape
    rows_per_temp = 1
    t_ptr = None
    if temperatures is not None:
        temperatures = temperatures.reshape(-1).to(torch.float32).contiguous()
        assert rows % temperatures.numel() == 0
        rows_per_temp = rows // temperatures.numel()
        t_ptr = temperatures.data_ptr()
    n_ptr, n_stride = None, 0
    if noise is not None:
        noise = noise.reshape(rows, vocab).to(torch.float32).contiguous()
        n_ptr, n_stride = noise.data_ptr(), noise.stride(0)
    x0 = torch.empty(rows, dtype=torch.int64, device=logits.device)
    x0_p = torch.empty(rows, dtype=torch.float32, device=logits.device)
    L = _lib.lib()
    ws_bytes = L.mdx_confidence_argmax_workspace_bytes(rows, vocab)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=logits.device)
    if seed is not None:
        rc = L.mdx_confidence_argmax_gumbel(l2.data_ptr(), l2.stride(0), _DTYPES[l2.dtype], t_ptr, rows_per_temp,
                                            *_generator_args(seed, offset, offset_dev, row_ids, rows),
                                            x0.data_ptr(), x0_p.data_ptr(), rows, vocab, ws.data_ptr(), ws_bytes, _stream(logits))
    else:
        rc = L.mdx_confidence_argmax(l2.data_ptr(), l2.stride(0), _DTYPES[l2.dtype], t_ptr, rows_per_temp, n_ptr, n_stride,
                                     x0.data_ptr(), x0_p.data_ptr(), rows, vocab, ws.data_ptr(), ws_bytes, _stream(logits))
    check(rc, "confidence_argmax")
    return x0.view(lead), x0_p.view(lead)


def lm_head_confidence(x: torch.Tensor, weight: torch.Tensor, temperatures: torch.Tensor | None = None,
                       rows_per_temp: int | None = None, row_ids: torch.Tensor | None = None):
    """ParallelLMHead.forward's F.linear(x, weight) (nanovllm/layers/embed_head.py:61-67) followed by
    Sampler.prepare without noise (layers/sampler.py:11-22), in one pass that never writes the logits:
    x [..., hidden] bf16, weight [vocab, hidden] bf16 -> (x0 int64 [...], x0_p fp32 [...]) = argmax and softmax
    confidence of bf16(x . weight^T) / T.  temperatures [n] fp32: row r uses entry (row_ids[r] if given else r)
    // rows_per_temp (default rows / n), so that compacted rows keep the temperature of their sequence."""
    _need_gpu(x, weight, temperatures, row_ids)
    assert x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16, "lm_head_confidence: bf16 only"
    lead = x.shape[:-1]
    x2 = x.reshape(-1, x.shape[-1])
    if x2.stride(-1) != 1:
        x2 = x2.contiguous()
    assert weight.dim() == 2 and weight.stride(-1) == 1 and weight.shape[1] == x2.shape[1]
    rows, hidden = x2.shape
    vocab = weight.shape[0]
    t_ptr, rpt = None, 1
    if temperatures is not None:
        temperatures = temperatures.reshape(-1).to(torch.float32).contiguous()
        if rows_per_temp is None:
            assert rows % temperatures.numel() == 0
            rows_per_temp = rows // temperatures.numel()
        t_ptr, rpt = temperatures.data_ptr(), int(rows_per_temp)
    ids_ptr = None
    if row_ids is not None:
        assert row_ids.dtype == torch.int64 and row_ids.is_contiguous() and row_ids.numel() >= rows
        ids_ptr = row_ids.data_ptr()
    x0 = torch.empty(rows, dtype=torch.int64, device=x.device)
    x0_p = torch.empty(rows, dtype=torch.float32, device=x.device)
    L = _lib.lib()
    ws_bytes = L.mdx_lm_head_confidence_workspace_bytes(rows, vocab)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=x.device)
    rc = L.mdx_lm_head_confidence(x2.data_ptr(), x2.stride(0), weight.data_ptr(), weight.stride(0), t_ptr, rpt, ids_ptr,
                                  x0.data_ptr(), x0_p.data_ptr(), rows, vocab, hidden, ws.data_ptr(), ws_bytes, _stream(x))
    check(rc, "lm_head_confidence")
    return x0.view(lead), x0_p.view(lead)


def filter_logits(logits: torch.Tensor, top_k: int = 0, top_p: float = 1.0,
                  temperatures: torch.Tensor | None = None, out: torch.Tensor | None = None) -> torch.Tensor:
    """top_k_logits then top_p_logits of the HF variant (modeling_mineru_diffusion.py:585-600, in the
    order of :608-611) on bf16 / fp16 logits [..., V]: a copy (or `out`, which may be `logits`) with
    every element below the row's cut-off set to -inf.  Feed the result to confidence_argmax /
    unmask_step; their `noise` input (Gumbel) then samples from the filtered distribution.  top_k = 0
    and top_p >= 1 switch the respective filter off.  temperatures as for confidence_argmax (they
    enter the top-p probabilities only)."""
    _need_gpu(logits, temperatures, out)
    l2 = _logits2d(logits)
    rows, vocab = l2.shape
    if out is None:
        out = torch.empty(logits.shape, dtype=logits.dtype, device=logits.device)
    assert out.shape == logits.shape and out.dtype == logits.dtype
    assert out.stride(-1) == 1, "out must have unit stride along the vocabulary"
    o2 = out if out.dim() == 2 else out.view(-1, vocab)          # raises if that would need a copy
    rows_per_temp, t_ptr = 1, None
    if temperatures is not None:
        temperatures = temperatures.reshape(-1).to(torch.float32).contiguous()
        assert rows % temperatures.numel() == 0
        rows_per_temp = rows // temperatures.numel()
        t_ptr = temperatures.data_ptr()
    rc = _lib.lib().mdx_filter_logits(l2.data_ptr(), l2.stride(0), _DTYPES[l2.dtype], t_ptr, rows_per_temp,
                                      int(top_k), float(top_p), o2.data_ptr(), o2.stride(0), rows, vocab, _stream(logits))
    check(rc, "filter_logits")
    return out


def num_transfer_tokens(block_length: int, steps: int) -> list[int]:
    """get_num_transfer_tokens (modeling_mineru_diffusion.py:617-623): how many positions each denoising step of a
    block commits at least -- block_length split over the steps, the remainder given to the first steps.  The k of
    unmask_step / select_transfer for step i is entry min(i, steps - 1) (modeling_mineru_diffusion.py:712)."""
    base, rem = divmod(int(block_length), int(steps))
    return [base + (1 if i < rem else 0) for i in range(int(steps))]


def select_transfer(x0: torch.Tensor, x0_p: torch.Tensor, tokens: torch.Tensor, mask_token_id: int,
                    threshold: float, k: int = 1):
    """Device form of the selection loop (sampler.py:32-54, modeling_mineru_diffusion.py:518-532).
    tokens [bs, S] int64 is updated in place; returns (transfer bool [bs, S], count int32 [bs])."""
    _need_gpu(x0, x0_p, tokens)
    assert tokens.dtype == torch.int64 and x0.dtype == torch.int64 and x0_p.dtype == torch.float32
    assert tokens.is_contiguous() and x0.is_contiguous() and x0_p.is_contiguous()
    bs, S = tokens.shape
    transfer = torch.empty((bs, S), dtype=torch.uint8, device=tokens.device)
    count = torch.empty(bs, dtype=torch.int32, device=tokens.device)
    rc = _lib.lib().mdx_select_transfer(x0.data_ptr(), x0_p.data_ptr(), tokens.data_ptr(), int(mask_token_id),
                                        float(threshold), int(k), transfer.data_ptr(), count.data_ptr(), bs, S,
                                        _stream(tokens))
    check(rc, "select_transfer")
    return transfer.view(torch.bool), count


def unmask_step(logits: torch.Tensor, tokens: torch.Tensor, mask_token_id: int, threshold: float, k: int = 1,
                temperatures: torch.Tensor | None = None, noise: torch.Tensor | None = None,
                top_k: int = 0, top_p: float = 1.0, seed: int | None = None, offset: int = 0,
                offset_dev: torch.Tensor | None = None):
    """One whole unmask step on the device: logits [bs, S, V], tokens [bs, S] int64 (in place).
    Returns (x0, x0_p, transfer, count).  top_k / top_p (off by default, as in
    modeling_mineru_diffusion.py:602,633-634) put filter_logits in front of the step; `noise` or
    (`seed`, `offset`, `offset_dev`) as for confidence_argmax."""
    _need_gpu(logits, tokens, temperatures, noise)
    assert noise is None or seed is None, "either a noise tensor or a seed"
    if top_k > 0 or top_p < 1.0:
        logits = filter_logits(logits, top_k, top_p, temperatures)
    assert tokens.dtype == torch.int64 and tokens.is_contiguous()
    bs, S = tokens.shape
    l2 = _logits2d(logits)
    rows, vocab = l2.shape
    assert rows == bs * S
    t_ptr = None
    if temperatures is not None:
        temperatures = temperatures.reshape(-1).to(torch.float32).contiguous()
        assert temperatures.numel() == bs
        t_ptr = temperatures.data_ptr()
    n_ptr, n_stride = None, 0
    if noise is not None:
        noise = noise.reshape(rows, vocab).to(torch.float32).contiguous()
        n_ptr, n_stride = noise.data_ptr(), noise.stride(0)
    dev = logits.device
    x0 = torch.empty((bs, S), dtype=torch.int64, device=dev)
    x0_p = torch.empty((bs, S), dtype=torch.float32, device=dev)
    transfer = torch.empty((bs, S), dtype=torch.uint8, device=dev)
    count = torch.empty(bs, dtype=torch.int32, device=dev)
    L = _lib.lib()
    ws_bytes = L.mdx_confidence_argmax_workspace_bytes(rows, vocab)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
    if seed is not None:
        rc = L.mdx_unmask_step_gumbel(l2.data_ptr(), l2.stride(0), _DTYPES[l2.dtype], t_ptr,
                                      *_generator_args(seed, offset, offset_dev, None, rows),
                                      tokens.data_ptr(), int(mask_token_id), float(threshold), int(k),
                                      x0.data_ptr(), x0_p.data_ptr(), transfer.data_ptr(), count.data_ptr(),
                                      bs, S, vocab, ws.data_ptr(), ws_bytes, _stream(logits))
    else:
        rc = L.mdx_unmask_step(l2.data_ptr(), l2.stride(0), _DTYPES[l2.dtype], t_ptr, n_ptr, n_stride,
                               tokens.data_ptr(), int(mask_token_id), float(threshold), int(k),
                               x0.data_ptr(), x0_p.data_ptr(), transfer.data_ptr(), count.data_ptr(),
                               bs, S, vocab, ws.data_ptr(), ws_bytes, _stream(logits))
    check(rc, "unmask_step")
    return x0, x0_p, transfer.view(torch.bool), count
