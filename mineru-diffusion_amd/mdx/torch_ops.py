"""torch.library registrations of the libmdx ops: `torch.ops.mdx.*`.

The engine calls the functions of `mdx.ops` directly (plain Python around one C call, which a HIP
graph capture records like any other launch).  Callers that TRACE their model -- torch.compile, as
the reference does around its small layer functions (nanovllm/layers/layernorm.py:16,28,
activation.py:12, sampler.py:11), or torch.export -- need each op to be opaque to the tracer and to
say what it returns without running: that is what this module adds.  Importing it registers

    torch.ops.mdx.sparse_attn_varlen(q, k, v, cu_seqlens_q, cu_seqlens_k, staircase_size, max_seqlen, softmax_scale) -> o
    torch.ops.mdx.store_kvcache(key, value, k_cache, v_cache, slot_mapping)            (writes the caches)
    torch.ops.mdx.paged_block_attn(q, k_cache, v_cache, cache_seqlens, block_table, softmax_scale) -> o
    torch.ops.mdx.confidence_argmax(logits, temperatures) -> (x0, x0_p)
    torch.ops.mdx.unmask_step(logits, tokens, mask_token_id, threshold, k, temperatures) -> (x0, x0_p, transfer, count)
                                                                                        (writes tokens)
    torch.ops.mdx.rms_norm(x, weight, eps) -> y
    torch.ops.mdx.add_rms_norm(x, residual, weight, eps) -> (y, new_residual)
    torch.ops.mdx.silu_and_mul(x) -> y
    torch.ops.mdx.lm_head_confidence(x, weight, temperatures) -> (x0, x0_p)

Same kernels, same results as the functions of `mdx.ops` they wrap; nothing here computes.
"""
from __future__ import annotations

import torch
from torch import Tensor
from torch.library import custom_op

from . import ops


@custom_op("mdx::sparse_attn_varlen", mutates_args=())
def sparse_attn_varlen(q: Tensor, k: Tensor, v: Tensor, cu_seqlens_q: Tensor, cu_seqlens_k: Tensor,
                       staircase_size: int, max_seqlen: int, softmax_scale: float) -> Tensor:
    return ops.sparse_attn_varlen(q, k, v, cu_seqlens_q, cu_seqlens_k, staircase_size,
                                  max_seqlen=max_seqlen or None, softmax_scale=softmax_scale)


@sparse_attn_varlen.register_fake
def _(q, k, v, cu_seqlens_q, cu_seqlens_k, staircase_size, max_seqlen, softmax_scale):
    return q.new_empty(q.shape)


@custom_op("mdx::store_kvcache", mutates_args=("k_cache", "v_cache"))
def store_kvcache(key: Tensor, value: Tensor, k_cache: Tensor, v_cache: Tensor, slot_mapping: Tensor) -> None:
    ops.store_kvcache_maybe4d(key, value, k_cache, v_cache, slot_mapping)


@store_kvcache.register_fake
def _(key, value, k_cache, v_cache, slot_mapping):
    return None


@custom_op("mdx::paged_block_attn", mutates_args=())
def paged_block_attn(q: Tensor, k_cache: Tensor, v_cache: Tensor, cache_seqlens: Tensor, block_table: Tensor,
                     softmax_scale: float) -> Tensor:
    # the stateless two-launch call: a traced graph may be run from any stream
    return ops.flash_attn_with_kvcache(q, k_cache, v_cache, cache_seqlens=cache_seqlens, block_table=block_table,
                                       softmax_scale=softmax_scale, causal=False, counters=False)


@paged_block_attn.register_fake
def _(q, k_cache, v_cache, cache_seqlens, block_table, softmax_scale):
    return q.new_empty(q.shape)


@custom_op("mdx::confidence_argmax", mutates_args=())
def confidence_argmax(logits: Tensor, temperatures: Tensor | None) -> tuple[Tensor, Tensor]:
    return ops.confidence_argmax(logits, temperatures)


@confidence_argmax.register_fake
def _(logits, temperatures):
    lead = logits.shape[:-1]
    return logits.new_empty(lead, dtype=torch.int64), logits.new_empty(lead, dtype=torch.float32)


@custom_op("mdx::unmask_step", mutates_args=("tokens",))
def unmask_step(logits: Tensor, tokens: Tensor, mask_token_id: int, threshold: float, k: int,
                temperatures: Tensor | None) -> tuple[Tensor, Tensor, Tensor, Tensor]:
    return ops.unmask_step(logits, tokens, mask_token_id, threshold, k, temperatures=temperatures)


@unmask_step.register_fake
def _(logits, tokens, mask_token_id, threshold, k, temperatures):
    return (tokens.new_empty(tokens.shape), tokens.new_empty(tokens.shape, dtype=torch.float32),
            tokens.new_empty(tokens.shape, dtype=torch.bool), tokens.new_empty(tokens.shape[:1], dtype=torch.int32))


@custom_op("mdx::rms_norm", mutates_args=())
def rms_norm(x: Tensor, weight: Tensor, eps: float) -> Tensor:
    return ops.rms_norm(x, weight, eps)


@rms_norm.register_fake
def _(x, weight, eps):
    return x.new_empty(x.shape)


@custom_op("mdx::add_rms_norm", mutates_args=())
def add_rms_norm(x: Tensor, residual: Tensor, weight: Tensor, eps: float) -> tuple[Tensor, Tensor]:
    return ops.rms_norm(x, weight, eps, residual)


@add_rms_norm.register_fake
def _(x, residual, weight, eps):
    return x.new_empty(x.shape), x.new_empty(x.shape)


@custom_op("mdx::silu_and_mul", mutates_args=())
def silu_and_mul(x: Tensor) -> Tensor:
    return ops.silu_and_mul(x)


@silu_and_mul.register_fake
def _(x):
    return x.new_empty((*x.shape[:-1], x.shape[-1] // 2))


@custom_op("mdx::lm_head_confidence", mutates_args=())
def lm_head_confidence(x: Tensor, weight: Tensor, temperatures: Tensor | None) -> tuple[Tensor, Tensor]:
    return ops.lm_head_confidence(x, weight, temperatures)


@lm_head_confidence.register_fake
def _(x, weight, temperatures):
    lead = x.shape[:-1]
    return x.new_empty(lead, dtype=torch.int64), x.new_empty(lead, dtype=torch.float32)
