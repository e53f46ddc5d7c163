"""The two layers that own the hot path, as the engine defines them."""
from __future__ import annotations

import torch
from torch import nn

from .context import get_context
from .ops import flash_attn_with_kvcache, sparse_attn_varlen, store_kvcache_maybe4d, unmask_step


_side_streams: dict = {}


def _side_stream(device: torch.device) -> torch.cuda.Stream:
    """One extra stream per device (default priority) for work that may run beside the caller's stream."""
    index = device.index if device.index is not None else torch.cuda.current_device()
    stream = _side_streams.get(index)
    if stream is None:
        stream = _side_streams[index] = torch.cuda.Stream(device=index)
    return stream


class Attention(nn.Module):
    """nanovllm/layers/sdar_attention.py:19-57: store the step's K/V into the paged cache,
    then staircase attention over the packed prompt (prefill) or non-causal attention of
    the current block over the cache (decode).  Inputs arrive through the global Context."""

    def __init__(self, num_heads, head_dim, scale, num_kv_heads):
        super().__init__()
        self.num_heads = num_heads
        self.head_dim = head_dim
        self.scale = scale
        self.num_kv_heads = num_kv_heads
        self.k_cache = self.v_cache = torch.tensor([])

    def forward(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor):
        context = get_context()
        k_cache, v_cache = self.k_cache, self.v_cache
        have_cache = bool(k_cache.numel() and v_cache.numel())
        if context.is_prefill:
            # The prefill attention reads k / v, not the cache: the store is independent of it and runs beside it on a
            # second stream (its small workgroups fill the gaps between the attention kernel's, which own whole CUs:
            # config 3, 0.820 -> 0.808 ms for the pair).  The caller's stream waits for both before it goes on.
            main = torch.cuda.current_stream(q.device)
            side = _side_stream(q.device) if have_cache else None
            if side is not None:
                side.wait_stream(main)
                with torch.cuda.stream(side):
                    store_kvcache_maybe4d(k, v, k_cache, v_cache, context.slot_mapping)
            o = sparse_attn_varlen(q, k, v, cu_seqlens_q=context.cu_seqlens_q, cu_seqlens_k=context.cu_seqlens_k,
                                   staircase_size=context.block_size,
                                   max_seqlen=context.max_seqlen_k or None, softmax_scale=self.scale)
            if side is not None:
                main.wait_stream(side)
            return o.flatten(1)
        if have_cache:
            store_kvcache_maybe4d(k, v, k_cache, v_cache, context.slot_mapping)
        o = flash_attn_with_kvcache(q, k_cache, v_cache, cache_seqlens=context.context_lens,
                                    block_table=context.block_tables, softmax_scale=self.scale, causal=False)
        return o.flatten(2)


class Sampler(nn.Module):
    """nanovllm/layers/sampler.py:6-61.  The device does the whole step (confidence, argmax,
    selection); only the [bs, S] results cross to the host to update the Sequence objects.

    `k` is the number of positions committed when fewer than k exceed the threshold
    (1 = the engine's rule, sampler.py:44-50).  The Gumbel term of sampler.py:15-18 comes from `seed`
    (drawn inside the kernel by a counter-based generator; every call takes the next offset, so a seed
    reproduces a run) or from `noise_fn(logits) -> fp32 noise`; neither = plain argmax."""

    def __init__(self, k: int = 1, noise_fn=None, seed: int | None = None):
        super().__init__()
        assert noise_fn is None or seed is None, "either a noise function or a seed"
        self.k = k
        self.noise_fn = noise_fn
        self.seed = seed
        self.calls = 0                                      # the generator offset of the next call

    def _noise_args(self, logits):
        if self.seed is not None:
            self.calls += 1
            return dict(seed=self.seed, offset=self.calls - 1)
        return dict(noise=self.noise_fn(logits) if self.noise_fn is not None else None)

    def prepare(self, logits: torch.Tensor, temperatures: torch.Tensor):
        from .ops import confidence_argmax
        return confidence_argmax(logits, temperatures, **self._noise_args(logits))

    def forward(self, logits: torch.Tensor, temperatures: torch.Tensor, seqs) -> int:
        strategy = seqs[0].sampling_params.denoising_strategy
        if strategy != 'low_confidence_dynamic':
            raise NotImplementedError(f"Denoising strategy {strategy} not implemented")
        threshold = seqs[0].sampling_params.dynamic_threshold
        x = torch.stack([seq.current_denoising_block for seq in seqs], dim=0).to(logits.device)
        _, _, transfer, count = unmask_step(logits, x, seqs[0].mask_token_id, threshold, self.k,
                                            temperatures=temperatures, **self._noise_args(logits))
        x_cpu, transfer_cpu = x.cpu(), transfer.cpu()
        for i, seq in enumerate(seqs):
            seq.current_denoising_block = x_cpu[i]
            seq.current_step_map[transfer_cpu[i]] = seq.current_denoise_step
            seq.current_denoise_step += 1
        return int(count.sum().item())
