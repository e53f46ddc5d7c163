"""mdx -- the block-diffusion attention hot path of the nano_dvlm engine as
hand-written gfx950 HIP kernels, behind the engine's own Python call sites.

Drop-in names (same arguments, layouts and in-place behaviour as the
reference functions they replace):

  sparse_attn_varlen        nanovllm/kernels/triton/attention/block_prefill_attention_v2.py:201
  store_kvcache             nanovllm/layers/attention.py:33
  store_kvcache_maybe4d     nanovllm/layers/sdar_attention.py:11
  flash_attn_with_kvcache   flash_attn (call at nanovllm/layers/sdar_attention.py:50-55)
  Attention                 nanovllm/layers/sdar_attention.py:19-57
  Sampler                   nanovllm/layers/sampler.py:6-61
  Context / set_context ..  nanovllm/utils/context.py
  rms_norm                  nanovllm/layers/layernorm.py:43-51 (RMSNorm.forward, with or without residual)
  silu_and_mul              nanovllm/layers/activation.py:13-16 (SiluAndMul.forward)
  qk_norm_rope_store        nanovllm/models/sdar.py:79-83 in one launch (q/k norm, rotary, KV store)

Every op runs in libmdx.so; importing an op works without a GPU, calling one
without the built library or on a non-GPU tensor raises.
"""
from .context import Context, get_context, set_context, reset_context  # noqa: F401
from .ops import (  # noqa: F401
    sparse_attn_varlen, sparse_attn_varlen_v2, store_kvcache, store_kvcache_maybe4d,
    flash_attn_with_kvcache, confidence_argmax, lm_head_confidence, gumbel_noise, filter_logits, num_transfer_tokens, select_transfer, unmask_step, qk_norm_rope_store, rms_norm, silu_and_mul,
)
from .layers import Attention, Sampler  # noqa: F401
from ._lib import lib, library_path, MdxError  # noqa: F401
