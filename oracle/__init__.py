"""CPU oracle for the block-diffusion attention hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package may import this
directory: it is the checker that the HIP kernels are compared against, used by
``tests/``, by ``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of
``bench.py``.  It is never the thing measured as the product and never a
fallback for a missing HIP library.

Each function restates, for the CPU, the arithmetic of one piece of the
reference's ``nano_dvlm`` engine (or of its HF twin) and cites the reference
file:line it follows.  The reference ships no tests, golden vectors or fixtures
for this path, so every function is pinned instead by closed forms, invariants,
library routines and brute force on tiny inputs (``tests/test_oracle_*.py``):

==========================  =====================================================
function                    pinned by
==========================  =====================================================
staircase_mask              second independent formula (tril-of-blocks, the HF
                            twin's construction), S=1 == causal, S>=L == full,
                            hand-written 7x7 case
pairs                       mask.sum() for every L<=200, closed form L(L+S)/2
masked_attention_f32        explicit fp64 softmax(QK^T)V loops on tiny shapes,
                            rows of P sum to 1, GQA == MHA with duplicated heads
staircase_attn_varlen       block-b output independent of later blocks,
                            S=1 == torch causal SDPA, S>=L == unmasked SDPA
paged_gather / paged attn   paged == contiguous, page permutation invariance
store_kvcache               torch index_copy_, untouched slots, -1 skipped
confidence_argmax           torch.softmax / torch.argmax, fp64 explicit sums
philox4x32_10               the known-answer vectors of the Random123 distribution (zeros, all ones, digits of pi),
                            distinct counters / keys give distinct outputs
gumbel_noise                built on philox4x32_10; its uniforms lie in (0, 1) on a 2^-23 grid, mean / variance of
                            the Gumbel law (Euler's constant, pi^2 / 6), Gumbel-max frequencies = softmax
filter_logits               torch.topk / sort / cumsum / scatter formulation on tie-free rows, kept count == k,
                            kept mass exceeds p and stops exceeding it without its smallest element,
                            brute force over all cut-offs on 8 values, ties at the cut-off all kept
select_transfer             torch.topk on tie-free inputs, brute force over all
                            subsets on 6 positions, counting invariants
slot_of / get_slots         brute force token-by-token formula
rms_norm_ref / rope_ref     unit RMS after norm, F.rms_norm, rotation preserves pair norms,
                            position 0 is the identity, complex-multiplication form
add_rms_norm                residual is the rounded sum; reduces to rms_norm_ref for a zero residual;
                            F.rms_norm of the fp32 sum; variance taken before the rounding (a case
                            where the two differ)
silu_and_mul                F.silu * other half; silu(0) = 0, silu(x) -> x and -> 0 in the tails
block_prepare               get_slots (brute-force slot formula) per position; idle lanes = graph padding
masked_rows                 numpy nonzero of the same mask
block_advance               driven with select_transfer over whole generations: pass count = the closed form
                            expected_passes, tokens / step maps / finish conditions equal to the host
                            engine's Sequence + postprocess (an independent implementation), stop tokens
dense_forward               built from the pinned attention oracle and plain matmuls; its mask
                            and SDPA are the functions above
==========================  =====================================================

The third-party arithmetic behind the reference's paged decode call
(flash-attn 2.8.3 ``flash_attn_with_kvcache``) is not under the reference tree;
its published semantics (dense softmax attention over the first
``cache_seqlens[b]`` keys gathered through ``block_table``) are restated here
and pinned by the contiguous closed form above.
"""
from .staircase import (  # noqa: F401
    staircase_mask, staircase_mask_tril, staircase_pairs, masked_attention_f32,
    attention_f64_explicit, staircase_attn_varlen, paged_gather, paged_block_attn,
)
from .kvstore import store_kvcache  # noqa: F401
from .unmask import confidence_argmax, filter_logits, philox4x32_10, gumbel_noise, select_transfer, unmask_step, num_transfer_tokens  # noqa: F401
from .slots import slot_of, get_slots  # noqa: F401
from .engine import dense_forward, expected_passes, block_prepare, masked_rows, block_advance  # noqa: F401
from .fused import qk_norm_rope, rms_norm_ref, rope_ref, add_rms_norm, silu_and_mul  # noqa: F401
