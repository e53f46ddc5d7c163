"""Oracle: token -> KV slot arithmetic of the paged cache.  Test infrastructure only.

Reference followed: engines/nano_dvlm/nanovllm/engine/sequence.py:117-141.
"""
from __future__ import annotations


def slot_of(block_table, t: int, page: int = 256) -> int:
    """Flat slot of token t: page id * page + offset in page."""
    return int(block_table[t // page]) * page + t % page


def get_slots(block_table, lo: int, hi: int, page: int = 256) -> list[int]:
    """Slots of tokens lo..hi-1; an empty page table (warm-up sequence,
    sequence.py:118-119) gives -1 for every token."""
    if len(block_table) == 0:
        return [-1] * (hi - lo)
    return [slot_of(block_table, t, page) for t in range(lo, hi)]
