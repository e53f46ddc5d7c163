"""Oracle: the store_kvcache scatter.  Test infrastructure only.

Reference followed: engines/nano_dvlm/nanovllm/layers/attention.py:10-40 and the
4-D flattening of layers/sdar_attention.py:11-16.
"""
from __future__ import annotations

import numpy as np


def store_kvcache(key: np.ndarray, value: np.ndarray, k_cache: np.ndarray, v_cache: np.ndarray,
                  slot_mapping: np.ndarray) -> None:
    """In place: for token i with slot = slot_mapping[i] != -1,
    k_cache.flat[slot*D:(slot+1)*D] = key[i].flat, same for V (attention.py:21-30).
    Arrays are raw 16-bit patterns (uint16) or any numpy dtype: a pure copy.
    key/value [N, Hkv, d] or [bs, S, Hkv, d]; caches [pages, page, Hkv, d]."""
    D = key.shape[-1] * key.shape[-2]
    kf = key.reshape(-1, D)
    vf = value.reshape(-1, D)
    slots = np.asarray(slot_mapping).reshape(-1)
    assert slots.size == kf.shape[0]
    kc = k_cache.reshape(-1, D)
    vc = v_cache.reshape(-1, D)
    for i, s in enumerate(slots):          # token order: a later duplicate slot wins
        if s == -1:
            continue
        kc[s] = kf[i]
        vc[s] = vf[i]
