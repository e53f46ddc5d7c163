"""Oracle: dense fp32 restatement of the decoder scaffold and of one block-diffusion pass.
Test infrastructure only.

The engine under test keeps a paged KV cache and feeds only the current 32-token block through
the model; this restatement recomputes the whole sequence with an explicit staircase mask and no
cache, the way the reference's HF twin does
(mineru_diffusion/modeling_mineru_diffusion.py:450-478 mask, :189-206 SDPA, :664-720 block loop;
layer structure engines/nano_dvlm/nanovllm/models/sdar.py:68-181).  Agreement of the two is the
check that store + paged attention + slot arithmetic implement the same function as a prefill.
"""
from __future__ import annotations

import numpy as np
import torch
import torch.nn.functional as F

from .staircase import masked_attention_f32, staircase_mask


def _rms(x, w, eps):
    x = x.float()
    return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w.float()


def _rope(x, cos, sin):
    x1, x2 = torch.chunk(x.float(), 2, dim=-1)
    return torch.cat((x1 * cos - x2 * sin, x2 * cos + x1 * sin), dim=-1)


def dense_forward(weights: dict, cfg, embeds: torch.Tensor):
    """embeds [L, hidden] fp32 for ONE sequence (prompt + committed blocks + current block).
    Returns (logits of the last block [S, V], per-layer k [layers][L, Hkv, d], per-layer v)."""
    L = embeds.shape[0]
    S = cfg.block_size
    W = {k: v.detach().float().cpu() for k, v in weights.items()}
    inv_freq = 1.0 / (cfg.rope_theta ** (torch.arange(0, cfg.head_dim, 2, dtype=torch.float) / cfg.head_dim))
    freqs = torch.einsum("i,j->ij", torch.arange(L, dtype=torch.float), inv_freq)
    cos, sin = freqs.cos().unsqueeze(1), freqs.sin().unsqueeze(1)
    mask = staircase_mask(L, S)
    x, residual = embeds.float(), None
    ks, vs = [], []
    for i in range(cfg.num_layers):
        p = f"layers.{i}."
        residual = x if residual is None else x + residual
        h = _rms(residual, W[p + "input_layernorm"], cfg.rms_norm_eps)
        qkv = h @ W[p + "qkv_proj"].T
        q, k, v = qkv.split([cfg.num_heads * cfg.head_dim, cfg.num_kv_heads * cfg.head_dim, cfg.num_kv_heads * cfg.head_dim], -1)
        q = _rope(_rms(q.view(L, -1, cfg.head_dim), W[p + "q_norm"], cfg.rms_norm_eps), cos, sin)
        k = _rope(_rms(k.view(L, -1, cfg.head_dim), W[p + "k_norm"], cfg.rms_norm_eps), cos, sin)
        v = v.view(L, -1, cfg.head_dim)
        ks.append(k)
        vs.append(v)
        o = masked_attention_f32(q, k, v, mask, cfg.head_dim ** -0.5).reshape(L, -1)
        x = o @ W[p + "o_proj"].T
        residual = x + residual
        h = _rms(residual, W[p + "post_attention_layernorm"], cfg.rms_norm_eps)
        gate, up = (h @ W[p + "gate_up_proj"].T).chunk(2, -1)
        x = (F.silu(gate) * up) @ W[p + "down_proj"].T
    hidden = _rms(x + residual, W["norm"], cfg.rms_norm_eps)
    return hidden[-S:] @ W["lm_head"].T, ks, vs


def expected_passes(block_len: int, k: int, n_blocks: int) -> int:
    """Model passes for one request when no confidence ever exceeds the threshold: every block
    takes ceil(block_len / k) denoising passes plus one pass that stores the committed block
    (engines/nano_dvlm/nanovllm/engine/scheduler.py:65-82)."""
    return n_blocks * (-(-block_len // k) + 1)


# ---- per-lane block state (the device loop's three small kernels) -----------------------------------------
IDLE, DENOISING, CACHING = 0, 1, 2


def block_prepare(lens, phase, block_table, page: int, block_len: int):
    """ModelRunner.prepare_decode (engines/nano_dvlm/nanovllm/engine/model_runner.py:169-185) per lane:
    positions = len .. len + S - 1, slots through the page table (engine/sequence.py:117-141),
    context length len + S; idle lanes are graph padding (model_runner.py:203-208): slots -1, context 0."""
    lens, phase, bt = np.asarray(lens), np.asarray(phase), np.asarray(block_table)
    bs = len(lens)
    pos = np.zeros((bs, block_len), dtype=np.int64)
    slots = np.full((bs, block_len), -1, dtype=np.int32)
    ctx = np.zeros(bs, dtype=np.int32)
    for b in range(bs):
        if phase[b] == IDLE:
            continue
        ctx[b] = lens[b] + block_len
        for p in range(block_len):
            t = int(lens[b]) + p
            pos[b, p] = t
            pg = t // page
            if pg < bt.shape[1] and bt[b, pg] >= 0:
                slots[b, p] = bt[b, pg] * page + t % page
    return pos, slots, ctx


def masked_rows(tokens, phase, mask_token_id: int, cap: int):
    """Flat indices of the still-masked positions of the denoising lanes, in order, padded to `cap`
    with the first entry (0 when there is none); and their count."""
    tokens, phase = np.asarray(tokens), np.asarray(phase)
    found = [b * tokens.shape[1] + p for b in range(tokens.shape[0]) if phase[b] == DENOISING
             for p in range(tokens.shape[1]) if tokens[b, p] == mask_token_id]
    fill = found[0] if found else 0
    rows = (found + [fill] * cap)[:cap]
    return np.asarray(rows, dtype=np.int64), len(found)


def block_advance(tokens, transfer, step_map, step, phase, lens, first_len, max_new, stop_ids, mask_token_id: int):
    """What follows the selection, per lane: Sampler.forward's bookkeeping (layers/sampler.py:56-59) and
    Scheduler.postprocess (engine/scheduler.py:65-82).  Works on copies; returns the new
    (tokens, step_map, step, phase, lens), the appended (tokens, steps) per lane (None when nothing
    was appended) and the status rows (phase, len, masked left, committed in this pass)."""
    tokens, step_map = np.array(tokens), np.array(step_map)
    step, phase, lens = np.array(step), np.array(phase), np.array(lens)
    transfer = np.asarray(transfer, dtype=bool)
    appended, status = [], []
    S = tokens.shape[1]
    for b in range(tokens.shape[0]):
        if phase[b] == IDLE:
            appended.append(None)
            status.append((IDLE, None, 0, 0))
            continue
        step_map[b][transfer[b]] = step[b]
        step[b] += 1
        moved = int(transfer[b].sum())
        if phase[b] == DENOISING:
            left = int((tokens[b] == mask_token_id).sum())
            if left == 0:
                phase[b] = CACHING
            appended.append(None)
        else:
            stop = any(s >= 0 and (tokens[b] == s).any() for s in stop_ids[b])
            appended.append((tokens[b].copy(), step_map[b].copy()))
            tokens[b] = mask_token_id
            lens[b] += S
            left = S
            phase[b] = IDLE if (stop or lens[b] - first_len[b] >= max_new[b]) else DENOISING
        status.append((int(phase[b]), int(lens[b]), 0 if phase[b] == IDLE else left, moved))
    return tokens, step_map, step, phase, lens, appended, status
