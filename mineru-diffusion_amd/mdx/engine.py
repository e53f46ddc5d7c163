"""A minimal block-diffusion decode loop around the mdx hot path.

This is the caller side of the hot path, restated from the nano_dvlm engine so that the
kernels can be driven exactly as the engine drives them:

  Sequence / slot arithmetic      nanovllm/engine/sequence.py:16-141
  page allocation                 nanovllm/engine/block_manager.py:59-102 (no prefix hashing: it is
                                  disabled in the reference, block_manager.py:65-66)
  prepare_prefill / prepare_decode nanovllm/engine/model_runner.py:121-185
  denoise -> CACHING -> append    nanovllm/engine/scheduler.py:24-82
  decoder layer structure         nanovllm/models/sdar.py:68-181, layers/layernorm.py:16-40,
                                  layers/rotary_embedding.py:6-48, layers/embed_head.py:61-67

The decoder is a random-init scaffold whose GEMMs are stock PyTorch (library) GEMMs; attention,
the KV store, the norms, the activation and the unmask step go through libmdx.  Decode passes can
replay a captured HIP graph (model_runner.py:198-259).  There is no vision tower, tokenizer,
weight loader or tensor parallelism here.
"""
from __future__ import annotations

import math
import time
from collections import deque
from dataclasses import dataclass, field
from enum import Enum, auto
from itertools import count

import torch
import torch.nn.functional as F
from torch import nn

from . import _lib
from .context import get_context, reset_context, set_context
from .layers import Attention
from .ops import (confidence_argmax, lm_head_confidence, flash_attn_with_kvcache, qk_norm_rope_store, rms_norm, select_transfer, silu_and_mul,
                  sparse_attn_varlen, unmask_step)

PAGE = 256                      # tokens per KV page (Sequence.kvcache_block_size, sequence.py:17)


# ----------------------------------------------------------------------------- requests
@dataclass
class SamplingParams:
    """nanovllm/sampling_params.py:4-15 plus the number of positions committed per step when
    fewer exceed the threshold (1 in the engine, block/steps in the HF generate loop)."""
    temperature: float = 1.0
    max_new_tokens: int = 64
    ignore_eos: bool = False
    denoising_strategy: str = "low_confidence_dynamic"
    dynamic_threshold: float = 0.9
    stop_token_ids: list = field(default_factory=list)
    transfer_count: int = 1

    def __post_init__(self):
        assert self.temperature > 1e-10, "greedy sampling is not permitted"


class SequenceStatus(Enum):
    WAITING = auto()
    RUNNING = auto()
    CACHING = auto()
    FINISHED = auto()


class Sequence:
    """Per-request state (sequence.py:16-141).  `prefix_embeds` ([n, hidden]) replaces the input
    embeddings of the first n prompt tokens (the engine splices vision embeddings there)."""
    counter = count()

    def __init__(self, token_ids, sampling_params=None, denoising_block_size=32, mask_token_id=151669,
                 prefix_embeds: torch.Tensor | None = None):
        self.seq_id = next(Sequence.counter)
        self.status = SequenceStatus.WAITING
        self.token_ids = list(token_ids)
        self.step_map = []
        self.num_tokens = len(self.token_ids)            # committed tokens, no mask tokens
        self.num_prompt_tokens = len(self.token_ids)
        self.block_table: list[int] = []
        self.sampling_params = sampling_params or SamplingParams()
        self.temperature = self.sampling_params.temperature
        self.max_new_tokens = self.sampling_params.max_new_tokens
        self.ignore_eos = self.sampling_params.ignore_eos
        self.denoising_block_size = denoising_block_size
        self.mask_token_id = mask_token_id
        self.prefix_embeds = prefix_embeds
        self.current_denoising_block = torch.full((denoising_block_size,), mask_token_id, dtype=torch.int64)
        self.current_step_map = torch.zeros((denoising_block_size,), dtype=torch.int32)
        self.current_denoise_step = 0

    def __len__(self):
        return self.num_tokens

    @property
    def is_finished(self):
        return self.status == SequenceStatus.FINISHED

    @property
    def is_caching(self):
        return self.status == SequenceStatus.CACHING

    @property
    def num_completion_tokens(self):
        return self.num_tokens - self.num_prompt_tokens

    @property
    def completion_token_ids(self):
        return self.token_ids[self.num_prompt_tokens:]

    @property
    def num_blocks(self):
        return (self.num_tokens + PAGE - 1) // PAGE

    def append_block(self):                               # sequence.py:97-101
        self.token_ids.extend(self.current_denoising_block.tolist())
        self.step_map.extend(self.current_step_map.tolist())
        self.num_tokens += self.denoising_block_size
        self.current_denoising_block = torch.full((self.denoising_block_size,), self.mask_token_id, dtype=torch.int64)

    def need_new_block(self):                             # sequence.py:114-115
        return self.num_tokens + self.denoising_block_size > PAGE * len(self.block_table)

    def get_slots(self, lo: int, hi: int):                # sequence.py:117-141
        if not self.block_table:
            return [-1] * (hi - lo)
        t = torch.arange(lo, hi)
        table = torch.tensor(self.block_table, dtype=torch.int64)
        return (table[t // PAGE] * PAGE + t % PAGE).tolist()


class BlockManager:
    """Free-list page allocator (block_manager.py:59-102 without the disabled prefix cache)."""

    def __init__(self, num_pages: int, shuffle_seed: int | None = None):
        ids = list(range(num_pages))
        if shuffle_seed is not None:                      # exercise non-contiguous page tables
            g = torch.Generator().manual_seed(shuffle_seed)
            ids = torch.randperm(num_pages, generator=g).tolist()
        self.free = deque(ids)

    def can_allocate(self, seq):
        return len(self.free) >= seq.num_blocks

    def allocate(self, seq):
        assert not seq.block_table
        seq.block_table.extend(self.free.popleft() for _ in range(seq.num_blocks))

    def can_append(self, seq):
        return len(self.free) >= int(seq.need_new_block())

    def may_append(self, seq):
        if seq.need_new_block():
            seq.block_table.append(self.free.popleft())

    def deallocate(self, seq):
        self.free.extend(reversed(seq.block_table))
        seq.block_table.clear()


# ----------------------------------------------------------------------------- decoder scaffold
@dataclass
class DecoderConfig:
    """Defaults = the language model of mineru_diffusion/configuration_mineru_diffusion.py:12-27."""
    num_layers: int = 28
    hidden_size: int = 2048
    num_heads: int = 16
    num_kv_heads: int = 8
    head_dim: int = 128
    intermediate_size: int = 6144
    vocab_size: int = 151936
    rope_theta: float = 1.0e6
    rms_norm_eps: float = 1e-6
    max_position: int = 8192
    block_size: int = 32
    mask_token_id: int = 151669
    fused_qk_rope_store: bool = True    # one libmdx launch for q/k norm + RoPE + KV store (else stock ops)
    fused_layer_ops: bool = True        # libmdx residual-add + RMSNorm and SiLU-and-multiply (else stock ops)


def _rms(x, w, eps):
    return F.rms_norm(x, (x.shape[-1],), w, eps)


class DecoderLayer(nn.Module):
    def __init__(self, c: DecoderConfig):
        super().__init__()
        self.c = c
        qkv_out = (c.num_heads + 2 * c.num_kv_heads) * c.head_dim
        self.qkv_proj = nn.Parameter(torch.empty(qkv_out, c.hidden_size))
        self.o_proj = nn.Parameter(torch.empty(c.hidden_size, c.num_heads * c.head_dim))
        self.gate_up_proj = nn.Parameter(torch.empty(2 * c.intermediate_size, c.hidden_size))
        self.down_proj = nn.Parameter(torch.empty(c.hidden_size, c.intermediate_size))
        self.q_norm = nn.Parameter(torch.ones(c.head_dim))
        self.k_norm = nn.Parameter(torch.ones(c.head_dim))
        self.input_layernorm = nn.Parameter(torch.ones(c.hidden_size))
        self.post_attention_layernorm = nn.Parameter(torch.ones(c.hidden_size))
        self.attn = Attention(c.num_heads, c.head_dim, c.head_dim ** -0.5, c.num_kv_heads)

    def _norm(self, x, residual, w):
        """layernorm.py:43-51: (normed, new residual)."""
        c = self.c
        if c.fused_layer_ops:
            if residual is None:
                return rms_norm(x, w, c.rms_norm_eps), x
            return rms_norm(x, w, c.rms_norm_eps, residual)
        residual = x if residual is None else x + residual
        return _rms(residual, w, c.rms_norm_eps), residual

    def forward(self, positions, x, residual, cos, sin, cos_table=None, sin_table=None):
        c = self.c
        h, residual = self._norm(x, residual, self.input_layernorm)       # sdar.py:147-150
        qkv = F.linear(h, self.qkv_proj)
        if c.fused_qk_rope_store:
            o = self._attend_fused(qkv, positions, cos_table, sin_table)
        else:
            q_size, kv_size = c.num_heads * c.head_dim, c.num_kv_heads * c.head_dim
            q, k, v = qkv.split([q_size, kv_size, kv_size], dim=-1)
            shape = (*positions.shape, -1, c.head_dim)
            q, k, v = q.view(shape), k.view(shape), v.view(shape)   # v stays a strided view of qkv
            q = _rms(q, self.q_norm, c.rms_norm_eps)
            k = _rms(k, self.k_norm, c.rms_norm_eps)
            q, k = _rope(q, cos, sin), _rope(k, cos, sin)
            o = self.attn(q, k, v)
        x = F.linear(o, self.o_proj)
        h, residual = self._norm(x, residual, self.post_attention_layernorm)
        gate_up = F.linear(h, self.gate_up_proj)
        if c.fused_layer_ops:
            act = silu_and_mul(gate_up)
        else:
            gate, up = gate_up.chunk(2, dim=-1)
            act = F.silu(gate) * up
        return F.linear(act, self.down_proj), residual

    def _attend_fused(self, qkv, positions, cos_table, sin_table):
        """sdar.py:79-83 + sdar_attention.py:34-57 with the q/k norm, RoPE and cache store done by
        one libmdx launch; the attention calls are the same two as in `Attention.forward`."""
        c, attn, ctx = self.c, self.attn, get_context()
        have_cache = attn.k_cache.numel() > 0
        q, k, v = qk_norm_rope_store(qkv, self.q_norm, self.k_norm, c.rms_norm_eps, cos_table, sin_table, positions,
                                     c.num_heads, c.num_kv_heads, c.head_dim,
                                     attn.k_cache if have_cache else None, attn.v_cache if have_cache else None,
                                     ctx.slot_mapping if have_cache else None, want_k=ctx.is_prefill)
        if ctx.is_prefill:
            o = sparse_attn_varlen(q, k, v, cu_seqlens_q=ctx.cu_seqlens_q, cu_seqlens_k=ctx.cu_seqlens_k,
                                   staircase_size=ctx.block_size, max_seqlen=ctx.max_seqlen_k or None, softmax_scale=attn.scale)
            return o.flatten(1)
        o = flash_attn_with_kvcache(q, attn.k_cache, attn.v_cache, cache_seqlens=ctx.context_lens,
                                    block_table=ctx.block_tables, softmax_scale=attn.scale, causal=False)
        return o.flatten(2)


def _rope(x, cos, sin):                                    # rotary_embedding.py:6-14
    x1, x2 = torch.chunk(x.float(), 2, dim=-1)
    return torch.cat((x1 * cos - x2 * sin, x2 * cos + x1 * sin), dim=-1).to(x.dtype)


class Decoder(nn.Module):
    """SDAR-shaped decoder-only model (sdar.py:157-216) with random weights (std 0.02)."""

    def __init__(self, c: DecoderConfig, device, dtype=torch.bfloat16, seed: int = 0):
        super().__init__()
        self.c = c
        self.embed_tokens = nn.Parameter(torch.empty(c.vocab_size, c.hidden_size))
        self.layers = nn.ModuleList(DecoderLayer(c) for _ in range(c.num_layers))
        self.norm = nn.Parameter(torch.ones(c.hidden_size))
        self.lm_head = nn.Parameter(torch.empty(c.vocab_size, c.hidden_size))
        self.to(device=device, dtype=dtype)
        g = torch.Generator(device=device).manual_seed(seed)
        with torch.no_grad():
            for name, p in self.named_parameters():
                if p.dim() == 2:
                    p.normal_(0.0, 0.02, generator=g)
        inv_freq = 1.0 / (c.rope_theta ** (torch.arange(0, c.head_dim, 2, dtype=torch.float) / c.head_dim))
        freqs = torch.einsum("i,j->ij", torch.arange(c.max_position, dtype=torch.float), inv_freq)
        self.register_buffer("cos", freqs.cos().to(device), persistent=False)
        self.register_buffer("sin", freqs.sin().to(device), persistent=False)

    def embed(self, input_ids):
        return F.embedding(input_ids, self.embed_tokens)

    @torch.inference_mode()
    def forward(self, inputs_embeds, positions):
        cos = sin = None
        if not self.c.fused_qk_rope_store:
            cos = self.cos[positions].unsqueeze(-2)
            sin = self.sin[positions].unsqueeze(-2)
        x, residual = inputs_embeds, None
        for layer in self.layers:
            x, residual = layer(positions, x, residual, cos, sin, self.cos, self.sin)
        if self.c.fused_layer_ops:
            return rms_norm(x, self.norm, self.c.rms_norm_eps, residual)[0]
        return _rms(x + residual, self.norm, self.c.rms_norm_eps)

    @torch.inference_mode()
    def compute_logits(self, hidden):                      # embed_head.py:61-67
        ctx = get_context()
        if ctx.is_prefill:
            starts = ctx.cu_seqlens_q[1:] - self.c.block_size
            idx = starts.unsqueeze(1) + torch.arange(self.c.block_size, device=starts.device)
            hidden = hidden[idx.long()].contiguous()
        return F.linear(hidden, self.lm_head)


# ----------------------------------------------------------------------------- engine
IDLE, DENOISING, CACHING = 0, 1, 2      # MDX_PHASE_* of include/mdx.h: the per-lane state of the device loop
N_STOP = 4                              # stop-token ids per sequence that the device loop can check


class _PagesShort(Exception):
    """The page pool cannot cover what the device loop wants ahead of a sequence."""


class BlockDiffusionEngine:
    """Scheduler + runner for block-diffusion decoding on one GPU (llm_engine.py:66-73 `step`,
    scheduler.py:24-82, model_runner.py:127-219).

    Two decode paths share the same kernels:
      * host-driven (decode_graphs=False, or a test hook is installed): every pass is prepared on the
        host, run eagerly, and its results are downloaded -- the reference's own control flow;
      * the device loop (decode_graphs=True): block tokens, lengths, step maps and the
        denoise -> caching -> append state machine live on the device (csrc/block_state.hip); a pass is two
        HIP-graph replays (decoder forward, then vocabulary projection + unmask step + state advance) with
        no upload and no blocking download, and the host reads a 16-byte status per sequence one
        pass late, while the next pass already runs."""

    def __init__(self, model: Decoder, num_pages: int, max_num_batched_tokens: int = 1 << 20,
                 max_num_seqs: int = 512, shuffle_pages_seed: int | None = None, on_logits=None, unmask=None,
                 decode_graphs: bool = False, max_model_len: int = 8192, masked_rows_only: bool = True,
                 replay_ahead: bool = True, gumbel_seed: int | None = None, fused_head: bool = True,
                 fused_head_min_rows: int = 384):
        self.model = model
        # device loop: vocabulary projection + confidence in one pass without logits in HBM, from this many rows on
        self.fused_head, self.fused_head_min_rows = fused_head, fused_head_min_rows
        self.decode_graphs = decode_graphs                 # decode through the device loop (HIP graphs per batch size)
        self.max_model_len = max_model_len
        # Gumbel noise on the scaled logits before the argmax, as Sampler.prepare draws it (sampler.py:15-18);
        # None = plain argmax, an int seeds the generator inside the unmask kernel: the noise of a pass is a
        # function of (seed, number of the sampling pass, row, column), so a seed reproduces a generation
        self.gumbel_seed = gumbel_seed
        self._rng_offset = 0                               # sampling passes so far: the generator offset of the next one
        self.replay_ahead = replay_ahead                   # device loop: enqueue pass p+1 before reading the status of pass p
        self.masked_rows_only = masked_rows_only           # device loop: logits for still-masked positions only
        self._graphs = {}                                  # captured batch size -> lane buffers and graphs
        self._loaded = None                                # the lanes that currently hold the running sequences
        self._temps = None
        self.c = model.c
        self.device = model.lm_head.device
        self.max_num_batched_tokens = max_num_batched_tokens
        self.max_num_seqs = max_num_seqs
        self.block_manager = BlockManager(num_pages, shuffle_pages_seed)
        self.waiting: deque[Sequence] = deque()
        self.running: deque[Sequence] = deque()
        self.on_logits = on_logits                         # test hook: (is_prefill, seqs, logits)
        self.unmask = unmask or unmask_step                # the device unmask step (replaceable in host-only tests)
        c = self.c
        dtype = model.lm_head.dtype
        # KV pool [2, layers, pages, 256, Hkv, d] (model_runner.py:113-119)
        self.kv_cache = torch.zeros(2, max(c.num_layers, 1), num_pages, PAGE, c.num_kv_heads, c.head_dim, dtype=dtype, device=self.device)
        for i, layer in enumerate(model.layers):
            layer.attn.k_cache = self.kv_cache[0, i]
            layer.attn.v_cache = self.kv_cache[1, i]
        self.stats = dict(prefill_passes=0, decode_passes=0, committed_tokens=0, prefill_s=0.0, decode_s=0.0)

    # ---- requests / scheduling ----
    def add_request(self, token_ids, sampling_params=None, prefix_embeds=None) -> Sequence:
        seq = Sequence(token_ids, sampling_params, self.c.block_size, self.c.mask_token_id, prefix_embeds)
        self.waiting.append(seq)
        return seq

    def is_finished(self):
        return not self.waiting and not self.running

    def _admit(self):
        """The prefill batch: requests from the head of the waiting queue, in arrival order, while the
        token budget, the sequence limit and the page pool allow (scheduler.py:24-42)."""
        batch, tokens = [], 0
        while self.waiting and len(batch) < self.max_num_seqs:
            seq = self.waiting[0]
            if tokens + len(seq) > self.max_num_batched_tokens or not self.block_manager.can_allocate(seq):
                break
            self.block_manager.allocate(seq)
            tokens += len(seq)
            seq.status = SequenceStatus.RUNNING
            self.running.append(self.waiting.popleft())
            batch.append(seq)
        return batch

    def _grow(self):
        """The decode batch of a host-driven pass: every running sequence gets the page its block needs; when
        the pool is empty, the sequence at the back of the queue gives its pages up (or, alone, the
        sequence itself) and goes back to the waiting queue (scheduler.py:44-63)."""
        batch = []
        while self.running and len(batch) < self.max_num_seqs:
            seq = self.running.popleft()
            evicted_itself = False
            while not self.block_manager.can_append(seq):
                if self.running:
                    self.preempt(self.running.pop())
                else:
                    self.preempt(seq)
                    evicted_itself = True
                    break
            if not evicted_itself:
                self.block_manager.may_append(seq)
                batch.append(seq)
        if not batch:
            raise RuntimeError("KV pool too small for a single sequence")
        self.running.extendleft(reversed(batch))
        return batch

    def schedule(self):
        """(sequences, is_prefill) of the next host-driven pass: prefill first (scheduler.py:24-58)."""
        batch = self._admit()
        if batch:
            return batch, True
        return self._grow(), False

    def preempt(self, seq):                                # scheduler.py:60-63: back to the queue, its pages freed;
        seq.status = SequenceStatus.WAITING                # the next prefill recomputes its cache (the block in
        self.block_manager.deallocate(seq)                 # progress keeps the tokens it has committed so far)
        self.waiting.appendleft(seq)
        self.stats["preemptions"] = self.stats.get("preemptions", 0) + 1

    def postprocess(self, seqs):
        """After a host-driven pass (scheduler.py:65-82): a sequence whose block has no mask left is due
        for its caching pass; one that just had it appends the block and either ends or starts a new one."""
        for seq in seqs:
            if seq.status != SequenceStatus.CACHING:
                if not bool((seq.current_denoising_block == seq.mask_token_id).any()):
                    seq.status = SequenceStatus.CACHING
                continue
            block = seq.current_denoising_block
            stopped = any(bool((block == s).any()) for s in seq.sampling_params.stop_token_ids)
            seq.append_block()
            self.stats["committed_tokens"] += seq.denoising_block_size
            if (stopped and not seq.ignore_eos) or seq.num_completion_tokens >= seq.max_new_tokens:
                self._retire(seq)
            else:
                seq.status = SequenceStatus.RUNNING

    def _retire(self, seq):
        seq.status = SequenceStatus.FINISHED
        self.block_manager.deallocate(seq)
        self.running.remove(seq)

    # ---- host-driven runner (model_runner.py:121-219) ----
    def _block_tables(self, seqs):
        n = max(len(s.block_table) for s in seqs)
        bt = torch.full((len(seqs), n), -1, dtype=torch.int32)
        for i, s in enumerate(seqs):
            bt[i, :len(s.block_table)] = torch.tensor(s.block_table, dtype=torch.int32)
        return bt.to(self.device, non_blocking=True)

    def _embed(self, seqs, input_ids, is_prefill):
        emb = self.model.embed(input_ids)
        if is_prefill:
            at = 0
            for s in seqs:
                if s.prefix_embeds is not None:
                    n = s.prefix_embeds.shape[0]
                    emb[at:at + n] = s.prefix_embeds.to(emb.dtype)
                at += len(s) + self.c.block_size
        return emb

    def prepare_prefill(self, seqs):                       # model_runner.py:127-167 (no prefix cache)
        S = self.c.block_size
        ids, pos, slots, cu, max_len = [], [], [], [0], 0
        for s in seqs:
            n = len(s) + S
            ids.extend(s.token_ids + s.current_denoising_block.tolist())
            pos.extend(range(n))
            cu.append(cu[-1] + n)
            max_len = max(max_len, n)
            slots.extend(s.get_slots(0, len(s)) + [-1] * S)
        dev = self.device
        cu = torch.tensor(cu, dtype=torch.int32).to(dev, non_blocking=True)
        set_context(True, cu, cu, max_len, max_len, torch.tensor(slots, dtype=torch.int32).to(dev, non_blocking=True),
                    None, None, block_size=S)
        return (torch.tensor(ids, dtype=torch.int64).to(dev, non_blocking=True),
                torch.tensor(pos, dtype=torch.int64).to(dev, non_blocking=True))

    def prepare_decode(self, seqs):                        # model_runner.py:169-185
        S = self.c.block_size
        ids = torch.stack([s.current_denoising_block for s in seqs])
        lens = torch.tensor([len(s) for s in seqs], dtype=torch.int64)
        pos = lens.unsqueeze(1) + torch.arange(S)
        slots = torch.tensor([s.get_slots(len(s), len(s) + S) for s in seqs], dtype=torch.int32)
        dev = self.device
        set_context(False, slot_mapping=slots.to(dev, non_blocking=True),
                    context_lens=(lens + S).to(torch.int32).to(dev, non_blocking=True),
                    block_tables=self._block_tables(seqs), block_size=S)
        return ids.to(dev, non_blocking=True), pos.to(dev, non_blocking=True)

    def _temperatures(self, seqs):
        key = tuple(s.temperature for s in seqs)
        if self._temps is None or self._temps[0] != key:
            self._temps = (key, torch.tensor(key, dtype=torch.float32, device=self.device))
        return self._temps[1]

    def sample(self, logits, seqs) -> int:                 # layers/sampler.py:24-61, selection on the device
        sp = seqs[0].sampling_params
        if sp.denoising_strategy != "low_confidence_dynamic":
            raise NotImplementedError(f"Denoising strategy {sp.denoising_strategy} not implemented")
        x = torch.stack([s.current_denoising_block for s in seqs]).to(self.device)
        extra = {} if self.gumbel_seed is None else {"seed": self.gumbel_seed, "offset": self._rng_offset}
        self._rng_offset += 1
        _, _, transfer, _n = self.unmask(logits, x, seqs[0].mask_token_id, sp.dynamic_threshold, sp.transfer_count,
                                         temperatures=self._temperatures(seqs), **extra)
        x_cpu, transfer_cpu = x.cpu(), transfer.cpu()
        for i, s in enumerate(seqs):
            s.current_denoising_block = x_cpu[i]
            s.current_step_map[transfer_cpu[i]] = s.current_denoise_step
            s.current_denoise_step += 1
        return int(transfer_cpu.sum().item())

    @torch.inference_mode()
    def run(self, seqs, is_prefill: bool) -> int:          # model_runner.py:213-219, host-driven
        ids, pos = self.prepare_prefill(seqs) if is_prefill else self.prepare_decode(seqs)
        hidden = self.model(self._embed(seqs, ids, is_prefill), pos)
        logits = self.model.compute_logits(hidden)
        if is_prefill:
            logits = logits.view(len(seqs), self.c.block_size, -1)
        if self.on_logits is not None:
            self.on_logits(is_prefill, seqs, logits)
        n = self.sample(logits, seqs)
        reset_context()
        return n

    # ---- the device loop ----------------------------------------------------------------------------------
    def _graph_batch(self, bs: int) -> int:
        """The captured batch size that serves `bs` sequences: 1, 2, 4, 8, then multiples of 16
        (model_runner.py:233,200); the lanes in excess are idle (slot -1, context length 0)."""
        for b in (1, 2, 4, 8):
            if bs <= b:
                return b
        return (bs + 15) // 16 * 16

    def _device_loop_usable(self, seqs) -> bool:
        if not self.decode_graphs or self.on_logits is not None or self.unmask is not unmask_step:
            return False
        sp = seqs[0].sampling_params
        if sp.denoising_strategy != "low_confidence_dynamic":
            raise NotImplementedError(f"Denoising strategy {sp.denoising_strategy} not implemented")
        S = self.c.block_size
        return all(s.num_prompt_tokens + -(-s.max_new_tokens // S) * S + S <= self.max_model_len and
                   len(s.sampling_params.stop_token_ids) <= N_STOP for s in seqs)

    def _make_lanes(self, gbs: int):
        """Static buffers of the lanes of one captured batch size and the graph of the decoder forward over them.
        The state a (re)load writes is one device buffer mirrored by one pinned host buffer (a single copy)."""
        S, dev = self.c.block_size, self.device
        width = (self.max_model_len + PAGE - 1) // PAGE
        i32, i64, f32 = torch.int32, torch.int64, torch.float32
        fields = [("ids", i64, (gbs, S)), ("stop_ids", i64, (gbs, N_STOP)), ("step_map", i32, (gbs, S)), ("lens", i32, (gbs,)),
                  ("phase", i32, (gbs,)), ("step", i32, (gbs,)), ("first_len", i32, (gbs,)), ("max_new", i32, (gbs,)),
                  ("temps", f32, (gbs,)), ("rng_step", i64, (1,)), ("bt", i32, (gbs, width))]
        offsets, at = {}, 0
        for name, dt, shape in fields:
            offsets[name] = at
            at += (math.prod(shape) * dt.itemsize + 15) // 16 * 16
        g = dict(bs=gbs, width=width, dev_buf=torch.zeros(at, dtype=torch.uint8, device=dev),
                 pin_buf=torch.zeros(at, dtype=torch.uint8, pin_memory=True), host={}, heads={}, pass_no=0)
        for name, dt, shape in fields:
            n = math.prod(shape) * dt.itemsize
            g[name] = g["dev_buf"][offsets[name]:offsets[name] + n].view(dt).view(shape)
            g["host"][name] = g["pin_buf"][offsets[name]:offsets[name] + n].view(dt).view(shape)
        g["pos"] = torch.zeros(gbs, S, dtype=i64, device=dev)                  # written by mdx_block_prepare every pass
        g["slots"] = torch.full((gbs, S), -1, dtype=i32, device=dev)
        g["ctx"] = torch.zeros(gbs, dtype=i32, device=dev)
        g["x0"] = torch.zeros(gbs * S, dtype=i64, device=dev)
        g["x0_p"] = torch.zeros(gbs * S, dtype=f32, device=dev)
        g["rows"] = torch.zeros(gbs * S, dtype=i64, device=dev)
        g["n_rows"] = torch.zeros(1, dtype=i32, device=dev)
        g["out_tokens"] = torch.zeros(gbs, self.max_model_len, dtype=i64, device=dev)
        g["out_steps"] = torch.zeros(gbs, self.max_model_len, dtype=i32, device=dev)
        g["status"] = torch.zeros(gbs, 4, dtype=i32, device=dev)
        g["status_host"] = torch.zeros(2, gbs, 4, dtype=i32, pin_memory=True)
        g["status_done"] = [torch.cuda.Event(), torch.cuda.Event()]
        g["bt_copied"] = torch.cuda.Event()
        g["host"]["bt"].fill_(-1)
        g["host"]["stop_ids"].fill_(-1)
        g["host"]["temps"].fill_(1.0)
        g["dev_buf"].copy_(g["pin_buf"])
        side = torch.cuda.Stream()
        g["stream"] = side
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):                      # warm-up outside the capture (library handles, autotuning)
            self._forward_lanes(g)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        g["fwd"] = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g["fwd"], stream=side):      # the stream of the warm-up: its per-stream buffers exist
            g["hidden"] = self._forward_lanes(g)
        torch.cuda.synchronize()
        return g

    def _forward_lanes(self, g):
        """prepare_decode on the device (positions, slots, context lengths from the lanes' lengths and page
        tables), then the decoder forward over the lanes' blocks."""
        S = self.c.block_size
        stream = torch.cuda.current_stream(self.device).cuda_stream
        _lib.check(_lib.lib().mdx_block_prepare(g["lens"].data_ptr(), g["phase"].data_ptr(), g["bt"].data_ptr(), g["bt"].stride(0),
                                                g["width"], PAGE, S, g["pos"].data_ptr(), g["slots"].data_ptr(), g["ctx"].data_ptr(),
                                                g["bs"], stream), "block_prepare")
        set_context(False, slot_mapping=g["slots"], context_lens=g["ctx"], block_tables=g["bt"], block_size=S)
        hidden = self.model(self.model.embed(g["ids"]), g["pos"])
        reset_context()
        return hidden

    def _logits_of_rows(self, g, cap: int):
        """Vocabulary projection + confidence / argmax on `cap` rows: the still-masked ones compacted on the device
        (cap < all rows), or all of them.  Results land in the lanes' x0 / x0_p."""
        S, gbs = self.c.block_size, g["bs"]
        flat = g["hidden"].flatten(0, 1)
        if cap < gbs * S:
            rows = g["rows"][:cap]
            stream = torch.cuda.current_stream(self.device).cuda_stream
            _lib.check(_lib.lib().mdx_masked_rows(g["ids"].data_ptr(), g["phase"].data_ptr(), self.c.mask_token_id, gbs, S,
                                                  rows.data_ptr(), cap, g["n_rows"].data_ptr(), stream), "masked_rows")
            if self._fused_head(cap):
                x0, p = lm_head_confidence(flat.index_select(0, rows), self.model.lm_head, g["temps"], rows_per_temp=S, row_ids=rows)
            else:
                logits = F.linear(flat.index_select(0, rows), self.model.lm_head)
                x0, p = confidence_argmax(logits, g["temps"].index_select(0, rows // S), **self._draw(g, rows))
            g["x0"].index_copy_(0, rows, x0)
            g["x0_p"].index_copy_(0, rows, p)
        else:
            if self._fused_head(cap):
                x0, p = lm_head_confidence(flat, self.model.lm_head, g["temps"], rows_per_temp=S)
            else:
                logits = F.linear(flat, self.model.lm_head).view(gbs, S, -1)
                x0, p = confidence_argmax(logits, g["temps"], **self._draw(g, None))
            g["x0"].copy_(x0.view(-1))
            g["x0_p"].copy_(p.view(-1))

    def _fused_head(self, rows: int) -> bool:
        """Projection and confidence in one pass that never writes the logits (mdx_lm_head_confidence): taken where it
        is the faster of the two (from a few hundred rows on; below that the library GEMM + the vocabulary pass
        win), for bf16 weights without sampling noise."""
        return (self.fused_head and self.gumbel_seed is None and rows >= self.fused_head_min_rows
                and self.model.lm_head.dtype == torch.bfloat16 and self.model.lm_head.shape[1] % 128 == 0)

    def _draw(self, g, rows):
        """Generator arguments of a device-loop pass: the lanes' own pass counter as the offset, and for compacted
        rows their places in the whole batch, so that compaction does not change the draw."""
        if self.gumbel_seed is None:
            return {}
        return dict(seed=self.gumbel_seed, offset=0, offset_dev=g["rng_step"], row_ids=rows)

    def _head(self, g, cap: int, threshold: float, k: int):
        """The second half of a pass: logits of (at most) `cap` masked rows, the selection rule, and the advance of
        every lane's state (sampler.py:24-61 + scheduler.py:65-82 on the device)."""
        S, gbs = self.c.block_size, g["bs"]
        if cap < gbs * S:
            # rows that get no fresh logits in this pass (the host's bound `cap` fell short of the masked rows: a
            # committed token that happens to be the mask token leaves its position masked) are not committed
            g["x0_p"].fill_(float("-inf"))
        if cap > 0:
            self._logits_of_rows(g, cap)
        transfer, _count = select_transfer(g["x0"].view(gbs, S), g["x0_p"].view(gbs, S), g["ids"], self.c.mask_token_id, threshold, k)
        stream = torch.cuda.current_stream(self.device).cuda_stream
        _lib.check(_lib.lib().mdx_block_advance(
            g["ids"].data_ptr(), transfer.data_ptr(), g["step_map"].data_ptr(), g["step"].data_ptr(), g["phase"].data_ptr(),
            g["lens"].data_ptr(), g["first_len"].data_ptr(), g["max_new"].data_ptr(), g["stop_ids"].data_ptr(), N_STOP,
            g["out_tokens"].data_ptr(), g["out_steps"].data_ptr(), g["out_tokens"].stride(0), g["status"].data_ptr(),
            self.c.mask_token_id, gbs, S, stream), "block_advance")
        g["rng_step"].add_(1)                               # the next pass draws other noise

    def _head_graph(self, g, cap, threshold, k):
        key = (cap, threshold, k)
        graph = g["heads"].get(key)
        if graph is None:
            outer = torch.cuda.current_stream()
            g["stream"].wait_stream(outer)
            with torch.cuda.stream(g["stream"]):           # warm the projection at this row count; touches scratch only, no lane state
                if cap > 0:
                    self._logits_of_rows(g, cap)
            outer.wait_stream(g["stream"])
            torch.cuda.synchronize()
            if "head_pool" not in g:                        # the variants hold temporaries only and never run together: one pool
                g["head_pool"] = torch.cuda.graph_pool_handle()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, pool=g["head_pool"], stream=g["stream"]):
                self._head(g, cap, threshold, k)
            torch.cuda.synchronize()
            g["heads"][key] = graph
        return graph

    def _load_lanes(self, seqs):
        """Puts the state of `seqs` (as the host knows it) into the lanes of the batch size that serves them."""
        S, mask = self.c.block_size, self.c.mask_token_id
        gbs = self._graph_batch(len(seqs))
        g = self._graphs.get(gbs)
        if g is None:
            g = self._graphs[gbs] = self._make_lanes(gbs)
        g["bt_copied"].synchronize()
        h = g["host"]
        h["phase"].zero_()
        h["lens"].zero_()
        h["bt"].fill_(-1)
        h["stop_ids"].fill_(-1)
        h["ids"].fill_(mask)
        h["rng_step"][0] = self._rng_offset
        for i, s in enumerate(seqs):
            h["ids"][i] = s.current_denoising_block
            h["step_map"][i] = s.current_step_map
            h["lens"][i] = len(s)
            h["phase"][i] = CACHING if s.status == SequenceStatus.CACHING else DENOISING
            h["step"][i] = s.current_denoise_step
            h["first_len"][i] = s.num_prompt_tokens
            h["max_new"][i] = s.max_new_tokens
            h["temps"][i] = s.temperature
            stops = [] if s.ignore_eos else list(s.sampling_params.stop_token_ids)
            h["stop_ids"][i, :len(stops)] = torch.tensor(stops, dtype=torch.int64)
            h["bt"][i, :len(s.block_table)] = torch.tensor(s.block_table, dtype=torch.int32)
        g["dev_buf"].copy_(g["pin_buf"], non_blocking=True)
        g["bt_copied"].record()
        masked = (h["ids"][:len(seqs)] == mask).sum(1).tolist()
        g["seqs"] = list(seqs)
        g["known"] = dict(at_pass=g["pass_no"], phase=h["phase"][:len(seqs)].tolist(), masked=masked, lens=h["lens"][:len(seqs)].tolist())
        g["live_at"] = {}                                   # pass number -> lanes that were live at its start, as far as known
        g["pending"] = []                                   # passes enqueued whose status has not been read yet
        self._loaded = g
        return g

    def _cover_pages(self, g):
        """Every live lane's page table must reach as far as the device can get before the host next looks:
        the block being denoised, the block after it, and one more block for the pass in flight."""
        S = self.c.block_size
        changed = False
        for i, s in enumerate(g["seqs"]):
            if g["known"]["phase"][i] == IDLE:
                continue
            last = min(g["known"]["lens"][i] + 3 * S, s.num_prompt_tokens + -(-s.max_new_tokens // S) * S)
            want = (last + PAGE - 1) // PAGE
            while len(s.block_table) < want:
                if not self.block_manager.free:
                    raise _PagesShort()
                if not changed:
                    g["bt_copied"].synchronize()             # the previous upload of the tables has left the pinned buffer
                    changed = True
                g["host"]["bt"][i, len(s.block_table)] = self.block_manager.free[0]
                s.block_table.append(self.block_manager.free.popleft())
        if changed:
            g["bt"].copy_(g["host"]["bt"], non_blocking=True)
            g["bt_copied"].record()

    def _rows_cap(self, g) -> int:
        """The number of rows that get logits in the pass about to be enqueued, rounded up to an eighth of all rows:
        what the host, one pass behind, expects to be masked at most -- a denoising pass commits min(k, masked)
        positions of a lane, a caching pass leaves a fresh block behind.  The expectation can fall short (a
        committed token that is the mask token itself leaves its position masked); rows beyond it get no logits and
        are not committed in that pass, and a denoising lane is never taken to be done before its status says so."""
        S, gbs = self.c.block_size, g["bs"]
        if not self.masked_rows_only:
            return gbs * S
        kn, k = g["known"], g["seqs"][0].sampling_params.transfer_count
        ahead = g["pass_no"] - kn["at_pass"]
        bound = 0
        for ph, m in zip(kn["phase"], kn["masked"]):
            if ahead == 0:
                bound += m if ph == DENOISING else 0
            else:
                bound += S if ph == CACHING else max(1, m - k) if ph == DENOISING else 0
        step = max(1, gbs * S // 8)
        return min(gbs * S, -(-bound // step) * step)

    def _read_status(self, g, pass_no):
        """Takes in the status that pass `pass_no` left: lengths, phases and masked counts of the lanes."""
        slot = pass_no % 2
        g["status_done"][slot].synchronize()
        st = g["status_host"][slot][:len(g["seqs"])].tolist()
        kn = g["known"]
        live_before = [ph != IDLE for ph in kn["phase"]]
        moved = 0
        for i, (ph, ln, masked, n_moved) in enumerate(st):
            if not live_before[i]:
                continue
            kn["phase"][i], kn["lens"][i], kn["masked"][i] = ph, ln, masked
            moved += n_moved
        kn["at_pass"] = pass_no + 1
        if any(live_before):
            self.stats["decode_passes"] += 1
        return moved, any(kn["phase"][i] == IDLE and live_before[i] for i in range(len(st)))

    def _drain(self):
        """Waits for the device loop, brings every loaded sequence's state back to the host and retires the finished ones."""
        g = self._loaded
        if g is None:
            return
        moved = 0
        for pass_no in g["pending"]:
            moved += self._read_status(g, pass_no)[0]
        g["pending"] = []
        torch.cuda.synchronize()
        n = len(g["seqs"])
        ids, step_map, step, lens = g["ids"][:n].cpu(), g["step_map"][:n].cpu(), g["step"][:n].tolist(), g["lens"][:n].tolist()
        phase = g["phase"][:n].tolist()
        for i, s in enumerate(g["seqs"]):
            have = s.num_tokens - s.num_prompt_tokens
            new = lens[i] - s.num_tokens
            if new > 0:
                s.token_ids.extend(g["out_tokens"][i, have:have + new].tolist())
                s.step_map.extend(g["out_steps"][i, have:have + new].tolist())
                s.num_tokens = lens[i]
                self.stats["committed_tokens"] += new
            s.current_denoising_block = ids[i].clone()
            s.current_step_map = step_map[i].clone()
            s.current_denoise_step = step[i]
            if phase[i] == IDLE:
                self._retire(s)
            else:
                s.status = SequenceStatus.CACHING if phase[i] == CACHING else SequenceStatus.RUNNING
        self._loaded = None
        return moved

    @torch.inference_mode()
    def _device_pass(self, seqs) -> int:
        """Enqueues one decode pass of the device loop and, one pass late, looks at what the passes before it did."""
        g = self._loaded
        moved = 0
        if g is None or g["seqs"] != seqs:
            moved += self._drain() or 0
            seqs = [s for s in seqs if not s.is_finished]   # the drain may have retired some of them
            if not seqs:
                return moved
            g = self._load_lanes(seqs)
        self._cover_pages(g)
        sp = seqs[0].sampling_params
        cap = self._rows_cap(g)
        head = self._head_graph(g, cap, float(sp.dynamic_threshold), int(sp.transfer_count))
        g["fwd"].replay()
        head.replay()
        self._rng_offset += 1
        slot = g["pass_no"] % 2
        g["status_host"][slot].copy_(g["status"], non_blocking=True)
        g["status_done"][slot].record()
        g["pending"].append(g["pass_no"])
        g["pass_no"] += 1
        finished = False
        keep = 1 if self.replay_ahead else 0               # passes that may stay unread while the next one is prepared
        while len(g["pending"]) > keep:
            n, fin = self._read_status(g, g["pending"].pop(0))
            moved += n
            finished |= fin
        if finished:
            moved += self._drain() or 0
        return moved

    def step(self):                                        # llm_engine.py:66-73
        t0 = time.perf_counter()
        batch = self._admit() if self.waiting else []
        if batch:
            self._drain()
            n = self.run(batch, True)
            self.postprocess(batch)
            self.stats["prefill_passes"] += 1
            self.stats["prefill_s"] += time.perf_counter() - t0
            return n, True
        seqs = list(self.running)[:self.max_num_seqs]
        if not seqs:
            return 0, False
        n = None
        if self._device_loop_usable(seqs):
            try:
                n = self._device_pass(seqs)
            except _PagesShort:
                self._drain()                               # the host-driven pass below needs less ahead and may preempt
        else:
            self._drain()
        if n is None:
            seqs = self._grow()
            n = self.run(seqs, False)
            self.postprocess(seqs)
            self.stats["decode_passes"] += 1
        self.stats["decode_s"] += time.perf_counter() - t0
        return n, False

    def generate(self):
        """Runs every queued request to completion; returns them in arrival order."""
        seqs = list(self.waiting)
        while not self.is_finished():
            self.step()
        return seqs
