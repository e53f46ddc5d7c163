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

from .context import get_context, reset_context, set_context
from .layers import Attention
from .ops import (confidence_argmax, flash_attn_with_kvcache, qk_norm_rope_store, rms_norm, select_transfer, silu_and_mul,
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
        self.block_has_mask = None                       # filled by the engine's sampler; see postprocess

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
class BlockDiffusionEngine:
    """Scheduler + runner for block-diffusion decoding (llm_engine.py:66-73 `step`, scheduler.py,
    model_runner.py:127-219), one GPU, eager."""

    def __init__(self, model: Decoder, num_pages: int, max_num_batched_tokens: int = 1 << 20,
                 max_num_seqs: int = 512, shuffle_pages_seed: int | None = None, on_logits=None, unmask=None,
                 decode_graphs: bool = False, max_model_len: int = 8192, masked_rows_only: bool = True,
                 replay_ahead: bool = True, gumbel_seed: int | None = None):
        self.model = model
        self.decode_graphs = decode_graphs                 # replay a captured HIP graph per decode batch size
        self.max_model_len = max_model_len
        # Gumbel noise on the scaled logits before the argmax, as Sampler.prepare draws it (sampler.py:15-18);
        # None = plain argmax (reproducible), an int seeds a device generator (reproducible per seed)
        self.gumbel = None if gumbel_seed is None else torch.Generator(device=model.lm_head.device).manual_seed(gumbel_seed)
        self.replay_ahead = replay_ahead                   # graph decode: enqueue the next forward before the host bookkeeping
        self.masked_rows_only = masked_rows_only           # graph decode: logits for still-masked positions only
        self._graphs = {}
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

    # ---- requests / scheduling (scheduler.py:21-63) ----
    def add_request(self, token_ids, sampling_params=None, prefix_embeds=None) -> Sequence:
        seq = Sequence(token_ids, sampling_params, self.c.block_size, self.c.mask_token_id, prefix_embeds)
        self.waiting.append(seq)
        return seq

    def is_finished(self):
        return not self.waiting and not self.running

    def schedule(self):
        scheduled, tokens = [], 0
        while self.waiting and len(scheduled) < self.max_num_seqs:
            seq = self.waiting[0]
            if tokens + len(seq) > self.max_num_batched_tokens or not self.block_manager.can_allocate(seq):
                break
            self.block_manager.allocate(seq)
            tokens += len(seq)
            seq.status = SequenceStatus.RUNNING
            self.waiting.popleft()
            self.running.append(seq)
            scheduled.append(seq)
        if scheduled:
            return scheduled, True
        # decode (scheduler.py:44-58): a sequence that cannot get the page its next block needs makes
        # room by preempting the sequence at the back of the queue (or itself, when it is alone)
        while self.running and len(scheduled) < self.max_num_seqs:
            seq = self.running.popleft()
            while not self.block_manager.can_append(seq):
                if self.running:
                    self.preempt(self.running.pop())
                else:
                    self.preempt(seq)
                    break
            else:
                self.block_manager.may_append(seq)
                scheduled.append(seq)
        if not scheduled:
            raise RuntimeError("KV pool too small for a single sequence")
        self.running.extendleft(reversed(scheduled))
        return scheduled, False

    def preempt(self, seq):                                # scheduler.py:60-63: back to the queue, its pages freed;
        seq.status = SequenceStatus.WAITING                # the next prefill recomputes its cache (the block in
        self.block_manager.deallocate(seq)                 # progress keeps the tokens it has committed so far)
        self.waiting.appendleft(seq)
        self.stats["preemptions"] = self.stats.get("preemptions", 0) + 1

    def postprocess(self, seqs):                           # scheduler.py:65-82
        for seq in seqs:
            if not seq.is_caching:
                probe = seq.block_has_mask                  # (block tensor, any mask left) noted by `sample`
                if probe is not None and probe[0] is seq.current_denoising_block:
                    masked = probe[1]
                else:
                    masked = bool((seq.current_denoising_block == seq.mask_token_id).any())
                if not masked:
                    seq.status = SequenceStatus.CACHING
                continue
            finished = any((seq.current_denoising_block == s).any() for s in seq.sampling_params.stop_token_ids)
            seq.append_block()
            self.stats["committed_tokens"] += seq.denoising_block_size
            if (not seq.ignore_eos and finished) or seq.num_completion_tokens >= seq.max_new_tokens:
                seq.status = SequenceStatus.FINISHED
                self.block_manager.deallocate(seq)
                self.running.remove(seq)
            else:
                seq.status = SequenceStatus.RUNNING

    # ---- runner (model_runner.py:121-219) ----
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

    # ---- decode graphs (model_runner.py:198-211 replay, :221-259 capture) ----
    def _capture_decode(self, bs: int):
        """Static input buffers + one captured forward of the decoder for `bs` sequences.  Every libmdx
        launch goes to torch's current stream and allocates nothing itself, so the capture records
        them like any torch op; page tables have their maximum width so that the split-KV launch
        geometry is the same for every replay.  The five inputs are views into one device buffer
        that mirrors one pinned host buffer: a pass uploads them with a single copy."""
        S, dev = self.c.block_size, self.device
        width = (self.max_model_len + PAGE - 1) // PAGE
        fields = [("ids", torch.int64, (bs, S)), ("pos", torch.int64, (bs, S)), ("slots", torch.int32, (bs, S)),
                  ("lens", torch.int32, (bs,)), ("bt", torch.int32, (bs, width))]
        offsets, at = {}, 0
        for name, dt, shape in fields:
            offsets[name] = at
            at += (math.prod(shape) * dt.itemsize + 15) // 16 * 16
        g = dict(dev_buf=torch.zeros(at, dtype=torch.uint8, device=dev),
                 pin_buf=torch.zeros(at, dtype=torch.uint8, pin_memory=True), host={})
        for name, dt, shape in fields:
            n = math.prod(shape) * dt.itemsize
            g[name] = g["dev_buf"][offsets[name]:offsets[name] + n].view(dt).view(shape)
            g["host"][name] = g["pin_buf"][offsets[name]:offsets[name] + n].view(dt).view(shape)
        g["host"]["slots"].fill_(-1)
        g["host"]["bt"].fill_(-1)
        g["dev_buf"].copy_(g["pin_buf"])
        g["result"] = torch.zeros(2, bs, S, dtype=torch.int64, device=dev)          # tokens, transfer flags
        g["result_host"] = torch.zeros(2, bs, S, dtype=torch.int64, pin_memory=True)
        g["downloaded"] = torch.cuda.Event()
        g["idx_host"] = torch.zeros(bs * S, dtype=torch.int64, pin_memory=True)       # rows still masked
        g["idx_dev"] = torch.zeros(bs * S, dtype=torch.int64, device=dev)
        set_context(False, slot_mapping=g["slots"], context_lens=g["lens"], block_tables=g["bt"], block_size=S)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):                      # warm-up outside the capture (library handles, autotuning)
            self.model(self.model.embed(g["ids"]), g["pos"])
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        g["graph"] = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g["graph"], stream=side):    # the stream of the warm-up: its per-stream buffers exist
            g["hidden"] = self.model(self.model.embed(g["ids"]), g["pos"])
        torch.cuda.synchronize()
        return g

    def _graph_batch(self, bs: int) -> int:
        """The captured batch size that serves `bs` sequences: 1, 2, 4, 8, then multiples of 16
        (model_runner.py:233,200); the rows in excess are padding (slot -1, context length 0)."""
        for b in (1, 2, 4, 8):
            if bs <= b:
                return b
        return (bs + 15) // 16 * 16

    def _run_decode_graph(self, seqs):
        """Uploads the pass inputs (one copy) and replays the graph.  Within a denoising block
        nothing has to be uploaded at all: lengths, slots and page tables are those of the previous
        pass, and the token block on the device is the one the unmask step just updated in place
        (the host rows handed to the sequences by `sample` are a download of exactly that buffer)."""
        S, bs = self.c.block_size, len(seqs)
        gbs = self._graph_batch(bs)
        g = self._graphs.get(gbs)
        if g is None:
            g = self._graphs[gbs] = self._capture_decode(gbs)
        signature = [(s.seq_id, s.num_tokens, len(s.block_table)) for s in seqs]
        rows = g.get("rows")
        fresh = (g.get("signature") == signature and rows is not None
                 and all(s.current_denoising_block is r for s, r in zip(seqs, rows)))
        if not fresh:
            h = g["host"]
            torch.stack([s.current_denoising_block for s in seqs], out=h["ids"][:bs])
            lens = torch.tensor([len(s) for s in seqs], dtype=torch.int64)
            torch.add(lens.unsqueeze(1), torch.arange(S), out=h["pos"][:bs])
            h["slots"].fill_(-1)                            # padding rows: nothing stored, no context (model_runner.py:203-206)
            h["slots"][:bs] = torch.tensor([s.get_slots(len(s), len(s) + S) for s in seqs], dtype=torch.int32)
            h["lens"].zero_()
            h["lens"][:bs] = lens + S
            h["ids"][bs:] = 0
            h["pos"][bs:] = 0
            h["bt"].fill_(-1)
            for i, s in enumerate(seqs):
                h["bt"][i, :len(s.block_table)] = torch.tensor(s.block_table, dtype=torch.int32)
            g["dev_buf"].copy_(g["pin_buf"], non_blocking=True)
            g["signature"] = signature
            g["x_host"] = h["ids"][:bs]                     # host copy of the device token blocks
        set_context(False, slot_mapping=g["slots"], context_lens=g["lens"], block_tables=g["bt"], block_size=S)
        ahead = g.pop("replayed_ahead", False)              # enqueued by the previous pass's `_download`?
        for other in self._graphs.values():
            other.pop("replayed_ahead", None)               # a forward enqueued ahead for another batch is void
        if not (fresh and ahead):
            g["graph"].replay()
        return g["hidden"], g

    def _noise(self, logits):
        if self.gumbel is None:
            return None
        e = torch.empty(logits.shape, dtype=torch.float32, device=logits.device).exponential_(generator=self.gumbel)
        return -e.log_()

    def _temperatures(self, seqs):
        key = tuple(s.temperature for s in seqs)
        if self._temps is None or self._temps[0] != key:
            self._temps = (key, torch.tensor(key, dtype=torch.float32, device=self.device))
        return self._temps[1]

    def sample(self, logits, seqs, g=None) -> int:         # layers/sampler.py:24-61 on the device
        """Unmask step on the device, then one download of (tokens, transfer flags).  With the
        buffers `g` of a decode graph, the token block is the graph's own input buffer (already
        on the device) and the download goes through one pinned buffer."""
        sp = seqs[0].sampling_params
        if sp.denoising_strategy != "low_confidence_dynamic":
            raise NotImplementedError(f"Denoising strategy {sp.denoising_strategy} not implemented")
        if g is not None:
            x = g["ids"][:len(seqs)]
        else:
            x = torch.stack([s.current_denoising_block for s in seqs]).to(self.device)
        extra = {} if self.gumbel is None else {"noise": self._noise(logits)}
        _, _, transfer, _n = self.unmask(logits, x, seqs[0].mask_token_id, sp.dynamic_threshold, sp.transfer_count,
                                         temperatures=self._temperatures(seqs), **extra)
        if g is None:
            x_cpu, transfer_cpu = x.cpu(), transfer.cpu()
            for i, s in enumerate(seqs):
                s.current_denoising_block = x_cpu[i]
                s.current_step_map[transfer_cpu[i]] = s.current_denoise_step
                s.current_denoise_step += 1
            return int(transfer_cpu.sum().item())
        return self._download(seqs, g, x, transfer)

    def _download(self, seqs, g, x, transfer) -> int:
        """One download of (tokens, transfer flags) through the pinned buffer, then the per-sequence
        bookkeeping of sampler.py:56-59 as batch operations."""
        bs = len(seqs)
        g["result"][0, :bs].copy_(x)
        g["result"][1, :bs].copy_(transfer)
        g["result_host"].copy_(g["result"], non_blocking=True)
        g["downloaded"].record()
        # The next pass's forward needs nothing from the host when no sequence of this pass is about
        # to append its block (then lengths, slots and page tables stay, and the token block is on
        # the device already): enqueue it now, so that the GPU runs it while the host does the
        # bookkeeping below.  `_run_decode_graph` checks that this really was the next pass.
        if self.replay_ahead and not any(s.is_caching for s in seqs):
            g["graph"].replay()
            g["replayed_ahead"] = True
        g["downloaded"].synchronize()
        x_cpu, transfer_cpu = g["result_host"][0, :bs].clone(), g["result_host"][1, :bs].bool()
        g["x_host"] = x_cpu
        # one indexed write for all step maps: the sequences' maps are rows of one batch tensor
        maps, map_rows = g.get("maps"), g.get("map_rows")
        if maps is None or not all(s.current_step_map is r for s, r in zip(seqs, map_rows)):
            maps = g["maps"] = torch.stack([s.current_step_map for s in seqs])
            map_rows = g["map_rows"] = list(maps.unbind(0))
            for s, r in zip(seqs, map_rows):
                s.current_step_map = r
        steps = torch.tensor([s.current_denoise_step for s in seqs], dtype=torch.int32)
        maps[transfer_cpu] = steps.unsqueeze(1).expand_as(maps)[transfer_cpu]
        rows = g["rows"] = list(x_cpu.unbind(0))
        has_mask = (x_cpu == seqs[0].mask_token_id).any(1).tolist()
        for s, r, m in zip(seqs, rows, has_mask):
            s.current_denoising_block = r
            s.block_has_mask = (r, m)
            s.current_denoise_step += 1
        return int(transfer_cpu.sum().item())

    def _sample_masked_rows(self, hidden, seqs, g) -> int:
        """The unmask step restricted to the positions that are still masked.  The selection reads
        confidences of masked positions only (sampler.py:39) and commits x0 only there (:54), so the
        logits of committed positions are never looked at: the vocabulary projection, the softmax
        and the argmax run on the masked rows alone (half the rows on average, none in the pass
        that only caches a finished block), with identical results."""
        sp = seqs[0].sampling_params
        if sp.denoising_strategy != "low_confidence_dynamic":
            raise NotImplementedError(f"Denoising strategy {sp.denoising_strategy} not implemented")
        S, bs, mask_id = self.c.block_size, len(seqs), seqs[0].mask_token_id
        idx = (g["x_host"].reshape(-1) == mask_id).nonzero().squeeze(1)
        if idx.numel() == 0:
            for s in seqs:
                s.current_denoise_step += 1
            return 0
        # through pinned memory: a copy from pageable memory would hold the host until the stream,
        # which may already hold the next forward, has drained
        n = idx.numel()
        g["idx_host"][:n].copy_(idx)
        idx_dev = g["idx_dev"][:n]
        idx_dev.copy_(g["idx_host"][:n], non_blocking=True)
        logits = F.linear(hidden.flatten(0, 1).index_select(0, idx_dev), self.model.lm_head)   # rows of the first bs sequences
        temps = self._temperatures(seqs)
        if len(set(self._temps[0])) == 1:
            temps = temps[:1]
        else:
            temps = temps.index_select(0, idx_dev // S)
        x0_rows, p_rows = confidence_argmax(logits, temps, self._noise(logits))
        if "x0" not in g:
            g["x0"] = torch.zeros(g["ids"].numel(), dtype=torch.int64, device=self.device)
            g["x0_p"] = torch.zeros(g["ids"].numel(), dtype=torch.float32, device=self.device)
        g["x0"].index_copy_(0, idx_dev, x0_rows)
        g["x0_p"].index_copy_(0, idx_dev, p_rows)
        transfer, _n = select_transfer(g["x0"][:bs * S].view(bs, S), g["x0_p"][:bs * S].view(bs, S), g["ids"][:bs], mask_id,
                                       sp.dynamic_threshold, sp.transfer_count)
        return self._download(seqs, g, g["ids"][:bs], transfer)

    @torch.inference_mode()
    def run(self, seqs, is_prefill: bool) -> int:          # model_runner.py:213-219
        if not is_prefill and self.decode_graphs and max(len(s) for s in seqs) + self.c.block_size <= self.max_model_len:
            hidden, g = self._run_decode_graph(seqs)
        else:
            g = None
            ids, pos = self.prepare_prefill(seqs) if is_prefill else self.prepare_decode(seqs)
            hidden = self.model(self._embed(seqs, ids, is_prefill), pos)
        if g is not None and self.masked_rows_only and self.on_logits is None and self.unmask is unmask_step:
            n = self._sample_masked_rows(hidden, seqs, g)
            reset_context()
            return n
        logits = self.model.compute_logits(hidden if g is None else hidden[:len(seqs)])
        if is_prefill:
            logits = logits.view(len(seqs), self.c.block_size, -1)
        if self.on_logits is not None:
            self.on_logits(is_prefill, seqs, logits)
        n = self.sample(logits, seqs, g)
        reset_context()
        return n

    def step(self):                                        # llm_engine.py:66-73
        seqs, is_prefill = self.schedule()
        t0 = time.perf_counter()
        n = self.run(seqs, is_prefill)
        self.postprocess(seqs)
        dt = time.perf_counter() - t0
        self.stats["prefill_passes" if is_prefill else "decode_passes"] += 1
        self.stats["prefill_s" if is_prefill else "decode_s"] += dt
        return n, is_prefill

    def generate(self):
        """Runs every queued request to completion; returns them in arrival order."""
        seqs = list(self.waiting)
        while not self.is_finished():
            self.step()
        return seqs
