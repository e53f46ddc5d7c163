"""Benchmark of the block-diffusion attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One "step" is one prefill pass of the attention layer over benchmark config 3 (8 packed
sequences, lengths U[1024, 8192], 32-token blocks, Hq 16 / Hkv 8 / d 128, bf16):
store_kvcache of the committed rows, then the staircase attention.  `value` is the
attention's ALGORITHMIC throughput (4*d*Hq flops per visible (query, key) pair, masked
pairs earn nothing) over the whole step time.  The same run also times, each with its own
roofline entry under "ops": store_kvcache alone (config 3), the paged single-block attention
(config 2) and the unmask step (config 4).  A bounded CPU leg runs the oracle (torch SDPA with
an explicit boolean mask, index_copy-style store, fp64 softmax) on the host cores as a baseline.

Prints ONE JSON line on stdout; progress goes to stderr.
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import threading
import time
from itertools import count
from pathlib import Path

ROOT = Path(__file__).resolve().parent
for p in (ROOT, ROOT / "mineru-diffusion_amd"):
    if str(p) not in sys.path:
        sys.path.insert(0, str(p))

import numpy as np  # noqa: E402
import torch  # noqa: E402

HQ, HKV, D, S, PAGE, VOCAB, MASK_ID = 16, 8, 128, 32, 256, 151936, 151669
PEAK_MFMA_TFLOPS = 2500.0          # MI355X dense bf16
PEAK_HBM_GBS = 8000.0              # MI355X HBM3E


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def ev_pair():
    return torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)


def time_kernel(fn, warmup, iters, graph=False, before_timed=None):
    """Average duration (ms) of fn's GPU work.  fn(i) must only enqueue work on torch's current
    stream (no allocation, no host sync); the `iters` calls are bracketed by ONE pair of HIP events
    recorded on that stream.  With graph=True the `iters` calls are first recorded into a HIP graph
    and the events bracket one replay of it: the figure is then the back-to-back duration of the
    launches themselves, whatever the host's launch rate (under a profiler the host falls behind
    the GPU on legs that take two short launches per call).  before_timed() runs (untimed) right
    before the timed launches, for legs whose calls consume their input.  A second number, the
    minimum over individually bracketed launches, is returned for reference."""
    for _ in range(warmup):
        fn(0)
    torch.cuda.synchronize()
    a, b = ev_pair()
    if graph:
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for i in range(iters):
                fn(i)
        g.replay()
        torch.cuda.synchronize()
        if before_timed is not None:
            before_timed()
        a.record()
        g.replay()
        b.record()
    else:
        if before_timed is not None:
            before_timed()
        a.record()
        for i in range(iters):
            fn(i)
        b.record()
    torch.cuda.synchronize()
    avg = a.elapsed_time(b) / iters
    pairs = []
    for i in range(min(iters, 10)):
        x, y = ev_pair()
        x.record()
        fn(i)
        y.record()
        pairs.append((x, y))
    torch.cuda.synchronize()
    return float(avg), float(min(x.elapsed_time(y) for x, y in pairs))


def op_entry(ms_graph, ms_single, bound, work, unit_div, peak, unit, extra=None):
    """One entry of "ops".  ms_graph: average duration of a launch inside one replay of a HIP graph of
    K back-to-back launches (launch gaps of the host excluded: the kernel's own time, what rocprofv3's
    kernel trace averages); ms_single: the fastest of ten individually bracketed eager launches (what a
    caller that launches one at a time sees, launch latency included).  `roofline` uses ms_graph,
    `roofline_single_launch` ms_single."""
    def roof(ms):
        a = work / ms / unit_div
        return dict(bound=bound, achieved=round(a, 2), peak=peak, unit=unit, frac=round(a / peak, 4), traffic=None)
    d = dict(ms_graph=round(ms_graph, 4), ms_single=round(ms_single, 4))
    d.update(extra or {})
    d["roofline"] = roof(ms_graph)
    d["roofline_single_launch"] = roof(ms_single)
    return d


def raw_stream():
    return torch.cuda.current_stream().cuda_stream


class PowerSampler:
    """Reads the socket power (hwmon power1_input, microwatts) and the shader clock (the starred line
    of pp_dpm_sclk) of card 0 from sysfs every few milliseconds on a host thread while a leg runs.
    Read-only files that an ordinary user may read; where they are missing the leg reports that."""

    def __init__(self, period_s=0.005):
        self.period = period_s
        self.power_file = self.sclk_file = self.cap_w = None
        for dev_dir in sorted(Path("/sys/class/drm").glob("card*/device")):
            for hw in sorted(dev_dir.glob("hwmon/hwmon*")):
                if (hw / "power1_input").exists() or (hw / "power1_average").exists():
                    self.power_file = hw / ("power1_input" if (hw / "power1_input").exists() else "power1_average")
                    if (hw / "power1_cap").exists():
                        try:
                            self.cap_w = int((hw / "power1_cap").read_text()) / 1e6
                        except (OSError, ValueError):
                            pass
                    if (dev_dir / "pp_dpm_sclk").exists():
                        self.sclk_file = dev_dir / "pp_dpm_sclk"
                    break
            if self.power_file is not None:
                break

    def available(self):
        return self.power_file is not None

    def _read(self):
        w = mhz = None
        try:
            w = int(self.power_file.read_text()) / 1e6
        except (OSError, ValueError):
            pass
        if self.sclk_file is not None:
            try:
                for line in self.sclk_file.read_text().splitlines():
                    if line.rstrip().endswith("*"):
                        mhz = float(line.split(":")[1].strip().split("M")[0])
            except (OSError, ValueError, IndexError):
                pass
        return w, mhz

    def run(self, enqueue, seconds):
        """Calls enqueue() (which replays a HIP graph of back-to-back launches and synchronizes) in a loop for
        about `seconds` while the thread samples; returns mean / max power and clock over the samples taken
        after the first third of the time (ramp), and the average duration of one enqueue() in that part."""
        samples, stop = [], threading.Event()

        def sample():
            while not stop.is_set():
                samples.append((time.perf_counter(),) + self._read())
                time.sleep(self.period)
        th = threading.Thread(target=sample, daemon=True)
        th.start()
        t0 = time.perf_counter()
        marks = []
        while time.perf_counter() - t0 < seconds:
            enqueue()
            marks.append(time.perf_counter())
        stop.set()
        th.join()
        cut = t0 + seconds / 3
        late = [s for s in samples if s[0] >= cut]
        ws = [s[1] for s in late if s[1] is not None]
        cs = [s[2] for s in late if s[2] is not None]
        late_marks = [m for m in marks if m >= cut]
        per_call = (late_marks[-1] - late_marks[0]) / (len(late_marks) - 1) if len(late_marks) > 1 else float("nan")
        return dict(samples=len(late), power_w_mean=round(float(np.mean(ws)), 1) if ws else None,
                    power_w_max=round(float(np.max(ws)), 1) if ws else None,
                    sclk_mhz_mean=round(float(np.mean(cs)), 1) if cs else None,
                    sclk_mhz_min=round(float(np.min(cs)), 1) if cs else None,
                    sclk_mhz_max=round(float(np.max(cs)), 1) if cs else None), per_call


# ----------------------------------------------------------------------------- config 3
def make_cfg3(dev, seed=3):
    """8 sequences, L ~ U{1024..8192} (not rounded to the block), packed; q/k contiguous as after
    RoPE, v a strided view of the fused projection output (row stride 4096), random page tables,
    last 32 tokens of each sequence uncommitted (slot -1) as in the engine's prefill."""
    import oracle
    g = torch.Generator().manual_seed(seed)
    lens = [int(x) for x in torch.randint(1024, 8193, (8,), generator=g)]
    N = sum(lens)
    cu = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32)
    fused = torch.empty(N, (HQ + 2 * HKV) * D, dtype=torch.bfloat16)
    for s in range(0, N, 4096):                      # chunked: keeps host memory flat
        fused[s:s + 4096] = torch.randn(min(4096, N - s), fused.shape[1], generator=g).bfloat16()
    n_pages = sum((L + PAGE - 1) // PAGE for L in lens) + 64
    perm = torch.randperm(n_pages, generator=g).tolist()
    slots = []
    for L in lens:
        n = (L + PAGE - 1) // PAGE
        table, perm = perm[:n], perm[n:]
        slots += oracle.get_slots(table, 0, L - S) + [-1] * S
    host = dict(lens=lens, cu=cu, fused=fused, slots=torch.tensor(slots, dtype=torch.int32), n_pages=n_pages)
    dfused = fused.to(dev)
    gpu = dict(
        q=dfused[:, :HQ * D].reshape(N, HQ, D).contiguous(),
        k=dfused[:, HQ * D:(HQ + HKV) * D].reshape(N, HKV, D).contiguous(),
        v=dfused[:, (HQ + HKV) * D:].view(N, HKV, D),
        cu=cu.to(dev), slots=host["slots"].to(dev),
        k_cache=torch.zeros(n_pages, PAGE, HKV, D, dtype=torch.bfloat16, device=dev),
        v_cache=torch.zeros(n_pages, PAGE, HKV, D, dtype=torch.bfloat16, device=dev),
    )
    return host, gpu


def cfg3_work(lens):
    import oracle
    pairs = sum(oracle.staircase_pairs(L, S) for L in lens)
    stored = sum(L - S for L in lens)
    return dict(pairs=pairs, flops=4 * D * HQ * pairs, store_bytes=2 * 2 * HKV * D * 2 * stored, tokens=sum(lens))


# ----------------------------------------------------------------------------- config 2
def make_cfg2(dev, n_sets=4, seed=2):
    """16 sequences, prefix U{512..4096} + 32, page 256, page tables = disjoint slices of a random
    permutation of a 64k-page pool (2 x 32 GiB, only the referenced pages are filled).  n_sets
    independent page sets are rotated so the 256 MB last-level cache does not hold the K/V."""
    g = torch.Generator().manual_seed(seed)
    bs, pool = 16, 65536
    ctxs = [int(x) + S for x in torch.randint(512, 4097, (bs,), generator=g)]
    maxp = max((c + PAGE - 1) // PAGE for c in ctxs)
    k_cache = torch.empty(pool, PAGE, HKV, D, dtype=torch.bfloat16, device=dev)
    v_cache = torch.empty(pool, PAGE, HKV, D, dtype=torch.bfloat16, device=dev)
    perm = torch.randperm(pool, generator=g)
    at, sets = 0, []
    for _ in range(n_sets):
        bt = torch.full((bs, maxp), -1, dtype=torch.int32)
        for b, c in enumerate(ctxs):
            n = (c + PAGE - 1) // PAGE
            bt[b, :n] = perm[at:at + n].to(torch.int32)
            at += n
        ids = bt[bt >= 0].long().to(dev)
        k_cache[ids] = torch.randn(ids.numel(), PAGE, HKV, D, device=dev, dtype=torch.float32).bfloat16()
        v_cache[ids] = torch.randn(ids.numel(), PAGE, HKV, D, device=dev, dtype=torch.float32).bfloat16()
        sets.append(bt.to(dev))
    q = torch.randn(bs, S, HQ, D, generator=g).bfloat16().to(dev)
    lens = torch.tensor(ctxs, dtype=torch.int32, device=dev)
    sum_ctx = sum(ctxs)
    work = dict(flops=4 * D * HQ * S * sum_ctx, bytes=2 * HKV * D * 2 * sum_ctx + 2 * bs * S * HQ * D * 2, sum_ctx=sum_ctx)
    return dict(q=q, k_cache=k_cache, v_cache=v_cache, tables=sets, lens=lens, ctxs=ctxs, work=work)


# ----------------------------------------------------------------------------- config 4
def make_cfg4(dev, n_sets=2, seed=4):
    """[32 x 32 x 151936] bf16 logits ~ N(0, 3^2), 50-100 % of each block masked; two logits
    buffers are rotated (622 MB > last-level cache)."""
    g = torch.Generator(device=dev).manual_seed(seed)
    gc = torch.Generator().manual_seed(seed)
    sets = []
    for _ in range(n_sets):
        logits = torch.empty(32, S, VOCAB, dtype=torch.bfloat16, device=dev)
        for b in range(32):
            logits[b] = (torch.randn(S, VOCAB, generator=g, device=dev) * 3).bfloat16()
        sets.append(logits)
    tokens = torch.randint(0, 1000, (32, S), generator=gc, dtype=torch.int64)
    for b in range(32):
        n = int(torch.randint(S // 2, S + 1, (1,), generator=gc))
        tokens[b, torch.randperm(S, generator=gc)[:n]] = MASK_ID
    return dict(logits=sets, tokens=tokens, bytes=32 * S * VOCAB * 2)


# ----------------------------------------------------------------------------- config 5
def run_cfg5(dev, layers=28, batch=32, new_tokens=2048, steps_per_block=8, masked_rows_only=True, gumbel_seed=None, fused_head=True):
    """Random-init SDAR-shaped decoder (28 layers, hidden 2048, Hq 16 / Hkv 8 / d 128, SwiGLU 6144,
    vocab 151936), batch 32, 1024 random prefix embeddings + 64 prompt tokens per sequence, 2048 new
    tokens in 32-token blocks, k = 32/8 = 4 committed positions per denoising pass, threshold 0.9.
    Returns committed tokens/s over the whole generation (prefill included), after an untimed
    two-block warm-up generation on the same prompts."""
    from mdx.engine import BlockDiffusionEngine, Decoder, DecoderConfig, SamplingParams
    cfg = DecoderConfig(num_layers=layers)
    model = Decoder(cfg, dev, seed=5)
    pages_per_seq = (1088 + new_tokens + PAGE - 1) // PAGE + 1
    eng = BlockDiffusionEngine(model, num_pages=batch * pages_per_seq + 8, shuffle_pages_seed=5, decode_graphs=True, max_model_len=4096,
                               masked_rows_only=masked_rows_only, gumbel_seed=gumbel_seed, fused_head=fused_head)
    g = torch.Generator().manual_seed(5)
    prompts = []
    for _ in range(batch):
        prompts.append(([0] * 1024 + torch.randint(0, 151000, (64,), generator=g).tolist(),
                        (torch.randn(1024, cfg.hidden_size, generator=g) * 0.02).to(dev)))
    # Untimed warm-up on the same prompts: two blocks per sequence, which takes the engine through
    # the prefill shape, the decode graph capture and the library's first-call set-up.
    warm = SamplingParams(max_new_tokens=2 * S, ignore_eos=True, transfer_count=S // steps_per_block)
    for ids, emb in prompts:
        eng.add_request(ids, warm, prefix_embeds=emb)
    eng.generate()
    for key in eng.stats:
        eng.stats[key] = type(eng.stats[key])()
    sp = SamplingParams(max_new_tokens=new_tokens, ignore_eos=True, transfer_count=S // steps_per_block)
    for ids, emb in prompts:
        eng.add_request(ids, sp, prefix_embeds=emb)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    seqs = eng.generate()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    done = sum(s.num_completion_tokens for s in seqs)
    st = eng.stats
    # what the run must have done, whatever its speed: every sequence complete, no mask token left, one step-map
    # entry per token, and (no confidence of a random-init model reaches the threshold) 8 denoising passes + 1
    # caching pass per block, the first denoising pass of the first block being the prefill
    blocks = new_tokens // S
    assert all(s.num_completion_tokens == new_tokens and len(s.step_map) == new_tokens for s in seqs), "incomplete generation"
    assert not any(cfg.mask_token_id in s.completion_token_ids for s in seqs), "mask token in the output"
    expected = blocks * (steps_per_block + 1) - 1
    if gumbel_seed is None:
        assert st["decode_passes"] == expected, f"unexpected pass count {st['decode_passes']}"
    else:
        # a sampled draw can be the mask token itself (1 in 151 936 per draw on these logits): the position then stays
        # masked for another pass, as in the reference (sampler.py:32 looks at the tokens, not at what was committed)
        assert expected <= st["decode_passes"] <= expected + blocks, f"unexpected pass count {st['decode_passes']}"
    out = dict(tokens_per_s=round(done / dt, 1), seconds=round(dt, 3), committed_tokens=done, batch=batch,
               prefill_passes=st["prefill_passes"], decode_passes=st["decode_passes"],
               prefill_s=round(st["prefill_s"], 3), decode_s=round(st["decode_s"], 3),
               ms_per_decode_pass=round(st["decode_s"] / max(1, st["decode_passes"]) * 1e3, 3), layers=layers,
               vocabulary_projection=("rows of still-masked positions only (the unmask rule reads no others; same tokens)"
                                      if masked_rows_only else "all 32 positions of every block, as the reference computes them"),
               model="random-init 28-layer SDAR-shaped decoder, stock PyTorch-ROCm GEMMs, libmdx attention/KV store/unmask")
    del eng, model
    torch.cuda.empty_cache()
    return out


# ----------------------------------------------------------------------------- CPU baseline
def cpu_baseline(host3):
    """The oracle on the host cores over the whole config-3 input (all 8 packed sequences, the
    same bytes the GPU step reads): SDPA with the explicit [L, L] staircase mask per sequence
    (bf16 inputs upcast to fp32), six timed passes after a short warm-up: about 10 s of CPU work
    on a 16-core host."""
    import oracle
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    lens = host3["lens"]
    N = sum(lens)
    fused = host3["fused"]
    q = fused[:, :HQ * D].reshape(N, HQ, D)
    k = fused[:, HQ * D:(HQ + HKV) * D].reshape(N, HKV, D)
    v = fused[:, (HQ + HKV) * D:].reshape(N, HKV, D)
    cu = [0] + list(np.cumsum(lens))
    oracle.staircase_attn_varlen(q[:512], k[:512], v[:512], [0, 512], S)      # warm-up
    ts = []
    for _ in range(6):
        t0 = time.perf_counter()
        oracle.staircase_attn_varlen(q, k, v, cu, S)
        ts.append(time.perf_counter() - t0)
    flops = sum(4 * D * HQ * oracle.staircase_pairs(L, S) for L in lens)
    t = float(np.mean(ts))
    return dict(value=round(flops / t / 1e12, 5), unit="TFLOP/s", cores=torch.get_num_threads(), kind="port",
                sample=f"oracle (torch SDPA fp32 + explicit boolean staircase mask) on the whole config-3 input "
                       f"({len(lens)} sequences, {N} tokens), mean of 6 passes of {t:.2f} s; flops counted on visible pairs only",
                ms=round(t * 1e3, 2))


def cpu_decode_pass(layers=2, batch=32, ctx=2112):
    """One decode pass of the config-5 decoder on the host cores, at reduced depth: `layers` decoder
    layers (of 28) on `batch` x 32 tokens against a cached context of `ctx` keys per sequence, plus the
    vocabulary projection and the unmask arithmetic, fp32, stock torch CPU ops (a port of the pass,
    not the reference's code).  Returns the pass time extrapolated to 28 layers and the committed
    tokens/s it implies at 8 denoising passes + 1 caching pass per 32-token block."""
    import torch.nn.functional as F
    import oracle
    g = torch.Generator().manual_seed(55)
    H, I, V = 2048, 6144, VOCAB
    rows = batch * S
    w = dict(qkv=torch.randn((HQ + 2 * HKV) * D, H, generator=g) * 0.02, o=torch.randn(H, HQ * D, generator=g) * 0.02,
             gu=torch.randn(2 * I, H, generator=g) * 0.02, down=torch.randn(H, I, generator=g) * 0.02, norm=torch.ones(H), hn=torch.ones(D))
    head = torch.randn(V, H, generator=g) * 0.02
    kc = torch.randn(batch, HKV, ctx, D, generator=g)
    vc = torch.randn(batch, HKV, ctx, D, generator=g)
    cos, sin = torch.ones(rows, 1, D // 2), torch.zeros(rows, 1, D // 2)
    x = torch.randn(rows, H, generator=g)

    def layer(x, res):
        res = x + res
        h = F.rms_norm(res, (H,), w["norm"], 1e-6)
        qkv = h @ w["qkv"].T
        q, k, v = qkv.split([HQ * D, HKV * D, HKV * D], -1)
        q = oracle.rope_ref(oracle.rms_norm_ref(q.reshape(rows, HQ, D), w["hn"], 1e-6), cos, sin)
        k = oracle.rope_ref(oracle.rms_norm_ref(k.reshape(rows, HKV, D), w["hn"], 1e-6), cos, sin)
        kc[:, :, -S:] = k.reshape(batch, S, HKV, D).transpose(1, 2)          # the block's K/V go into the cache
        vc[:, :, -S:] = v.reshape(batch, S, HKV, D).transpose(1, 2)
        o = F.scaled_dot_product_attention(q.reshape(batch, S, HQ, D).transpose(1, 2), kc, vc, enable_gqa=True)
        x = o.transpose(1, 2).reshape(rows, HQ * D) @ w["o"].T
        res = x + res
        h = F.rms_norm(res, (H,), w["norm"], 1e-6)
        gate, up = (h @ w["gu"].T).chunk(2, -1)
        return (F.silu(gate) * up) @ w["down"].T, res

    def run(n_layers):
        t0 = time.perf_counter()
        h, res = x, torch.zeros_like(x)
        for _ in range(n_layers):
            h, res = layer(h, res)
        t_layers = time.perf_counter() - t0
        t0 = time.perf_counter()
        logits = F.rms_norm(h + res, (H,), w["norm"], 1e-6) @ head.T
        p = torch.softmax(logits, -1)
        x0 = logits.argmax(-1)
        conf = p.gather(-1, x0[:, None])
        t_head = time.perf_counter() - t0
        return t_layers, t_head, float(conf.sum())

    run(1)                                                                    # warm-up
    t_layers, t_head, _ = run(layers)
    t_pass = t_layers / layers * 28 + t_head
    return dict(seconds_per_pass_28_layers=round(t_pass, 3), tokens_per_s=round(batch * S / 9 / t_pass, 1), cores=torch.get_num_threads(),
                sample=f"{layers} of 28 decoder layers ({t_layers:.2f} s) extrapolated + vocabulary projection and softmax/argmax ({t_head:.2f} s), "
                       f"batch {batch} x {S} tokens, cached context {ctx} keys, fp32 torch CPU ops; 8 denoising + 1 caching pass per block")


def cpu_side_ops(host3, cfg4_tokens):
    """Bounded CPU timings of the two bandwidth ops, reported next to their GPU numbers."""
    import oracle
    out = {}
    N = 4096
    fused = host3["fused"][:N]
    k = fused[:, HQ * D:(HQ + HKV) * D].reshape(N, HKV * D)
    v = fused[:, (HQ + HKV) * D:].reshape(N, HKV * D).contiguous()
    kc = torch.zeros(N + 512, HKV * D, dtype=torch.bfloat16)
    vc = torch.zeros_like(kc)
    idx = torch.randperm(N + 512)[:N]
    t0 = time.perf_counter()
    for _ in range(5):
        kc.index_copy_(0, idx, k)
        vc.index_copy_(0, idx, v)
    t = (time.perf_counter() - t0) / 5
    out["store_kvcache"] = dict(value=round(N * 2 * 2 * HKV * D * 2 / t / 1e9, 3), unit="GB/s",
                                sample=f"index_copy_ of {N} rows, 5 runs")
    g = torch.Generator().manual_seed(0)
    rows = (torch.randn(64, VOCAB, generator=g) * 3).bfloat16()
    t0 = time.perf_counter()
    x0, p = oracle.confidence_argmax(rows.float().numpy()[None])
    t = time.perf_counter() - t0
    out["unmask"] = dict(value=round(rows.numel() * 2 / t / 1e9, 3), unit="GB/s", sample="oracle softmax+argmax on 64 rows")
    return out


# ----------------------------------------------------------------------------- main
def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--skip-cpu", action="store_true", help="leave out the CPU baseline leg (profiling runs)")
    ap.add_argument("--no-full-logits-leg", action="store_true",
                    help="decode leg: skip the second generation that projects all 32 positions of every block")
    ap.add_argument("--only", default="", help="comma list of legs to run: calib,step,store,paged,unmask,gumbel,filter,lmhead,decode (default all; gumbel and filter run inside unmask), plus power (only when named: socket power and clock under the attention kernel and the library GEMM) and f32 (only when named: the attention calls on fp32 tensors)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (no collectives, no sharding); run with --gpus 1")
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    import mdx
    if not mdx.library_path().exists():
        sys.exit("bench.py: libmdx.so is missing; build it first (python mineru-diffusion_amd/build.py)")
    only = set(filter(None, args.only.split(",")))
    want = lambda leg: not only or leg in only      # noqa: E731
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    K, W = args.steps, args.warmup
    result_ops = {}
    calibration = None

    # A plain 1 GiB device copy: the yardstick against which FETCH_SIZE / WRITE_SIZE counter
    # readings of the kernels below are scaled when this command runs under rocprofv3 --pmc.
    if want("calib"):
        src = torch.ones(1 << 28, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        # the same copy as the yardstick of the HBM-bound legs: what the runtime's own copy kernel moves
        copy_ms, _ = time_kernel(lambda i: dst.copy_(src), 2, 5)
        del src, dst
        torch.cuda.empty_cache()
        # What the matrix pipe sustains on this box: the clock is power-limited and operand bit
        # toggling sets the power, so the library GEMM is timed on N(0,1) data and on zeros.
        calibration = {"device_copy_1GiB": dict(gbs=round(2 * (1 << 30) / copy_ms / 1e6, 1), ms=round(copy_ms, 4),
                                                note="bytes read + bytes written over the copy kernel's time")}
        for name, fill in (("gemm_bf16_8192_random", None), ("gemm_bf16_8192_zeros", 0.0)):
            a_ = torch.randn(8192, 8192, device=dev).bfloat16() if fill is None else torch.zeros(8192, 8192, device=dev, dtype=torch.bfloat16)
            b_ = a_.clone()
            # 60 untimed launches first: the GEMM is the first matrix work after an idle stretch, and the clock
            # needs some tens of milliseconds under load to settle (timed cold, the random-data figure reads a fifth low)
            ms_, _ = time_kernel(lambda i: torch.matmul(a_, b_), 60, 10, graph=True)
            calibration[name] = dict(tflops=round(2 * 8192 ** 3 / ms_ / 1e9, 1), ms=round(ms_, 3))
            del a_, b_
        torch.cuda.empty_cache()

    # ---------------- config 3: the step (store + staircase attention) -----------------------------
    log("[bench] building config 3 inputs")
    host3, g3 = make_cfg3(dev)
    work3 = cfg3_work(host3["lens"])
    max_len = max(host3["lens"])
    attn = mdx.Attention(HQ, D, 1 / math.sqrt(D), HKV)
    attn.k_cache, attn.v_cache = g3["k_cache"], g3["v_cache"]
    mdx.set_context(True, g3["cu"], g3["cu"], max_len, max_len, g3["slots"], None, None, block_size=S)

    o3 = torch.empty_like(g3["q"])

    def attn_only(_, zeros=None):
        q, k, v = zeros if zeros is not None else (g3["q"], g3["k"], g3["v"])
        rc = mdx.lib().mdx_staircase_attn_varlen(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), o3.data_ptr(), q.stride(0), q.stride(1), k.stride(0), k.stride(1),
            v.stride(0), v.stride(1), o3.stride(0), o3.stride(1), g3["cu"].data_ptr(), g3["cu"].data_ptr(), len(host3["lens"]),
            max_len, q.shape[0], HQ, HKV, D, S, 1 / math.sqrt(D), 0, raw_stream())
        assert rc == 0

    ms_step = attn_ms = float("nan")
    if want("step"):
        log("[bench] timing the step")
        # The inputs were built on the host while the GPU sat idle: the first 20 to 30 steps after that
        # run about 10 % slower (clock ramp, first use of the allocator's blocks).  Thirty untimed
        # steps come before the W warm-up steps so that a small W does not time that ramp.
        for _ in range(30 + W):
            attn(g3["q"], g3["k"], g3["v"])
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(K):
            attn(g3["q"], g3["k"], g3["v"])
        torch.cuda.synchronize()
        ms_step = (time.perf_counter() - t0) * 1e3 / K
        attn_ms, attn_min = time_kernel(attn_only, 2, K, graph=True)
        result_ops["staircase_attn"] = op_entry(attn_ms, attn_min, "mfma", work3["flops"], 1e9, PEAK_MFMA_TFLOPS, "TFLOP/s")
        if calibration is not None:
            # the same launch on all-zero q/k/v (same strides): less bit toggling, higher clock
            zf = torch.zeros(g3["q"].shape[0], (HQ + 2 * HKV) * D, dtype=torch.bfloat16, device=dev)
            z = (torch.zeros_like(g3["q"]), torch.zeros_like(g3["k"]), zf[:, (HQ + HKV) * D:].view(-1, HKV, D))
            z_ms, _ = time_kernel(lambda i: attn_only(i, z), 2, K, graph=True)
            calibration["staircase_attn_zero_inputs"] = dict(tflops=round(work3["flops"] / z_ms / 1e9, 1), ms=round(z_ms, 4))
            del zf
            del z
    power = None
    if "power" in only:
        # Socket power and shader clock while the attention kernel (and, beside it, the library GEMM) runs back to
        # back for a few seconds each, on N(0,1) data and on zeros: the evidence for "the clock is power-limited and
        # operand bit toggling sets the power".  Off by default (it adds 15 s); profiles/ keeps a summary of one run.
        ps = PowerSampler()
        if not ps.available():
            power = {"error": "no readable hwmon power file under /sys/class/drm/card*/device"}
        else:
            power = {"power_cap_w": ps.cap_w, "source": f"{ps.power_file} and {ps.sclk_file}, sampled every 5 ms on a host thread; "
                     "figures are over the last two thirds of a 3 s loop of HIP-graph replays (20 launches each)"}
            time.sleep(1.0)
            idle_w, idle_mhz = ps._read()
            power["idle"] = dict(power_w=idle_w, sclk_mhz=idle_mhz)
            zf = torch.zeros(g3["q"].shape[0], (HQ + 2 * HKV) * D, dtype=torch.bfloat16, device=dev)
            z = (torch.zeros_like(g3["q"]), torch.zeros_like(g3["k"]), zf[:, (HQ + HKV) * D:].view(-1, HKV, D))
            a_r = torch.randn(8192, 8192, device=dev).bfloat16()
            a_z = torch.zeros(8192, 8192, device=dev, dtype=torch.bfloat16)
            gemm_flops = 2 * 8192 ** 3
            # the matrix pipe alone: register-only loops of back-to-back MFMAs (two wavefronts per SIMD) on N(0,1) bf16
            # operands -- no kernel that feeds such data through these instructions can run faster under the power limit
            Lc = mdx.lib()
            pb, pit = 512, 1600
            p_ops = torch.randn(pb * 256 * 128, device=dev).bfloat16().view(torch.int16)
            p_out = torch.empty(pb * 256, device=dev)

            def mfma_loop(shape):
                rc = Lc.mdx_calib_mfma_loop(shape, p_ops.data_ptr(), p_out.data_ptr(), pb, pit, raw_stream())
                assert rc == 0
            # the fused vocabulary projection at 1024 rows (config 5's head), the library's GEMM structure without a softmax
            hw = (torch.randn(VOCAB, 2048, device=dev) * 0.02).bfloat16()
            hx = torch.randn(1024, 2048, device=dev).bfloat16()
            h0 = torch.empty(1024, dtype=torch.int64, device=dev)
            hp = torch.empty(1024, dtype=torch.float32, device=dev)
            hws_b = Lc.mdx_lm_head_confidence_workspace_bytes(1024, VOCAB)
            hws = torch.empty(hws_b, dtype=torch.uint8, device=dev)

            def head_fused():
                rc = Lc.mdx_lm_head_confidence(hx.data_ptr(), 2048, hw.data_ptr(), 2048, None, 1, None, h0.data_ptr(), hp.data_ptr(),
                                               1024, VOCAB, 2048, hws.data_ptr(), hws_b, raw_stream())
                assert rc == 0
            for name, fn, flops in (("staircase_attn_config3_random", lambda: attn_only(0), work3["flops"]),
                                    ("lm_head_confidence_1024_rows", head_fused, 2 * 1024 * VOCAB * 2048),
                                    ("staircase_attn_config3_zeros", lambda: attn_only(0, z), work3["flops"]),
                                    ("library_gemm_bf16_8192_random", lambda: torch.matmul(a_r, a_r), gemm_flops),
                                    ("library_gemm_bf16_8192_zeros", lambda: torch.matmul(a_z, a_z), gemm_flops),
                                    ("mfma_32x32x16_register_loop_random", lambda: mfma_loop(32), Lc.mdx_calib_mfma_loop_flops(32, pb, pit)),
                                    ("mfma_16x16x32_register_loop_random", lambda: mfma_loop(16), Lc.mdx_calib_mfma_loop_flops(16, pb, pit))):
                for _ in range(3):
                    fn()
                torch.cuda.synchronize()
                gr = torch.cuda.CUDAGraph()
                with torch.cuda.graph(gr):
                    for _ in range(20):
                        fn()

                def replay():
                    gr.replay()
                    torch.cuda.synchronize()
                stats, per_call = ps.run(replay, 3.0)
                stats["ms_per_launch"] = round(per_call * 1e3 / 20, 4)
                stats["tflops"] = round(flops / (per_call / 20) / 1e12, 1)
                power[name] = stats
                log(f"[bench] power leg {name}: {stats}")
                del gr
                time.sleep(0.5)
            del zf, z, a_r, a_z, p_ops, p_out, hw, hx, hws
            torch.cuda.empty_cache()
    if "f32" in only:
        # The two attention calls in fp32 arithmetic (fp32 tensors; the path of head widths outside the 16-bit kernels):
        # a compatibility path, timed only when named.  Prefill: four sequences of 2048 tokens and one of 8192, fp32,
        # d = 128; paged: 16 sequences of 2700 keys.  Roofline: the fp32 matrix instruction's published peak.
        f32 = {}
        for name, lens in (("prefill_4x2048", [2048] * 4), ("prefill_1x8192", [8192])):
            n_tok = sum(lens)
            qf = torch.randn(n_tok, HQ, D, device=dev)
            kf = torch.randn(n_tok, HKV, D, device=dev)
            vf = torch.randn(n_tok, HKV, D, device=dev)
            cu = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32, device=dev)
            ms, _ = time_kernel(lambda i: mdx.sparse_attn_varlen(qf, kf, vf, cu, cu, S, max_seqlen=max(lens)), 2, 5, graph=True)
            flops = cfg3_work(lens)["flops"]
            f32[name] = dict(ms=round(ms, 4), roofline=dict(bound="mfma", achieved=round(flops / ms / 1e9, 1), peak=157.3, unit="TFLOP/s",
                                                            frac=round(flops / ms / 1e9 / 157.3, 4), traffic=None))
            del qf, kf, vf
        bs_p, ctx_p = 16, 2700
        pages_p = (ctx_p + PAGE - 1) // PAGE
        qp = torch.randn(bs_p, S, HQ, D, device=dev)
        kcp = torch.randn(bs_p * pages_p, PAGE, HKV, D, device=dev)
        vcp = torch.randn(bs_p * pages_p, PAGE, HKV, D, device=dev)
        btp = torch.arange(bs_p * pages_p, dtype=torch.int32, device=dev).view(bs_p, pages_p)
        lens_p = torch.full((bs_p,), ctx_p, dtype=torch.int32, device=dev)
        ms, _ = time_kernel(lambda i: mdx.flash_attn_with_kvcache(qp, kcp, vcp, cache_seqlens=lens_p, block_table=btp, softmax_scale=D ** -0.5,
                                                                  causal=False), 2, 5, graph=True)
        flops = 4.0 * S * HQ * D * bs_p * ctx_p
        f32["paged_16x2700"] = dict(ms=round(ms, 4), roofline=dict(bound="mfma", achieved=round(flops / ms / 1e9, 1), peak=157.3, unit="TFLOP/s",
                                                                    frac=round(flops / ms / 1e9 / 157.3, 4), traffic=None))
        result_ops["attention_fp32_arithmetic"] = f32
        log(f"[bench] fp32-arithmetic attention: {f32}")
        del qp, kcp, vcp
        torch.cuda.empty_cache()
    if want("store"):
        # three rotating (source, cache) sets, about 900 MB touched per round trip, so the 256 MB
        # last-level cache cannot serve the next launch; the C ABI is called directly
        L = mdx.lib()
        N = g3["k"].shape[0]
        sets = [(g3["k"], g3["v"], g3["k_cache"], g3["v_cache"])]
        for _ in range(2):
            f2 = host3["fused"].to(dev)
            sets.append((f2[:, HQ * D:(HQ + HKV) * D].reshape(N, HKV, D).contiguous(), f2[:, (HQ + HKV) * D:].view(N, HKV, D),
                         torch.zeros_like(g3["k_cache"]), torch.zeros_like(g3["v_cache"])))
        num_slots = g3["k_cache"].shape[0] * PAGE

        def store_only(i):
            k, v, kc, vc = sets[i % 3]
            L.mdx_store_kvcache(k.data_ptr(), v.data_ptr(), k.stride(0), v.stride(0), kc.data_ptr(), vc.data_ptr(),
                                g3["slots"].data_ptr(), N, HKV * D, 2, num_slots, raw_stream())
        st_ms, st_min = time_kernel(store_only, W, K, graph=True)
        result_ops["store_kvcache"] = op_entry(st_ms, st_min, "hbm", work3["store_bytes"], 1e6, PEAK_HBM_GBS, "GB/s")
        del sets
        torch.cuda.empty_cache()
    mdx.reset_context()

    # ---------------- config 4: unmask step -----------------------------------------------------------
    cfg4_tokens = None
    if want("unmask"):
        log("[bench] building config 4 inputs")
        c4 = make_cfg4(dev)
        cfg4_tokens = c4["tokens"]
        L = mdx.lib()
        rows4 = 32 * S
        ws_bytes4 = L.mdx_confidence_argmax_workspace_bytes(rows4, VOCAB)
        ws4 = torch.empty(max(ws_bytes4, 16), dtype=torch.uint8, device=dev)
        # every step starts from the same masked blocks: one copy of them per call, made beforehand
        n_calls = W + K + 10
        dtoks = c4["tokens"].to(dev).unsqueeze(0).repeat(n_calls, 1, 1).contiguous()
        calls = count()
        x0_4 = torch.empty(32, S, dtype=torch.int64, device=dev)
        p_4 = torch.empty(32, S, dtype=torch.float32, device=dev)
        tr_4 = torch.empty(32, S, dtype=torch.uint8, device=dev)
        cnt_4 = torch.empty(32, dtype=torch.int32, device=dev)

        def unmask(i):
            lg = c4["logits"][i % len(c4["logits"])]
            dtok = dtoks[next(calls) % n_calls]
            rc = L.mdx_unmask_step(lg.data_ptr(), VOCAB, 0, None, None, 0, dtok.data_ptr(), MASK_ID, 0.9, 4,
                                   x0_4.data_ptr(), p_4.data_ptr(), tr_4.data_ptr(), cnt_4.data_ptr(), 32, S, VOCAB,
                                   ws4.data_ptr(), ws_bytes4, raw_stream())
            assert rc == 0
        fresh4 = dtoks.clone()

        def remask():                                   # every timed call starts from the masked blocks
            dtoks.copy_(fresh4)
        um_ms, um_min = time_kernel(unmask, W, K, graph=True, before_timed=remask)
        result_ops["unmask_step"] = op_entry(um_ms, um_min, "hbm", c4["bytes"], 1e6, PEAK_HBM_GBS, "GB/s")
        if want("gumbel"):
            # the reference's own sampling (sampler.py:15-18: Gumbel noise on every logit before the argmax), the noise
            # drawn inside the kernel: bound by the generator's integer multiplies and the two logarithms per logit
            def unmask_gumbel(i):
                lg = c4["logits"][i % len(c4["logits"])]
                dtok = dtoks[next(calls) % n_calls]
                rc = L.mdx_unmask_step_gumbel(lg.data_ptr(), VOCAB, 0, None, 2024, i, None, None, dtok.data_ptr(), MASK_ID, 0.9, 4,
                                              x0_4.data_ptr(), p_4.data_ptr(), tr_4.data_ptr(), cnt_4.data_ptr(), 32, S, VOCAB,
                                              ws4.data_ptr(), ws_bytes4, raw_stream())
                assert rc == 0
            gm_ms, gm_min = time_kernel(unmask_gumbel, 2, max(3, K // 4), graph=True, before_timed=remask)
            result_ops["unmask_step_gumbel"] = op_entry(gm_ms, gm_min, "hbm", c4["bytes"], 1e6, PEAK_HBM_GBS, "GB/s",
                                                        dict(note="Gumbel noise drawn in the kernel (Philox-4x32-10 per 4 logits): compute-bound, "
                                                                  "not a bandwidth figure; the same step with the noise made by torch ops and "
                                                                  "passed as a tensor takes about 1 ms"))
        if want("filter"):
            # the HF variant's optional top-k / top-p filter in front of the step (off by default there): a filtered
            # copy of the same logits, algorithmic bytes = one read + one write of them
            flt_out = torch.empty_like(c4["logits"][0])

            def logit_filter(i):
                lg = c4["logits"][i % len(c4["logits"])]
                rc = L.mdx_filter_logits(lg.data_ptr(), VOCAB, 0, None, 1, 50, 0.9, flt_out.data_ptr(), VOCAB, rows4, VOCAB, raw_stream())
                assert rc == 0
            fl_ms, fl_min = time_kernel(logit_filter, 2, max(3, K // 4), graph=True)
            # the sampled step on the filtered copy: the generator runs only where a kept logit could still win
            def unmask_gumbel_filtered(i):
                dtok = dtoks[next(calls) % n_calls]
                rc = L.mdx_unmask_step_gumbel(flt_out.data_ptr(), VOCAB, 0, None, 2024, i, None, None, dtok.data_ptr(), MASK_ID, 0.9, 4,
                                              x0_4.data_ptr(), p_4.data_ptr(), tr_4.data_ptr(), cnt_4.data_ptr(), 32, S, VOCAB,
                                              ws4.data_ptr(), ws_bytes4, raw_stream())
                assert rc == 0
            gf_ms, _ = time_kernel(unmask_gumbel_filtered, 2, max(3, K // 4), graph=True, before_timed=remask)
            result_ops["filter_logits"] = op_entry(fl_ms, fl_min, "hbm", 2 * c4["bytes"], 1e6, PEAK_HBM_GBS, "GB/s",
                                                   dict(top_k=50, top_p=0.9, sampled_step_on_the_filtered_logits_ms=round(gf_ms, 4),
                                                        note="off by default in the reference; with both filters on a row is read five times (four counting passes and the writing pass)"))
            del flt_out
        del c4
        torch.cuda.empty_cache()

    # (the 64 GiB page pool of config 2 is built after the other operator legs: buffers allocated from what the pool
    # leaves behind when it is freed have measured up to 10 % slower streams in the legs that followed)
    # ---------------- config 2: paged single-block attention ---------------------------------------
    if want("paged"):
        log("[bench] building config 2 inputs (64 GiB page pool, referenced pages only are filled)")
        c2 = make_cfg2(dev)

        L = mdx.lib()
        bs2, maxp = c2["tables"][0].shape
        ws_bytes = L.mdx_paged_block_attn_workspace_bytes(bs2, S, HQ, HKV, D, maxp, PAGE)
        ws2 = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
        o2 = torch.empty_like(c2["q"])
        kc2, vc2, q2 = c2["k_cache"], c2["v_cache"], c2["q"]

        def paged(i):
            bt = c2["tables"][i % len(c2["tables"])]
            rc = L.mdx_paged_block_attn(q2.data_ptr(), o2.data_ptr(), kc2.data_ptr(), vc2.data_ptr(),
                                        q2.stride(0), q2.stride(1), q2.stride(2), o2.stride(0), o2.stride(1), o2.stride(2),
                                        kc2.stride(0), kc2.stride(1), kc2.stride(2), bt.data_ptr(), bt.stride(0),
                                        c2["lens"].data_ptr(), bs2, S, HQ, HKV, D, maxp, PAGE, kc2.shape[0],
                                        1 / math.sqrt(D), 0, ws2.data_ptr(), ws_bytes, raw_stream())
            assert rc == 0
        pg_ms, pg_min = time_kernel(paged, W, K, graph=True)
        result_ops["paged_block_attn"] = op_entry(
            pg_ms, pg_min, "hbm", c2["work"]["bytes"], 1e6, PEAK_HBM_GBS, "GB/s",
            dict(tflops=round(c2["work"]["flops"] / pg_ms / 1e9, 2),
                 mfma_frac=round(c2["work"]["flops"] / pg_ms / 1e9 / PEAK_MFMA_TFLOPS, 4), sum_ctx=c2["work"]["sum_ctx"]))
        del c2
        torch.cuda.empty_cache()

    # ---------------- vocabulary projection fused with the confidence reduction ------------------------------
    if want("lmhead"):
        # config 5's head: [rows, 2048] x [151936, 2048]^T at the row counts the decode loop projects (eighths of the
        # 1024 positions of a pass); fused (no logits in memory) against the library GEMM + the vocabulary pass
        L = mdx.lib()
        hid = 2048
        gh = torch.Generator(device=dev).manual_seed(6)
        w_head = (torch.randn(VOCAB, hid, generator=gh, device=dev) * 0.02).bfloat16()
        head = {}
        for rows_h in (1024, 512, 256):
            xh = torch.randn(rows_h, hid, generator=gh, device=dev).bfloat16()
            x0h = torch.empty(rows_h, dtype=torch.int64, device=dev)
            ph = torch.empty(rows_h, dtype=torch.float32, device=dev)
            wsb = L.mdx_lm_head_confidence_workspace_bytes(rows_h, VOCAB)
            wsh = torch.empty(wsb, dtype=torch.uint8, device=dev)
            lg = torch.empty(rows_h, VOCAB, dtype=torch.bfloat16, device=dev)
            wsb2 = L.mdx_confidence_argmax_workspace_bytes(rows_h, VOCAB)
            ws2h = torch.empty(max(wsb2, 16), dtype=torch.uint8, device=dev)
            x0t = torch.empty_like(x0h)
            pt = torch.empty_like(ph)

            def fused(i):
                rc = L.mdx_lm_head_confidence(xh.data_ptr(), xh.stride(0), w_head.data_ptr(), w_head.stride(0), None, 1, None,
                                              x0h.data_ptr(), ph.data_ptr(), rows_h, VOCAB, hid, wsh.data_ptr(), wsb, raw_stream())
                assert rc == 0

            def two_step(i):
                torch.matmul(xh, w_head.t(), out=lg)
                rc = L.mdx_confidence_argmax(lg.data_ptr(), VOCAB, 0, None, 1, None, 0, x0t.data_ptr(), pt.data_ptr(), rows_h, VOCAB,
                                             ws2h.data_ptr(), wsb2, raw_stream())
                assert rc == 0
            f_ms, f_min = time_kernel(fused, 20 + W, max(5, K // 2), graph=True)
            t_ms, _ = time_kernel(two_step, 20 + W, max(5, K // 2), graph=True)
            flops_h = 2 * rows_h * VOCAB * hid
            e = op_entry(f_ms, f_min, "mfma", flops_h, 1e9, PEAK_MFMA_TFLOPS, "TFLOP/s",
                         dict(rows=rows_h, library_gemm_plus_confidence_pass_ms=round(t_ms, 4),
                              same_tokens=round(float((x0h == x0t).float().mean()), 4)))
            head[f"rows_{rows_h}"] = e
            if rows_h == 1024:
                result_ops["lm_head_confidence"] = e
        result_ops["lm_head_confidence"]["other_row_counts"] = {k: v for k, v in head.items() if k != "rows_1024"}
        del w_head
        torch.cuda.empty_cache()

    # ---------------- config 5: end-to-end block-diffusion decode ---------------------------------------
    decode = None
    if want("decode"):
        log("[bench] config 5: end-to-end block-diffusion decode (32 x 2048 tokens)")
        del g3, attn
        torch.cuda.empty_cache()
        decode = run_cfg5(dev)
        if not args.no_full_logits_leg:
            full = run_cfg5(dev, masked_rows_only=False)
            decode["with_full_logits"] = {k: full[k] for k in ("tokens_per_s", "seconds", "ms_per_decode_pass", "vocabulary_projection")}
            noisy = run_cfg5(dev, gumbel_seed=5)
            decode["with_gumbel_sampling"] = {k: noisy[k] for k in ("tokens_per_s", "seconds", "ms_per_decode_pass")}
            two = run_cfg5(dev, fused_head=False)
            decode["with_library_projection_and_separate_confidence_pass"] = {k: two[k] for k in ("tokens_per_s", "seconds", "ms_per_decode_pass")}

    # ---------------- CPU baseline (bounded) -------------------------------------------------------------
    cpu = None
    if not args.skip_cpu:
        log("[bench] CPU baseline (oracle on host cores)")
        cpu = cpu_baseline(host3)
        try:
            cpu["other_ops"] = cpu_side_ops(host3, cfg4_tokens)
            if decode is not None:
                cpu["other_ops"]["decode"] = cpu_decode_pass()
        except Exception as e:  # the side numbers are informative only
            cpu["other_ops"] = {"error": str(e)}

    # HBM bytes per launch: NOT measured by this run (counters need the profiler); copied from the
    # summary of the rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this same command under profiles/
    tfile = ROOT / "profiles" / "hbm_traffic_per_call.txt"
    if tfile.exists():
        measured = json.loads("".join(l for l in tfile.read_text().splitlines(True) if not l.startswith("#")))
        for name, op in result_ops.items():
            if name in measured:
                op["roofline"]["traffic"] = measured[name]["bytes"]
                op["roofline"]["traffic_source"] = "profiles/hbm_traffic_per_call.txt"
    value = work3["flops"] / ms_step / 1e9 if ms_step == ms_step else None
    line = {
        "metric": "staircase-attn TFLOP/s (%MFMA peak) + block-diffusion decode tokens/s, 1 GPU",
        "value": None if value is None else round(value, 2), "unit": "TFLOP/s",
        "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": None if value is None else round(ms_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "config 3: one prefill pass of the attention layer (store_kvcache + staircase "
                               "block-prefill attention) over 8 packed sequences; mdx.Attention launches the store on a second stream beside "
                               "the attention kernel and joins both before it returns",
                   "seq_lens": host3["lens"], "total_tokens": work3["tokens"], "block": S, "num_q_heads": HQ,
                   "num_kv_heads": HKV, "head_dim": D, "page_size": PAGE, "visible_pairs": work3["pairs"],
                   "algorithmic_gflop": round(work3["flops"] / 1e9, 2)},
        "roofline": result_ops.get("staircase_attn", {}).get("roofline"),
        "cpu_baseline": cpu,
        "ops": result_ops,
        "calibration": calibration,
        "decode": decode,
        "power": power,
        "host": {"cpu_count": os.cpu_count(), "torch_threads": torch.get_num_threads()},
    }
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
