"""GPU parity of the two drop-in layer classes, driven the way the engine drives them:

  mdx.Sampler.forward / .prepare   engines/nano_dvlm/nanovllm/layers/sampler.py:24-61, called at
                                   engine/model_runner.py:217 with temperatures [bs, 1] and the scheduled Sequences
  mdx.Attention.forward            engines/nano_dvlm/nanovllm/layers/sdar_attention.py:34-57, inputs through the
                                   global Context in both of its modes (prefill / decode)

Every field the reference mutates and every return value is compared with the oracle."""
import math
from types import SimpleNamespace

import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu
MASK_ID, V, S = 151669, 151936, 32


def _fake_seqs(tokens: torch.Tensor, threshold: float, steps):
    """Objects with exactly the attributes Sampler.forward touches (sequence.py:20-48)."""
    sp = SimpleNamespace(denoising_strategy="low_confidence_dynamic", dynamic_threshold=threshold)
    return [SimpleNamespace(current_denoising_block=tokens[i].clone(), current_step_map=torch.zeros(S, dtype=torch.int32),
                            current_denoise_step=int(steps[i]), sampling_params=sp, mask_token_id=MASK_ID)
            for i in range(tokens.shape[0])]


def _engine_rule(conf: np.ndarray, masked: np.ndarray, threshold: float) -> np.ndarray:
    """sampler.py:39-50 restated on its own (not through oracle.select_transfer): rows without a masked
    position are skipped; all positions above the threshold if there is one, else the single best."""
    out = np.zeros(conf.shape, dtype=bool)
    for j in range(conf.shape[0]):
        if not masked[j].any():
            continue
        c = np.where(masked[j], conf[j], -np.inf)
        hi = c > threshold
        if hi.sum() >= 1:
            out[j] = hi
        else:
            out[j, int(np.argmax(c))] = True
    return out


def _sampler_case(seed=21, bs=6):
    logits, tokens, temps = _sampler_case6(seed)
    return logits[:bs].contiguous(), tokens[:bs].contiguous(), temps[:bs].contiguous()


def _sampler_case6(seed):
    bs = 6
    g = torch.Generator().manual_seed(seed)
    logits = (torch.randn(bs, S, V, generator=g) * 3).bfloat16()
    logits[0, 3, 777] += 40.0                       # two positions far above the threshold in sequence 0
    logits[0, 9, 12345] += 40.0
    logits[4, 30, 5] += 40.0                        # above the threshold but already committed (not masked)
    tokens = torch.randint(0, 1000, (bs, S), generator=g, dtype=torch.int64)
    for b, n in enumerate((32, 20, 5, 0, 16, 1)):   # sequence 3 has nothing left to unmask
        tokens[b, torch.randperm(S, generator=g)[:n]] = MASK_ID
    tokens[0, 3] = tokens[0, 9] = MASK_ID
    tokens[4, 30] = 17
    temps = torch.tensor([1.0, 0.7, 1.0, 1.3, 1.0, 2.0]).unsqueeze(1)      # [bs, 1] as prepare_sample builds it
    return logits, tokens, temps


@pytest.mark.parametrize("k", [1, 4])
def test_sampler_forward_mutates_sequences_like_the_reference(dev, k):
    import mdx
    logits, tokens, temps = _sampler_case()
    bs = tokens.shape[0]
    steps = [0, 3, 7, 2, 1, 5]
    seqs = _fake_seqs(tokens, 0.9, steps)
    n = mdx.Sampler(k=k).forward(logits.to(dev), temps.to(dev), seqs)

    ex0, ep, etr, etok = oracle.unmask_step(logits.to(torch.float64).numpy(), tokens.numpy(), MASK_ID, 0.9, k,
                                            temperatures=temps.numpy().reshape(-1))
    if k == 1:       # the oracle's rule with k = 1 must be the engine's loop
        assert np.array_equal(etr, _engine_rule(ep.astype(np.float32), tokens.numpy() == MASK_ID, 0.9))
    assert isinstance(n, int) and n == int(etr.sum())
    assert etr[0, 3] and etr[0, 9] and not etr[4, 30] and not etr[3].any()
    for i, s in enumerate(seqs):
        assert s.current_denoising_block.device.type == "cpu" and s.current_denoising_block.dtype == torch.int64
        assert np.array_equal(s.current_denoising_block.numpy(), etok[i]), f"tokens of sequence {i}"
        want_map = np.where(etr[i], steps[i], 0).astype(np.int32)
        assert np.array_equal(s.current_step_map.numpy(), want_map), f"step map of sequence {i}"
        assert s.current_denoise_step == steps[i] + 1


def test_sampler_forward_over_several_steps_unmasks_the_block(dev):
    """The same Sequences through consecutive calls (as the scheduler re-schedules them): with k = 4 and
    confidences below the threshold the block of 32 empties in exactly 8 steps, and the step map records
    the step of every commit."""
    import mdx
    logits, tokens, temps = _sampler_case(seed=5, bs=2)
    tokens[:] = MASK_ID
    seqs = _fake_seqs(tokens, 0.9, [0, 0])
    sampler, d_logits, d_temps = mdx.Sampler(k=4), logits.to(dev), temps[:2].to(dev)
    cur = tokens.numpy().copy()
    total = 0
    for step in range(8):
        n = sampler(d_logits, d_temps, seqs)
        _, _, etr, cur = oracle.unmask_step(logits.to(torch.float64).numpy(), cur, MASK_ID, 0.9, 4,
                                            temperatures=temps[:2].numpy().reshape(-1))
        assert n == int(etr.sum())
        total += n
        for i, s in enumerate(seqs):
            assert np.array_equal(s.current_denoising_block.numpy(), cur[i])
            assert (s.current_step_map.numpy()[etr[i]] == step).all()
    assert total == 2 * S and not (cur == MASK_ID).any()        # 4 per step x 8 steps


def test_sampler_with_a_seed_samples_like_the_reference_prepare(dev):
    """Sampler(seed=) draws the Gumbel noise of sampler.py:15-16 inside the kernel: the Sequences change exactly as the
    oracle's step on the oracle's restatement of that noise says, every call takes the next offset, and the same
    seed replays the same calls."""
    import mdx
    logits, tokens, temps = _sampler_case(seed=9)
    bs, S, V = logits.shape
    l64 = logits.to(torch.float64).numpy()
    for attempt in range(2):
        sampler = mdx.Sampler(k=1, seed=4242)
        cur = tokens.numpy().copy()
        seqs = _fake_seqs(tokens.clone(), 0.9, [0] * bs)
        for call in range(3):
            noise = oracle.gumbel_noise(bs * S, V, 4242, offset=call).reshape(bs, S, V)
            ex0, ep, etr, etok = oracle.unmask_step(l64, cur, MASK_ID, 0.9, 1, temperatures=temps.numpy().reshape(-1), noise=noise)
            n = sampler.forward(logits.to(dev), temps.to(dev), seqs)
            assert n == int(etr.sum())
            for i, s in enumerate(seqs):
                assert np.array_equal(s.current_denoising_block.numpy(), etok[i]), f"call {call}, sequence {i}"
            cur = etok
        assert sampler.calls == 3
    x0_plain, _ = mdx.Sampler().prepare(logits.to(dev), temps.to(dev))
    x0_noisy, _ = mdx.Sampler(seed=4242).prepare(logits.to(dev), temps.to(dev))
    assert not torch.equal(x0_plain, x0_noisy)


def test_sampler_prepare_is_the_confidence_pass(dev):
    import mdx
    logits, _, temps = _sampler_case(seed=8, bs=3)
    x0, p = mdx.Sampler().prepare(logits.to(dev), temps[:3].to(dev))
    ex0, ep = oracle.confidence_argmax(logits.to(torch.float64).numpy(), temps[:3].numpy().reshape(-1))
    assert x0.dtype == torch.int64 and p.dtype == torch.float32 and x0.shape == (3, S)
    assert np.array_equal(x0.cpu().numpy(), ex0)
    np.testing.assert_allclose(p.cpu().numpy(), ep, rtol=2e-5)


def test_sampler_rejects_other_strategies(dev):
    import mdx
    logits, tokens, temps = _sampler_case(bs=1)
    seqs = _fake_seqs(tokens, 0.9, [0])
    seqs[0].sampling_params.denoising_strategy = "random"
    with pytest.raises(NotImplementedError):
        mdx.Sampler()(logits.to(dev), temps[:1].to(dev), seqs)


# ----------------------------------------------------------------------------- Attention.forward
HQ, HKV, D, PAGE = 16, 8, 128, 256


def _i16(t):
    return t.contiguous().view(torch.int16).cpu().numpy()


def test_attention_forward_prefill_context(dev):
    """Prefill mode (sdar_attention.py:37-47): store the prompt rows (the trailing mask block has slot -1),
    staircase attention over the packed sequences, output flattened to [N, Hq * d].  V arrives as the
    strided view of the fused QKV projection (sdar.py:73-78)."""
    import mdx
    g = torch.Generator().manual_seed(31)
    lens = [700 + S, 129 + S, 33 + S]
    N = sum(lens)
    fused = torch.randn(N, (HQ + 2 * HKV) * D, generator=g).bfloat16()
    dfused = fused.to(dev)
    q = dfused[:, :HQ * D].view(N, HQ, D)
    k = dfused[:, HQ * D:(HQ + HKV) * D].reshape(N, HKV, D).contiguous()
    v = dfused[:, (HQ + HKV) * D:].view(N, HKV, D)
    cu = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32)
    tables = [[5, 2, 7], [0], [3]]
    slots = []
    for b, L in enumerate(lens):
        slots += oracle.get_slots(tables[b], 0, L - S) + [-1] * S
    slots = torch.tensor(slots, dtype=torch.int32)
    attn = mdx.Attention(HQ, D, 1 / math.sqrt(D), HKV)
    attn.k_cache = torch.zeros(8, PAGE, HKV, D, dtype=torch.bfloat16, device=dev)
    attn.v_cache = torch.zeros_like(attn.k_cache)
    mdx.set_context(True, cu.to(dev), cu.to(dev), max(lens), max(lens), slots.to(dev), None, None, block_size=S)
    try:
        o = attn(q, k, v)
    finally:
        mdx.reset_context()
    assert o.shape == (N, HQ * D) and o.dtype == torch.bfloat16
    hq, hk, hv = (fused[:, :HQ * D].view(N, HQ, D), fused[:, HQ * D:(HQ + HKV) * D].view(N, HKV, D),
                  fused[:, (HQ + HKV) * D:].view(N, HKV, D))
    ref = oracle.staircase_attn_varlen(hq, hk, hv, cu, S)
    assert (o.view(N, HQ, D).float().cpu() - ref).abs().max().item() < 2e-2
    ek = np.zeros((8, PAGE, HKV, D), dtype=np.int16)
    ev = np.zeros_like(ek)
    oracle.store_kvcache(_i16(hk), _i16(hv), ek, ev, slots.numpy())
    assert np.array_equal(_i16(attn.k_cache), ek) and np.array_equal(_i16(attn.v_cache), ev)


def test_attention_forward_decode_context(dev):
    """Decode mode (sdar_attention.py:37-38,48-56): the 4-D block K/V is stored into its pages first,
    then the block attends, non-causally, to prefix + block through the page table; output [bs, S, Hq * d].
    A graph-padding row (slots -1, context 0, model_runner.py:205-208) stores nothing and yields zeros."""
    import mdx
    g = torch.Generator().manual_seed(32)
    prefix = [1000, 300, 0]
    bs = len(prefix)
    tables = [[4, 9, 1, 6, 2], [8, 3], [7]]
    n_pages = 12
    kc = torch.randn(n_pages, PAGE, HKV, D, generator=g).bfloat16()
    vc = torch.randn(n_pages, PAGE, HKV, D, generator=g).bfloat16()
    q = torch.randn(bs, S, HQ, D, generator=g).bfloat16()
    k = torch.randn(bs, S, HKV, D, generator=g).bfloat16()
    v = torch.randn(bs, S, HKV, D, generator=g).bfloat16()
    slots = torch.tensor([oracle.get_slots(tables[b], prefix[b], prefix[b] + S) for b in range(bs)], dtype=torch.int32)
    ctx = torch.tensor([p + S for p in prefix], dtype=torch.int32)
    slots[2] = -1
    ctx[2] = 0
    bt = torch.full((bs, 5), -1, dtype=torch.int32)
    for b, t in enumerate(tables):
        bt[b, :len(t)] = torch.tensor(t, dtype=torch.int32)
    attn = mdx.Attention(HQ, D, 1 / math.sqrt(D), HKV)
    attn.k_cache, attn.v_cache = kc.to(dev), vc.to(dev)
    mdx.set_context(False, slot_mapping=slots.to(dev), context_lens=ctx.to(dev), block_tables=bt.to(dev), block_size=S)
    try:
        o = attn(q.to(dev), k.to(dev), v.to(dev))
    finally:
        mdx.reset_context()
    assert o.shape == (bs, S, HQ * D)
    ek, ev = _i16(kc).copy(), _i16(vc).copy()
    oracle.store_kvcache(_i16(k).reshape(bs * S, HKV, D), _i16(v).reshape(bs * S, HKV, D), ek, ev, slots.numpy().reshape(-1))
    assert np.array_equal(_i16(attn.k_cache), ek) and np.array_equal(_i16(attn.v_cache), ev)
    ref = oracle.paged_block_attn(q, torch.from_numpy(ek).view(torch.bfloat16), torch.from_numpy(ev).view(torch.bfloat16),
                                  bt, ctx, 1 / math.sqrt(D))
    got = o.view(bs, S, HQ, D).float().cpu()
    assert (got - ref).abs().max().item() < 2e-2
    assert got[2].abs().max().item() == 0
