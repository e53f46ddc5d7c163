"""GPU: the mini engine (paged KV cache, block-at-a-time decode through libmdx) against a dense
fp32 recomputation of the same decoder with an explicit staircase mask and no cache."""
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu


def _tiny(dev):
    from mdx.engine import Decoder, DecoderConfig
    cfg = DecoderConfig(num_layers=2, hidden_size=256, num_heads=4, num_kv_heads=2, head_dim=128,
                        intermediate_size=512, vocab_size=1000, max_position=1024, mask_token_id=999)
    return cfg, Decoder(cfg, dev, seed=3)


def test_engine_logits_and_cache_match_dense_recompute(dev):
    from mdx.engine import PAGE, BlockDiffusionEngine, SamplingParams
    cfg, model = _tiny(dev)
    weights = dict(model.named_parameters())
    seen = []

    def on_logits(is_prefill, seqs, logits):
        for i, s in enumerate(seqs):
            seen.append((s.seq_id, list(s.token_ids), s.current_denoising_block.clone(), logits[i].float().cpu()))

    eng = BlockDiffusionEngine(model, num_pages=12, shuffle_pages_seed=5, on_logits=on_logits)
    g = torch.Generator().manual_seed(0)
    sp = SamplingParams(max_new_tokens=64, ignore_eos=True, transfer_count=8)
    prefix = torch.randn(20, cfg.hidden_size, generator=g) * 0.02
    a = eng.add_request(torch.randint(0, 900, (250,), generator=g).tolist(), sp, prefix_embeds=prefix)
    b = eng.add_request(torch.randint(0, 900, (37,), generator=g).tolist(), sp)
    tables = {}
    orig_dealloc = eng.block_manager.deallocate
    eng.block_manager.deallocate = lambda s: (tables.__setitem__(s.seq_id, list(s.block_table)), orig_dealloc(s))
    eng.generate()
    assert a.num_completion_tokens == 64 and b.num_completion_tokens == 64
    assert len(seen) == 2 * oracle.expected_passes(32, 8, 2)

    emb_w = weights["embed_tokens"].detach().float().cpu()

    def embeds_of(seq, tokens, block):
        e = emb_w[torch.tensor(tokens + block.tolist())]
        if seq is a:
            e[:20] = prefix.to(torch.bfloat16).float()
        return e

    # every pass: the block's logits from the cached engine == dense recompute on the same tokens
    worst = 0.0
    for sid, tokens, block, logits in seen[::3] + seen[-2:]:
        seq = a if sid == a.seq_id else b
        ref, _, _ = oracle.dense_forward(weights, cfg, embeds_of(seq, tokens, block))
        scale = ref.abs().max().item()
        worst = max(worst, (logits - ref).abs().max().item() / scale)
    assert worst < 0.06, f"relative logits error {worst}"

    # the pass that runs on a fully committed block stores that block's K/V: cache == K/V of final tokens
    for seq in (a, b):
        final = seq.token_ids
        e = emb_w[torch.tensor(final)]
        if seq is a:
            e[:20] = prefix.to(torch.bfloat16).float()
        # dense K/V over the committed tokens (a trailing mask block would not change earlier rows)
        _, ks, vs = oracle.dense_forward(weights, cfg, torch.cat([e, emb_w[torch.full((32,), cfg.mask_token_id)]]))
        table = tables[seq.seq_id]
        for layer in range(cfg.num_layers):
            kc = oracle.paged_gather(eng.kv_cache[0, layer].float().cpu(), table, len(final))
            vc = oracle.paged_gather(eng.kv_cache[1, layer].float().cpu(), table, len(final))
            assert (kc - ks[layer][:len(final)]).abs().max().item() < 0.08
            assert (vc - vs[layer][:len(final)]).abs().max().item() < 0.02 * max(1.0, vs[layer].abs().max().item())


def test_engine_is_deterministic_and_independent_of_page_placement(dev):
    from mdx.engine import BlockDiffusionEngine, SamplingParams
    cfg, model = _tiny(dev)
    outs = []
    for seed in (None, 11):
        eng = BlockDiffusionEngine(model, num_pages=10, shuffle_pages_seed=seed)
        sp = SamplingParams(max_new_tokens=32, ignore_eos=True, transfer_count=4)
        s = eng.add_request(list(range(5, 300)), sp)
        eng.generate()
        outs.append(s.completion_token_ids)
    assert outs[0] == outs[1]


def test_device_loop_forward_replays_match_eager(dev):
    """The captured forward of the device loop (pass inputs computed on the device from lengths and page tables,
    then the decoder), replayed on different blocks, lengths and page tables with eager work and
    synchronisations in between: its pass inputs equal the host's prepare_decode and its hidden states equal
    the eager forward on the same inputs, bit for bit."""
    from mdx.context import reset_context, set_context
    from mdx.engine import BlockDiffusionEngine, SamplingParams
    cfg, model = _tiny(dev)
    eng = BlockDiffusionEngine(model, num_pages=24, shuffle_pages_seed=7, decode_graphs=True, max_model_len=1024)
    sp = SamplingParams(max_new_tokens=96, ignore_eos=True, transfer_count=8)
    g = torch.Generator().manual_seed(1)
    seqs = [eng.add_request(torch.randint(0, 900, (n,), generator=g).tolist(), sp) for n in (300, 41, 129)]
    eng.step()                                             # prefill: fills the caches, allocates pages
    for rep in range(6):
        for s in seqs:                                     # a different partly unmasked block every time
            blk = torch.full((32,), cfg.mask_token_id, dtype=torch.int64)
            blk[: 4 * rep] = torch.randint(0, 900, (4 * rep,), generator=g)
            s.current_denoising_block = blk
            eng.block_manager.may_append(s)
        gr = eng._load_lanes(seqs)                         # three sequences run in the lanes captured for four
        assert gr["bs"] == 4
        gr["fwd"].replay()
        hidden = gr["hidden"].clone()
        torch.cuda.synchronize()
        ids, pos = eng.prepare_decode(seqs)                # the host's version of the same pass inputs
        from mdx.context import get_context
        ctx = get_context()
        assert torch.equal(gr["ids"][:3], ids) and torch.equal(gr["pos"][:3], pos)
        assert torch.equal(gr["slots"][:3], ctx.slot_mapping) and torch.equal(gr["ctx"][:3], ctx.context_lens)
        assert gr["ctx"][3].item() == 0 and (gr["slots"][3] == -1).all()        # the idle lane
        set_context(False, slot_mapping=gr["slots"], context_lens=gr["ctx"], block_tables=gr["bt"], block_size=32)
        ref = model(model.embed(gr["ids"].clone()), gr["pos"].clone())          # same launch geometry as the capture
        reset_context()
        torch.cuda.synchronize()
        assert torch.equal(hidden, ref), f"replay {rep}: max diff {(hidden.float() - ref.float()).abs().max().item()}"
        assert torch.isfinite(hidden[3].float()).all()                          # idle lane: finite
        eng._loaded = None
        if rep == 2:                                       # sequences grow between replays
            for s in seqs:
                s.current_denoising_block = torch.randint(0, 900, (32,), generator=g)
                s.append_block()
                eng.block_manager.may_append(s)


def test_device_loop_generates_like_the_host_driven_engine(dev):
    """The same requests through the host-driven engine and through the device loop, with and without the one-pass
    lag of the status reads and with the projection on all rows or on the masked rows: same number of passes, and
    the same tokens and step maps up to near-ties (the lanes' page tables have their full width, which moves the
    split points of the paged attention)."""
    from mdx.engine import BlockDiffusionEngine, SamplingParams
    cfg, model = _tiny(dev)
    outs = []
    for kw in (dict(decode_graphs=False), dict(decode_graphs=True, replay_ahead=False), dict(decode_graphs=True),
               dict(decode_graphs=True, masked_rows_only=False)):
        eng = BlockDiffusionEngine(model, num_pages=24, shuffle_pages_seed=9, max_model_len=1024, **kw)
        g = torch.Generator().manual_seed(12)
        seqs = [eng.add_request(torch.randint(0, 900, (n,), generator=g).tolist(),
                                SamplingParams(max_new_tokens=96, ignore_eos=True, transfer_count=4, temperature=t))
                for n, t in ((250, 1.0), (33, 0.8), (140, 1.2))]
        eng.generate()
        assert all(s.num_completion_tokens == 96 and len(s.step_map) == 96 for s in seqs)
        assert eng.stats["decode_passes"] == 3 * 9 - 1 and eng.stats["committed_tokens"] == 3 * 96
        assert len(eng.block_manager.free) == 24 and not eng.running
        outs.append([(s.completion_token_ids, list(s.step_map)) for s in seqs])
    for other in outs[1:]:
        for (ta, ma), (tb, mb) in zip(outs[0], other):
            assert sum(int(a == b) for a, b in zip(ta, tb)) >= 90
            assert sum(int(a == b) for a, b in zip(ma, mb)) >= 90
    assert outs[1] == outs[2]                               # the lag is pure scheduling


def test_engine_with_decode_graphs_generates_like_eager(dev):
    from mdx.engine import BlockDiffusionEngine, SamplingParams
    cfg, model = _tiny(dev)
    outs = []
    for graphs in (False, True):
        eng = BlockDiffusionEngine(model, num_pages=10, shuffle_pages_seed=3, decode_graphs=graphs, max_model_len=1024)
        sp = SamplingParams(max_new_tokens=64, ignore_eos=True, transfer_count=4)
        s = eng.add_request(list(range(5, 300)), sp)
        eng.generate()
        outs.append(s.completion_token_ids)
        assert len(outs[-1]) == 64
    # same kernels; only the split-KV geometry may differ (page table width), which can flip a near-tie
    same = sum(int(a == b) for a, b in zip(*outs))
    assert same >= 60, f"only {same}/64 tokens agree"


@pytest.mark.parametrize("temps", [(1.0, 1.0, 1.0), (1.0, 0.7, 1.3)])
def test_masked_rows_only_sampling_matches_full_logits(dev, temps):
    """Graph decode with the vocabulary projection and the unmask step restricted to the still
    masked positions vs the same engine on full [bs, 32, V] logits: same committed tokens and step
    maps (the projection runs on fewer rows, which may pick another GEMM tiling and flip a near-tie)."""
    from mdx.engine import BlockDiffusionEngine, SamplingParams
    cfg, model = _tiny(dev)
    outs = []
    for rows_only in (False, True):
        eng = BlockDiffusionEngine(model, num_pages=16, shuffle_pages_seed=3, decode_graphs=True, max_model_len=1024,
                                   masked_rows_only=rows_only)
        g = torch.Generator().manual_seed(2)
        seqs = [eng.add_request(torch.randint(0, 900, (n,), generator=g).tolist(),
                                SamplingParams(max_new_tokens=96, ignore_eos=True, transfer_count=4, temperature=t))
                for n, t in zip((290, 33, 150), temps)]
        eng.generate()
        outs.append([(s.completion_token_ids, list(s.step_map)) for s in seqs])
        assert eng.stats["decode_passes"] == 3 * 9 - 1      # 3 blocks x (8 denoise + 1 caching pass); the prefill pass is the first denoise
    for (ta, ma), (tb, mb) in zip(*outs):
        assert len(ta) == len(tb) == 96 and len(ma) == len(mb)
        same = sum(int(a == b) for a, b in zip(ta, tb))
        assert same >= 90, f"only {same}/96 tokens agree"
        assert sum(int(a == b) for a, b in zip(ma, mb)) >= 90


@pytest.mark.parametrize("rows_only", [False, True])
@pytest.mark.parametrize("temps", [(1.0, 1.0, 1.0), (1.0, 0.7, 1.3)])
def test_fused_head_generates_like_projection_plus_confidence_pass(dev, temps, rows_only):
    """The device loop with the vocabulary projection fused into the confidence reduction (no logits in memory,
    mdx_lm_head_confidence; forced on for this small batch) against the same engine on the library GEMM + the
    vocabulary pass: same pass count, same committed tokens and step maps up to near-ties (the two sum the
    products in different orders, which can move a logit to the neighbouring bf16 value)."""
    from mdx.engine import BlockDiffusionEngine, SamplingParams
    cfg, model = _tiny(dev)
    outs = []
    for fused in (False, True):
        eng = BlockDiffusionEngine(model, num_pages=16, shuffle_pages_seed=3, decode_graphs=True, max_model_len=1024,
                                   masked_rows_only=rows_only, fused_head=fused, fused_head_min_rows=1)
        g = torch.Generator().manual_seed(2)
        seqs = [eng.add_request(torch.randint(0, 900, (n,), generator=g).tolist(),
                                SamplingParams(max_new_tokens=96, ignore_eos=True, transfer_count=4, temperature=t))
                for n, t in zip((290, 33, 150), temps)]
        eng.generate()
        outs.append([(s.completion_token_ids, list(s.step_map)) for s in seqs])
        assert eng.stats["decode_passes"] == 3 * 9 - 1
    for (ta, ma), (tb, mb) in zip(*outs):
        assert len(ta) == len(tb) == 96 and cfg.mask_token_id not in tb
        assert sum(int(a == b) for a, b in zip(ta, tb)) >= 90
        assert sum(int(a == b) for a, b in zip(ma, mb)) >= 90


def test_replay_ahead_changes_nothing(dev):
    """Enqueuing the next decode forward before the host bookkeeping of the current pass is pure
    scheduling: same tokens, same step maps, same pass count, with a request that arrives late
    (its prefill runs between two decode passes) and sequences of different lengths."""
    from mdx.engine import BlockDiffusionEngine, SamplingParams
    cfg, model = _tiny(dev)
    outs = []
    for ahead in (False, True):
        eng = BlockDiffusionEngine(model, num_pages=20, shuffle_pages_seed=4, decode_graphs=True, max_model_len=1024,
                                   replay_ahead=ahead)
        g = torch.Generator().manual_seed(6)
        sp = SamplingParams(max_new_tokens=64, ignore_eos=True, transfer_count=4)
        seqs = [eng.add_request(torch.randint(0, 900, (n,), generator=g).tolist(), sp) for n in (200, 45)]
        for _ in range(5):
            eng.step()
        seqs.append(eng.add_request(torch.randint(0, 900, (77,), generator=g).tolist(),
                                    SamplingParams(max_new_tokens=32, ignore_eos=True, transfer_count=8)))
        eng.generate()
        outs.append(([s.completion_token_ids for s in seqs], [list(s.step_map) for s in seqs], dict(eng.stats)))
    (ta, ma, sa), (tb, mb, sb) = outs
    assert set(eng._graphs) <= {1, 2, 4}                   # batches of 3, 2, 1 run in the graphs for 4, 2, 1
    assert ta == tb and ma == mb
    assert sa["decode_passes"] == sb["decode_passes"] and sa["prefill_passes"] == sb["prefill_passes"] == 2


def test_gumbel_noise_is_reproducible_per_seed(dev):
    """Sampler.prepare adds Gumbel noise to the scaled logits before the argmax (sampler.py:15-18);
    here the noise is drawn inside the unmask kernel as a function of (seed, sampling pass, row, column):
    same seed, same tokens -- through the device loop with logits of the masked rows only, with logits of
    all rows, and through the host-driven passes; another seed or no noise, other tokens (temperature 1
    on a random-weight model: the argmax is far from certain)."""
    from mdx.engine import BlockDiffusionEngine, SamplingParams
    cfg, model = _tiny(dev)
    outs = {}
    for key, kw in (("a", dict(gumbel_seed=7)), ("b", dict(gumbel_seed=7)), ("c", dict(gumbel_seed=8)), ("plain", {}),
                    ("full", dict(gumbel_seed=7, masked_rows_only=False)), ("host", dict(gumbel_seed=7, decode_graphs=False)),
                    ("lockstep", dict(gumbel_seed=7, replay_ahead=False))):
        kw = {"decode_graphs": True, **kw}
        eng = BlockDiffusionEngine(model, num_pages=10, shuffle_pages_seed=3, max_model_len=1024, **kw)
        s = eng.add_request(list(range(5, 200)), SamplingParams(max_new_tokens=64, ignore_eos=True, transfer_count=4))
        eng.generate()
        outs[key] = s.completion_token_ids
        assert len(outs[key]) == 64 and cfg.mask_token_id not in outs[key]
    assert outs["a"] == outs["b"]
    assert outs["a"] != outs["c"] and outs["a"] != outs["plain"]
    assert outs["full"] == outs["a"] == outs["host"] == outs["lockstep"]   # the draw does not depend on how the pass is run


@pytest.mark.parametrize("graphs", [False, True])
def test_preemption_on_the_device_keeps_the_tokens(dev, graphs):
    """scheduler.py:44-63 on the GPU: with too few pages for both sequences to grow, one is preempted, its
    pages freed, and it is prefilled again later together with the tokens it had committed (the
    prefill then runs over a partly unmasked current block).  Both sequences must finish, and with
    the tokens of a run that had pages to spare (a near-tie may flip with the changed pass order)."""
    from mdx.engine import BlockDiffusionEngine, SamplingParams
    cfg, model = _tiny(dev)
    outs = []
    for pages in (12, 4):
        eng = BlockDiffusionEngine(model, num_pages=pages, shuffle_pages_seed=2, decode_graphs=graphs, max_model_len=1024)
        sp = SamplingParams(max_new_tokens=288, ignore_eos=True, transfer_count=8)
        s1 = eng.add_request([5 + (i * 7) % 900 for i in range(300)], sp)      # grows from 2 to 3 pages
        s2 = eng.add_request([11 + (i * 13) % 900 for i in range(40)], sp)     # grows from 1 to 2 pages: 5 > 4 in total
        eng.generate()
        assert s1.num_completion_tokens == 288 and s2.num_completion_tokens == 288
        assert (eng.stats.get("preemptions", 0) >= 1) == (pages == 4)
        assert len(eng.block_manager.free) == pages and not eng.running and not eng.waiting
        outs.append(s1.completion_token_ids + s2.completion_token_ids)
    same = sum(int(a == b) for a, b in zip(*outs))
    assert same >= 0.9 * len(outs[0]), f"only {same}/{len(outs[0])} tokens agree"


def test_sequences_that_finish_at_different_times(dev):
    """Five requests of different lengths and budgets: as they finish one by one the decode batch shrinks
    through the captured sizes 8, 4, 2, 1 (padding rows in between), page tables and lengths change
    under the graphs, and every sequence must still produce what the eager engine produces."""
    from mdx.engine import BlockDiffusionEngine, SamplingParams
    cfg, model = _tiny(dev)
    outs = []
    for graphs in (False, True):
        eng = BlockDiffusionEngine(model, num_pages=24, shuffle_pages_seed=4, decode_graphs=graphs, max_model_len=1024)
        seqs = []
        for i, (n_prompt, budget) in enumerate(((17, 32), (250, 160), (64, 96), (300, 64), (5, 128))):
            sp = SamplingParams(max_new_tokens=budget, ignore_eos=True, transfer_count=8)
            seqs.append(eng.add_request([3 + (j * (5 + i)) % 900 for j in range(n_prompt)], sp))
        eng.generate()
        assert [s.num_completion_tokens for s in seqs] == [32, 160, 96, 64, 128]
        if graphs:
            assert {1, 2, 4, 8} <= set(eng._graphs)
        outs.append([t for s in seqs for t in s.completion_token_ids])
    same = sum(int(a == b) for a, b in zip(*outs))
    assert same >= 0.95 * len(outs[0]), f"only {same}/{len(outs[0])} tokens agree"


def test_stop_token_ends_the_sequence_at_its_block(dev):
    """scheduler.py:71-78: a sequence whose finished block holds a stop token ends with that block
    (unless ignore_eos), whatever its token budget."""
    from mdx.engine import BlockDiffusionEngine, SamplingParams
    cfg, model = _tiny(dev)
    prompt = [7 + (j * 3) % 900 for j in range(100)]
    eng = BlockDiffusionEngine(model, num_pages=8, decode_graphs=True, max_model_len=1024)
    free = eng.add_request(prompt, SamplingParams(max_new_tokens=160, ignore_eos=True, transfer_count=8))
    eng.generate()
    tokens = free.completion_token_ids
    # the stop token: the one whose first appearance comes latest (the tiny random model repeats itself a lot)
    first = {}
    for i, t in enumerate(tokens):
        first.setdefault(t, i)
    stop, at = max(first.items(), key=lambda kv: kv[1])
    end = (at // 32 + 1) * 32
    eng = BlockDiffusionEngine(model, num_pages=8, decode_graphs=True, max_model_len=1024)
    sp = SamplingParams(max_new_tokens=160, ignore_eos=False, transfer_count=8, stop_token_ids=(stop,))
    s = eng.add_request(prompt, sp)
    eng.generate()
    assert s.num_completion_tokens == end and s.completion_token_ids == tokens[:end]
    assert len(eng.block_manager.free) == 8
