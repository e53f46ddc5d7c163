"""Host logic of the mini engine on the CPU: slot arithmetic, page allocation, the tensors the
runner hands to the kernels, and the denoise -> CACHING -> append state machine, driven by a
scripted model and an oracle-backed unmask step (no GPU, no libmdx call)."""
import numpy as np
import pytest
import torch

import oracle
from mdx import get_context
from mdx.engine import PAGE, BlockDiffusionEngine, BlockManager, DecoderConfig, SamplingParams, Sequence, SequenceStatus

MASK = 99


def test_get_slots_matches_brute_force():
    s = Sequence(list(range(700)), mask_token_id=MASK)
    assert s.get_slots(0, 5) == [-1] * 5                     # no pages yet (warm-up sequences)
    s.block_table = [7, 2, 9]
    for lo, hi in [(0, 700), (250, 262), (255, 257), (512, 700), (300, 301), (10, 10)]:
        assert s.get_slots(lo, hi) == oracle.get_slots(s.block_table, lo, hi)


def test_block_manager_and_need_new_block():
    bm = BlockManager(8)
    s = Sequence(list(range(500)), mask_token_id=MASK)       # 2 pages for the prompt
    assert bm.can_allocate(s)
    bm.allocate(s)
    assert s.block_table == [0, 1] and len(bm.free) == 6
    assert s.need_new_block()                                # 500 + 32 > 512
    bm.may_append(s)
    assert s.block_table == [0, 1, 2] and not s.need_new_block()
    bm.deallocate(s)
    assert len(bm.free) == 8 and not s.block_table


class ScriptedModel:
    """Stands in for the decoder: records the runner's inputs and returns logits whose argmax at
    block position p is token 10 + p, with a confidence chosen by the test."""

    def __init__(self, vocab=64, peak=0.0):
        self.c = DecoderConfig(num_layers=0, hidden_size=8, vocab_size=vocab, block_size=32, mask_token_id=MASK)
        self.lm_head = torch.zeros(1)
        self.layers = []
        self.peak = peak
        self.calls = []

    def embed(self, ids):
        return torch.zeros(*ids.shape, 8)

    def __call__(self, embeds, positions):
        ctx = get_context()
        self.calls.append(dict(prefill=ctx.is_prefill, positions=positions.clone(), slots=ctx.slot_mapping.clone(),
                               cu=None if ctx.cu_seqlens_q is None else ctx.cu_seqlens_q.clone(),
                               ctx_lens=None if ctx.context_lens is None else ctx.context_lens.clone(),
                               tables=None if ctx.block_tables is None else ctx.block_tables.clone()))
        return embeds

    def compute_logits(self, hidden):
        n = len(self.calls[-1]["cu"]) - 1 if self.calls[-1]["prefill"] else hidden.shape[0]
        logits = torch.zeros(n, 32, self.c.vocab_size)
        for p in range(32):
            logits[:, p, 10 + p] = 1.0 + 0.01 * p + self.peak      # later positions slightly more confident
        return logits.view(-1, self.c.vocab_size) if self.calls[-1]["prefill"] else logits


def oracle_unmask(logits, x, mask_id, thr, k, temperatures=None):
    x0, p, tr, new = oracle.unmask_step(logits.double().numpy(), x.numpy(), mask_id, thr, k,
                                        None if temperatures is None else temperatures.numpy())
    x.copy_(torch.from_numpy(new))
    return torch.from_numpy(x0), torch.from_numpy(p), torch.from_numpy(tr), torch.from_numpy(tr.sum(-1).astype(np.int32))


def _engine(model, **kw):
    return BlockDiffusionEngine(model, num_pages=16, unmask=oracle_unmask, **kw)


@pytest.mark.parametrize("k", [1, 4])
def test_topk_schedule_and_state_machine(k):
    model = ScriptedModel()
    eng = _engine(model)
    sp = SamplingParams(max_new_tokens=64, ignore_eos=True, transfer_count=k)
    s1 = eng.add_request(list(range(300)), sp)
    s2 = eng.add_request(list(range(40)), sp)
    eng.generate()
    # flat logits: top-k branch, so each block needs 32/k denoising passes + 1 caching pass
    assert len(model.calls) == oracle.expected_passes(32, k, 2)
    assert model.calls[0]["prefill"] and not any(c["prefill"] for c in model.calls[1:])
    for s in (s1, s2):
        assert s.status == SequenceStatus.FINISHED and s.num_completion_tokens == 64
        assert s.completion_token_ids == [10 + p for p in range(32)] * 2
        # most confident positions (the last ones) are committed first
        assert s.step_map[31] < s.step_map[0]
    assert len(eng.block_manager.free) == 16


def test_threshold_branch_commits_a_block_in_one_pass():
    model = ScriptedModel(peak=30.0)                         # every position above 0.9
    eng = _engine(model)
    s = eng.add_request(list(range(100)), SamplingParams(max_new_tokens=96, ignore_eos=True, transfer_count=4))
    eng.generate()
    assert len(model.calls) == 3 * 2                         # one denoising pass + one caching pass per block
    assert s.completion_token_ids == [10 + p for p in range(32)] * 3


def test_runner_tensors_follow_the_reference_layout():
    model = ScriptedModel()
    eng = _engine(model, shuffle_pages_seed=1)
    sp = SamplingParams(max_new_tokens=32, ignore_eos=True, transfer_count=4)
    s1 = eng.add_request(list(range(250)), sp)               # crosses a page when the block is appended
    s2 = eng.add_request(list(range(10)), sp)
    eng.step()
    pre = model.calls[0]
    assert pre["cu"].tolist() == [0, 282, 324]               # prompt + 32 mask tokens per sequence
    assert pre["positions"].tolist() == list(range(282)) + list(range(42))
    t1, t2 = list(s1.block_table), list(s2.block_table)
    want = oracle.get_slots(t1, 0, 250) + [-1] * 32 + oracle.get_slots(t2, 0, 10) + [-1] * 32
    assert pre["slots"].tolist() == want                     # the uncommitted block is not stored in prefill
    eng.step()
    dec = model.calls[1]
    assert len(s1.block_table) == 2 and len(s2.block_table) == 1      # 250 + 32 > 256 -> second page
    assert dec["ctx_lens"].tolist() == [282, 42]
    assert dec["positions"].tolist() == [list(range(250, 282)), list(range(10, 42))]
    assert dec["slots"].tolist() == [oracle.get_slots(s1.block_table, 250, 282), oracle.get_slots(s2.block_table, 10, 42)]
    assert dec["tables"].tolist() == [s1.block_table, s2.block_table + [-1]]


def test_stop_token_finishes_a_sequence():
    model = ScriptedModel(peak=30.0)
    eng = _engine(model)
    s = eng.add_request(list(range(5)), SamplingParams(max_new_tokens=320, stop_token_ids=[10 + 7], transfer_count=4))
    eng.generate()
    assert s.num_completion_tokens == 32 and s.status == SequenceStatus.FINISHED


def test_preemption_when_the_page_pool_runs_out():
    """scheduler.py:44-63: with too few pages for both sequences to grow, the one at the back of the
    queue is preempted (pages freed, back to the waiting queue), prefilled again later with the
    tokens it has committed so far, and both still finish with the right tokens."""
    model = ScriptedModel()
    eng = BlockDiffusionEngine(model, num_pages=4, unmask=oracle_unmask)
    sp = SamplingParams(max_new_tokens=288, ignore_eos=True, transfer_count=8)
    s1 = eng.add_request(list(range(300)), sp)              # grows from 2 to 3 pages
    s2 = eng.add_request(list(range(40)), sp)               # grows from 1 to 2 pages: 5 > 4 in total
    eng.generate()
    assert eng.stats["preemptions"] >= 1
    assert sum(c["prefill"] for c in model.calls) >= 2      # the preempted sequence was prefilled again
    for s in (s1, s2):
        assert s.status == SequenceStatus.FINISHED and s.num_completion_tokens == 288
        assert s.completion_token_ids == [10 + p for p in range(32)] * 9
    assert len(eng.block_manager.free) == 4 and not eng.running and not eng.waiting


# ---- the per-lane block state machine of the device loop, on the CPU ---------------------------------------
def test_oracle_block_prepare_is_get_slots_per_lane():
    lens, phase = [250, 10, 700, 0], [1, 2, 0, 1]
    bt = np.array([[7, 2, -1, -1], [5, -1, -1, -1], [1, 3, 4, -1], [6, -1, -1, -1]], dtype=np.int32)
    pos, slots, ctx = oracle.block_prepare(lens, phase, bt, PAGE, 32)
    assert ctx.tolist() == [282, 42, 0, 32]
    for b in (0, 1, 3):
        assert pos[b].tolist() == list(range(lens[b], lens[b] + 32))
        assert slots[b].tolist() == oracle.get_slots([int(x) for x in bt[b] if x >= 0], lens[b], lens[b] + 32)
    assert (slots[2] == -1).all() and (pos[2] == 0).all()                  # idle lane = graph padding
    # a block that runs past the last page of the table has no slot there
    _, s2, _ = oracle.block_prepare([250], [1], np.array([[9, -1]], dtype=np.int32), PAGE, 32)
    assert s2[0, :6].tolist() == [9 * PAGE + 250 + i for i in range(6)] and (s2[0, 6:] == -1).all()


def test_oracle_masked_rows():
    tok = np.full((3, 8), 5)
    tok[0, [1, 6]] = MASK
    tok[1, :] = MASK                                                       # idle lane: not listed
    tok[2, 3] = MASK
    rows, n = oracle.masked_rows(tok, [1, 0, 1], MASK, 6)
    assert n == 3 and rows.tolist() == [1, 6, 19, 1, 1, 1]
    rows, n = oracle.masked_rows(tok, [2, 0, 2], MASK, 4)                  # caching lanes have nothing masked to project
    assert n == 0 and rows.tolist() == [0, 0, 0, 0]
    rows, n = oracle.masked_rows(tok, [1, 1, 1], MASK, 2)                  # more than the list holds: count says so
    assert n == 11 and rows.tolist() == [1, 6]


@pytest.mark.parametrize("k,peak", [(1, 0.0), (4, 0.0), (8, 0.0), (4, 30.0)])
def test_oracle_block_advance_runs_the_same_generation_as_the_host_engine(k, peak):
    """select_transfer + block_advance, pass after pass, against the host engine's Sequence / postprocess on the
    same scripted confidences: same pass count (the closed form), same tokens, same step maps."""
    model = ScriptedModel(peak=peak)
    eng = _engine(model)
    budgets = [64, 96]
    sp = [SamplingParams(max_new_tokens=b, ignore_eos=True, transfer_count=k) for b in budgets]
    seqs = [eng.add_request(list(range(300)), sp[0]), eng.add_request(list(range(40)), sp[1])]
    eng.generate()

    S = 32
    logits = model.compute_logits(torch.zeros(2, S, 8)).double().numpy()      # the scripted logits of a decode pass
    _, conf = oracle.confidence_argmax(logits)
    x0 = logits.argmax(-1)
    tokens = np.full((2, S), MASK, dtype=np.int64)
    step_map = np.zeros((2, S), dtype=np.int32)
    step, phase, lens = np.zeros(2, dtype=np.int32), np.array([1, 1]), np.array([300, 40])
    first, stop = np.array([300, 40]), np.full((2, 4), -1)
    out_tok, out_step, passes = [[], []], [[], []], 0
    while (phase != 0).any():
        transfer = oracle.select_transfer(conf.astype(np.float32), (tokens == MASK) & (phase[:, None] == 1), 0.9, k)
        tokens = np.where(transfer, x0, tokens)
        tokens, step_map, step, phase, lens, appended, status = oracle.block_advance(
            tokens, transfer, step_map, step, phase, lens, first, np.array(budgets), stop, MASK)
        for b, a in enumerate(appended):
            if a is not None:
                out_tok[b] += a[0].tolist()
                out_step[b] += a[1].tolist()
        passes += 1
    per_block = 2 if peak else oracle.expected_passes(S, k, 1)
    assert passes == 3 * per_block                                           # the longer request: three blocks
    assert passes == len(model.calls)                                        # the host engine's prefill pass is its first denoising pass
    for b, s in enumerate(seqs):
        assert out_tok[b] == s.completion_token_ids and out_step[b] == s.step_map
        assert lens[b] == s.num_tokens


def test_oracle_block_advance_stop_token_and_idle_lanes():
    S = 32
    tokens = np.tile(np.arange(10, 10 + S), (3, 1)).astype(np.int64)          # complete blocks
    zeros = np.zeros((3, S), dtype=bool)
    stop = np.array([[17, -1, -1, -1], [-1, -1, -1, -1], [17, -1, -1, -1]])
    t, m, step, phase, lens, appended, status = oracle.block_advance(
        tokens, zeros, np.zeros((3, S), dtype=np.int32), [4, 4, 4], [2, 2, 0], [5, 5, 5], [5, 5, 5], [320, 320, 320], stop, MASK)
    assert phase.tolist() == [0, 1, 0] and lens.tolist() == [37, 37, 5]      # lane 0 stops, lane 1 goes on, lane 2 was idle
    assert appended[2] is None and appended[0][0].tolist() == list(range(10, 42))
    assert (t[0] == MASK).all() and (t[2] == tokens[2]).all() and step.tolist() == [5, 5, 4]
    assert status[1] == (1, 37, S, 0)


def test_transfer_schedule_helper_matches_the_oracle():
    """mdx.num_transfer_tokens is host arithmetic (modeling_mineru_diffusion.py:617-623): same lists as the oracle's,
    which sum to the block length, differ by at most one and may hold zeros when a block is shorter than its steps."""
    import mdx
    for block, steps in ((32, 8), (32, 32), (10, 4), (32, 5), (3, 8), (1, 1)):
        got = mdx.num_transfer_tokens(block, steps)
        assert got == oracle.num_transfer_tokens(block, steps)
        assert sum(got) == block and max(got) - min(got) <= 1 and got == sorted(got, reverse=True)
    assert mdx.num_transfer_tokens(3, 8) == [1, 1, 1, 0, 0, 0, 0, 0]



def test_oracle_block_advance_against_a_hand_written_trace():
    """One lane, a block of 4 positions, budget of one block, written out by hand from layers/sampler.py:56-59 and
    engine/scheduler.py:65-82 (no engine code involved).  Pass 0 commits positions 2 and 0, pass 1 commits 1 and 3
    and thereby ends the denoising (phase -> caching), pass 2 is the caching pass: the block is appended, the
    length grows by 4, the budget is spent (phase -> idle), the lane's tokens become a fresh all-mask block."""
    M = MASK
    tokens = np.array([[M, M, M, M]], dtype=np.int64)
    step_map = np.zeros((1, 4), dtype=np.int32)
    step, phase, lens = np.array([0], dtype=np.int32), np.array([1]), np.array([10])
    first, budget, stop = np.array([10]), np.array([4]), np.full((1, 4), -1)

    # pass 0: the sampler wrote tokens 7 and 5 at positions 2 and 0
    tokens[0, 2], tokens[0, 0] = 7, 5
    transfer = np.array([[True, False, True, False]])
    tokens, step_map, step, phase, lens, appended, status = oracle.block_advance(
        tokens, transfer, step_map, step, phase, lens, first, budget, stop, M)
    assert tokens.tolist() == [[5, M, 7, M]] and step_map.tolist() == [[0, 0, 0, 0]]     # committed at step 0
    assert step.tolist() == [1] and phase.tolist() == [1] and lens.tolist() == [10] and appended == [None]
    assert status == [(1, 10, 2, 2)]                                                    # denoising, 2 masked left, 2 committed

    # pass 1: positions 1 and 3 get 8 and 9: nothing masked is left, the next pass only caches
    tokens[0, 1], tokens[0, 3] = 8, 9
    transfer = np.array([[False, True, False, True]])
    tokens, step_map, step, phase, lens, appended, status = oracle.block_advance(
        tokens, transfer, step_map, step, phase, lens, first, budget, stop, M)
    assert tokens.tolist() == [[5, 8, 7, 9]] and step_map.tolist() == [[0, 1, 0, 1]]
    assert step.tolist() == [2] and phase.tolist() == [2] and lens.tolist() == [10] and appended == [None]
    assert status == [(2, 10, 0, 2)]

    # pass 2 (caching): nothing is committed; the block is appended and the budget of 4 new tokens is spent
    transfer = np.zeros((1, 4), dtype=bool)
    tokens, step_map, step, phase, lens, appended, status = oracle.block_advance(
        tokens, transfer, step_map, step, phase, lens, first, budget, stop, M)
    assert appended[0][0].tolist() == [5, 8, 7, 9] and appended[0][1].tolist() == [0, 1, 0, 1]
    assert tokens.tolist() == [[M, M, M, M]] and lens.tolist() == [14] and phase.tolist() == [0] and step.tolist() == [3]
    assert status == [(0, 14, 0, 0)]

    # the same lane with a budget of two blocks goes back to denoising instead, with 4 masked positions
    t2, _, _, p2, l2, _, s2 = oracle.block_advance(np.array([[5, 8, 7, 9]]), transfer, np.array([[0, 1, 0, 1]], dtype=np.int32),
                                                   np.array([2], dtype=np.int32), np.array([2]), np.array([10]), first, np.array([8]), stop, M)
    assert p2.tolist() == [1] and l2.tolist() == [14] and s2 == [(1, 14, 4, 0)] and t2.tolist() == [[M, M, M, M]]
