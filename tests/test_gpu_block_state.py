"""GPU parity of the three per-lane block-state kernels (csrc/block_state.hip) through the C ABI, bit-exact
against the oracle: the pass inputs of prepare_decode, the masked-row list, and the state advance that
follows the selection (sampler.py:56-59 + scheduler.py:65-82)."""
import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu
MASK, PAGE = 151669, 256


def _stream():
    return torch.cuda.current_stream().cuda_stream


@pytest.mark.parametrize("S", [32, 4, 100])
def test_block_prepare_matches_oracle(dev, S):
    import mdx
    rng = np.random.default_rng(S)
    bs, width = 9, 6
    lens = rng.integers(0, 1300, bs).astype(np.int32)
    lens[3] = 256 - S // 2                                 # a block straddling a page boundary
    phase = rng.integers(0, 3, bs).astype(np.int32)
    phase[3] = 1
    bt = np.full((bs, width + 2), -1, dtype=np.int32)      # row stride wider than the table
    for b in range(bs):
        n = rng.integers(1, width + 1)
        bt[b, :n] = rng.permutation(64)[:n]
    d = lambda a: torch.from_numpy(a).to(dev)             # noqa: E731
    dl, dp, dbt = d(lens), d(phase), d(bt)
    pos = torch.full((bs, S), -7, dtype=torch.int64, device=dev)
    slots = torch.full((bs, S), -7, dtype=torch.int32, device=dev)
    ctx = torch.full((bs,), -7, dtype=torch.int32, device=dev)
    rc = mdx.lib().mdx_block_prepare(dl.data_ptr(), dp.data_ptr(), dbt.data_ptr(), dbt.stride(0), width, PAGE, S,
                                     pos.data_ptr(), slots.data_ptr(), ctx.data_ptr(), bs, _stream())
    assert rc == 0
    epos, eslots, ectx = oracle.block_prepare(lens, phase, bt[:, :width], PAGE, S)
    assert np.array_equal(pos.cpu().numpy(), epos) and np.array_equal(slots.cpu().numpy(), eslots)
    assert np.array_equal(ctx.cpu().numpy(), ectx)


@pytest.mark.parametrize("bs,S,cap", [(3, 32, 96), (40, 32, 640), (40, 32, 64), (2, 7, 14), (70, 32, 2240)])
def test_masked_rows_matches_oracle(dev, bs, S, cap):
    import mdx
    rng = np.random.default_rng(bs * S + cap)
    tok = rng.integers(0, 1000, (bs, S)).astype(np.int64)
    tok[rng.random((bs, S)) < 0.4] = MASK
    phase = rng.integers(0, 3, bs).astype(np.int32)
    dt, dp = torch.from_numpy(tok).to(dev), torch.from_numpy(phase).to(dev)
    rows = torch.full((cap,), -1, dtype=torch.int64, device=dev)
    n = torch.full((1,), -1, dtype=torch.int32, device=dev)
    rc = mdx.lib().mdx_masked_rows(dt.data_ptr(), dp.data_ptr(), MASK, bs, S, rows.data_ptr(), cap, n.data_ptr(), _stream())
    assert rc == 0
    erows, en = oracle.masked_rows(tok, phase, MASK, cap)
    assert int(n.item()) == en
    assert np.array_equal(rows.cpu().numpy(), erows)
    # nothing masked at all: the list is all zeros
    dt.fill_(5)
    mdx.lib().mdx_masked_rows(dt.data_ptr(), dp.data_ptr(), MASK, bs, S, rows.data_ptr(), cap, n.data_ptr(), _stream())
    assert int(n.item()) == 0 and int(rows.abs().sum().item()) == 0


@pytest.mark.parametrize("S", [32, 8, 80])
def test_block_advance_matches_oracle(dev, S):
    import mdx
    rng = np.random.default_rng(100 + S)
    bs, n_stop, out_stride = 12, 4, 40 * S
    for trial in range(4):
        tok = rng.integers(0, 50, (bs, S)).astype(np.int64)
        phase = rng.integers(0, 3, bs).astype(np.int32)
        for b in range(bs):
            if phase[b] == 1 and rng.random() < 0.7:                    # most denoising lanes still hold masks
                tok[b, rng.random(S) < 0.5] = MASK
        transfer = ((rng.random((bs, S)) < 0.3) & (phase[:, None] == 1)).astype(np.uint8)
        step_map = rng.integers(0, 9, (bs, S)).astype(np.int32)
        step = rng.integers(0, 20, bs).astype(np.int32)
        first = rng.integers(1, 300, bs).astype(np.int32)
        blocks_done = rng.integers(0, 5, bs)
        lens = (first + blocks_done * S).astype(np.int32)
        max_new = rng.choice([S, 3 * S, 5 * S - 3, 30 * S], bs).astype(np.int32)
        stop = np.full((bs, n_stop), -1, dtype=np.int64)
        stop[::3, 0] = 7                                                # some lanes stop on token 7
        stop[1::4, 2] = 49
        d = lambda a: torch.from_numpy(a.copy()).to(dev)               # noqa: E731
        dtok, dtr, dmap, dstep, dph, dlen = d(tok), d(transfer), d(step_map), d(step), d(phase), d(lens)
        dfirst, dmax, dstop = d(first), d(max_new), d(stop)              # kept alive until the launch has run
        out_tok = torch.full((bs, out_stride), -1, dtype=torch.int64, device=dev)
        out_step = torch.full((bs, out_stride), -1, dtype=torch.int32, device=dev)
        status = torch.full((bs, 4), -9, dtype=torch.int32, device=dev)
        rc = mdx.lib().mdx_block_advance(dtok.data_ptr(), dtr.data_ptr(), dmap.data_ptr(), dstep.data_ptr(), dph.data_ptr(), dlen.data_ptr(),
                                         dfirst.data_ptr(), dmax.data_ptr(), dstop.data_ptr(), n_stop,
                                         out_tok.data_ptr(), out_step.data_ptr(), out_stride, status.data_ptr(), MASK, bs, S, _stream())
        assert rc == 0, mdx.lib().mdx_last_error()
        et, em, es, eph, el, appended, est = oracle.block_advance(tok, transfer, step_map, step, phase, lens, first, max_new, stop, MASK)
        assert np.array_equal(dtok.cpu().numpy(), et) and np.array_equal(dmap.cpu().numpy(), em)
        assert np.array_equal(dstep.cpu().numpy(), es) and np.array_equal(dph.cpu().numpy(), eph) and np.array_equal(dlen.cpu().numpy(), el)
        got_status = status.cpu().numpy()
        ot, os_ = out_tok.cpu().numpy(), out_step.cpu().numpy()
        for b in range(bs):
            ph, ln, left, moved = est[b]
            assert got_status[b, 0] == ph and got_status[b, 2] == left and got_status[b, 3] == moved
            if ln is not None:
                assert got_status[b, 1] == ln
            at = lens[b] - first[b]
            if appended[b] is None:
                assert (ot[b] == -1).all()
            else:
                assert np.array_equal(ot[b, at:at + S], appended[b][0]) and np.array_equal(os_[b, at:at + S], appended[b][1])
                assert (ot[b, :at] == -1).all() and (ot[b, at + S:] == -1).all()
