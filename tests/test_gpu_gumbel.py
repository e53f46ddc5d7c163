"""GPU parity: Gumbel noise drawn inside the kernel (Philox-4x32-10 keyed by seed, counted by
offset / row / column) against the oracle's restatement of the generator, and the sampling calls that
use it against the same calls fed the noise as a tensor."""
import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu
MASK_ID = 151669


def _f64(t):
    return t.detach().cpu().to(torch.float64).numpy()


@pytest.mark.parametrize("rows,vocab,seed,offset", [(3, 1, 0, 0), (5, 7, 1, 0), (4, 4096, 123456789, 17), (40, 151936, 2 ** 40 + 3, 2 ** 35 + 1)])
def test_noise_tensor_matches_the_oracle_generator(dev, rows, vocab, seed, offset):
    import mdx
    got = mdx.gumbel_noise(rows, vocab, seed, offset, device=dev)
    torch.cuda.synchronize()
    want = oracle.gumbel_noise(rows, vocab, seed, offset)
    # same random bits (a wrong word would be off by O(1)); fp32 logarithms against fp64 ones.  The largest case
    # holds 6 million draws: its largest noise values (above 14, from u within 1e-6 of 1, the draws that decide an
    # argmax) are as accurate as the rest.
    np.testing.assert_allclose(_f64(got), want, rtol=0, atol=3e-6)
    if rows * vocab > 10 ** 6:
        assert want.max() > 14


def test_noise_row_ids_and_device_offset(dev):
    import mdx
    ids = torch.tensor([9, 0, 4], dtype=torch.int64, device=dev)
    bump = torch.tensor([5], dtype=torch.int64, device=dev)
    got = mdx.gumbel_noise(3, 1001, 77, 20, device=dev, offset_dev=bump, row_ids=ids)
    torch.cuda.synchronize()
    np.testing.assert_allclose(_f64(got), oracle.gumbel_noise(3, 1001, 77, 25, row_ids=[9, 0, 4]), rtol=0, atol=3e-6)
    full = mdx.gumbel_noise(10, 1001, 77, 25, device=dev)
    assert torch.equal(got, full[ids])                      # the same bits as the uncompacted layout


def _case(dev, dtype, bs, S, V, seed, offset, temps=None, stride=None):
    g = torch.Generator().manual_seed(V + bs)
    if stride is None:
        logits = (torch.randn(bs, S, V, generator=g) * 3).to(dtype).to(dev)
    else:                                                    # rows off the 16-byte grid
        buf = (torch.randn(bs * S, stride, generator=g) * 3).to(dtype).to(dev)
        logits = buf[:, :V].unflatten(0, (bs, S))
    return logits


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("bs,S,V,stride", [(2, 4, 1, None), (2, 4, 37, None), (1, 8, 5000, 5003), (2, 32, 40000, None), (40, 32, 4096, None), (1, 4, 151936, None)])
def test_seeded_sampling_equals_sampling_with_the_noise_tensor(dev, dtype, bs, S, V, stride):
    """confidence_argmax(seed, offset) draws the tokens of confidence_argmax(noise = gumbel_noise(seed, offset)),
    all of them (rows split over several workgroups, one workgroup per row, rows off the 16-byte grid; the
    confidences are the same sums taken in another order), and those of the oracle's sampling on the oracle's
    noise wherever the best two noisy logits are not within rounding."""
    import mdx
    logits = _case(dev, dtype, bs, S, V, 5, 9, stride=stride)
    temps = torch.linspace(0.6, 1.5, bs, device=dev)
    x0, p = mdx.confidence_argmax(logits, temps, seed=5, offset=9)
    noise = mdx.gumbel_noise(bs * S, V, 5, 9, device=dev)
    x0n, pn = mdx.confidence_argmax(logits, temps, noise=noise.view(bs, S, V))
    torch.cuda.synchronize()
    assert torch.equal(x0, x0n)
    torch.testing.assert_close(p, pn, rtol=3e-6, atol=0)
    l = _f64(logits)
    gn = oracle.gumbel_noise(bs * S, V, 5, 9).reshape(bs, S, V)
    ex0, ep = oracle.confidence_argmax(l, temps.cpu().numpy(), gn)
    noisy = (l.astype(np.float32) / temps.cpu().numpy().reshape(-1, 1, 1)).astype(np.float64) + gn
    top2 = np.sort(noisy, axis=-1)[..., -2:] if V > 1 else np.stack([noisy[..., 0] - 1, noisy[..., 0]], -1)
    clear = (top2[..., 1] - top2[..., 0]) > 1e-4
    assert clear.mean() > 0.95
    assert np.array_equal(x0.cpu().numpy()[clear], ex0[clear])
    np.testing.assert_allclose(p.cpu().numpy()[clear], ep[clear], rtol=3e-5, atol=1e-30)
    if V > 100:
        assert not np.array_equal(x0.cpu().numpy(), l.argmax(-1))          # the noise moved some picks
        x0b, _ = mdx.confidence_argmax(logits, temps, seed=5, offset=10)
        assert not torch.equal(x0, x0b)                                     # another offset, another draw


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_seeded_sampling_of_peaked_rows_skips_only_what_cannot_win(dev, dtype):
    """The seeded kernel leaves the generator alone for chunks none of whose elements could take the lead (largest
    element + the largest possible draw below the lane's best so far): rows with a few candidates far above a bulk 20
    to 60 below them, with stretches of -inf, with the candidates early, late or clustered, at several temperatures
    -- the picks must be those of the kernel that reads the same noise from a tensor and skips nothing."""
    import mdx
    g = torch.Generator().manual_seed(77)
    bs, S, V = 3, 16, 50000
    logits = torch.randn(bs, S, V, generator=g) * 2 - 40
    for b in range(bs):
        for r in range(S):
            n = int(torch.randint(1, 40, (1,), generator=g))
            where = torch.randint(0, V, (n,), generator=g) if r % 3 else torch.arange(V - n, V) if r % 2 else torch.arange(n)
            logits[b, r, where] = torch.randn(n, generator=g) * 3 + (0 if r % 4 else 15)
            if r % 5 == 0:
                lo = int(torch.randint(0, V - 9000, (1,), generator=g))
                keep = logits[b, r, where].clone()
                logits[b, r, lo:lo + 9000] = float("-inf")
                logits[b, r, where] = keep
    logits = logits.to(dtype).to(dev)
    temps = torch.tensor([0.5, 1.0, 2.5], device=dev)
    for offset in range(3):
        x0, p = mdx.confidence_argmax(logits, temps, seed=11, offset=offset)
        noise = mdx.gumbel_noise(bs * S, V, 11, offset, device=dev)
        x0n, pn = mdx.confidence_argmax(logits, temps, noise=noise.view(bs, S, V))
        torch.cuda.synchronize()
        assert torch.equal(x0, x0n)
        torch.testing.assert_close(p, pn, rtol=3e-6, atol=0)
    assert len(set(x0.flatten().tolist())) > 10


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("bs,S,V", [(1, 4, 151936), (2, 8, 50001), (40, 32, 5000), (3, 5, 2048 * 3 + 8 * 70)])
def test_seeded_sampling_of_rows_whose_noisy_logits_are_all_negative(dev, dtype, bs, S, V):
    """Rows shifted to about -60, so that every noisy logit is negative, with chunk counts that are not a multiple
    of the workgroup's width: on the last, partly filled trip of a row the wavefront's lead is not published (a
    shuffle over switched-off lanes reads 0, which would beat every real value here and let the other wavefronts
    skip the winner).  Picks must be those of the tensor-noise path, which skips nothing."""
    import mdx
    g = torch.Generator().manual_seed(V)
    logits = (torch.randn(bs, S, V, generator=g) * 2 - 60)
    # winners late in the row and inside the last trips of other wavefronts
    for b in range(bs):
        for r in range(S):
            at = V - 1 - int(torch.randint(0, min(V, 4096), (1,), generator=g))
            logits[b, r, at] += 14.0
    logits = logits.to(dtype).to(dev)
    temps = torch.linspace(0.7, 1.4, bs, device=dev)
    for offset in range(4):
        x0, p = mdx.confidence_argmax(logits, temps, seed=21, offset=offset)
        noise = mdx.gumbel_noise(bs * S, V, 21, offset, device=dev)
        x0n, pn = mdx.confidence_argmax(logits, temps, noise=noise.view(bs, S, V))
        torch.cuda.synchronize()
        assert torch.equal(x0, x0n)
        torch.testing.assert_close(p, pn, rtol=3e-6, atol=0)
        assert float(((logits.float() / temps.view(-1, 1, 1)) + noise.view(bs, S, V)).max()) < 0


def test_seeded_unmask_step_equals_the_step_with_the_noise_tensor(dev):
    import mdx
    g = torch.Generator().manual_seed(3)
    bs, S, V = 6, 32, 30011
    logits = (torch.randn(bs, S, V, generator=g) * 3).bfloat16().to(dev)
    tokens = torch.where(torch.rand(bs, S, generator=g) < 0.6, torch.tensor(MASK_ID), torch.randint(0, V, (bs, S), generator=g))
    temps = torch.linspace(0.7, 1.3, bs, device=dev)
    bump = torch.tensor([3], dtype=torch.int64, device=dev)
    t1, t2 = tokens.clone().to(dev), tokens.clone().to(dev)
    a = mdx.unmask_step(logits, t1, MASK_ID, 0.3, 2, temps, seed=99, offset=4, offset_dev=bump)
    noise = mdx.gumbel_noise(bs * S, V, 99, 7, device=dev).view(bs, S, V)
    b = mdx.unmask_step(logits, t2, MASK_ID, 0.3, 2, temps, noise=noise)
    torch.cuda.synchronize()
    assert torch.equal(a[0], b[0]) and torch.equal(a[2], b[2]) and torch.equal(a[3], b[3])
    torch.testing.assert_close(a[1], b[1], rtol=3e-6, atol=0)
    assert torch.equal(t1, t2) and int(a[3].sum()) > 0


def test_draws_follow_the_softmax(dev):
    """Gumbel-max over many rows with the same logits: token frequencies = softmax(logits / T), and the reported
    confidence is that softmax at the drawn token."""
    import mdx
    l = torch.tensor([0.0, 1.0, 2.0, -1.0, 0.5, 1.5, -3.0, 0.25])
    rows = 60000
    logits = l.repeat(rows, 1).bfloat16().to(dev)
    T = 0.8
    temps = torch.full((1,), T, device=dev)
    x0, p = mdx.confidence_argmax(logits, temps, seed=2024, offset=1)
    torch.cuda.synchronize()
    want = torch.softmax(l.bfloat16().double() / T, -1).numpy()
    freq = np.bincount(x0.cpu().numpy(), minlength=8) / rows
    assert np.abs(freq - want).max() < 0.008                                 # about 4 sigma of the largest bin
    np.testing.assert_allclose(p.cpu().numpy(), want[x0.cpu().numpy()], rtol=1e-5)


def test_seeded_sampling_inside_a_graph_steps_with_the_device_offset(dev):
    """A captured call draws new noise on every replay when a device counter is stepped between replays, and the
    draw of replay i equals the eager call at offset + i."""
    import mdx
    g = torch.Generator().manual_seed(8)
    logits = (torch.randn(2, 32, 20000, generator=g) * 3).bfloat16().to(dev)
    step = torch.zeros(1, dtype=torch.int64, device=dev)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        mdx.confidence_argmax(logits, seed=1, offset=100, offset_dev=step)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        x0, p = mdx.confidence_argmax(logits, seed=1, offset=100, offset_dev=step)
        step.add_(1)
    seen = []
    for i in range(4):
        graph.replay()
        torch.cuda.synchronize()
        ex0, ep = mdx.confidence_argmax(logits, seed=1, offset=100 + i)
        torch.cuda.synchronize()
        assert torch.equal(x0, ex0) and torch.equal(p, ep)
        seen.append(x0.clone())
    assert not torch.equal(seen[0], seen[1])
