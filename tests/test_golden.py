"""The committed fixtures of tests/golden/ (made by tests/golden/make_golden.py from the CPU oracle):
on the CPU the oracle must still reproduce them; on the GPU the HIP path is checked against the
stored numbers, through the same entry points as the other parity tests."""
import math
import pathlib

import numpy as np
import pytest
import torch

import oracle

GOLD = pathlib.Path(__file__).resolve().parent / "golden"
TOL = 2e-2            # attention, max-abs against the stored fp32 answer


def bf16(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)


def load(name):
    return np.load(GOLD / name, allow_pickle=False)


# ----------------------------------------------------------------------------- CPU: oracle == fixtures
def test_oracle_reproduces_attention_fixtures():
    f = load("staircase_attn.npz")
    o = oracle.staircase_attn_varlen(bf16(f["q"]), bf16(f["k"]), bf16(f["v"]), f["cu"].tolist(), int(f["block"]))
    assert np.allclose(o.float().numpy(), f["o"], atol=1e-5)
    p = load("paged_block_attn.npz")
    o = oracle.paged_block_attn(bf16(p["q"]), bf16(p["k_cache"]), bf16(p["v_cache"]), torch.from_numpy(p["block_table"]),
                                torch.from_numpy(p["context_lens"]), 1 / math.sqrt(128))
    assert np.allclose(o.float().numpy(), p["o"], atol=1e-5)
    assert np.all(p["o"][1] == 0)                                # the padding row


def test_oracle_reproduces_store_and_unmask_fixtures():
    f = load("store_kvcache.npz")
    hkv = int(f["hkv"])
    n = f["fused"].shape[0]
    key = f["fused"][:, :hkv * 128].reshape(n, hkv, 128)
    val = f["fused"][:, 2 * hkv * 128:].reshape(n, hkv, 128)
    kc, vc = f["k_cache"].copy(), f["v_cache"].copy()
    oracle.store_kvcache(key, val, kc, vc, f["slot_mapping"])
    assert np.array_equal(kc, f["k_after"]) and np.array_equal(vc, f["v_after"])
    u = load("unmask_step.npz")
    x0, x0_p, transfer, after = oracle.unmask_step(bf16(u["logits"]).float().numpy(), u["tokens"], int(u["mask_id"]),
                                                   float(u["threshold"]), int(u["k"]), temperatures=u["temperatures"])
    assert np.array_equal(x0, u["x0"]) and np.allclose(x0_p, u["x0_p"], rtol=1e-6)
    assert np.array_equal(transfer.astype(np.uint8), u["transfer"]) and np.array_equal(after, u["tokens_after"])
    # the fixture covers both branches of the rule: a row set above the threshold and top-k rows
    assert u["count"].tolist() == [4, int(u["transfer"][1].sum()), 3] and u["count"][1] > 4


def test_oracle_reproduces_layer_op_fixtures():
    f = load("layer_ops.npz")
    y, nr = oracle.add_rms_norm(bf16(f["x"]), bf16(f["residual"]), bf16(f["weight"]), float(f["eps"]))
    assert torch.equal(y, bf16(f["normed"])) and torch.equal(nr, bf16(f["new_residual"]))
    assert torch.equal(oracle.add_rms_norm(bf16(f["x"]), None, bf16(f["weight"]), float(f["eps"]))[0], bf16(f["normed_no_residual"]))
    assert torch.equal(oracle.silu_and_mul(bf16(f["gate_up"])), bf16(f["act"]))


def test_oracle_reproduces_sampling_and_block_state_fixtures():
    f = load("sampling.npz")
    x = bf16(f["logits"]).to(torch.float64).numpy().reshape(8, -1)
    T8 = np.repeat(f["temperatures"].astype(np.float64), 4)
    filt = oracle.filter_logits(x, top_k=int(f["top_k"]), top_p=float(f["top_p"]), temperatures=T8)
    assert np.array_equal(np.isfinite(filt).astype(np.uint8), f["kept"])
    assert 1 <= f["kept"].sum(1).min() and f["kept"].sum(1).max() <= int(f["top_k"])
    noise = oracle.gumbel_noise(8, x.shape[1], int(f["seed"]), int(f["offset"]))
    assert np.array_equal(noise.astype(np.float32), f["noise"])
    x0, p = oracle.confidence_argmax(filt.reshape(2, 4, -1), f["temperatures"], noise.reshape(2, 4, -1))
    assert np.array_equal(x0, f["x0"]) and np.allclose(p, f["x0_p"], rtol=1e-6)
    assert f["kept"].reshape(2, 4, -1)[np.arange(2)[:, None], np.arange(4)[None], x0].all()      # every drawn token survived the filter
    b = load("block_state.npz")
    pos, slots, ctx = oracle.block_prepare(b["lens"], b["phase"], b["block_table"], int(b["page"]), int(b["block_len"]))
    assert np.array_equal(pos, b["positions"]) and np.array_equal(slots, b["slot_mapping"]) and np.array_equal(ctx, b["context_lens"])
    rows, n = oracle.masked_rows(b["tokens"], b["phase"], int(b["mask_id"]), len(b["rows"]))
    assert np.array_equal(rows, b["rows"]) and n == int(b["n_rows"])
    tok, smap, step, phase, lens, appended, status = oracle.block_advance(
        b["tokens_selected"], b["transfer"], b["step_map"], b["step"], b["phase"], b["lens"], b["first_len"], b["max_new"],
        b["stop_ids"], int(b["mask_id"]))
    assert np.array_equal(tok, b["tokens_after"]) and np.array_equal(smap, b["step_map_after"]) and np.array_equal(step, b["step_after"])
    assert np.array_equal(phase, b["phase_after"]) and np.array_equal(lens, b["lens_after"])
    # the fixture walks every transition: denoising -> caching, caching -> idle by stop token and by budget, idle stays idle
    assert b["phase"].tolist() == [1, 2, 1, 0, 2] and b["phase_after"].tolist() == [2, 0, 1, 0, 0]


def test_oracle_reproduces_fused_head_fixture():
    f = load("lm_head.npz")
    x, w = bf16(f["x"]), bf16(f["w"])
    logits = (x.float() @ w.float().T).bfloat16().to(torch.float64).numpy()
    rpt = int(f["rows_per_temp"])
    x0, p = oracle.confidence_argmax(logits.reshape(-1, rpt, logits.shape[1]), f["temperatures"])
    assert np.array_equal(x0.reshape(-1), f["x0"]) and np.allclose(p.reshape(-1), f["x0_p"], rtol=1e-12)
    # independent of the oracle: argmax / softmax by torch on the same exact logits, and the forced tie resolves to the lower index
    t = torch.from_numpy(logits) / torch.from_numpy(f["temperatures"].astype(np.float32)).double().repeat_interleave(rpt)[:, None]
    assert np.array_equal(torch.argmax(t, -1).numpy(), f["x0"])
    np.testing.assert_allclose(torch.softmax(t, -1).max(-1).values.numpy(), f["x0_p"], rtol=1e-6)
    assert 250 not in f["x0"].tolist()


# ----------------------------------------------------------------------------- GPU: HIP path == fixtures
@pytest.mark.gpu
def test_hip_sampling_matches_fixtures(dev):
    import mdx
    f = load("sampling.npz")
    logits = bf16(f["logits"]).to(dev)
    temps = torch.from_numpy(f["temperatures"]).to(dev)
    V = logits.shape[-1]
    filt = mdx.filter_logits(logits, top_k=int(f["top_k"]), top_p=float(f["top_p"]), temperatures=temps)
    assert np.array_equal(torch.isfinite(filt.float()).cpu().numpy().reshape(8, V).astype(np.uint8), f["kept"])
    assert torch.equal(filt[torch.isfinite(filt.float())], logits[torch.isfinite(filt.float())])
    noise = mdx.gumbel_noise(8, V, int(f["seed"]), int(f["offset"]), device=dev)
    np.testing.assert_allclose(noise.cpu().numpy(), f["noise"], rtol=0, atol=3e-6)
    x0, p = mdx.confidence_argmax(filt, temps, seed=int(f["seed"]), offset=int(f["offset"]))
    assert np.array_equal(x0.cpu().numpy(), f["x0"])
    np.testing.assert_allclose(p.cpu().numpy(), f["x0_p"], rtol=3e-5)


@pytest.mark.gpu
def test_hip_block_state_matches_fixtures(dev):
    import mdx
    b = load("block_state.npz")
    L = mdx.lib()
    stream = torch.cuda.current_stream().cuda_stream
    d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)      # noqa: E731
    bs, S, width = len(b["lens"]), int(b["block_len"]), b["block_table"].shape[1]
    lens, phase, bt = d(b["lens"]), d(b["phase"]), d(b["block_table"])
    pos = torch.empty(bs, S, dtype=torch.int64, device=dev)
    slots = torch.empty(bs, S, dtype=torch.int32, device=dev)
    ctx = torch.empty(bs, dtype=torch.int32, device=dev)
    assert L.mdx_block_prepare(lens.data_ptr(), phase.data_ptr(), bt.data_ptr(), width, width, int(b["page"]), S,
                               pos.data_ptr(), slots.data_ptr(), ctx.data_ptr(), bs, stream) == 0
    assert np.array_equal(pos.cpu().numpy(), b["positions"]) and np.array_equal(slots.cpu().numpy(), b["slot_mapping"])
    assert np.array_equal(ctx.cpu().numpy(), b["context_lens"])
    cap = len(b["rows"])
    rows = torch.empty(cap, dtype=torch.int64, device=dev)
    n = torch.empty(1, dtype=torch.int32, device=dev)
    tok = d(b["tokens"])
    assert L.mdx_masked_rows(tok.data_ptr(), phase.data_ptr(), int(b["mask_id"]), bs, S, rows.data_ptr(), cap, n.data_ptr(), stream) == 0
    assert np.array_equal(rows.cpu().numpy(), b["rows"]) and int(n.item()) == int(b["n_rows"])
    tok2, tr, smap, step = d(b["tokens_selected"]), d(b["transfer"]), d(b["step_map"]), d(b["step"])
    first, mx, stop = d(b["first_len"]), d(b["max_new"]), d(b["stop_ids"])
    out_tok = torch.full((bs, 64), -1, dtype=torch.int64, device=dev)
    out_step = torch.full((bs, 64), -1, dtype=torch.int32, device=dev)
    status = torch.zeros(bs, 4, dtype=torch.int32, device=dev)
    assert L.mdx_block_advance(tok2.data_ptr(), tr.data_ptr(), smap.data_ptr(), step.data_ptr(), phase.data_ptr(), lens.data_ptr(),
                               first.data_ptr(), mx.data_ptr(), stop.data_ptr(), stop.shape[1], out_tok.data_ptr(), out_step.data_ptr(),
                               64, status.data_ptr(), int(b["mask_id"]), bs, S, stream) == 0
    torch.cuda.synchronize()
    live = b["phase"] != 0
    assert np.array_equal(tok2.cpu().numpy(), b["tokens_after"]) and np.array_equal(smap.cpu().numpy(), b["step_map_after"])
    assert np.array_equal(step.cpu().numpy()[live], b["step_after"][live])
    assert np.array_equal(phase.cpu().numpy(), b["phase_after"]) and np.array_equal(lens.cpu().numpy(), b["lens_after"])
    assert np.array_equal(out_tok.cpu().numpy(), b["out_tokens"]) and np.array_equal(out_step.cpu().numpy(), b["out_steps"])
    st = status.cpu().numpy()
    assert np.array_equal(st[live], b["status"][live]) and st[~live][:, 0].tolist() == [0] * int((~live).sum())
@pytest.mark.gpu
def test_hip_attention_matches_fixtures(dev):
    import mdx
    f = load("staircase_attn.npz")
    cu = torch.from_numpy(f["cu"]).to(dev)
    o = mdx.sparse_attn_varlen(bf16(f["q"]).to(dev), bf16(f["k"]).to(dev), bf16(f["v"]).to(dev), cu, cu, staircase_size=int(f["block"]))
    assert np.abs(o.float().cpu().numpy() - f["o"]).max() < TOL
    p = load("paged_block_attn.npz")
    o = mdx.flash_attn_with_kvcache(bf16(p["q"]).to(dev), bf16(p["k_cache"]).to(dev), bf16(p["v_cache"]).to(dev),
                                    cache_seqlens=torch.from_numpy(p["context_lens"]).to(dev),
                                    block_table=torch.from_numpy(p["block_table"]).to(dev), softmax_scale=1 / math.sqrt(128), causal=False)
    assert np.abs(o.float().cpu().numpy() - p["o"]).max() < TOL
    assert o[1].abs().sum().item() == 0


@pytest.mark.gpu
def test_hip_store_and_unmask_match_fixtures(dev):
    import mdx
    f = load("store_kvcache.npz")
    hkv = int(f["hkv"])
    fused = bf16(f["fused"]).to(dev)
    n = fused.shape[0]
    key = fused[:, :hkv * 128].reshape(n, hkv, 128).contiguous()
    val = fused[:, 2 * hkv * 128:].unflatten(1, (hkv, 128))       # strided view, as in the engine
    kc, vc = bf16(f["k_cache"]).to(dev), bf16(f["v_cache"]).to(dev)
    mdx.store_kvcache(key, val, kc, vc, torch.from_numpy(f["slot_mapping"]).to(dev))
    assert torch.equal(kc.cpu(), bf16(f["k_after"])) and torch.equal(vc.cpu(), bf16(f["v_after"]))
    u = load("unmask_step.npz")
    tokens = torch.from_numpy(u["tokens"]).to(dev)
    x0, x0_p, transfer, count = mdx.unmask_step(bf16(u["logits"]).to(dev), tokens, int(u["mask_id"]), float(u["threshold"]), int(u["k"]),
                                                temperatures=torch.from_numpy(u["temperatures"]).to(dev))
    masked = u["tokens"] == int(u["mask_id"])
    assert np.array_equal(x0.cpu().numpy(), u["x0"])
    assert np.allclose(x0_p.cpu().numpy(), u["x0_p"], rtol=2e-5)
    assert np.array_equal(transfer.cpu().numpy().astype(np.uint8), u["transfer"])
    assert np.array_equal(tokens.cpu().numpy(), u["tokens_after"]) and np.array_equal(count.cpu().numpy(), u["count"])
    assert masked.any()


@pytest.mark.gpu
def test_hip_layer_ops_match_fixtures(dev):
    import mdx
    f = load("layer_ops.npz")
    y, nr = mdx.rms_norm(bf16(f["x"]).to(dev), bf16(f["weight"]).to(dev), float(f["eps"]), bf16(f["residual"]).to(dev))
    assert torch.equal(nr.cpu(), bf16(f["new_residual"]))
    for got, want in ((y, f["normed"]), (mdx.rms_norm(bf16(f["x"]).to(dev), bf16(f["weight"]).to(dev), float(f["eps"])), f["normed_no_residual"]),
                      (mdx.silu_and_mul(bf16(f["gate_up"]).to(dev)), f["act"])):
        w = bf16(want).float()
        diff = (got.float().cpu() - w).abs()
        assert (diff <= w.abs() * 2 ** -7 + 1e-30).all() and (diff == 0).float().mean() > 0.97


@pytest.mark.gpu
def test_hip_fused_head_matches_fixture(dev):
    import mdx
    f = load("lm_head.npz")
    x0, p = mdx.lm_head_confidence(bf16(f["x"]).to(dev), bf16(f["w"]).to(dev), torch.from_numpy(f["temperatures"]).to(dev),
                                   rows_per_temp=int(f["rows_per_temp"]))
    assert np.array_equal(x0.cpu().numpy(), f["x0"])
    np.testing.assert_allclose(p.cpu().numpy(), f["x0_p"], rtol=3e-5)
