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


# ----------------------------------------------------------------------------- GPU: HIP path == fixtures
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
