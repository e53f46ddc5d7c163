"""The C ABI without a GPU: the library loads, exports every symbol include/mdx.h declares,
and refuses bad arguments before launching anything."""
import ctypes
import re
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent


@pytest.fixture(scope="module")
def L():
    import mdx
    if not mdx.library_path().exists():
        from importlib import import_module
        import sys
        sys.path.insert(0, str(ROOT))
        import_module("__graft_entry__").build()
    return mdx.lib()


def _declared():
    text = (ROOT / "include" / "mdx.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mdx_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree(L):
    from mdx import _lib
    names = _declared()
    assert names, "no declarations found in include/mdx.h"
    assert sorted(_lib.SIGNATURES) == names
    for n in names:
        assert hasattr(L, n), f"libmdx.so does not export {n}"


def test_version_matches_header(L):
    text = (ROOT / "include" / "mdx.h").read_text()
    assert L.mdx_version() == int(re.search(r"#define MDX_VERSION (\d+)", text).group(1))


def test_workspace_queries_are_pure_host_arithmetic(L):
    assert L.mdx_confidence_argmax_workspace_bytes(1024, 151936) == 0 or \
        L.mdx_confidence_argmax_workspace_bytes(1024, 151936) % 24 == 0
    few = L.mdx_confidence_argmax_workspace_bytes(32, 151936)
    assert few > 0 and few % (32 * 24) == 0            # small batches split rows over workgroups
    ws = L.mdx_paged_block_attn_workspace_bytes(16, 32, 16, 8, 128, 17, 256)
    assert ws > 16 and (ws - 16) % (16 * 16 * 32 * 130 * 4) == 0      # partial slots + the split-size word
    assert L.mdx_paged_block_attn_workspace_bytes(0, 32, 16, 8, 128, 17, 256) == 0


def test_bad_arguments_are_refused_without_a_launch(L):
    null = None
    one = ctypes.c_void_p(16)     # never dereferenced: every call below must fail validation first
    assert L.mdx_store_kvcache(null, null, 0, 0, null, null, null, 5, 1024, 2, 10, null) == -1
    assert b"null" in L.mdx_last_error()
    assert L.mdx_store_kvcache(one, one, 0, 0, one, one, one, 5, 1024, 3, 10, null) == -2
    assert L.mdx_store_kvcache(null, null, 0, 0, null, null, null, 0, 1024, 2, 10, null) == 0   # empty: no-op
    sa = lambda **kw: L.mdx_staircase_attn_varlen(                                            # noqa: E731
        one, one, one, one, 2048, 128, 1024, 128, 1024, 128, 2048, 128, one, one, 1, 100, 100,
        kw.get("hq", 16), kw.get("hkv", 8), kw.get("d", 128), kw.get("S", 32), kw.get("scale", 0.1), kw.get("dtype", 0), null)
    assert sa(d=260) == -2 and b"head_dim" in L.mdx_last_error()    # up to 256 columns (above 128: the fp32-arithmetic kernel)
    assert sa(d=70) == -2 and b"head_dim" in L.mdx_last_error()     # multiples of 4 only
    assert sa(S=48) == -1 and b"staircase_size" in L.mdx_last_error()
    assert sa(hq=12) == -1
    assert sa(dtype=3) == -2 and b"dtype" in L.mdx_last_error()     # bf16, fp16 and fp32 are the element types
    assert sa(scale=-1.0) == -1
    pa = lambda **kw: L.mdx_paged_block_attn(                                                  # noqa: E731
        one, one, one, one, 65536, 2048, 128, 65536, 2048, 128, 262144, 1024, 128, one, 17, one,
        4, kw.get("sq", 32), 16, 8, kw.get("d", 128), 17, kw.get("page", 256), 100, 0.1, 0, kw.get("ws", null), kw.get("ws_bytes", 0), null)
    assert pa(sq=129) == -2 and b"queries per sequence" in L.mdx_last_error()    # up to four tiles of 32 queries
    assert pa(page=100) == -2
    assert pa(d=260) == -2 and b"head_dim" in L.mdx_last_error()    # up to 256 columns (above 128: the fp32-arithmetic kernel)
    assert pa(d=42) == -2                                           # multiples of 4 only
    assert L.mdx_paged_block_attn_workspace_bytes(16, 32, 16, 8, 256, 17, 256) == 0     # that kernel never splits a sequence
    assert pa() == -3 and b"workspace" in L.mdx_last_error()
    assert L.mdx_select_transfer(one, one, one, 7, 0.9, -1, one, one, 2, 32, null) == -1      # k < 0
    assert L.mdx_select_transfer(one, one, one, 7, 0.9, 1, one, one, 2, 2000, null) == -2      # block too long
    assert L.mdx_confidence_argmax(one, 10, 0, null, 1, null, 0, one, one, 4, 20, null, 0, null) == -2   # stride < vocab
    fl = lambda **kw: L.mdx_filter_logits(one, kw.get("stride", 100), kw.get("dtype", 0), null, 1,           # noqa: E731
                                          kw.get("k", 5), kw.get("p", 0.9), one, 100, kw.get("rows", 4), 100, null)
    assert fl(dtype=2) == -2 and b"16-bit" in L.mdx_last_error()      # fp32 logits: the cut-off is found by counting 16-bit values
    assert fl(k=-1) == -1 and fl(p=-0.5) == -1 and fl(p=float("nan")) == -1
    assert fl(stride=50) == -2
    assert fl(rows=0) == 0
    # the single-launch paged call: with about a pair per CU (32 sequences x 8 head groups) it needs the counters
    big = ctypes.c_void_p(1 << 20)
    ws32 = L.mdx_paged_block_attn_workspace_bytes(32, 32, 16, 8, 128, 17, 256)
    sl = lambda counters, nbytes: L.mdx_paged_block_attn_single_launch(                          # noqa: E731
        one, one, one, one, 65536, 2048, 128, 65536, 2048, 128, 262144, 1024, 128, one, 17, one,
        32, 32, 16, 8, 128, 17, 256, 100, 0.1, 0, big, ws32, counters, nbytes, null)
    # one counter per (sequence, head group, query tile), sized for the longest block (four tiles of 32 queries)
    assert ws32 > 0 and L.mdx_paged_block_attn_counter_bytes(32, 16, 8) == 32 * 8 * 4 * 4
    assert sl(null, 0) == -3 and b"counters" in L.mdx_last_error()
    assert sl(one, 32 * 8 * 4 - 4) == -3
    assert sl(ctypes.c_void_p(18), 4096) == -3 and b"aligned" in L.mdx_last_error()


def test_fused_head_and_calibration_arguments_are_validated(L):
    null = None
    one = ctypes.c_void_p(16)
    ws = L.mdx_lm_head_confidence_workspace_bytes(1024, 151936)
    assert ws == 1024 * 1188 * 16 and L.mdx_lm_head_confidence_workspace_bytes(0, 151936) == 0     # one record per row and 128-entry slice
    big = ctypes.c_void_p(1 << 20)
    head = lambda **kw: L.mdx_lm_head_confidence(                                                   # noqa: E731
        kw.get("x", one), kw.get("xs", 2048), one, 2048, null, 1, null, one, one, kw.get("rows", 1024), 151936, kw.get("hidden", 2048),
        kw.get("ws", big), kw.get("ws_bytes", ws), null)
    assert head(x=null) == -1 and b"null" in L.mdx_last_error()
    assert head(hidden=2000) == -2 and b"hidden" in L.mdx_last_error()
    assert head(xs=2047) == -2
    assert head(ws_bytes=ws - 16) == -3 and b"workspace" in L.mdx_last_error()
    assert head(rows=0) == 0
    assert L.mdx_calib_mfma_loop(7, one, one, 4, 8, null) == -1
    assert L.mdx_calib_mfma_loop(32, null, one, 4, 8, null) == -1
    assert L.mdx_calib_mfma_loop_flops(32, 256, 8) == 256 * 4 * 8 * 8 * 32 * 32 * 16 * 2
    assert L.mdx_calib_mfma_loop_flops(16, 256, 3) == 256 * 4 * 8 * 16 * 16 * 16 * 32 * 2              # iterations rounded up to 8


def test_ops_fail_loudly_off_gpu():
    import torch
    import mdx
    x = torch.zeros(4, 8, 128, dtype=torch.bfloat16)
    with pytest.raises(mdx.MdxError):
        mdx.store_kvcache(x, x, torch.zeros(1, 256, 8, 128, dtype=torch.bfloat16),
                          torch.zeros(1, 256, 8, 128, dtype=torch.bfloat16), torch.zeros(4, dtype=torch.int32))
    with pytest.raises(mdx.MdxError):
        mdx.sparse_attn_varlen(x, x, x, torch.tensor([0, 4], dtype=torch.int32), torch.tensor([0, 4], dtype=torch.int32), 32)


def test_context_mirror():
    import mdx
    mdx.set_context(True, max_seqlen_q=5, block_size=32)
    assert mdx.get_context().is_prefill and mdx.get_context().max_seqlen_q == 5
    mdx.reset_context()
    assert not mdx.get_context().is_prefill and mdx.get_context().slot_mapping is None


def test_generated_kernel_core_is_current():
    """staircase_pair_core.inc, its fp16 twin and lm_head_core.inc are the committed outputs of their generators: regenerate and compare."""
    import subprocess
    import sys
    from pathlib import Path
    csrc = Path(__file__).resolve().parents[1] / "mineru-diffusion_amd" / "csrc"
    out = subprocess.run([sys.executable, str(csrc / "gen_staircase_pair_core.py")], capture_output=True, text=True, check=True)
    assert out.stdout == (csrc / "staircase_pair_core.inc").read_text()
    out = subprocess.run([sys.executable, str(csrc / "gen_staircase_pair_core.py"), "f16"], capture_output=True, text=True, check=True)
    assert out.stdout == (csrc / "staircase_pair_core_f16.inc").read_text()
    # the core of the fused vocabulary projection
    out = subprocess.run([sys.executable, str(csrc / "gen_lm_head_core.py")], capture_output=True, text=True, check=True)
    assert out.stdout == (csrc / "lm_head_core.inc").read_text()
