"""Builds libmdx.so (the HIP kernels + C ABI) for gfx950 with hipcc, in-tree.

Usage: python build.py [--force]
The library lands next to the Python package (mdx/libmdx.so) so that it travels
with the source tree; nothing is installed.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

ROOT = Path(__file__).resolve().parent
CSRC = ROOT / "csrc"
OBJ = ROOT / "build"
LIB = ROOT / "mdx" / "libmdx.so"

SOURCES = ["mdx_api.hip", "store_kvcache.hip", "unmask.hip", "logit_filter.hip", "staircase_attn.hip", "staircase_attn_f32.hip", "paged_attn.hip", "paged_attn_f32.hip", "paged_attn_static.hip", "qk_norm_rope_store.hip", "layer_ops.hip", "block_state.hip", "lm_head_unmask.hip", "calib_probe.hip"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # hipcc -O3 forms packed fp32 ops on its own; they are kept out of every kernel here.
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-attributes",
]


def _compile(src: str) -> Path:
    obj = OBJ / (src.rsplit(".", 1)[0] + ".o")
    cmd = [HIPCC, *FLAGS, "-c", str(CSRC / src), "-o", str(obj)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in r.stderr.splitlines() if noise not in l and l.strip() != "1 warning generated when compiling for host.")
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        print(err, file=sys.stderr)
    return obj


def build_all(verbose: bool = True) -> Path:
    """Compiles every HIP source and links libmdx.so; always recompiles."""
    OBJ.mkdir(exist_ok=True)
    srcs = [s for s in SOURCES if (CSRC / s).exists()]
    missing = [s for s in SOURCES if not (CSRC / s).exists()]
    if missing:
        raise RuntimeError(f"missing sources: {missing}")
    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        objs = list(ex.map(_compile, srcs))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB), *map(str, objs)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr}")
    if verbose:
        print(f"built {LIB} ({LIB.stat().st_size} bytes) from {len(srcs)} sources")
    return LIB


if __name__ == "__main__":
    build_all()
