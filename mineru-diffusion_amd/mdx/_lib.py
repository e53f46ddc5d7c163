"""ctypes binding of libmdx.so (C ABI declared in include/mdx.h)."""
from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_float, c_int32, c_int64, c_uint64, c_void_p
from pathlib import Path

_HERE = Path(__file__).resolve().parent

MDX_BF16, MDX_F16, MDX_F32 = 0, 1, 2


class MdxError(RuntimeError):
    """A libmdx entry point refused its arguments (nothing was launched)."""


def library_path() -> Path:
    return _HERE / "libmdx.so"


# name -> (restype, argtypes); mirrors include/mdx.h one to one
_P, _I32, _I64, _F, _U64 = c_void_p, c_int32, c_int64, c_float, c_uint64
SIGNATURES = {
    "mdx_version": (c_int32, []),
    "mdx_last_error": (c_char_p, []),
    "mdx_store_kvcache": (c_int32, [_P, _P, _I64, _I64, _P, _P, _P, _I64, _I64, _I32, _I64, _P]),
    "mdx_staircase_attn_varlen": (c_int32, [_P, _P, _P, _P] + [_I64] * 8 + [_P, _P, _I32, _I32, _I64,
                                                                           _I32, _I32, _I32, _I32, _F, _I32, _P]),
    "mdx_paged_block_attn_workspace_bytes": (c_int64, [_I32] * 7),
    "mdx_paged_block_attn": (c_int32, [_P, _P, _P, _P] + [_I64] * 9 + [_P, _I64, _P] + [_I32] * 7 + [_I64, _F, _I32,
                                                                                                      _P, _I64, _P]),
    "mdx_paged_block_attn_counter_bytes": (c_int64, [_I32] * 3),
    "mdx_paged_block_attn_single_launch": (c_int32, [_P, _P, _P, _P] + [_I64] * 9 + [_P, _I64, _P] + [_I32] * 7 + [_I64, _F, _I32,
                                                                                                                    _P, _I64, _P, _I64, _P]),
    "mdx_paged_block_attn_static": (c_int32, [_P, _P, _P, _P] + [_I64] * 9 + [_P, _I64, _P] + [_I32] * 7 + [_I64, _F, _I32, _P]),
    "mdx_confidence_argmax_workspace_bytes": (c_int64, [_I64, _I64]),
    "mdx_confidence_argmax": (c_int32, [_P, _I64, _I32, _P, _I32, _P, _I64, _P, _P, _I64, _I64, _P, _I64, _P]),
    "mdx_confidence_argmax_gumbel": (c_int32, [_P, _I64, _I32, _P, _I32, _U64, _U64, _P, _P, _P, _P, _I64, _I64, _P, _I64, _P]),
    "mdx_unmask_step_gumbel": (c_int32, [_P, _I64, _I32, _P, _U64, _U64, _P, _P, _P, _I64, _F, _I32, _P, _P, _P, _P,
                                         _I32, _I32, _I64, _P, _I64, _P]),
    "mdx_gumbel_noise": (c_int32, [_P, _I64, _I64, _I64, _U64, _U64, _P, _P, _P]),
    "mdx_select_transfer": (c_int32, [_P, _P, _P, _I64, _F, _I32, _P, _P, _I32, _I32, _P]),
    "mdx_qk_norm_rope_store": (c_int32, [_P, _I64, _P, _P, _F, _P, _P, _I64, _P, _P, _I64, _P, _I64, _P, _P, _P, _I64,
                                         _I64, _I32, _I32, _I32, _I32, _P]),
    "mdx_add_rms_norm": (c_int32, [_P, _I64, _P, _I64, _P, _I64, _P, _F, _P, _I64, _I64, _I32, _I32, _P]),
    "mdx_silu_and_mul": (c_int32, [_P, _I64, _P, _I64, _I64, _I32, _I32, _P]),
    "mdx_block_prepare": (c_int32, [_P, _P, _P, _I64, _I32, _I32, _I32, _P, _P, _P, _I32, _P]),
    "mdx_masked_rows": (c_int32, [_P, _P, _I64, _I32, _I32, _P, _I32, _P, _P]),
    "mdx_block_advance": (c_int32, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _I32, _P, _P, _I64, _P, _I64, _I32, _I32, _P]),
    "mdx_filter_logits": (c_int32, [_P, _I64, _I32, _P, _I32, _I32, _F, _P, _I64, _I64, _I64, _P]),
    "mdx_lm_head_confidence_workspace_bytes": (c_int64, [_I64, _I64]),
    "mdx_lm_head_confidence": (c_int32, [_P, _I64, _P, _I64, _P, _I32, _P, _P, _P, _I64, _I64, _I64, _P, _I64, _P]),
    "mdx_calib_mfma_loop_flops": (c_int64, [_I32, _I32, _I32]),
    "mdx_calib_mfma_loop": (c_int32, [_I32, _P, _P, _I32, _I32, _P]),
    "mdx_unmask_step": (c_int32, [_P, _I64, _I32, _P, _P, _I64, _P, _I64, _F, _I32, _P, _P, _P, _P,
                                  _I32, _I32, _I64, _P, _I64, _P]),
}

_lib = None


def lib() -> ctypes.CDLL:
    """The loaded library; raises if it has not been built (no fallback path exists)."""
    global _lib
    if _lib is None:
        path = library_path()
        if not path.exists():
            raise MdxError(f"{path} is missing: build it with `python mineru-diffusion_amd/build.py` "
                           "(hipcc, gfx950); there is no non-HIP fallback")
        handle = ctypes.CDLL(str(path))
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = lib().mdx_last_error()
        raise MdxError(f"{what} failed ({rc}): {msg.decode() if msg else ''}")
