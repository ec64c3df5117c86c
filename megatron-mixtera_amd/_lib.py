"""ctypes binding of ``libmi355_decode.so`` (the C ABI declared in ``include/mi355_decode.h``).

The library is the product path: when it is missing every op raises -- there is no
eager / CPU fallback behind these functions.
"""
from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_float, c_int, c_int32, c_int64, c_void_p
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
LIB_PATH = PKG_DIR / "libmi355_decode.so"

MI_DTYPE_BF16, MI_DTYPE_FP16 = 0, 1
MI_KV_16BIT, MI_KV_BF16, MI_KV_FP8_E4M3 = 0, 0, 1
MI_NORM_NONE, MI_NORM_RMS, MI_NORM_L2 = 0, 1, 2


class MiTuning(ctypes.Structure):
    """Per-call experiment knobs (``MiTuning`` of the header); all zero = the defaults."""
    _fields_ = [(name, c_int32) for name in (
        "decode_tile_subtiles", "decode_min_waves", "decode_wgs_per_cu", "decode_grid", "decode_waves_per_block",
        "prefill_two_phase", "prefill_tile_subtiles", "prefill_row_tiles", "prefill_kv_split",
        "norm_rope_vectorised", "mla_decode_lds")] + [("reserved", c_int32 * 5)]


_P, _I32, _I64, _F = c_void_p, c_int32, c_int64, c_float

# name -> (restype, argtypes); mirrors include/mi355_decode.h declaration by declaration.
SIGNATURES = {
    "mi_version": (c_int, []),
    "mi_last_error": (c_char_p, []),
    "mi_profile_enable": (c_int, [_I32]),
    "mi_profile_collect": (_I32, [_P, _I32]),
    "mi_kv_append": (c_int, [_P, _P, _I64, _P, _P, _I64, _I64, _P, _P, _I32, _I32, _I32, _P]),
    "mi_kv_append_decode": (
        c_int, [_P, _P, _I64, _P, _P, _I64, _I64, _P, _I64, _P, _I32, _I32, _I32, _I32, _P]),
    "mi_kv_quantize_chunks_fp8": (
        c_int, [_P, _I64, _I64, _P, _I64, _I64, _P, _I32, _I32, _I32, _I32, _I32, _P]),
    "mi_kv_append_decode_fp8": (
        c_int, [_P, _P, _I64, _P, _P, _I64, _I64, _P, _P, _P, _I64, _P, _I32, _I32, _I32, _I32, _F, _I32, _P]),
    "mi_kv_append_fp8": (
        c_int, [_P, _P, _I64, _P, _P, _I64, _I64, _P, _P, _P, _P, _I32, _I32, _I32, _I32, _F, _I32, _P]),
    "mi_decode_workspace_bytes": (_I64, [_I32, _I32, _I32, _I32, _I32, _I32, _I32, _P]),
    "mi_paged_decode_attention": (
        c_int,
        [_P, _I64, _I64, _P, _P, _I64, _I64, _I64, _P, _I64, _P, _P, _I64, _I64, _P, _I64,
         _I32, _I32, _I32, _I32, _I32, _I32, _I32, _F, _I32, _P, _P, _I32, _P, _P]),
    "mi_decode_step_attention": (
        c_int,
        [_P, _I64, _I64, _P, _I64, _I64, _P, _I64, _I64, _P, _P, _F, _I32, _P, _I64, _I32, _I32, _F, _P, _P, _P,
         _I64, _I64, _I64, _P, _I64, _P, _P, _I64, _I64, _P, _I64, _I32, _I32, _I32, _I32, _I32, _I32, _F, _I32,
         _I32, _P, _P]),
    "mi_decode_step_attention_fp8": (
        c_int,
        [_P, _I64, _I64, _P, _I64, _I64, _P, _I64, _I64, _P, _P, _F, _I32, _P, _I64, _I32, _I32, _F, _P, _P, _P,
         _I64, _I64, _I64, _P, _P, _F, _P, _I64, _P, _P, _I64, _I64, _P, _I64, _I32, _I32, _I32, _I32, _I32, _I32, _F,
         _I32, _I32, _P, _P]),
    "mi_paged_decode_attention_noalloc": (
        c_int,
        [_P, _I64, _I64, _P, _P, _I64, _I64, _I64, _P, _I64, _P, _P, _I64, _I64,
         _I32, _I32, _I32, _I32, _I32, _I32, _I32, _F, _I32, _P, _P, _I32, _P, _P]),
    "mi_mla_decode_workspace_bytes": (_I64, [_I32, _I32, _I32, _P]),
    "mi_paged_mla_decode_attention": (
        c_int, [_P, _I64, _I64, _P, _I64, _I64, _P, _I64, _P, _P, _I64, _I64, _P, _I64,
                _I32, _I32, _I32, _I32, _I32, _I32, _F, _I32, _P, _P]),
    "mi_prefill_workspace_bytes": (_I64, [_I32, _I32, _I32, _I32, _I32, _I32, _I32, _P]),
    "mi_paged_prefill_attention": (
        c_int,
        [_P, _I64, _I64, _P, _P, _I64, _I64, _I64, _P, _I64, _P, _P, _P, _I64, _I64, _P, _I64,
         _I32, _I32, _I32, _I32, _I32, _I32, _I32, _I32, _F, _I32, _P, _P]),
    "mi_paged_prefill_attention_fp8": (
        c_int,
        [_P, _I64, _I64, _P, _P, _I64, _I64, _I64, _P, _P, _P, _I64, _P, _P, _P, _I64, _I64, _P, _I64,
         _I32, _I32, _I32, _I32, _I32, _I32, _I32, _I32, _F, _I32, _P, _P]),
    "mi_paged_prefill_attention_mla": (
        c_int,
        [_P, _I64, _I64, _P, _I64, _I64, _I64, _P, _I64, _I64, _I64, _P, _I64, _P, _P, _P, _I64, _I64,
         _P, _I64, _I32, _I32, _I32, _I32, _I32, _I32, _I32, _I32, _F, _I32, _P, _P]),
    "mi_update_requests": (
        c_int, [_P] * 8 + [_I64, _I32] + [_P] * 15 + [_I32] * 7 + [_P]),
    "mi_step_attention_state": (
        c_int, [_P, _P, _P, _I64, _I32, _P, _P, _P, _P, _P, _I64, _P, _P, _P, _P] + [_I32] * 6 + [_P]),
    "mi_add_request": (c_int, [_P] * 8 + [_I64] + [_P] * 8 + [_I32] * 8 + [_P]),
    "mi_decode_attention_state": (
        c_int, [_P, _P, _P, _I64, _I32, _P, _P, _P, _I64, _P, _P, _P, _I32, _I32, _I32, _I32, _I32, _P]),
    "mi_last_token_gather": (c_int, [_P, _I64, _P, _I64, _P, _I32, _I32, _I32, _P]),
    "mi_selected_log_probs": (c_int, [_P, _I64, _I32, _I32, _I32, _P, _P, _P]),
    "mi_sample_from_logits": (
        c_int, [_P, _I64, _I32, _I32, _I32, _I32, _F, _F, _P, _I32, _P, _P, _P, _P, _P, _I64, _P, _P]),
    "mi_norm_rope_append": (
        c_int,
        [_P, _I64, _P, _I64, _P, _I64, _P, _I64, _P, _I64, _P, _P, _F, _I32, _P, _I64, _I32, _I32, _F,
         _P, _P, _P, _P, _I64, _I64, _P, _P, _P, _I64, _P, _I32, _I32, _I32, _I32, _I32, _I32, _I32, _P, _P]),
    "mi_linear_decode_workspace_bytes": (_I64, [_I32, _I32, _I32]),
    "mi_linear_decode": (c_int, [_P, _I64, _P, _I64, _P, _P, _I64, _P, _I64, _I32, _I32, _I32, _I32, _P]),
    "mi_linear_qkv_decode_step": (
        c_int, [_P, _I64, _P, _I64, _P, _P, _I64, _P, _I64, _I32, _I32, _I32, _I32, _I32, _I32, _P]),
    "mi_attention_out_linear_proj": (
        c_int, [_P, _I64, _P, _I64, _P, _I64, _P, _I64, _I32, _I32, _I32, _I32, _I32, _P]),
    "mi_qkv_norm_rope_append": (
        c_int,
        [_P, _I64, _P, _I64, _P, _I64, _P, _P, _F, _I32, _P, _I64, _I32, _I32, _F,
         _P, _P, _P, _P, _I64, _I64, _P, _P, _P, _I64, _P, _I32, _I32, _I32, _I32, _I32, _I32, _I32, _P, _P]),
}


class LibraryMissingError(RuntimeError):
    """The HIP library has not been built (run ``__graft_entry__.build()``)."""


class KernelError(RuntimeError):
    """An entry point rejected its arguments or the launch failed."""


_lib = None


def load() -> ctypes.CDLL:
    """Load the shared library once and attach the prototypes."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise LibraryMissingError(
            f"{LIB_PATH} not found: build the HIP kernels first (python {PKG_DIR / 'build.py'}); "
            "there is no fallback path.")
    lib = ctypes.CDLL(str(LIB_PATH))
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError here means header and library disagree
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(code: int, what: str) -> None:
    if code != 0:
        msg = load().mi_last_error().decode(errors="replace")
        raise KernelError(f"{what} failed with code {code}: {msg}")
