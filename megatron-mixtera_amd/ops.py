"""Torch-level wrappers over the C ABI: tensors in, raw pointers + strides out.

Each function validates what only the host can see (dtypes, devices, contiguity of
the innermost dimension), then enqueues exactly one C-ABI call on torch's current
stream.  Nothing here computes: without the HIP library these functions raise.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch
from torch import Tensor

import ctypes
import threading

from . import _lib
from ._lib import (MI_DTYPE_BF16, MI_DTYPE_FP16, MI_KV_16BIT, MI_KV_BF16, MI_KV_FP8_E4M3,  # noqa: F401
                   MI_NORM_L2, MI_NORM_NONE, MI_NORM_RMS)

_NORM_KINDS = {None: MI_NORM_NONE, "none": MI_NORM_NONE, "rms": MI_NORM_RMS, "l2": MI_NORM_L2}


def _stream(t: Tensor) -> int:
    if t.device.type != "cuda":
        raise RuntimeError(
            f"the HIP kernels need device tensors, got a tensor on {t.device}; there is no CPU path")
    return torch.cuda.current_stream(t.device).cuda_stream


def _ptr(t: Optional[Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _require(cond: bool, msg: str) -> None:
    if not cond:
        raise ValueError(msg)


def _cache_strides(cache: Tensor) -> Tuple[int, int, int]:
    """(chunk, token, head) element strides of a ``[N, C, Hkv, d]`` cache view."""
    _require(cache.dim() == 4 and cache.stride(3) == 1, "KV cache must be [N, C, Hkv, d] with contiguous d")
    return cache.stride(0), cache.stride(1), cache.stride(2)


# Split-K workspaces, one per (device, stream) and grown on demand (owned here, handed to the C ABI as caller
# memory).  Calls on one stream are ordered and may share a buffer; calls on different streams of a device may
# overlap, so each stream gets its own.
_workspaces: dict = {}
_retired_workspaces: list = []   # outgrown buffers stay alive: work already enqueued may still use them
_override_local = threading.local()   # ``use_workspace`` buffers of THIS thread (innermost last)


def _override_stack() -> list:
    stack = getattr(_override_local, "stack", None)
    if stack is None:
        stack = _override_local.stack = []
    return stack


def _workspace(device: torch.device, nbytes: int, stream: Optional[int] = None) -> Optional[Tensor]:
    """Scratch for a call on ``stream`` (the handle the caller already looked up; default: the current one)."""
    if nbytes <= 0:
        return None
    override = _override_stack()
    if override:
        ws = override[-1]
        _require(ws.device == device and ws.numel() >= nbytes, "the workspace given to use_workspace is too small")
        return ws
    key = (device, torch.cuda.current_stream(device).cuda_stream if stream is None else stream)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        if ws is not None:
            _retired_workspaces.append(ws)
            if len(_retired_workspaces) > 8:  # enqueued work may still use them: wait for it once, then let them go
                torch.cuda.synchronize(device)
                _retired_workspaces.clear()
        ws = torch.empty(max(nbytes, 2 * (0 if ws is None else ws.numel())), dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws


class use_workspace:
    """Context manager: attention calls this thread makes inside use ``buffer`` as their scratch instead of the
    per-stream one (graph capture needs a buffer that is never re-allocated).  Other threads are not affected."""

    def __init__(self, buffer: Tensor):
        self.buffer = buffer

    def __enter__(self):
        _override_stack().append(self.buffer)
        return self.buffer

    def __exit__(self, *exc):
        _override_stack().pop()
        return False


# ---------------------------------------------------------------------------------------------
# experiment knobs: the C ABI takes them per call (MiTuning); this module keeps the set that its own calls pass
# ---------------------------------------------------------------------------------------------
_TUNING_FIELDS = tuple(name for name, _ in _lib.MiTuning._fields_ if name != "reserved")
_tuning_defaults: dict = {}          # set_tuning: every thread, until changed back
_tuning_local = threading.local()    # tuning(...): this thread, inside the with block


def set_tuning(name: str, value: int) -> None:
    """Knob ``name`` (a field of ``MiTuning`` in the header) for every later call of this module; 0 = the default.
    A sweep / test hook: the library itself keeps no such state."""
    _require(name in _TUNING_FIELDS, f"unknown knob {name!r}; the knobs are {', '.join(_TUNING_FIELDS)}")
    if int(value) == 0:
        _tuning_defaults.pop(name, None)
    else:
        _tuning_defaults[name] = int(value)


class tuning:
    """``with ops.tuning(decode_grid=7, prefill_two_phase=-1): ...`` -- knobs for the calls this thread makes
    inside the block (on top of :func:`set_tuning`)."""

    def __init__(self, **knobs: int):
        for name in knobs:
            _require(name in _TUNING_FIELDS, f"unknown knob {name!r}")
        self.knobs = {k: int(v) for k, v in knobs.items()}

    def __enter__(self):
        stack = getattr(_tuning_local, "stack", None)
        if stack is None:
            stack = _tuning_local.stack = []
        stack.append(self.knobs)
        return self

    def __exit__(self, *exc):
        _tuning_local.stack.pop()
        return False


def current_tuning() -> dict:
    """The knobs a call made now would pass (name -> non-zero value)."""
    merged = dict(_tuning_defaults)
    for layer in getattr(_tuning_local, "stack", None) or ():
        merged.update(layer)
    return {k: v for k, v in merged.items() if v != 0}


def _tuning_arg():
    """``const MiTuning*`` for a C call: NULL when every knob is at its default."""
    knobs = current_tuning()
    return ctypes.byref(_lib.MiTuning(**knobs)) if knobs else None


_DTYPE_CODES = {torch.bfloat16: MI_DTYPE_BF16, torch.float16: MI_DTYPE_FP16}


_LOGIT_CODES = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}


def _dtype_code(t: Tensor, name: str) -> int:
    _require(t.dtype in _DTYPE_CODES, f"{name} must be bf16 or fp16, got {t.dtype}")
    return _DTYPE_CODES[t.dtype]


# ---------------------------------------------------------------------------------------------
# KV append
# ---------------------------------------------------------------------------------------------
def _rows(x: Tensor, name: str) -> Tuple[Tensor, int, int]:
    """View ``[T, (1,) Hkv, d]`` as T rows of Hkv*d contiguous elements."""
    if x.dim() == 4:
        _require(x.size(1) == 1, f"{name}.size(1) must be 1")
        x = x.squeeze(1)
    _require(x.dim() == 3, f"{name} must be [T, Hkv, d]")
    _require(x.stride(2) == 1 and x.stride(1) == x.size(2), f"{name} rows must be contiguous")
    return x, x.size(1) * x.size(2), x.stride(0)


def kv_append(key: Tensor, value: Optional[Tensor], k_cache: Tensor, v_cache: Optional[Tensor],
              token_to_chunk_idx: Tensor, token_to_local_pos: Tensor) -> None:
    """``k_cache[chunk_idx[t], local[t]] = key[t]`` (and value): bit-exact scatter.  ``value`` and
    ``v_cache`` may both be ``None`` (a cache with one tensor, e.g. MLA latents ``[N, C, 1, r]``)."""
    lib = _lib.load()
    _stream(key)  # device check first: there is no CPU path
    key, row, k_st = _rows(key, "key")
    T = key.size(0)
    _require((value is None) == (v_cache is None), "value and v_cache go together")
    sc, st, sh = _cache_strides(k_cache)
    _require(key.dtype == k_cache.dtype, "dtype mismatch between K/V and cache")
    if value is not None:
        value, row_v, v_st = _rows(value, "value")
        _require(row == row_v and value.size(0) == T and k_st == v_st, "key/value shapes differ")
        _require(key.dtype == v_cache.dtype == value.dtype, "dtype mismatch between K/V and cache")
        _require(_cache_strides(v_cache) == (sc, st, sh), "k_cache / v_cache strides differ")
    _require(sh == k_cache.size(3) and row == k_cache.size(2) * k_cache.size(3), "cache rows must be contiguous [Hkv, d]")
    _require(token_to_chunk_idx.dtype == torch.int64 and token_to_local_pos.dtype == torch.int64,
             "slot index tensors must be int64")
    _require(token_to_chunk_idx.numel() >= T and token_to_local_pos.numel() >= T, "slot index tensors too short")
    _require(token_to_chunk_idx.is_contiguous() and token_to_local_pos.is_contiguous(), "slot index tensors must be contiguous")
    _lib.check(lib.mi_kv_append(key.data_ptr(), _ptr(value), k_st, k_cache.data_ptr(), _ptr(v_cache),
                                sc, st, token_to_chunk_idx.data_ptr(), token_to_local_pos.data_ptr(),
                                T, row, key.element_size(), _stream(key)), "mi_kv_append")


def kv_append_decode(key: Tensor, value: Tensor, k_cache: Tensor, v_cache: Tensor,
                     block_table: Tensor, kv_lens: Tensor) -> None:
    """Decode-step append with the slot derived on the GPU from block table + kv length."""
    lib = _lib.load()
    _stream(key)  # device check first: there is no CPU path
    key, row, k_st = _rows(key, "key")
    value, row_v, v_st = _rows(value, "value")
    R = key.size(0)
    _require(row == row_v and value.size(0) == R and k_st == v_st, "key/value shapes differ")
    _require(key.dtype == k_cache.dtype == v_cache.dtype == value.dtype, "dtype mismatch between K/V and cache")
    sc, st, sh = _cache_strides(k_cache)
    _require(_cache_strides(v_cache) == (sc, st, sh), "k_cache / v_cache strides differ")
    _require(sh == k_cache.size(3) and row == k_cache.size(2) * k_cache.size(3), "cache rows must be contiguous [Hkv, d]")
    _require(block_table.dtype == torch.int32 and kv_lens.dtype == torch.int32, "block_table / kv_lens must be int32")
    _require(block_table.dim() == 2 and block_table.stride(1) == 1 and block_table.size(0) >= R, "bad block_table")
    _require(kv_lens.is_contiguous() and kv_lens.numel() >= R, "bad kv_lens")
    _lib.check(lib.mi_kv_append_decode(key.data_ptr(), value.data_ptr(), k_st, k_cache.data_ptr(), v_cache.data_ptr(),
                                       sc, st, block_table.data_ptr(), block_table.stride(0), kv_lens.data_ptr(),
                                       R, k_cache.size(1), row, key.element_size(), _stream(key)),
               "mi_kv_append_decode")


# ---------------------------------------------------------------------------------------------
# fp8 KV storage
# ---------------------------------------------------------------------------------------------
def quantize_chunks_fp8(src: Tensor, dst: Tensor, scales: Tensor) -> None:
    """Quantise whole 16-bit chunks ``[N, C, Hkv, d]`` into an e4m3fn byte cache + ``[N, Hkv]`` scales."""
    lib = _lib.load()
    _stream(src)  # device check first: there is no CPU path
    _require(src.dtype in (torch.bfloat16, torch.float16), "source chunks must be bf16 or fp16")
    _require(dst.element_size() == 1, "destination cache must hold one byte per element")
    _require(scales.dtype == torch.float32 and scales.is_contiguous(), "scales must be contiguous fp32")
    ssc, sst, ssh = _cache_strides(src)
    dsc, dst_t, dsh = _cache_strides(dst)
    N, C, H, D = src.shape
    _require(tuple(dst.shape) == (N, C, H, D) and tuple(scales.shape) == (N, H), "shape mismatch")
    _require(ssh == D and dsh == D, "heads must be contiguous")
    _lib.check(lib.mi_kv_quantize_chunks_fp8(src.data_ptr(), ssc, sst, dst.data_ptr(), dsc, dst_t,
                                             scales.data_ptr(), N, C, H, D, _dtype_code(src, "src"), _stream(src)),
               "mi_kv_quantize_chunks_fp8")


def kv_append_decode_fp8(key: Tensor, value: Tensor, k_cache: Tensor, v_cache: Tensor, k_scales: Tensor,
                         v_scales: Tensor, block_table: Tensor, kv_lens: Tensor, headroom: float = 2.0) -> None:
    """Quantise and append one new 16-bit token per request into an fp8 cache."""
    lib = _lib.load()
    _stream(key)  # device check first: there is no CPU path
    key, row, k_st = _rows(key, "key")
    value, _, v_st = _rows(value, "value")
    _require(key.dtype in (torch.bfloat16, torch.float16) and value.dtype == key.dtype and k_st == v_st,
             "K/V must share one 16-bit type and have equal strides")
    _require(k_cache.element_size() == 1 and v_cache.element_size() == 1, "fp8 caches hold one byte per element")
    sc, st, sh = _cache_strides(k_cache)
    _require(_cache_strides(v_cache) == (sc, st, sh) and sh == k_cache.size(3), "cache layout")
    _require(k_scales.dtype == torch.float32 and v_scales.dtype == torch.float32, "scales must be fp32")
    _require(k_scales.is_contiguous() and v_scales.is_contiguous(), "scales must be contiguous")
    _require(block_table.dtype == torch.int32 and kv_lens.dtype == torch.int32, "block_table / kv_lens must be int32")
    _lib.check(lib.mi_kv_append_decode_fp8(key.data_ptr(), value.data_ptr(), k_st, k_cache.data_ptr(), v_cache.data_ptr(),
                                           sc, st, k_scales.data_ptr(), v_scales.data_ptr(), block_table.data_ptr(),
                                           block_table.stride(0), kv_lens.data_ptr(), key.size(0), k_cache.size(1),
                                           k_cache.size(2), k_cache.size(3), float(headroom), _dtype_code(key, "key"),
                                           _stream(key)), "mi_kv_append_decode_fp8")


def kv_append_fp8(key: Tensor, value: Tensor, k_cache: Tensor, v_cache: Tensor, k_scales: Tensor, v_scales: Tensor,
                  token_to_chunk_idx: Tensor, token_to_local_pos: Tensor, headroom: float = 2.0) -> None:
    """Quantise and append 16-bit tokens with explicit slots into an fp8 cache (prefill / mixed steps)."""
    lib = _lib.load()
    _stream(key)  # device check first: there is no CPU path
    key, row, k_st = _rows(key, "key")
    value, _, v_st = _rows(value, "value")
    T = key.size(0)
    _require(key.dtype in (torch.bfloat16, torch.float16) and value.dtype == key.dtype and k_st == v_st
             and value.size(0) == T, "K/V must share one 16-bit type and have equal shapes and strides")
    _require(k_cache.element_size() == 1 and v_cache.element_size() == 1, "fp8 caches hold one byte per element")
    sc, st, sh = _cache_strides(k_cache)
    _require(_cache_strides(v_cache) == (sc, st, sh) and sh == k_cache.size(3) and row == k_cache.size(2) * sh,
             "cache layout")
    _require(k_scales.dtype == torch.float32 and v_scales.dtype == torch.float32, "scales must be fp32")
    _require(k_scales.is_contiguous() and v_scales.is_contiguous(), "scales must be contiguous")
    for rows in (token_to_chunk_idx, token_to_local_pos):
        _require(rows.dtype == torch.int64 and rows.is_contiguous() and rows.numel() >= T, "slot rows must be int64 [>=T]")
    _lib.check(lib.mi_kv_append_fp8(key.data_ptr(), value.data_ptr(), k_st, k_cache.data_ptr(), v_cache.data_ptr(),
                                    sc, st, k_scales.data_ptr(), v_scales.data_ptr(), token_to_chunk_idx.data_ptr(),
                                    token_to_local_pos.data_ptr(), T, k_cache.size(1), k_cache.size(2),
                                    k_cache.size(3), float(headroom), _dtype_code(key, "key"), _stream(key)),
               "mi_kv_append_fp8")


# ---------------------------------------------------------------------------------------------
# attention
# ---------------------------------------------------------------------------------------------
def _qo_view(x: Tensor, name: str) -> Tensor:
    if x.dim() == 4:
        _require(x.size(1) == 1, f"{name} must be [T, 1, Hq, d] or [T, Hq, d]")
        x = x.squeeze(1)
    _require(x.dim() == 3 and x.stride(2) == 1, f"{name} must be [T, Hq, d] with contiguous d")
    _require(x.dtype in _DTYPE_CODES, f"{name} must be bf16 or fp16, got {x.dtype}")
    return x


def decode_workspace_bytes(R: int, Hq: int, Hkv: int, head_dim: int, chunk: int, max_kv_len: int,
                           split_tokens: int = 0) -> int:
    return int(_lib.load().mi_decode_workspace_bytes(R, Hq, Hkv, head_dim, chunk, max_kv_len, split_tokens,
                                                     _tuning_arg()))


def prefill_workspace_bytes(T: int, R: int, Hq: int, Hkv: int, head_dim: int, max_kv_len: int,
                            split_tokens: int = 0) -> int:
    """Scratch of one varlen attention call over ``T`` query rows of ``R`` requests: the decode part's
    partials and, when the tile kernel splits the keys, its partials behind them."""
    return int(_lib.load().mi_prefill_workspace_bytes(T, R, Hq, Hkv, head_dim, max_kv_len, split_tokens,
                                                      _tuning_arg()))


def paged_decode_attention(q: Tensor, k_cache: Tensor, v_cache: Tensor, kv_lens: Tensor, block_table: Tensor,
                           *, softmax_scale: Optional[float] = None, max_kv_len: Optional[int] = None,
                           split_tokens: int = 0, out: Optional[Tensor] = None,
                           workspace: Optional[Tensor] = None, k_scales: Optional[Tensor] = None,
                           v_scales: Optional[Tensor] = None) -> Tensor:
    """One query token per request against the paged cache; returns a tensor shaped like ``q``."""
    lib = _lib.load()
    stream = _stream(q)  # device check first: there is no CPU path
    q3 = _qo_view(q, "q")
    R, Hq, D = q3.shape
    N, C, Hkv, Dk = k_cache.shape
    _require(Dk == D and tuple(v_cache.shape) == tuple(k_cache.shape), "cache shape mismatch")
    fp8 = k_cache.element_size() == 1
    _require(fp8 or k_cache.dtype == q3.dtype, "the KV cache must have the queries' 16-bit type, or be a one-byte fp8 type")
    _require(v_cache.dtype == k_cache.dtype, "k_cache / v_cache dtypes differ")
    sc, st, sh = _cache_strides(k_cache)
    _require(_cache_strides(v_cache) == (sc, st, sh), "k_cache / v_cache strides differ")
    _require(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.stride(1) == 1, "bad block_table")
    _require(kv_lens.dtype == torch.int32 and kv_lens.is_contiguous(), "kv_lens must be contiguous int32")
    _require(block_table.size(0) >= R and kv_lens.numel() >= R, "block_table / kv_lens shorter than the batch")
    if fp8:
        _require(k_scales is not None and v_scales is not None, "fp8 cache needs k_scales and v_scales")
        _require(k_scales.dtype == torch.float32 and v_scales.dtype == torch.float32, "scales must be fp32")
        _require(tuple(k_scales.shape) == (N, Hkv) and tuple(v_scales.shape) == (N, Hkv), "scales must be [N, Hkv]")
        _require(k_scales.is_contiguous() and v_scales.is_contiguous(), "scales must be contiguous")
    if max_kv_len is None:
        max_kv_len = block_table.size(1) * C
    if softmax_scale is None:
        softmax_scale = D ** -0.5
    if out is None:
        out = torch.empty_like(q)
    o3 = _qo_view(out, "out")
    _require(tuple(o3.shape) == (R, Hq, D) and o3.dtype == q3.dtype, "out shape / dtype mismatch")
    tune = _tuning_arg()
    need = lib.mi_decode_workspace_bytes(R, Hq, Hkv, D, C, max_kv_len, split_tokens, tune)
    if workspace is None:
        workspace = _workspace(q.device, need, stream)
    ws_bytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    _lib.check(lib.mi_paged_decode_attention(
        q3.data_ptr(), q3.stride(0), q3.stride(1), k_cache.data_ptr(), v_cache.data_ptr(), sc, st, sh,
        block_table.data_ptr(), block_table.stride(0), kv_lens.data_ptr(), o3.data_ptr(), o3.stride(0), o3.stride(1),
        _ptr(workspace), ws_bytes, R, Hq, Hkv, D, C, int(max_kv_len), int(split_tokens), float(softmax_scale),
        MI_KV_FP8_E4M3 if fp8 else MI_KV_16BIT, _ptr(k_scales), _ptr(v_scales), _dtype_code(q3, "q"), tune,
        stream), "mi_paged_decode_attention")
    return out


def paged_decode_attention_noalloc(q: Tensor, k_cache: Tensor, v_cache: Tensor, kv_lens: Tensor, block_table: Tensor,
                                   out: Tensor, *, softmax_scale: Optional[float] = None,
                                   max_kv_len: Optional[int] = None, split_tokens: int = 0,
                                   k_scales: Optional[Tensor] = None, v_scales: Optional[Tensor] = None) -> Tensor:
    """:func:`paged_decode_attention` through the entry point that allocates nothing: the caller brings
    ``out``, the partials live in the library's built-in device scratch (16 MiB per GPU; larger problems are
    rejected).  Calls that overlap on one GPU share that scratch and race."""
    lib = _lib.load()
    stream = _stream(q)
    q3 = _qo_view(q, "q")
    R, Hq, D = q3.shape
    N, C, Hkv, Dk = k_cache.shape
    _require(Dk == D and tuple(v_cache.shape) == tuple(k_cache.shape), "cache shape mismatch")
    fp8 = k_cache.element_size() == 1
    _require(fp8 or k_cache.dtype == q3.dtype, "the KV cache must have the queries' 16-bit type, or be a one-byte fp8 type")
    _require(v_cache.dtype == k_cache.dtype, "k_cache / v_cache dtypes differ")
    sc, st, sh = _cache_strides(k_cache)
    _require(_cache_strides(v_cache) == (sc, st, sh), "k_cache / v_cache strides differ")
    _require(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.stride(1) == 1, "bad block_table")
    _require(kv_lens.dtype == torch.int32 and kv_lens.is_contiguous(), "kv_lens must be contiguous int32")
    _require(block_table.size(0) >= R and kv_lens.numel() >= R, "block_table / kv_lens shorter than the batch")
    if fp8:
        _require(k_scales is not None and v_scales is not None, "fp8 cache needs k_scales and v_scales")
        _require(k_scales.dtype == torch.float32 and v_scales.dtype == torch.float32
                 and k_scales.is_contiguous() and v_scales.is_contiguous()
                 and tuple(k_scales.shape) == (N, Hkv) and tuple(v_scales.shape) == (N, Hkv),
                 "scales must be contiguous fp32 [N, Hkv]")
    o3 = _qo_view(out, "out")
    _require(tuple(o3.shape) == (R, Hq, D) and o3.dtype == q3.dtype, "out shape / dtype mismatch")
    if max_kv_len is None:
        max_kv_len = block_table.size(1) * C
    if softmax_scale is None:
        softmax_scale = D ** -0.5
    _lib.check(lib.mi_paged_decode_attention_noalloc(
        q3.data_ptr(), q3.stride(0), q3.stride(1), k_cache.data_ptr(), v_cache.data_ptr(), sc, st, sh,
        block_table.data_ptr(), block_table.stride(0), kv_lens.data_ptr(), o3.data_ptr(), o3.stride(0), o3.stride(1),
        R, Hq, Hkv, D, C, int(max_kv_len), int(split_tokens), float(softmax_scale),
        MI_KV_FP8_E4M3 if fp8 else MI_KV_16BIT, _ptr(k_scales), _ptr(v_scales), _dtype_code(q3, "q"), _tuning_arg(),
        stream), "mi_paged_decode_attention_noalloc")
    return out


def paged_mla_decode_attention(q: Tensor, kv_cache: Tensor, kv_lens: Tensor, block_table: Tensor, *,
                               softmax_scale: float, head_dim_v: int = 512, max_kv_len: Optional[int] = None,
                               out: Optional[Tensor] = None) -> Tensor:
    """Absorbed multi-latent decode attention: ``q`` ``[R, (1,) Hq, 576]`` over the latent cache
    ``[N, C, 576]`` (or ``[N, C, 1, 576]``); returns ``[R, (1,) Hq, head_dim_v]``."""
    lib = _lib.load()
    stream = _stream(q)
    q3 = _qo_view(q, "q")
    R, Hq, Dk = q3.shape
    if kv_cache.dim() == 4:
        _require(kv_cache.size(2) == 1, "the latent cache has one row per token")
        kv_cache = kv_cache.squeeze(2)
    _require(kv_cache.dim() == 3 and kv_cache.stride(2) == 1 and kv_cache.size(2) == Dk
             and kv_cache.dtype == q3.dtype, "kv_cache must be [N, C, 576] of the queries' type with contiguous rows")
    _require(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.stride(1) == 1, "bad block_table")
    _require(kv_lens.dtype == torch.int32 and kv_lens.is_contiguous() and kv_lens.numel() >= R, "bad kv_lens")
    C = kv_cache.size(1)
    if max_kv_len is None:
        max_kv_len = block_table.size(1) * C
    if out is None:
        out = torch.empty(q.shape[:-1] + (head_dim_v,), dtype=q.dtype, device=q.device)
    o3 = _qo_view(out, "out")
    _require(tuple(o3.shape) == (R, Hq, head_dim_v), "out shape mismatch")
    tune = _tuning_arg()
    workspace = _workspace(q.device, lib.mi_mla_decode_workspace_bytes(R, Hq, head_dim_v, tune), stream)
    _lib.check(lib.mi_paged_mla_decode_attention(
        q3.data_ptr(), q3.stride(0), q3.stride(1), kv_cache.data_ptr(), kv_cache.stride(0), kv_cache.stride(1),
        block_table.data_ptr(), block_table.stride(0), kv_lens.data_ptr(), o3.data_ptr(), o3.stride(0), o3.stride(1),
        _ptr(workspace), 0 if workspace is None else workspace.numel(), R, Hq, Dk, head_dim_v, C, int(max_kv_len),
        float(softmax_scale), _dtype_code(q3, "q"), tune, stream), "mi_paged_mla_decode_attention")
    return out


def paged_prefill_attention_mla(q: Tensor, k_cache: Tensor, v_cache: Tensor, cu_seqlens_q: Tensor, kv_lens: Tensor,
                                block_table: Tensor, *, softmax_scale: float, max_kv_len: Optional[int] = None,
                                out: Optional[Tensor] = None) -> Tensor:
    """Varlen causal attention over the decompressed caches of multi-latent attention: ``q`` ``[T, Hq, 192]``,
    ``k_cache`` ``[N, C, H, 192]``, ``v_cache`` ``[N, C, H, 128]`` (each with its own strides) -> ``[T, Hq, 128]``.
    ``max_kv_len`` (an upper bound of ``kv_lens``; default: what the block table can hold) sizes the split of
    the keys when few query rows meet long contexts."""
    lib = _lib.load()
    stream = _stream(q)
    q3 = _qo_view(q, "q")
    T, Hq, Dk = q3.shape
    _require(k_cache.dim() == 4 and v_cache.dim() == 4 and k_cache.shape[:3] == v_cache.shape[:3],
             "key / value caches must be [N, C, H, d] with equal leading dimensions")
    _require(k_cache.dtype == q3.dtype and v_cache.dtype == q3.dtype, "the caches must have the queries' 16-bit type")
    N, C, Hkv, _ = k_cache.shape
    Dv = v_cache.size(3)
    _require(k_cache.size(3) == Dk, "query and key widths differ")
    ksc, kst, ksh = _cache_strides(k_cache)
    vsc, vst, vsh = _cache_strides(v_cache)
    _require(cu_seqlens_q.dtype == torch.int32 and cu_seqlens_q.is_contiguous(), "cu_seqlens_q must be contiguous int32")
    R = cu_seqlens_q.numel() - 1
    _require(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.stride(1) == 1, "bad block_table")
    _require(kv_lens.dtype == torch.int32 and kv_lens.is_contiguous(), "kv_lens must be contiguous int32")
    _require(block_table.size(0) >= R and kv_lens.numel() >= R, "block_table / kv_lens shorter than the batch")
    if out is None:
        out = torch.empty(q.shape[:-1] + (Dv,), dtype=q.dtype, device=q.device)
    o3 = _qo_view(out, "out")
    _require(tuple(o3.shape) == (T, Hq, Dv) and o3.dtype == q3.dtype, "out shape / dtype mismatch")
    if max_kv_len is None:
        max_kv_len = block_table.size(1) * C
    tune = _tuning_arg()
    need = lib.mi_prefill_workspace_bytes(T, R, Hq, Hkv, Dv, int(max_kv_len), 0, tune)
    override = _override_stack()
    if override and override[-1].numel() < need:
        workspace = None  # the split of the keys is optional here: a caller-sized workspace that is too small turns it off
    else:
        workspace = _workspace(q.device, need, stream)
    ws_bytes = 0 if workspace is None else workspace.numel()
    _lib.check(lib.mi_paged_prefill_attention_mla(
        q3.data_ptr(), q3.stride(0), q3.stride(1), k_cache.data_ptr(), ksc, kst, ksh, v_cache.data_ptr(), vsc, vst, vsh,
        block_table.data_ptr(), block_table.stride(0), cu_seqlens_q.data_ptr(), kv_lens.data_ptr(),
        o3.data_ptr(), o3.stride(0), o3.stride(1), _ptr(workspace), ws_bytes, T, R, Hq, Hkv, Dk, Dv, C,
        int(max_kv_len), float(softmax_scale), _dtype_code(q3, "q"), tune, stream),
        "mi_paged_prefill_attention_mla")
    return out


def paged_prefill_attention(q: Tensor, k_cache: Tensor, v_cache: Tensor, cu_seqlens_q: Tensor, kv_lens: Tensor,
                            block_table: Tensor, *, softmax_scale: Optional[float] = None,
                            max_kv_len: Optional[int] = None, out: Optional[Tensor] = None,
                            k_scales: Optional[Tensor] = None, v_scales: Optional[Tensor] = None) -> Tensor:
    """Varlen causal attention of new tokens over the paged cache (bottom-right aligned mask).
    Byte caches with ``k_scales`` / ``v_scales`` ``[N, Hkv]`` select the fp8-e4m3 path."""
    lib = _lib.load()
    _stream(q)  # device check first: there is no CPU path
    q3 = _qo_view(q, "q")
    T, Hq, D = q3.shape
    N, C, Hkv, Dk = k_cache.shape
    _require(Dk == D and tuple(v_cache.shape) == tuple(k_cache.shape), "cache shape mismatch")
    fp8 = k_scales is not None
    if fp8:
        _require(k_cache.element_size() == 1 and v_cache.element_size() == 1, "fp8 caches hold one byte per element")
        _require(v_scales is not None and k_scales.dtype == torch.float32 and v_scales.dtype == torch.float32
                 and k_scales.is_contiguous() and v_scales.is_contiguous() and tuple(k_scales.shape) == (N, Hkv)
                 and tuple(v_scales.shape) == (N, Hkv), "scales must be contiguous fp32 [N, Hkv]")
    else:
        _require(k_cache.dtype == q3.dtype and v_cache.dtype == q3.dtype,
                 "the cache must have the queries' 16-bit type, or be bytes with scales")
    sc, st, sh = _cache_strides(k_cache)
    _require(_cache_strides(v_cache) == (sc, st, sh), "k_cache / v_cache strides differ")
    _require(cu_seqlens_q.dtype == torch.int32 and cu_seqlens_q.is_contiguous(), "cu_seqlens_q must be contiguous int32")
    R = cu_seqlens_q.numel() - 1
    _require(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.stride(1) == 1, "bad block_table")
    _require(kv_lens.dtype == torch.int32 and kv_lens.is_contiguous(), "kv_lens must be contiguous int32")
    _require(block_table.size(0) >= R and kv_lens.numel() >= R, "block_table / kv_lens shorter than the batch")
    if max_kv_len is None:
        max_kv_len = block_table.size(1) * C
    if softmax_scale is None:
        softmax_scale = D ** -0.5
    if out is None:
        out = torch.empty_like(q)
    o3 = _qo_view(out, "out")
    _require(tuple(o3.shape) == (T, Hq, D) and o3.dtype == q3.dtype, "out shape / dtype mismatch")
    tune = _tuning_arg()
    stream = _stream(q)
    workspace = _workspace(q.device, lib.mi_prefill_workspace_bytes(T, R, Hq, Hkv, D, int(max_kv_len), 0, tune), stream)
    ws_bytes = 0 if workspace is None else workspace.numel()
    if fp8:
        _lib.check(lib.mi_paged_prefill_attention_fp8(
            q3.data_ptr(), q3.stride(0), q3.stride(1), k_cache.data_ptr(), v_cache.data_ptr(), sc, st, sh,
            k_scales.data_ptr(), v_scales.data_ptr(), block_table.data_ptr(), block_table.stride(0),
            cu_seqlens_q.data_ptr(), kv_lens.data_ptr(), o3.data_ptr(), o3.stride(0), o3.stride(1),
            _ptr(workspace), ws_bytes, T, R, Hq, Hkv, D, C, int(max_kv_len), 0, float(softmax_scale),
            _dtype_code(q3, "q"), tune, stream), "mi_paged_prefill_attention_fp8")
        return out
    _lib.check(lib.mi_paged_prefill_attention(
        q3.data_ptr(), q3.stride(0), q3.stride(1), k_cache.data_ptr(), v_cache.data_ptr(), sc, st, sh,
        block_table.data_ptr(), block_table.stride(0), cu_seqlens_q.data_ptr(), kv_lens.data_ptr(),
        o3.data_ptr(), o3.stride(0), o3.stride(1), _ptr(workspace), ws_bytes, T, R, Hq, Hkv, D, C,
        int(max_kv_len), 0,
        float(softmax_scale), _dtype_code(q3, "q"), tune, stream), "mi_paged_prefill_attention")
    return out


# ---------------------------------------------------------------------------------------------
# fused head norm + rotary embedding (+ append)
# ---------------------------------------------------------------------------------------------
def _angles(emb: Optional[Tensor]) -> Tuple[Optional[Tensor], int, int]:
    """Accept the reference's ``[max_seq, 1, 1, rot]`` fp32 table (or ``[max_seq, rot]``)."""
    if emb is None:
        return None, 0, 0
    _require(emb.dtype == torch.float32, "rotary table must be fp32 angles")
    e2 = emb.reshape(emb.size(0), emb.size(-1)) if emb.dim() != 2 else emb
    _require(e2.stride(1) == 1, "rotary table rows must be contiguous")
    return e2, e2.stride(0), e2.size(1)


def norm_rope_append(query: Optional[Tensor], key: Optional[Tensor], *, value: Optional[Tensor] = None,
                     q_weight: Optional[Tensor] = None, k_weight: Optional[Tensor] = None,
                     eps: float = 1e-5, norm: Optional[str] = None, rotary_emb: Optional[Tensor] = None,
                     q_positions: Optional[Tensor] = None, k_positions: Optional[Tensor] = None,
                     rotary_interleaved: bool = False, mscale: float = 1.0, query_out: Optional[Tensor] = None,
                     key_out: Optional[Tensor] = None,
                     k_cache: Optional[Tensor] = None, v_cache: Optional[Tensor] = None,
                     token_to_chunk_idx: Optional[Tensor] = None, token_to_local_pos: Optional[Tensor] = None,
                     block_table: Optional[Tensor] = None, kv_lens: Optional[Tensor] = None,
                     faithful_rounding: bool = True) -> None:
    """Norm (none / rms / l2) then RoPE on ``query`` (in place unless ``query_out`` is given) and on
    ``key`` (result to ``key_out`` and/or straight into the cache slot, together with ``value``)."""
    lib = _lib.load()
    ref = query if query is not None else key
    _require(ref is not None, "need query and/or key")
    T = Hq = Hkv = 0
    D = ref.size(-1)
    q3 = k3 = None
    if query is not None:
        q3 = _qo_view(query, "query")
        _require(q3.stride(1) == D, "query heads must be contiguous")
        T, Hq = q3.size(0), q3.size(1)
    if key is not None:
        k3 = _qo_view(key, "key")
        _require(k3.stride(1) == D, "key heads must be contiguous")
        T, Hkv = k3.size(0), k3.size(1)
        _require(query is None or q3.size(0) == T, "query / key token counts differ")
    qo3 = q3
    if query_out is not None:
        qo3 = _qo_view(query_out, "query_out")
        _require(q3 is not None and tuple(qo3.shape) == tuple(q3.shape) and qo3.stride(1) == D, "query_out shape")
    ko3 = None
    if key_out is not None:
        ko3 = _qo_view(key_out, "key_out")
        _require(tuple(ko3.shape) == tuple(k3.shape) and ko3.stride(1) == D, "key_out shape")
    v3 = None
    if value is not None:
        v3 = _qo_view(value, "value")
        _require(tuple(v3.shape) == tuple(k3.shape) and v3.stride(1) == D, "value shape")
    ang, a_stride, rot = _angles(rotary_emb)
    for w in (q_weight, k_weight):
        _require(w is None or (w.dtype == ref.dtype and w.numel() == D and w.is_contiguous()),
                 "norm weights must be [d] of the tensors' 16-bit type")
    for pz in (q_positions, k_positions, token_to_chunk_idx, token_to_local_pos):
        _require(pz is None or (pz.dtype == torch.int64 and pz.is_contiguous() and pz.numel() >= T), "index rows must be int64 [>=T]")
    sc = st = 0
    chunk = 0
    if k_cache is not None:
        _require(k_cache.dtype == ref.dtype and v_cache is not None and v_cache.dtype == ref.dtype,
                 "the caches must have the tensors' 16-bit type")
        sc, st, sh = _cache_strides(k_cache)
        _require(_cache_strides(v_cache) == (sc, st, sh) and sh == D, "cache layout")
        chunk = k_cache.size(1)
        if block_table is not None:
            _require(block_table.dtype == torch.int32 and block_table.stride(1) == 1, "bad block_table")
            _require(kv_lens is not None and kv_lens.dtype == torch.int32 and kv_lens.is_contiguous(), "bad kv_lens")
    for other in (q3, k3, qo3, ko3, v3):
        _require(other is None or other.dtype == ref.dtype, "query / key / value / outputs must share one 16-bit type")
    _lib.check(lib.mi_norm_rope_append(
        _ptr(q3), 0 if q3 is None else q3.stride(0), _ptr(qo3), 0 if qo3 is None else qo3.stride(0),
        _ptr(k3), 0 if k3 is None else k3.stride(0),
        _ptr(ko3), 0 if ko3 is None else ko3.stride(0), _ptr(v3), 0 if v3 is None else v3.stride(0),
        _ptr(q_weight), _ptr(k_weight), float(eps), _NORM_KINDS[norm], _ptr(ang), a_stride, rot,
        int(bool(rotary_interleaved)), float(mscale), _ptr(q_positions), _ptr(k_positions),
        _ptr(k_cache), _ptr(v_cache), sc, st, _ptr(token_to_chunk_idx), _ptr(token_to_local_pos),
        _ptr(block_table), 0 if block_table is None else block_table.stride(0), _ptr(kv_lens), chunk,
        T, Hq, Hkv, D, int(bool(faithful_rounding)), _dtype_code(ref, "query / key"), _tuning_arg(), _stream(ref)),
        "mi_norm_rope_append")


def qkv_norm_rope_append(mixed_qkv: Tensor, *, num_query_heads: int, num_kv_heads: int, query_out: Tensor,
                         key_out: Optional[Tensor] = None, q_weight: Optional[Tensor] = None,
                         k_weight: Optional[Tensor] = None, eps: float = 1e-5, norm: Optional[str] = None,
                         rotary_emb: Optional[Tensor] = None, q_positions: Optional[Tensor] = None,
                         k_positions: Optional[Tensor] = None, rotary_interleaved: bool = False,
                         mscale: float = 1.0, k_cache: Optional[Tensor] = None, v_cache: Optional[Tensor] = None,
                         token_to_chunk_idx: Optional[Tensor] = None, token_to_local_pos: Optional[Tensor] = None,
                         block_table: Optional[Tensor] = None, kv_lens: Optional[Tensor] = None,
                         faithful_rounding: bool = True) -> None:
    """:func:`norm_rope_append` reading the QKV projection's output ``[T, (1,) (Hq + 2 Hkv) * d]`` (per
    query group: its query heads, then its key head, then its value head -- the layout that
    ``get_query_key_value_tensors`` splits, attention.py:985-1030) without materialising the split."""
    lib = _lib.load()
    _require(mixed_qkv.is_cuda and mixed_qkv.dtype in _DTYPE_CODES, "mixed_qkv must be a bf16 or fp16 device tensor")
    if mixed_qkv.dim() == 3:
        _require(mixed_qkv.size(1) == 1, "mixed_qkv must be [T, 1, W]")
        mixed_qkv = mixed_qkv[:, 0]
    _require(mixed_qkv.dim() == 2 and mixed_qkv.stride(1) == 1, "mixed_qkv must be [T, W] with contiguous rows")
    T, W = mixed_qkv.shape
    Hq, Hkv = int(num_query_heads), int(num_kv_heads)
    _require(Hq > 0 and Hkv > 0 and Hq % Hkv == 0 and W % (Hq + 2 * Hkv) == 0, "mixed_qkv width / head counts")
    D = W // (Hq + 2 * Hkv)
    qo3 = _qo_view(query_out, "query_out")
    _require(tuple(qo3.shape) == (T, Hq, D) and qo3.stride(1) == D and qo3.dtype == mixed_qkv.dtype,
             "query_out must be [T, Hq, d] of the projection's type")
    ko3 = None
    if key_out is not None:
        ko3 = _qo_view(key_out, "key_out")
        _require(tuple(ko3.shape) == (T, Hkv, D) and ko3.stride(1) == D, "key_out must be [T, Hkv, d]")
    _require(ko3 is not None or k_cache is not None, "the key needs a destination: key_out and/or the cache")
    ang, a_stride, rot = _angles(rotary_emb)
    for w in (q_weight, k_weight):
        _require(w is None or (w.dtype == mixed_qkv.dtype and w.numel() == D and w.is_contiguous()),
                 "norm weights must be [d] of the tensors' 16-bit type")
    for pz in (q_positions, k_positions, token_to_chunk_idx, token_to_local_pos):
        _require(pz is None or (pz.dtype == torch.int64 and pz.is_contiguous() and pz.numel() >= T), "index rows must be int64 [>=T]")
    sc = st = 0
    chunk = 0
    if k_cache is not None:
        _require(k_cache.dtype == mixed_qkv.dtype and v_cache is not None and v_cache.dtype == mixed_qkv.dtype,
                 "the caches must have the projection's 16-bit type")
        sc, st, sh = _cache_strides(k_cache)
        _require(_cache_strides(v_cache) == (sc, st, sh) and sh == D, "cache layout")
        chunk = k_cache.size(1)
        if block_table is not None:
            _require(block_table.dtype == torch.int32 and block_table.stride(1) == 1, "bad block_table")
            _require(kv_lens is not None and kv_lens.dtype == torch.int32 and kv_lens.is_contiguous(), "bad kv_lens")
    _lib.check(lib.mi_qkv_norm_rope_append(
        _ptr(mixed_qkv), mixed_qkv.stride(0), _ptr(qo3), qo3.stride(0), _ptr(ko3), 0 if ko3 is None else ko3.stride(0),
        _ptr(q_weight), _ptr(k_weight), float(eps), _NORM_KINDS[norm], _ptr(ang), a_stride, rot,
        int(bool(rotary_interleaved)), float(mscale), _ptr(q_positions), _ptr(k_positions),
        _ptr(k_cache), _ptr(v_cache), sc, st, _ptr(token_to_chunk_idx), _ptr(token_to_local_pos),
        _ptr(block_table), 0 if block_table is None else block_table.stride(0), _ptr(kv_lens), chunk,
        T, Hq, Hkv, D, int(bool(faithful_rounding)), _dtype_code(mixed_qkv, "mixed_qkv"), _tuning_arg(),
        _stream(mixed_qkv)), "mi_qkv_norm_rope_append")


# ---------------------------------------------------------------------------------------------
# context bookkeeping on the GPU
# ---------------------------------------------------------------------------------------------
def decode_step_supported(head_dim: int, rot_dim: int, rotary_interleaved: bool, fp8_cache: bool) -> bool:
    """Whether :func:`decode_step_attention` has a kernel for these shapes (else: the separate calls)."""
    if head_dim not in (64, 96, 128, 192, 256) or (fp8_cache and head_dim != 128):
        return False
    # half-split pairs must sit a whole number of a lane's fragments apart (fp8 key bytes: 64 elements)
    return rot_dim == 0 or rotary_interleaved or (rot_dim // 2) % (64 if fp8_cache else 32) == 0


def decode_step_attention(query: Optional[Tensor], key: Optional[Tensor], value: Optional[Tensor], k_cache: Tensor,
                          v_cache: Tensor, kv_lens: Tensor, block_table: Tensor, *,
                          mixed_qkv: Optional[Tensor] = None, num_query_heads: int = 0, num_kv_heads: int = 0,
                          q_weight: Optional[Tensor] = None, k_weight: Optional[Tensor] = None, eps: float = 1e-5,
                          norm: Optional[str] = None, rotary_emb: Optional[Tensor] = None,
                          positions: Optional[Tensor] = None, rotary_interleaved: bool = False, mscale: float = 1.0,
                          softmax_scale: Optional[float] = None, max_kv_len: Optional[int] = None,
                          split_tokens: int = 0, out: Optional[Tensor] = None, workspace: Optional[Tensor] = None,
                          faithful_rounding: bool = True, k_scales: Optional[Tensor] = None,
                          v_scales: Optional[Tensor] = None, headroom: float = 2.0) -> Tensor:
    """One decode step of a layer in two launches: head norm + RoPE of the raw queries and of the step's new key
    rows, the append of the new key / value rows at position ``kv_lens - 1`` and the attention over the cache --
    what :func:`norm_rope_append` (or :func:`qkv_norm_rope_append`) followed by :func:`paged_decode_attention`
    computes.  Inputs: ``query`` ``[R, (1,) Hq, d]``, ``key`` / ``value`` ``[R, (1,) Hkv, d]``, or ``mixed_qkv``
    ``[R, (1,) (Hq + 2 Hkv) d]`` (the QKV projection's output) with the head counts.  Returns ``[R, (1,) Hq, d]``.
    Byte caches with ``k_scales`` / ``v_scales`` hold e4m3 values: the append then quantises like
    :func:`kv_append_decode_fp8` (``headroom`` as there)."""
    lib = _lib.load()
    if mixed_qkv is not None:
        _require(query is None and key is None and value is None, "give either query / key / value or mixed_qkv")
        _require(mixed_qkv.is_cuda and mixed_qkv.dtype in _DTYPE_CODES, "mixed_qkv must be a bf16 or fp16 device tensor")
        four_d = mixed_qkv.dim() == 3
        m2 = mixed_qkv[:, 0] if four_d else mixed_qkv
        _require(not four_d or mixed_qkv.size(1) == 1, "mixed_qkv must be [R, 1, W]")
        _require(m2.dim() == 2 and m2.stride(1) == 1, "mixed_qkv must be [R, W] with contiguous rows")
        R, W = m2.shape
        Hq, Hkv = int(num_query_heads), int(num_kv_heads)
        _require(Hq > 0 and Hkv > 0 and Hq % Hkv == 0 and W % (Hq + 2 * Hkv) == 0, "mixed_qkv width / head counts")
        D = W // (Hq + 2 * Hkv)
        G = Hq // Hkv
        group = (G + 2) * D
        ref = m2
        q_ptr, q_st, q_gst = m2.data_ptr(), m2.stride(0), group
        k_ptr, k_st, k_hst = m2.data_ptr() + 2 * G * D, m2.stride(0), group
        v_ptr, v_st, v_hst = m2.data_ptr() + 2 * (G + 1) * D, m2.stride(0), group
        out_shape = (R, 1, Hq, D) if four_d else (R, Hq, D)
    else:
        q3, k3, v3 = _qo_view(query, "query"), _qo_view(key, "key"), _qo_view(value, "value")
        R, Hq, D = q3.shape
        Hkv = k3.size(1)
        _require(tuple(k3.shape) == (R, Hkv, D) and tuple(v3.shape) == (R, Hkv, D) and Hq % max(Hkv, 1) == 0,
                 "query / key / value shapes")
        _require(q3.stride(1) == D, "query heads must be contiguous")
        _require(k3.dtype == q3.dtype and v3.dtype == q3.dtype, "query / key / value must share one 16-bit type")
        ref = q3
        q_ptr, q_st, q_gst = q3.data_ptr(), q3.stride(0), (Hq // Hkv) * D
        k_ptr, k_st, k_hst = k3.data_ptr(), k3.stride(0), k3.stride(1)
        v_ptr, v_st, v_hst = v3.data_ptr(), v3.stride(0), v3.stride(1)
        out_shape = tuple(query.shape)
    stream = _stream(ref)
    N, C, Hkv_c, Dk = k_cache.shape
    _require(Dk == D and Hkv_c == Hkv and tuple(v_cache.shape) == tuple(k_cache.shape), "cache shape mismatch")
    fp8 = k_cache.element_size() == 1
    if fp8:
        _require(v_cache.element_size() == 1 and k_scales is not None and v_scales is not None,
                 "byte caches hold e4m3 values and need k_scales / v_scales")
        for t in (k_scales, v_scales):
            _require(t.dtype == torch.float32 and t.is_contiguous() and tuple(t.shape) == (N, Hkv), "scales must be fp32 [n_chunks, Hkv]")
    else:
        _require(k_cache.dtype == ref.dtype and v_cache.dtype == ref.dtype, "the caches must have the tensors' 16-bit type")
    sc, st, sh = _cache_strides(k_cache)
    _require(_cache_strides(v_cache) == (sc, st, sh), "k_cache / v_cache strides differ")
    _require(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.stride(1) == 1, "bad block_table")
    _require(kv_lens.dtype == torch.int32 and kv_lens.is_contiguous(), "kv_lens must be contiguous int32")
    _require(block_table.size(0) >= R and kv_lens.numel() >= R, "block_table / kv_lens shorter than the batch")
    ang, a_stride, rot = _angles(rotary_emb)
    _require(positions is None or (positions.dtype == torch.int64 and positions.is_contiguous()
                                   and positions.numel() >= R), "positions must be int64 [>= R] (None: kv_lens - 1)")
    for w in (q_weight, k_weight):
        _require(w is None or (w.dtype == ref.dtype and w.numel() == D and w.is_contiguous()),
                 "norm weights must be [d] of the tensors' 16-bit type")
    if max_kv_len is None:
        max_kv_len = block_table.size(1) * C
    if softmax_scale is None:
        softmax_scale = D ** -0.5
    if out is None:
        out = torch.empty(out_shape, dtype=ref.dtype, device=ref.device)
    o3 = _qo_view(out, "out")
    _require(tuple(o3.shape) == (R, Hq, D) and o3.dtype == ref.dtype, "out shape / dtype mismatch")
    tune = _tuning_arg()
    need = lib.mi_decode_workspace_bytes(R, Hq, Hkv, D, C, max_kv_len, split_tokens, tune)
    if workspace is None:
        workspace = _workspace(ref.device, need, stream)
    ws_bytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    if fp8:
        _lib.check(lib.mi_decode_step_attention_fp8(
            q_ptr, q_st, q_gst, k_ptr, k_st, k_hst, v_ptr, v_st, v_hst, _ptr(q_weight), _ptr(k_weight), float(eps),
            _NORM_KINDS[norm], _ptr(ang), a_stride, rot, int(bool(rotary_interleaved)), float(mscale), _ptr(positions),
            k_cache.data_ptr(), v_cache.data_ptr(), sc, st, sh, k_scales.data_ptr(), v_scales.data_ptr(), float(headroom),
            block_table.data_ptr(), block_table.stride(0), kv_lens.data_ptr(), o3.data_ptr(), o3.stride(0), o3.stride(1),
            _ptr(workspace), ws_bytes, R, Hq, Hkv, D, C, int(split_tokens), float(softmax_scale),
            int(bool(faithful_rounding)), _dtype_code(ref, "query"), tune, stream), "mi_decode_step_attention_fp8")
        return out
    _lib.check(lib.mi_decode_step_attention(
        q_ptr, q_st, q_gst, k_ptr, k_st, k_hst, v_ptr, v_st, v_hst, _ptr(q_weight), _ptr(k_weight), float(eps),
        _NORM_KINDS[norm], _ptr(ang), a_stride, rot, int(bool(rotary_interleaved)), float(mscale), _ptr(positions),
        k_cache.data_ptr(), v_cache.data_ptr(), sc, st, sh, block_table.data_ptr(), block_table.stride(0),
        kv_lens.data_ptr(), o3.data_ptr(), o3.stride(0), o3.stride(1), _ptr(workspace), ws_bytes, R, Hq, Hkv, D, C,
        int(split_tokens), float(softmax_scale), int(bool(faithful_rounding)), _dtype_code(ref, "query"), tune,
        stream), "mi_decode_step_attention")
    return out


def update_requests(ctx, mask_i32: Tensor, new_tokens_i64: Tensor) -> None:
    """Enqueue the single-kernel ``update_requests`` on the state tensors of ``ctx`` (results land in
    ``ctx._counters`` / ``ctx._newly_paused_buf`` / ``ctx._finished_ids_buf`` / ``ctx._paused_tokens_buf``)."""
    lib = _lib.load()
    table = ctx.request_to_kv_chunk_ids
    _require(table.stride(1) == 1, "request_to_kv_chunk_ids rows must be contiguous")
    _lib.check(lib.mi_update_requests(
        ctx.request_ids.data_ptr(), ctx.request_query_lengths.data_ptr(), ctx.request_output_lengths.data_ptr(),
        ctx.request_kv_length_offsets.data_ptr(), ctx.request_kv_chunk_counts.data_ptr(),
        ctx.request_last_kv_chunk_id.data_ptr(), ctx.request_last_kv_chunk_offset.data_ptr(),
        table.data_ptr(), table.stride(0), table.size(1),
        ctx.token_to_input_ids.data_ptr(), ctx.token_to_pos_ids.data_ptr(), ctx.token_to_request_idx.data_ptr(),
        ctx.token_to_position_in_request.data_ptr(), ctx.token_to_chunk_idx.data_ptr(),
        ctx.token_to_local_position_within_kv_chunk.data_ptr(), ctx.chunk_allocator.chunk_bag.data_ptr(),
        mask_i32.data_ptr(), new_tokens_i64.data_ptr(), ctx._paused_tokens_buf.data_ptr(),
        ctx._next_tokens_buf.data_ptr(), ctx._update_scratch.data_ptr(), ctx._newly_paused_buf.data_ptr(),
        ctx._finished_ids_buf.data_ptr(), ctx._counters.data_ptr(), ctx.total_request_count, ctx.paused_request_count,
        ctx.chunk_allocator.chunk_count_avail, ctx.gtd_chunk_count, ctx.gtd_request_count,
        ctx.chunk_size_tokens, ctx.max_requests, _stream(table)), "mi_update_requests")


def add_request(ctx, row: int, token_begin: int, tokens_i64: Tensor, n_chunks: int, stack_first: int,
                request_id: int, output_length: int) -> None:
    """The tensor writes of ``add_request`` in one launch: request row ``row``, its chunk-table entries
    ``chunk_bag[stack_first : stack_first + n_chunks]`` and the token rows from ``token_begin`` on."""
    lib = _lib.load()
    table = ctx.request_to_kv_chunk_ids
    _require(tokens_i64.dtype == torch.int64 and tokens_i64.is_contiguous() and tokens_i64.device == table.device,
             "prompt tokens must be a contiguous int64 tensor on the context's device")
    _lib.check(lib.mi_add_request(
        ctx.request_ids.data_ptr(), ctx.request_query_lengths.data_ptr(), ctx.request_output_lengths.data_ptr(),
        ctx.request_kv_length_offsets.data_ptr(), ctx.request_kv_chunk_counts.data_ptr(),
        ctx.request_last_kv_chunk_id.data_ptr(), ctx.request_last_kv_chunk_offset.data_ptr(), table.data_ptr(),
        table.stride(0), ctx.token_to_input_ids.data_ptr(), ctx.token_to_pos_ids.data_ptr(),
        ctx.token_to_request_idx.data_ptr(), ctx.token_to_position_in_request.data_ptr(),
        ctx.token_to_chunk_idx.data_ptr(), ctx.token_to_local_position_within_kv_chunk.data_ptr(),
        ctx.chunk_allocator.chunk_bag.data_ptr(), tokens_i64.data_ptr(), int(row), int(token_begin),
        tokens_i64.numel(), int(n_chunks), int(stack_first), ctx.chunk_size_tokens, int(request_id),
        int(output_length), _stream(table)), "mi_add_request")


def decode_attention_state(ctx, n_active_requests: int, padded_tokens: int) -> None:
    """Fill the fixed-address length / block-table mirrors and the padded token rows in one launch."""
    lib = _lib.load()
    table = ctx.request_to_kv_chunk_ids
    mirror = ctx.request_to_kv_chunk_ids_cudagraph_only
    _lib.check(lib.mi_decode_attention_state(
        ctx.request_kv_length_offsets.data_ptr(), ctx.request_query_lengths.data_ptr(), table.data_ptr(),
        table.stride(0), table.size(1), ctx.query_seq_lengths_cudagraph_only.data_ptr(),
        ctx.kv_seq_lengths_cudagraph_only.data_ptr(), mirror.data_ptr(), mirror.stride(0),
        ctx.token_to_chunk_idx.data_ptr(), ctx.token_to_local_position_within_kv_chunk.data_ptr(),
        ctx.token_to_position_in_request.data_ptr(), ctx.paused_request_count, n_active_requests,
        ctx.active_token_count, padded_tokens, ctx.dummy_chunk_idx, _stream(table)), "mi_decode_attention_state")


def step_attention_state(ctx, n_active_requests: int, padded_requests: int, padded_tokens: int) -> None:
    """Prefill / mixed steps: the fixed-address mirrors of lengths, their running sums and the block table, the
    padded token rows and the two maxima (into ``ctx._max_lengths``) in one launch."""
    lib = _lib.load()
    table = ctx.request_to_kv_chunk_ids
    mirror = ctx.request_to_kv_chunk_ids_cudagraph_only
    _lib.check(lib.mi_step_attention_state(
        ctx.request_kv_length_offsets.data_ptr(), ctx.request_query_lengths.data_ptr(), table.data_ptr(),
        table.stride(0), table.size(1), ctx.query_seq_lengths_cudagraph_only.data_ptr(),
        ctx.kv_seq_lengths_cudagraph_only.data_ptr(), ctx.cu_query_seq_lengths_cudagraph_only.data_ptr(),
        ctx.cu_kv_seq_lengths_cudagraph_only.data_ptr(), mirror.data_ptr(), mirror.stride(0),
        ctx.token_to_chunk_idx.data_ptr(), ctx.token_to_local_position_within_kv_chunk.data_ptr(),
        ctx.token_to_position_in_request.data_ptr(), ctx._max_lengths.data_ptr(), ctx.paused_request_count,
        n_active_requests, padded_requests, ctx.active_token_count, padded_tokens, ctx.dummy_chunk_idx,
        _stream(table)), "mi_step_attention_state")


# ---------------------------------------------------------------------------------------------
# tail of a decode step: last-token rows, sampling, finished-request mask
# ---------------------------------------------------------------------------------------------
def last_token_gather(rows: Tensor, request_query_lengths: Tensor, out: Optional[Tensor] = None) -> Tensor:
    """``rows[cumsum(request_query_lengths) - 1]`` in one launch (``rows`` is ``[T, E]``; the
    lengths are those of the active requests, int32)."""
    lib = _lib.load()
    stream = _stream(rows)
    _require(rows.dim() == 2 and rows.stride(1) == 1, "rows must be [T, E] with contiguous E")
    _require(rows.element_size() in (2, 4), "rows must have 2- or 4-byte elements")
    _require(request_query_lengths.dtype == torch.int32 and request_query_lengths.dim() == 1
             and request_query_lengths.is_contiguous(), "request_query_lengths must be a contiguous int32 row")
    R, E = request_query_lengths.numel(), rows.size(1)
    if out is None:
        out = torch.empty(R, E, dtype=rows.dtype, device=rows.device)
    _require(out.dtype == rows.dtype and tuple(out.shape) == (R, E) and out.stride(1) == 1, "out must be [R, E]")
    _lib.check(lib.mi_last_token_gather(rows.data_ptr(), rows.stride(0), out.data_ptr(), out.stride(0),
                                        request_query_lengths.data_ptr(), R, E, rows.element_size(), stream),
               "mi_last_token_gather")
    return out


def selected_log_probs(logits: Tensor, token_ids: Tensor) -> Tensor:
    """``log_softmax(logits.float(), -1)[arange(T), token_ids]`` (fp32 ``[T]``) with one read of each row of
    ``logits`` ``[T, V]`` (fp32, bf16 or fp16) and no ``[T, V]`` intermediate."""
    lib = _lib.load()
    stream = _stream(logits)
    _require(logits.dim() == 2 and logits.stride(1) == 1, "logits must be [T, V] with contiguous V")
    _require(logits.dtype in _LOGIT_CODES, "logits must be fp32, bf16 or fp16")
    T, V = logits.shape
    _require(token_ids.dtype == torch.int64 and token_ids.dim() == 1 and token_ids.numel() == T
             and token_ids.is_contiguous() and token_ids.device == logits.device,
             "token_ids must be a contiguous int64 row with one id per row of logits")
    out = torch.empty(T, dtype=torch.float32, device=logits.device)
    _lib.check(lib.mi_selected_log_probs(logits.data_ptr(), logits.stride(0),
                                         _LOGIT_CODES[logits.dtype], T, V,
                                         token_ids.data_ptr(), out.data_ptr(), stream), "mi_selected_log_probs")
    return out


def sample_from_logits(logits: Tensor, *, top_k: int = 0, top_p: float = 0.0, temperature: float = 1.0,
                       uniform: Optional[Tensor] = None, vocab_size: Optional[int] = None,
                       termination_id: Optional[int] = None, kv_length_offsets: Optional[Tensor] = None,
                       query_lengths: Optional[Tensor] = None, output_lengths: Optional[Tensor] = None,
                       return_cut: bool = False):
    """One launch: filter + draw per row of ``logits`` ``[R, V]`` (fp32, bf16 or fp16) and, when
    ``termination_id`` is given, the uint8 mask of requests that go on generating.

    Returns ``(samples int64 [R], mask uint8 [R] or None)`` and, with ``return_cut``, also the
    smallest kept value per row (fp32, -inf where nothing was filtered)."""
    lib = _lib.load()
    stream = _stream(logits)
    _require(logits.dim() == 2 and logits.stride(1) == 1, "logits must be [R, V] with contiguous V")
    _require(logits.dtype in _LOGIT_CODES, "logits must be fp32, bf16 or fp16")
    R, V = logits.shape
    dev = logits.device
    if top_k != 1:
        _require(uniform is not None, "sampling needs one uniform number per row")
        _require(uniform.dtype == torch.float32 and uniform.is_contiguous() and uniform.numel() >= R
                 and uniform.device == dev, "uniform must be a contiguous fp32 row of at least R numbers")
    samples = torch.empty(R, dtype=torch.int64, device=dev)
    mask = None
    lens = (kv_length_offsets, query_lengths, output_lengths)
    if termination_id is not None:
        mask = torch.empty(R, dtype=torch.uint8, device=dev)
        _require(all(t is None for t in lens) or all(t is not None for t in lens),
                 "the three request length rows go together")
        for t in lens:
            _require(t is None or (t.dtype == torch.int32 and t.is_contiguous() and t.numel() >= R and t.device == dev),
                     "request length rows must be contiguous int32 rows of at least R entries")
    else:
        _require(all(t is None for t in lens), "request lengths without a termination id")
    cut = torch.empty(R, dtype=torch.float32, device=dev) if return_cut else None
    _lib.check(lib.mi_sample_from_logits(
        logits.data_ptr(), logits.stride(0), _LOGIT_CODES[logits.dtype], R, V, int(top_k),
        float(top_p), float(temperature), _ptr(uniform), int(vocab_size or 0), samples.data_ptr(), _ptr(cut),
        _ptr(kv_length_offsets), _ptr(query_lengths), _ptr(output_lengths),
        int(termination_id) if termination_id is not None else -1, _ptr(mask), stream), "mi_sample_from_logits")
    return (samples, mask, cut) if return_cut else (samples, mask)


def linear_decode(x: Tensor, weight: Tensor, bias: Optional[Tensor] = None, out: Optional[Tensor] = None) -> Tensor:
    """``x @ weight.T (+ bias)`` for a decode-sized step (at most 256 rows of ``x``): the weight matrix streams from
    HBM once.  ``x`` is ``[..., K]`` (leading dimensions are flattened to rows), ``weight`` ``[N, K]``; the result
    has ``x``'s leading dimensions and ``N`` columns.  What ``linear_qkv`` / ``linear_proj`` of the attention layer
    compute at tensor-parallel size 1 (``mi_linear_decode`` of the header)."""
    _require(weight.dim() == 2 and weight.stride(1) == 1, "weight must be [N, K] with contiguous rows")
    N, K = weight.shape
    _require(x.size(-1) == K and x.stride(-1) == 1, "x must be [..., K] with a contiguous last dimension")
    _require(x.dtype == weight.dtype and (bias is None or bias.dtype == x.dtype), "x, weight and bias share one 16-bit type")
    x2 = x.reshape(-1, K)
    T = x2.size(0)
    if out is None:
        out = torch.empty(*x.shape[:-1], N, dtype=x.dtype, device=x.device)
    o2 = out.view(-1, N)
    _require(o2.size(0) == T and o2.stride(1) == 1, "out must be [..., N] with a contiguous last dimension")
    if bias is not None:
        _require(bias.numel() == N and bias.is_contiguous(), "bias must be a contiguous [N] vector")
    lib = _lib.load()
    stream = _stream(x)
    nbytes = lib.mi_linear_decode_workspace_bytes(T, N, K)
    ws = _workspace(x.device, nbytes, stream)
    _lib.check(lib.mi_linear_decode(x2.data_ptr(), x2.stride(0), weight.data_ptr(), weight.stride(0), _ptr(bias),
                                    o2.data_ptr(), o2.stride(0), _ptr(ws), 0 if ws is None else ws.numel(), T, N, K,
                                    _dtype_code(x, "x"), stream), "mi_linear_decode")
    return out
