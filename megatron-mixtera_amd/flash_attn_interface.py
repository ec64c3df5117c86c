"""The flash-attn entry points the reference's dynamic path calls, on MI355X kernels.

``Attention.flash_decode_and_prefill`` (megatron/core/transformer/attention.py:470-601)
resolves the module-level names ``flash_attn_with_kvcache`` and ``flash_attn_varlen_func``;
these functions accept the keyword surface used there and run the paged kernels of
``libmi355_decode.so``.  Arguments the reference never passes on this path (dropout,
windows, alibi, rotary fusion, new-token append inside the call) are rejected rather than
silently ignored.
"""
from __future__ import annotations

import weakref
from typing import Optional

import torch
from torch import Tensor

from . import ops


# Per-request kv lengths that belong to a cu_seqlens_k tensor, published by the context that built both
# (DynamicInferenceContext.initialize_attention_state).  The reference's call site hands flash_attn_varlen_func only
# the running sums (attention.py:546-557); with a note the lengths need not be recomputed by a subtraction + copy in
# every layer.  Notes are keyed by the identity of the sums tensor OBJECT and die with it (a weak reference), so a
# later tensor that happens to reuse the address never inherits them, and several contexts keep one note each.
_kv_lengths_notes = {}


def note_kv_lengths(cu_seqlens_k: Optional[Tensor], kv_lens: Optional[Tensor]) -> None:
    """Remember that ``kv_lens`` are the differences of ``cu_seqlens_k``; ``kv_lens=None`` forgets that tensor's
    note, ``cu_seqlens_k=None`` is a no-op."""
    if cu_seqlens_k is None:
        return
    key = id(cu_seqlens_k)
    if kv_lens is None:
        _kv_lengths_notes.pop(key, None)
        return
    ref = weakref.ref(cu_seqlens_k, lambda _r, key=key: _kv_lengths_notes.pop(key, None))
    _kv_lengths_notes[key] = (ref, kv_lens)


def _lengths_of(cu_seqlens_k: Tensor) -> Tensor:
    note = _kv_lengths_notes.get(id(cu_seqlens_k))
    if note is not None and note[0]() is cu_seqlens_k:
        return note[1]
    return (cu_seqlens_k[1:] - cu_seqlens_k[:-1]).contiguous()


def _reject(**unsupported) -> None:
    # (a tensor is an argument given, whatever it holds: `tensor in (...)` would compare element values)
    bad = [k for k, v in unsupported.items() if isinstance(v, Tensor) or v not in (None, False, 0, 0.0, (-1, -1))]
    if bad:
        raise NotImplementedError(f"unsupported flash-attn arguments on the paged MI355X path: {bad}")


def flash_attn_with_kvcache(q: Tensor, k_cache: Tensor, v_cache: Tensor, k: Optional[Tensor] = None,
                            v: Optional[Tensor] = None, rotary_cos=None, rotary_sin=None,
                            cache_seqlens: Optional[Tensor] = None, cache_batch_idx=None,
                            cache_leftpad=None, block_table: Optional[Tensor] = None,
                            softmax_scale: Optional[float] = None, causal: bool = False,
                            window_size=(-1, -1), softcap: float = 0.0, rotary_interleaved: bool = True,
                            alibi_slopes=None, num_splits: int = 0, return_softmax_lse: bool = False,
                            *, page_table: Optional[Tensor] = None, k_scales: Optional[Tensor] = None,
                            v_scales: Optional[Tensor] = None, max_seqlen_k: Optional[int] = None) -> Tensor:
    """Paged decode attention: ``q`` is ``[batch, 1, Hq, d]``, one query token per request.

    ``cache_seqlens`` (int32 ``[batch]``) already counts the token appended this step;
    ``block_table`` / ``page_table`` is int32 ``[batch, max_chunks]``.  With a single query
    token the causal mask is a no-op, so ``causal`` is accepted either way.
    """
    _reject(k=k, v=v, rotary_cos=rotary_cos, rotary_sin=rotary_sin, cache_batch_idx=cache_batch_idx,
            cache_leftpad=cache_leftpad, window_size=window_size, softcap=softcap, alibi_slopes=alibi_slopes,
            return_softmax_lse=return_softmax_lse)
    table = block_table if block_table is not None else page_table
    if table is None or cache_seqlens is None:
        raise ValueError("the paged path needs block_table (or page_table) and cache_seqlens")
    if q.dim() != 4 or q.size(1) != 1:
        raise NotImplementedError("flash_attn_with_kvcache on this path takes one query token per request: q [B,1,Hq,d]")
    return ops.paged_decode_attention(q, k_cache, v_cache, cache_seqlens, table, softmax_scale=softmax_scale,
                                      max_kv_len=max_seqlen_k, k_scales=k_scales, v_scales=v_scales)


def flash_attn_varlen_func(q: Tensor, k: Tensor, v: Tensor, cu_seqlens_q: Tensor, cu_seqlens_k: Optional[Tensor],
                           max_seqlen_q: int, max_seqlen_k: int, dropout_p: float = 0.0,
                           softmax_scale: Optional[float] = None, causal: bool = False, window_size=(-1, -1),
                           softcap: float = 0.0, alibi_slopes=None, deterministic: bool = False,
                           return_attn_probs: bool = False, block_table: Optional[Tensor] = None,
                           *, seqused_k: Optional[Tensor] = None, k_scales: Optional[Tensor] = None,
                           v_scales: Optional[Tensor] = None) -> Tensor:
    """Paged varlen causal attention: ``q`` is ``[T, Hq, d]``, ``k``/``v`` are the paged caches.

    Per-request key counts come from ``seqused_k`` if given, else from the differences of
    ``cu_seqlens_k``.  The mask is flash-attn's bottom-right aligned causal mask.
    """
    _reject(dropout_p=dropout_p, window_size=window_size, softcap=softcap, alibi_slopes=alibi_slopes,
            return_attn_probs=return_attn_probs)
    if block_table is None:
        raise NotImplementedError("only the paged form (block_table given) exists on this path")
    if not causal:
        raise NotImplementedError("the paged prefill kernel is causal")
    if seqused_k is not None:
        kv_lens = seqused_k
    elif cu_seqlens_k is not None:
        kv_lens = _lengths_of(cu_seqlens_k)
    else:
        raise ValueError("need cu_seqlens_k or seqused_k")
    if k.size(-1) != v.size(-1):
        # decompressed multi-latent caches: keys carry the shared rotary slice, values do not
        if k_scales is not None or v_scales is not None:
            raise NotImplementedError("no fp8 variant for caches with different key / value widths")
        return ops.paged_prefill_attention_mla(
            q, k, v, cu_seqlens_q, kv_lens.to(torch.int32), block_table, max_kv_len=max_seqlen_k,
            softmax_scale=softmax_scale if softmax_scale is not None else q.shape[-1] ** -0.5)
    return ops.paged_prefill_attention(q, k, v, cu_seqlens_q, kv_lens.to(torch.int32), block_table,
                                       softmax_scale=softmax_scale, max_kv_len=max_seqlen_k,
                                       k_scales=k_scales, v_scales=v_scales)


def _flash_attn_forward(q: Tensor, k: Tensor, v: Tensor, k_new=None, v_new=None, qv=None, out: Optional[Tensor] = None,
                        cu_seqlens_q: Optional[Tensor] = None, cu_seqlens_k: Optional[Tensor] = None,
                        cu_seqlens_k_new=None, seqused_q=None, seqused_k: Optional[Tensor] = None,
                        max_seqlen_q: Optional[int] = None, max_seqlen_k: Optional[int] = None,
                        page_table: Optional[Tensor] = None, kv_batch_idx=None, leftpad_k=None, rotary_cos=None,
                        rotary_sin=None, seqlens_rotary=None, q_descale=None, k_descale=None, v_descale=None,
                        softmax_scale: Optional[float] = None, causal: bool = False, window_size=(-1, -1),
                        attention_chunk: int = 0, softcap: float = 0.0, rotary_interleaved: bool = True,
                        scheduler_metadata=None, num_splits: int = 0, pack_gqa=None, sm_margin: int = 0):
    """The flash-attention-3 form of the paged varlen call (attention.py:510-544, taken when the reference finds
    ``flashattn_hopper``): ``q`` ``[T, Hq, d]``, paged caches, ``cu_seqlens_q``, per-request key counts in
    ``seqused_k`` (or the running sums ``cu_seqlens_k``), the block table as ``page_table``.  Returns
    ``(out, None)``: the reference keeps the first element and discards the rest, and the log-sum-exp is not
    produced.  Scheduling hints (``scheduler_metadata``, ``num_splits``, ``pack_gqa``, ``sm_margin``) have no
    meaning here and are ignored; arguments that would change the result are rejected."""
    _reject(k_new=k_new, v_new=v_new, qv=qv, cu_seqlens_k_new=cu_seqlens_k_new, seqused_q=seqused_q,
            kv_batch_idx=kv_batch_idx, leftpad_k=leftpad_k, rotary_cos=rotary_cos, rotary_sin=rotary_sin,
            seqlens_rotary=seqlens_rotary, q_descale=q_descale, k_descale=k_descale, v_descale=v_descale,
            window_size=window_size, attention_chunk=attention_chunk, softcap=softcap)
    if cu_seqlens_q is None:
        raise NotImplementedError("only the varlen form (cu_seqlens_q given) exists on this path")
    res = flash_attn_varlen_func(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k,
                                 softmax_scale=softmax_scale, causal=causal, block_table=page_table,
                                 seqused_k=seqused_k)
    if out is not None:
        out.copy_(res)
        res = out
    return res, None


def get_mla_metadata(cache_seqlens: Tensor, num_heads_per_head_k: int, num_heads_k: int):
    """Counterpart of ``flash_mla.get_mla_metadata`` (called at attention.py:571-575): the streaming
    kernel splits the work on the GPU by itself, so there is no schedule to precompute."""
    return None, None


def flash_mla_with_kvcache(q: Tensor, k_cache: Tensor, block_table: Tensor, cache_seqlens: Tensor, head_dim_v: int,
                           tile_scheduler_metadata=None, num_splits=None, softmax_scale: Optional[float] = None,
                           causal: bool = False):
    """Absorbed multi-latent decode attention with flash_mla's call shape (attention.py:576-587):
    ``q`` ``[batch, 1, Hq, 576]``, ``k_cache`` ``[chunks, chunk_tokens, 1, 576]`` (the latent cache with a
    head dimension added), ``cache_seqlens`` int32 ``[batch]`` counting this step's token.  Returns
    ``(out [batch, 1, Hq, head_dim_v], None)``: the log-sum-exp the reference discards is not produced."""
    if q.dim() != 4 or q.size(1) != 1:
        raise NotImplementedError("flash_mla_with_kvcache on this path takes one query token per request: q [B,1,Hq,d]")
    if softmax_scale is None:
        softmax_scale = q.shape[-1] ** -0.5
    out = ops.paged_mla_decode_attention(q, k_cache, cache_seqlens, block_table, softmax_scale=softmax_scale,
                                         head_dim_v=head_dim_v)
    return out, None
