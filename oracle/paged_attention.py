"""fp32 oracle for paged attention, KV append, LSE merge and fp8 KV storage.

Restates, on CPU tensors:
* ``key_value_cache`` + block-table addressing: ``K_r[j] = k_cache[block_table[r, j // C], j % C]``
  (megatron/core/inference/contexts/dynamic_context.py:547-564, 811-825);
* the unfused core attention the reference documents as its math -- GQA by repeating KV
  heads, scores scaled by ``d**-0.5``, fp32 softmax, weighted sum of V
  (megatron/core/transformer/dot_product_attention.py:159-235,
  megatron/core/fusions/fused_softmax.py:299-342);
* flash-attn's call contract at megatron/core/transformer/attention.py:546-557,589-600:
  bottom-right aligned causal mask, kv length includes the token appended this step;
* ``append_key_value_cache`` (dynamic_context.py:511-545).

Pinned by (tests/test_oracle_attention.py): torch.nn.functional.scaled_dot_product_attention
on gathered K/V (library routine, incl. an explicit bottom-right mask and GQA), fp64 brute
force loops on tiny cases, invariance under chunk-id permutation, all-equal-K => mean of V,
single-key => V itself, split + LSE merge == single pass, zero-length row => zeros.
fp8: torch's own ``float8_e4m3fn`` cast is the rounding reference.
"""
from __future__ import annotations

import math
from typing import List, Optional, Sequence, Tuple

import torch
from torch import Tensor

E4M3_MAX = 448.0


def gather_request_kv(cache: Tensor, block_table_row: Tensor, length: int) -> Tensor:
    """Logical ``[length, Hkv, d]`` view of one request's keys (or values) as fp32."""
    C = cache.size(1)
    n_chunks = (length + C - 1) // C
    ids = block_table_row[:n_chunks].long()
    flat = cache[ids].reshape(n_chunks * C, cache.size(2), cache.size(3))
    return flat[:length].float()


def attention_one_request(q: Tensor, k: Tensor, v: Tensor, scale: float, causal_shift: Optional[int]) -> Tensor:
    """``q`` [Lq,Hq,d], ``k`` [Lk,Hkv,d], ``v`` [Lk,Hkv,dv] fp32 -> [Lq,Hq,dv] fp32 (dv = d except for the
    decompressed caches of multi-latent attention, whose keys are wider than their values).

    ``causal_shift`` = Lk - Lq for the bottom-right aligned mask (query i sees keys
    j <= i + shift); ``None`` disables masking.
    """
    Lq, Hq, d = q.shape
    Lk, Hkv, _ = k.shape
    G = Hq // Hkv
    if Lk == 0:
        return torch.zeros(Lq, Hq, v.size(-1))
    # Query head h reads KV head h // G: the same pairing as repeating every KV head G times
    # (dot_product_attention.py:159-165), written without materialising the copies.
    qg = q.reshape(Lq, Hkv, G, d)
    scores = torch.einsum("qhgd,khd->hgqk", qg, k) * scale
    if causal_shift is not None:
        qi = torch.arange(Lq).view(Lq, 1)
        kj = torch.arange(Lk).view(1, Lk)
        scores = scores.masked_fill(kj > qi + causal_shift, float("-inf"))
    probs = torch.softmax(scores, dim=-1)
    probs = torch.nan_to_num(probs, nan=0.0)  # rows with no visible key
    return torch.einsum("hgqk,khd->qhgd", probs, v).reshape(Lq, Hq, v.size(-1))


def paged_decode_attention(q: Tensor, k_cache: Tensor, v_cache: Tensor, kv_lens: Tensor, block_table: Tensor,
                           softmax_scale: Optional[float] = None, k_scales: Optional[Tensor] = None,
                           v_scales: Optional[Tensor] = None) -> Tensor:
    """Decode: ``q`` [R,Hq,d] (one token per request) -> fp32 [R,Hq,d]."""
    R, Hq, d = q.shape
    scale = d ** -0.5 if softmax_scale is None else softmax_scale
    out = torch.zeros(R, Hq, d, dtype=torch.float32)
    if k_scales is not None:
        k_cache = dequantize_fp8(k_cache, k_scales)
        v_cache = dequantize_fp8(v_cache, v_scales)
    for r in range(R):
        L = int(kv_lens[r])
        if L <= 0:
            continue
        k = gather_request_kv(k_cache, block_table[r], L)
        v = gather_request_kv(v_cache, block_table[r], L)
        out[r] = attention_one_request(q[r : r + 1].float(), k, v, scale, None)[0]
    return out


def mla_decode_attention(q: Tensor, latent_cache: Tensor, kv_lens: Tensor, block_table: Tensor,
                         softmax_scale: float, head_dim_v: int) -> Tensor:
    """Absorbed multi-latent decode attention, the arithmetic flash_mla_with_kvcache is called for at
    megatron/core/transformer/attention.py:561-587: ``q`` [R,Hq,dk]; ``latent_cache`` [N,C,dk] holds one
    row per token shared by every head; scores over all dk values, output = weighted sum of the first
    ``head_dim_v`` values of the rows.  fp32 [R,Hq,head_dim_v]."""
    R, Hq, dk = q.shape
    C = latent_cache.size(1)
    out = torch.zeros(R, Hq, head_dim_v, dtype=torch.float32)
    for r in range(R):
        L = int(kv_lens[r])
        if L <= 0:
            continue
        n = (L + C - 1) // C
        rows = latent_cache[block_table[r, :n].long()].reshape(n * C, dk)[:L].float()
        probs = torch.softmax(q[r].float() @ rows.T * softmax_scale, dim=-1)
        out[r] = probs @ rows[:, :head_dim_v]
    return out


def paged_varlen_attention(q: Tensor, k_cache: Tensor, v_cache: Tensor, cu_seqlens_q: Tensor, kv_lens: Tensor,
                           block_table: Tensor, softmax_scale: Optional[float] = None,
                           k_scales: Optional[Tensor] = None, v_scales: Optional[Tensor] = None) -> Tensor:
    """Prefill / mixed: ``q`` [T,Hq,d]; request r owns rows cu_q[r]:cu_q[r+1] and kv_lens[r] keys.
    With scales the caches are e4m3fn bytes, dequantised to fp32 first."""
    if k_scales is not None:
        k_cache = dequantize_fp8(k_cache, k_scales)
        v_cache = dequantize_fp8(v_cache, v_scales)
    T, Hq, d = q.shape
    scale = d ** -0.5 if softmax_scale is None else softmax_scale
    out = torch.zeros(T, Hq, v_cache.size(-1), dtype=torch.float32)
    for r in range(cu_seqlens_q.numel() - 1):
        a, b = int(cu_seqlens_q[r]), int(cu_seqlens_q[r + 1])
        L = int(kv_lens[r])
        if b <= a:
            continue
        if L <= 0:
            continue
        k = gather_request_kv(k_cache, block_table[r], L)
        v = gather_request_kv(v_cache, block_table[r], L)
        out[a:b] = attention_one_request(q[a:b].float(), k, v, scale, L - (b - a))
    return out


def kv_append(k_cache: Tensor, v_cache: Tensor, key: Tensor, value: Tensor, chunk_idx: Tensor,
              local_pos: Tensor) -> None:
    """In-place scatter ``cache[chunk_idx[t], local_pos[t]] = row[t]`` (token order; last writer wins)."""
    for t in range(key.size(0)):
        k_cache[int(chunk_idx[t]), int(local_pos[t])] = key[t]
        v_cache[int(chunk_idx[t]), int(local_pos[t])] = value[t]


def decode_slots(block_table: Tensor, kv_lens: Tensor, chunk: int) -> Tuple[Tensor, Tensor, Tensor]:
    """(rows, chunk ids, local positions) of the token appended this step for rows with len > 0."""
    rows = torch.nonzero(kv_lens > 0, as_tuple=True)[0]
    pos = kv_lens[rows].long() - 1
    ids = block_table[rows, pos // chunk].long()
    return rows, ids, pos % chunk


def lse_merge(partials: Sequence[Tensor], lses: Sequence[Tensor]) -> Tensor:
    """o = sum_s e^{lse_s - m} o_s / sum_s e^{lse_s - m}; ``partials[s]`` [..., d], ``lses[s]`` [...]."""
    lse = torch.stack(list(lses), dim=0).double()
    o = torch.stack(list(partials), dim=0).double()
    w = torch.exp(lse - lse.max(dim=0, keepdim=True).values)
    return ((w.unsqueeze(-1) * o).sum(0) / w.sum(0).unsqueeze(-1)).float()


def attention_with_lse(q: Tensor, k: Tensor, v: Tensor, scale: float) -> Tuple[Tensor, Tensor]:
    """Unmasked single-request attention returning (out [Lq,Hq,d], natural-log LSE [Lq,Hq])."""
    Lq, Hq, d = q.shape
    Hkv = k.size(1)
    qg = q.reshape(Lq, Hkv, Hq // Hkv, d)
    s = torch.einsum("qhgd,khd->hgqk", qg, k) * scale
    lse = torch.logsumexp(s, dim=-1)  # [Hkv, G, Lq]
    out = torch.einsum("hgqk,khd->qhgd", torch.softmax(s, dim=-1), v).reshape(Lq, Hq, d)
    return out, lse.permute(2, 0, 1).reshape(Lq, Hq)


# --------------------------------------------------------------------------------------------
# fp8 (OCP e4m3fn) KV storage with one fp32 scale per (chunk, KV head)
# --------------------------------------------------------------------------------------------
def quantize_chunks_fp8(cache: Tensor) -> Tuple[Tensor, Tensor]:
    """``cache`` [N,C,Hkv,d] -> (uint8 e4m3fn bytes, fp32 scales [N,Hkv]); scale = amax / 448."""
    x = cache.float()
    amax = x.abs().amax(dim=(1, 3))
    scale = torch.where(amax > 0, amax / E4M3_MAX, torch.ones_like(amax))
    y = (x / scale[:, None, :, None]).clamp(-E4M3_MAX, E4M3_MAX)
    return y.to(torch.float8_e4m3fn).view(torch.uint8), scale


def dequantize_fp8(cache_bytes: Tensor, scales: Tensor) -> Tensor:
    return cache_bytes.view(torch.float8_e4m3fn).float() * scales[:, None, :, None]


def quantize_token_fp8(row: Tensor, scale: Tensor) -> Tensor:
    """``row`` [Hkv,d], ``scale`` [Hkv] -> uint8 e4m3fn bytes (saturating)."""
    y = (row.float() / scale[:, None]).clamp(-E4M3_MAX, E4M3_MAX)
    return y.to(torch.float8_e4m3fn).view(torch.uint8)


def kv_append_fp8(cache_bytes: Tensor, scales: Tensor, rows: Tensor, chunk_idx: Tensor, local: Tensor,
                  headroom: float = 2.0) -> None:
    """The library's fp8 append policy for many tokens per call, in scalar loops (in place).

    ``cache_bytes`` uint8 [N,C,Hkv,d], ``scales`` fp32 [N,Hkv], ``rows`` bf16 [T,Hkv,d]; token t goes to
    (chunk_idx[t], local[t]).  Consecutive tokens of one chunk with rising local positions form a run.
    A run starting at local 0 opens the chunk: per head, scale = amax(run) / 448, times ``headroom`` unless
    the run fills the chunk (zero amax -> scale 1); a run starting further in reuses the stored scale.
    Values are divided by the scale in fp32, clamped to +-448 and rounded to e4m3fn (nearest even).
    This policy has no counterpart in the reference (its cache is never quantised)."""
    C = cache_bytes.size(1)
    T = rows.size(0)
    t = 0
    while t < T:
        c, l0 = int(chunk_idx[t]), int(local[t])
        n = 1
        while t + n < T and int(chunk_idx[t + n]) == c and int(local[t + n]) == l0 + n and l0 + n < C:
            n += 1
        if l0 == 0:
            amax = rows[t:t + n].float().abs().amax(dim=(0, 2))
            hr = 1.0 if n == C else headroom
            scales[c] = torch.where(amax > 0, (torch.tensor(hr, dtype=torch.float32) * amax) / E4M3_MAX,
                                    torch.ones_like(amax))
        for i in range(n):
            cache_bytes[c, l0 + i] = quantize_token_fp8(rows[t + i], scales[c])
        t += n


def decode_attention_bytes(kv_lens: Sequence[int], Hq: int, Hkv: int, d: int, chunk: int, kv_bytes: int = 2,
                           fp8_scales: bool = False) -> int:
    """Algorithmic HBM bytes of one decode-attention call (KV once, q in, out, table, lengths)."""
    lens = [int(x) for x in kv_lens]
    total = sum(lens) * Hkv * d * 2 * kv_bytes
    total += len(lens) * Hq * d * (2 + 2)
    chunks = sum((l + chunk - 1) // chunk for l in lens)
    total += chunks * 4 + len(lens) * 4
    if fp8_scales:
        total += chunks * Hkv * 2 * 4
    return total
