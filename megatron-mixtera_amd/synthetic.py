"""Seeded synthetic inputs for the five benchmark / parity configurations.

Shapes follow the configuration list of the headline benchmark: a paged KV cache
``[N, C, Hkv, d]`` whose chunks are handed to requests through a seeded random permutation,
context lengths drawn uniformly from a range, one new token per request.  Generation works
on any device: small cases are drawn on the CPU (so a CPU checker sees identical values)
and moved; large cases are drawn slab by slab directly on the GPU.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

import torch
from torch import Tensor


@dataclass(frozen=True)
class DecodeConfig:
    name: str
    batch: int
    Hq: int
    Hkv: int
    d: int
    len_lo: int
    len_hi: int
    chunk: int = 256
    fp8: bool = False
    qk_norm: Optional[str] = None
    rope_theta: Optional[float] = None
    seed: int = 1000


CONFIGS: Dict[str, DecodeConfig] = {
    "cfg1": DecodeConfig("cfg1: B4 8/8 heads d64 len U[64,1024]", 4, 8, 8, 64, 64, 1024, seed=1001),
    "cfg2": DecodeConfig("cfg2: Llama-3-8B layer B64 32/8 d128 len U[512,8192]", 64, 32, 8, 128, 512, 8192,
                         qk_norm="rms", rope_theta=500000.0, seed=1002),
    "cfg3_decode": DecodeConfig("cfg3 decode part: B120 32/8 d128 len U[512,8192]", 120, 32, 8, 128, 512, 8192,
                                seed=1003),
    "cfg4": DecodeConfig("cfg4: 70B layer B16 64/8 d128 len 131072", 16, 64, 8, 128, 131072, 131072, seed=1004),
    "cfg5": DecodeConfig("cfg5: fp8 KV B256 32/8 d128 len U[1024,32768]", 256, 32, 8, 128, 1024, 32768, fp8=True,
                         seed=1005),
}


def draw_lengths(batch: int, lo: int, hi: int, gen: torch.Generator) -> Tensor:
    if lo == hi:
        return torch.full((batch,), lo, dtype=torch.int32)
    return torch.randint(lo, hi + 1, (batch,), generator=gen, dtype=torch.int64).to(torch.int32)


def build_block_table(lens: Tensor, chunk: int, gen: torch.Generator, pool_chunks: Optional[int] = None,
                      max_chunks: Optional[int] = None) -> Tuple[Tensor, int]:
    """Random assignment of physical chunks; id ``N-1`` stays free as the dummy chunk.

    Returns ``(block_table int32 [R, M] padded with -1, N)``.
    """
    need = [(int(l) + chunk - 1) // chunk for l in lens]
    total = sum(need)
    N = max(pool_chunks or 0, total + 1)
    perm = torch.randperm(N - 1, generator=gen)[:total].to(torch.int32)
    M = max_chunks or max(max(need), 1)
    table = torch.full((len(need), M), -1, dtype=torch.int32)
    at = 0
    for r, n in enumerate(need):
        table[r, :n] = perm[at : at + n]
        at += n
    return table, N


def randn_fill_(t: Tensor, gen: torch.Generator, slab_bytes: int = 1 << 28) -> Tensor:
    """Fill ``t`` with N(0,1) through fp32 slabs of bounded size (works for bf16 and large tensors)."""
    flat = t.view(-1)
    step = max(1, slab_bytes // 4)
    for a in range(0, flat.numel(), step):
        b = min(a + step, flat.numel())
        flat[a:b] = torch.randn(b - a, generator=gen, device=t.device, dtype=torch.float32).to(t.dtype)
    return t


@dataclass
class DecodeCase:
    cfg: DecodeConfig
    q: Tensor            # [R, 1, Hq, d] bf16
    k_new: Tensor        # [R, 1, Hkv, d] bf16 -- this step's key / value rows
    v_new: Tensor
    k_cache: Tensor      # [N, C, Hkv, d] bf16 (or uint8 when fp8)
    v_cache: Tensor
    block_table: Tensor  # int32 [R, M]
    kv_lens: Tensor      # int32 [R], counts the token appended this step
    k_scales: Optional[Tensor] = None
    v_scales: Optional[Tensor] = None
    extras: dict = field(default_factory=dict)


def make_decode_case(cfg: DecodeConfig, device, *, batch: Optional[int] = None, seed: Optional[int] = None,
                     on_device_rng: bool = False, pool_chunks: Optional[int] = None,
                     lens: Optional[Tensor] = None, dtype: torch.dtype = torch.bfloat16) -> DecodeCase:
    """Build q, the new K/V rows, a bf16 cache filled with N(0,1), block table and lengths.

    ``on_device_rng=False`` draws values on the CPU and moves them (bit-identical inputs
    for a CPU checker); ``True`` draws the cache on ``device`` (for full-size runs).
    The cache has ``dtype`` (bf16 or fp16) here; fp8 configurations quantise a bf16 one afterwards with the
    library's own kernel or the checker's quantiser.
    """
    device = torch.device(device)
    B = batch or cfg.batch
    cpu_gen = torch.Generator().manual_seed(cfg.seed if seed is None else seed)
    if lens is None:
        lens = draw_lengths(B, cfg.len_lo, cfg.len_hi, cpu_gen)
    table, N = build_block_table(lens, cfg.chunk, cpu_gen, pool_chunks)
    q = torch.randn(B, 1, cfg.Hq, cfg.d, generator=cpu_gen).to(dtype)
    k_new = torch.randn(B, 1, cfg.Hkv, cfg.d, generator=cpu_gen).to(dtype)
    v_new = torch.randn(B, 1, cfg.Hkv, cfg.d, generator=cpu_gen).to(dtype)
    shape = (N, cfg.chunk, cfg.Hkv, cfg.d)
    if on_device_rng and device.type != "cpu":
        dgen = torch.Generator(device=device).manual_seed((cfg.seed if seed is None else seed) + 7)
        k_cache = randn_fill_(torch.empty(shape, dtype=dtype, device=device), dgen)
        v_cache = randn_fill_(torch.empty(shape, dtype=dtype, device=device), dgen)
    else:
        k_cache = randn_fill_(torch.empty(shape, dtype=dtype), cpu_gen).to(device)
        v_cache = randn_fill_(torch.empty(shape, dtype=dtype), cpu_gen).to(device)
    return DecodeCase(cfg, q.to(device), k_new.to(device), v_new.to(device), k_cache, v_cache,
                      table.to(device), lens.to(device))


def make_prefill_case(device, *, n_prefill: int, new_tokens: int, ctx_lo: int, ctx_hi: int, n_decode: int,
                      dec_lo: int, dec_hi: int, Hq: int, Hkv: int, d: int, chunk: int = 256, seed: int = 1003,
                      on_device_rng: bool = False, dtype: torch.dtype = torch.bfloat16):
    """Mixed batch: ``n_prefill`` requests with ``new_tokens`` new tokens over an existing context
    of U[ctx_lo, ctx_hi] tokens, followed by ``n_decode`` one-token requests with total length
    U[dec_lo, dec_hi].  Returns (q [T,Hq,d], k_cache, v_cache, cu_seqlens_q, kv_lens, block_table)."""
    device = torch.device(device)
    gen = torch.Generator().manual_seed(seed)
    ctx = draw_lengths(n_prefill, ctx_lo, ctx_hi, gen) if n_prefill else torch.zeros(0, dtype=torch.int32)
    dec = draw_lengths(n_decode, dec_lo, dec_hi, gen) if n_decode else torch.zeros(0, dtype=torch.int32)
    q_lens = torch.cat([torch.full((n_prefill,), new_tokens, dtype=torch.int32),
                        torch.ones(n_decode, dtype=torch.int32)])
    kv_lens = torch.cat([ctx + new_tokens, dec]).to(torch.int32)
    cu_q = torch.zeros(q_lens.numel() + 1, dtype=torch.int32)
    cu_q[1:] = torch.cumsum(q_lens, 0)
    table, N = build_block_table(kv_lens, chunk, gen)
    T = int(cu_q[-1])
    q = torch.randn(T, Hq, d, generator=gen).to(dtype)
    shape = (N, chunk, Hkv, d)
    if on_device_rng and device.type != "cpu":
        dgen = torch.Generator(device=device).manual_seed(seed + 7)
        k_cache = randn_fill_(torch.empty(shape, dtype=dtype, device=device), dgen)
        v_cache = randn_fill_(torch.empty(shape, dtype=dtype, device=device), dgen)
    else:
        k_cache = randn_fill_(torch.empty(shape, dtype=dtype), gen).to(device)
        v_cache = randn_fill_(torch.empty(shape, dtype=dtype), gen).to(device)
    return q.to(device), k_cache, v_cache, cu_q.to(device), kv_lens.to(device), table.to(device)


def prefill_token_rows(cu_seqlens_q: Tensor, kv_lens: Tensor, block_table: Tensor, chunk: int):
    """Per-token rows of a mixed batch, as the context would hold them: position in the request,
    physical chunk id and position inside the chunk of every new token (int64, on the inputs' device).
    Token i of request r (Lq new tokens over Lk - Lq cached ones) sits at position Lk - Lq + i."""
    cu = cu_seqlens_q.long()
    lq = cu[1:] - cu[:-1]
    T = int(cu[-1])
    req = torch.repeat_interleave(torch.arange(lq.numel(), device=cu.device), lq)
    pos = torch.arange(T, device=cu.device) - cu[req] + (kv_lens.long() - lq)[req]
    chunk_idx = block_table.long()[req, pos // chunk]
    return pos.contiguous(), chunk_idx.contiguous(), (pos % chunk).contiguous()


def rotary_angle_table(max_seq_len: int, dim: int, base: float = 10000.0) -> Tensor:
    """fp32 ``[max_seq_len, 1, 1, dim]`` table of rotary angles in the layout the model hands to the
    context (``emb = cat(freqs, freqs)`` with ``freqs = outer(positions, 1 / base^(2i/dim))``,
    rotary_pos_embedding.py:79-81,151-181) -- a synthetic input for benchmarks and examples."""
    inv_freq = 1.0 / (base ** (torch.arange(0, dim, 2, dtype=torch.float32) / dim))
    freqs = torch.outer(torch.arange(max_seq_len, dtype=torch.float32), inv_freq)
    return torch.cat((freqs, freqs), dim=-1)[:, None, None, :]


def decode_attention_bytes(kv_lens, Hq: int, Hkv: int, d: int, chunk: int, kv_bytes: int = 2,
                           fp8_scales: bool = False) -> int:
    """Bytes one decode-attention call has to move: every cached K and V row once, q in, out back,
    the block-table entries and lengths in use (and the per-chunk scales of an fp8 cache)."""
    lens = [int(x) for x in kv_lens]
    chunks = sum((l + chunk - 1) // chunk for l in lens)
    total = sum(lens) * Hkv * d * 2 * kv_bytes + len(lens) * Hq * d * (2 + 2) + chunks * 4 + len(lens) * 4
    if fp8_scales:
        total += chunks * Hkv * 2 * 4
    return total
