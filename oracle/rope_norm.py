"""Oracle for the rotary table, RoPE application and the q/k head norms.

Restates:
* ``RotaryEmbedding``: inv_freq = 1 / base^(2i/dim), optional llama-3 frequency scaling,
  angles = outer(positions, inv_freq), table = cat(angles, angles) (or pairwise repeated when
  interleaved)  (megatron/core/models/common/embeddings/rotary_pos_embedding.py:58-181);
* ``_rotate_half`` / ``_apply_rotary_pos_emb_bshd``: cos and sin are cast to the tensor dtype
  BEFORE the multiply, pass-through tail beyond rot_dim
  (megatron/core/models/common/embeddings/rope_utils.py:73-126);
* gather of the table by per-token positions (dynamic_context.py:587-589, 619-621);
* q/k layernorm = torch RMSNorm over the head dim or L2Norm
  (megatron/core/transformer/attention.py:1026-1030, torch_norm.py:15-96);
* the split of the QKV projection's output into per-head query / key / value
  (``SelfAttention.get_query_key_value_tensors``, megatron/core/transformer/attention.py:985-1024).

Pinned by (tests/test_oracle_rope_norm.py): position 0 is the identity; fp64 complex
multiplication by e^{i theta}; pairwise norm preservation; torch.nn.functional.rms_norm
(library routine); llama-3 scaling against the published three-band formula evaluated in
fp64 for a low, a medium and a high frequency; the QKV split against hand-computed element
offsets of an ``arange`` row and a scalar triple loop.
"""
from __future__ import annotations

import math
from typing import Optional

import torch
from torch import Tensor


def inv_freq(dim: int, base: float = 10000.0, rope_scaling: bool = False, factor: float = 8.0,
             low_freq_factor: float = 1.0, high_freq_factor: float = 4.0, original_max_pos: int = 8192) -> Tensor:
    f = 1.0 / (base ** (torch.arange(0, dim, 2, dtype=torch.float32) / dim))
    if not rope_scaling:
        return f
    wavelen = 2 * math.pi / f
    low_w = original_max_pos / low_freq_factor
    high_w = original_max_pos / high_freq_factor
    scaled = torch.where(wavelen > low_w, f / factor, f)
    smooth = (original_max_pos / wavelen - low_freq_factor) / (high_freq_factor - low_freq_factor)
    mid = (1 - smooth) * scaled / factor + smooth * scaled
    is_mid = ~(wavelen < high_w) & ~(wavelen > low_w)
    return torch.where(is_mid, mid, scaled)


def rotary_table(max_seq_len: int, dim: int, base: float = 10000.0, interleaved: bool = False,
                 rope_scaling: bool = False, factor: float = 8.0, offset: int = 0,
                 seq_len_interpolation_factor: Optional[float] = None) -> Tensor:
    """fp32 ``[max_seq_len, 1, 1, dim]`` table of angles as RotaryEmbedding.forward returns it."""
    f = inv_freq(dim, base, rope_scaling, factor)
    seq = torch.arange(max_seq_len, dtype=torch.float32) + offset
    if seq_len_interpolation_factor is not None:
        seq = seq * (1 / seq_len_interpolation_factor)
    ang = torch.outer(seq, f)
    if interleaved:
        emb = torch.stack((ang.view(-1, 1), ang.view(-1, 1)), dim=-1).view(ang.shape[0], -1)
    else:
        emb = torch.cat((ang, ang), dim=-1)
    return emb[:, None, None, :]


def rotate_half(x: Tensor, interleaved: bool) -> Tensor:
    if not interleaved:
        x1, x2 = torch.chunk(x, 2, dim=-1)
        return torch.cat((-x2, x1), dim=-1)
    x1, x2 = x[..., ::2], x[..., 1::2]
    return torch.stack((-x2, x1), dim=-1).reshape(x.shape)


def apply_rope(t: Tensor, angles: Tensor, interleaved: bool = False, mscale: float = 1.0) -> Tensor:
    """``t`` [T, H, d] (any float dtype), ``angles`` [T, rot] fp32 -> same dtype as ``t``.

    Evaluated op by op in ``t.dtype`` exactly like the reference chain.
    """
    rot = angles.shape[-1]
    a = angles[:, None, :]
    tr, tp = t[..., :rot], t[..., rot:]
    cos_ = (torch.cos(a) * mscale).to(t.dtype)
    sin_ = (torch.sin(a) * mscale).to(t.dtype)
    tr = (tr * cos_) + (rotate_half(tr, interleaved) * sin_)
    return torch.cat((tr, tp), dim=-1)


def apply_rope_fp32(t: Tensor, angles: Tensor, interleaved: bool = False, mscale: float = 1.0) -> Tensor:
    """Same formula, everything in fp32, no intermediate rounding (returns fp32)."""
    return apply_rope(t.float(), angles, interleaved, mscale)


def rms_norm(x: Tensor, weight: Optional[Tensor], eps: float) -> Tensor:
    """RMSNorm over the last dim: fp32 internally, weight applied in fp32, one final rounding."""
    xf = x.float()
    y = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    if weight is not None:
        y = y * weight.float()
    return y.to(x.dtype)


def l2_norm(x: Tensor, eps: float = 1e-6) -> Tensor:
    xf = x.float()
    return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)).type_as(x)


def norm_rope(x: Tensor, positions: Tensor, table: Optional[Tensor], *, norm: Optional[str] = None,
              weight: Optional[Tensor] = None, eps: float = 1e-5, interleaved: bool = False,
              mscale: float = 1.0) -> Tensor:
    """Head norm then RoPE on ``x`` [T,H,d], op by op in ``x.dtype`` (the unfused reference chain)."""
    if norm == "rms":
        x = rms_norm(x, weight, eps)
    elif norm == "l2":
        x = l2_norm(x, eps)
    if table is None:
        return x
    tab = table.reshape(table.shape[0], table.shape[-1])
    return apply_rope(x, tab[positions.long()], interleaved, mscale)


def split_mixed_qkv(mixed_qkv: Tensor, num_query_heads: int, num_kv_heads: int):
    """``[T, 1, (Hq + 2 Hkv) d]`` -> query ``[T, 1, Hq, d]``, key and value ``[T, 1, Hkv, d]``.

    The projection's columns are ordered by query group: the G = Hq/Hkv query heads of the group,
    then its key head, then its value head (attention.py:989-1024: view as
    ``[sq, b, ng, (np/ng + 2) hn]``, split ``[np/ng * hn, hn, hn]`` along the last dim, reshape the
    query to ``[sq, b, np, hn]``).
    """
    t, b, w = mixed_qkv.shape
    g = num_query_heads // num_kv_heads
    d = w // (num_query_heads + 2 * num_kv_heads)
    grouped = mixed_qkv.view(t, b, num_kv_heads, (g + 2) * d)
    query, key, value = torch.split(grouped, [g * d, d, d], dim=3)
    return query.reshape(t, b, num_query_heads, d), key, value
