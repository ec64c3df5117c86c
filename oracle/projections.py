"""CPU restatement of the two projections around the attention path -- TEST INFRASTRUCTURE ONLY.

``linear`` follows ColumnParallelLinear / RowParallelLinear at tensor-parallel size 1
(megatron/core/tensor_parallel/layers.py:946-1010 and :1225-1290): ``output = input @ weight.T`` with the bias added
unless ``skip_bias_add``, in which case it is handed back; the result has the inputs' 16-bit type.  ``qkv_split``
follows Attention.get_query_key_value_tensors (megatron/core/transformer/attention.py:985-1030): the projection's
output ``[T, ng * (np/ng + 2) * hn]`` viewed per KV group and split into query ``[T, np, hn]``, key and value
``[T, ng, hn]``.

Pinned by: ``torch.nn.functional.linear`` in float64 (a library routine) on random inputs and the closed forms
``linear(x, I) == x`` and ``linear(x, W, b)[t, n] == dot(x[t], W[n]) + b[n]`` as Python loops on tiny inputs
(``tests/test_oracle_projections.py``); ``qkv_split`` by a hand-laid-out tensor whose entries name their own
(group, role, head, element).
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch
from torch import Tensor


def linear(x: Tensor, weight: Tensor, bias: Optional[Tensor] = None, skip_bias_add: bool = False) -> Tuple[Tensor, Optional[Tensor]]:
    """``(output, output_bias)`` as the reference's linear layers return them (layers.py:1004-1010, 1283-1290):
    fp32 accumulation here, rounded once to the inputs' type."""
    y = x.float() @ weight.float().t()
    if bias is not None and not skip_bias_add:
        y = y + bias.float()
    return y.to(x.dtype), (bias if skip_bias_add else None)


def qkv_split(mixed_qkv: Tensor, num_query_heads: int, num_kv_heads: int, head_dim: int) -> Tuple[Tensor, Tensor, Tensor]:
    """attention.py:994-1020: ``[T, ng * (np/ng + 2) * hn]`` -> query ``[T, np, hn]``, key / value ``[T, ng, hn]``."""
    T = mixed_qkv.size(0)
    G = num_query_heads // num_kv_heads
    grouped = mixed_qkv.reshape(T, num_kv_heads, (G + 2) * head_dim)
    q, k, v = torch.split(grouped, [G * head_dim, head_dim, head_dim], dim=2)
    return q.reshape(T, num_query_heads, head_dim), k, v
