"""Attention-side glue of the dynamic inference path, as free functions and a small module.

Mirrors the pieces of ``Attention`` that run between the QKV projection and the output
projection when ``inference_context`` is a dynamic context
(megatron/core/transformer/attention.py:394-414 ``_adjust_key_value_for_inference`` dynamic
branch, :470-601 ``flash_decode_and_prefill``, :740-790 rotary on the query), so a
``SelfAttention`` subclass injected through a ModuleSpec only has to forward to them.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch
from torch import Tensor

from .flash_attn_interface import (
    flash_attn_varlen_func,
    flash_attn_with_kvcache,
    flash_mla_with_kvcache,
    get_mla_metadata,
)


def adjust_key_value_for_inference(inference_context, layer_number: int, query: Tensor, key: Tensor, value: Tensor,
                                   rotary_pos_emb, config, cp_group=None):
    """RoPE(K) -> append(K, V) -> fetch cache views, in the reference's order.

    Returns ``(query, k_cache, v_cache, rotary_pos_emb, block_table)`` where the returned
    ``rotary_pos_emb`` is ``(q_pos_emb, None)``: the key half has been applied.
    """
    if rotary_pos_emb is not None:
        q_pos_emb, k_pos_emb = rotary_pos_emb
        key = inference_context.apply_rotary_emb_key(key, k_pos_emb, config, cp_group)
        rotary_pos_emb = (q_pos_emb, None)
    inference_context.append_key_value_cache(layer_number, key, value)
    k_cache, v_cache, block_table = inference_context.key_value_cache(layer_number)
    return query, k_cache, v_cache, rotary_pos_emb, block_table


def flash_decode_and_prefill(q: Tensor, k: Tensor, v: Tensor, max_seqlen_q, max_seqlen_k, cu_seqlens_q,
                             cu_seqlens_k, seqlens_k, block_table, softmax_scale: Optional[float] = None, *,
                             k_scales: Optional[Tensor] = None, v_scales: Optional[Tensor] = None,
                             mla_head_dim_v: Optional[int] = None) -> Tensor:
    """Same contract as ``Attention.flash_decode_and_prefill`` (attention.py:470-601).

    ``q`` is ``[T, 1, Hq, d]``; ``k`` / ``v`` are the paged caches.  ``max_seqlen_q == 1``
    selects the decode kernel, anything else the varlen causal kernel.  ``k_scales`` / ``v_scales``
    (an addition) go with byte caches holding e4m3 values.  ``mla_head_dim_v`` (the reference tests
    ``isinstance(self.config, MLATransformerConfig)`` and reads ``config.kv_lora_rank`` instead) selects the
    absorbed multi-latent decode: ``k`` is then the latent cache and ``v`` is ``None``.
    """
    if max_seqlen_q > 1:
        out = flash_attn_varlen_func(q.squeeze(1), k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k,
                                     softmax_scale=softmax_scale if softmax_scale is not None else q.shape[-1] ** -0.5,
                                     causal=True, block_table=block_table, seqused_k=seqlens_k,
                                     k_scales=k_scales, v_scales=v_scales)
        return out.unsqueeze(1)
    if mla_head_dim_v is not None:
        metadata, num_splits = get_mla_metadata(seqlens_k, q.size(2), 1)
        out, _ = flash_mla_with_kvcache(q, k.unsqueeze(-2), block_table, seqlens_k, mla_head_dim_v, metadata,
                                        num_splits, softmax_scale=softmax_scale, causal=True)
        return out
    return flash_attn_with_kvcache(q=q, k_cache=k, v_cache=v, cache_seqlens=seqlens_k, causal=True,
                                   block_table=block_table, softmax_scale=softmax_scale, max_seqlen_k=max_seqlen_k,
                                   k_scales=k_scales, v_scales=v_scales)


class PagedSelfAttentionCore(torch.nn.Module):
    """Everything between ``get_query_key_value_tensors`` and ``linear_proj`` for one layer.

    ``forward(query, key, value, inference_context, rotary_pos_emb)`` takes the split,
    per-head tensors ``[T, 1, H, d]`` and returns ``[T, 1, Hq*d]`` like
    ``Attention.forward`` does before the output projection (attention.py:815-829).
    With ``fused=True`` the q/k norm, both RoPE applications and the KV-append run as one
    launch; otherwise the reference's call sequence on the context is kept.
    """

    def __init__(self, layer_number: int, head_dim: int, *, qk_norm: Optional[str] = None, eps: float = 1e-5,
                 softmax_scale: Optional[float] = None, rotary_interleaved: bool = False, fused: bool = True,
                 dtype: torch.dtype = torch.bfloat16, device=None):
        super().__init__()
        self.layer_number = layer_number
        self.head_dim = head_dim
        self.qk_norm = qk_norm
        self.eps = eps
        self.softmax_scale = softmax_scale
        self.fused = fused
        self.config = type("RopeConfig", (), {"rotary_interleaved": rotary_interleaved,
                                                "multi_latent_attention": False})()
        if qk_norm == "rms":
            self.q_layernorm_weight = torch.nn.Parameter(torch.ones(head_dim, dtype=dtype, device=device))
            self.k_layernorm_weight = torch.nn.Parameter(torch.ones(head_dim, dtype=dtype, device=device))
        else:
            self.q_layernorm_weight = self.k_layernorm_weight = None

    def forward_mixed_qkv(self, mixed_qkv: Tensor, num_query_heads: int, inference_context,
                          rotary_pos_emb: Optional[Tuple[Tensor, Tensor]] = None) -> Tensor:
        """Same as :meth:`forward`, starting from the QKV projection's output ``[T, 1, (Hq + 2 Hkv) d]``:
        the split of ``get_query_key_value_tensors`` (attention.py:985-1030) is folded into the fused
        norm / RoPE / append launch, so no per-head q / k / v tensors are materialised."""
        ctx = inference_context
        emb = None
        if rotary_pos_emb is not None:
            q_emb, k_emb = rotary_pos_emb if isinstance(rotary_pos_emb, tuple) else (rotary_pos_emb,) * 2
            assert q_emb is k_emb or q_emb is None or k_emb is None or q_emb.data_ptr() == k_emb.data_ptr(), \
                "the fused path takes one rotary table for query and key"
            emb = q_emb if q_emb is not None else k_emb
        if self.fused and self._step_fusable(ctx, emb):
            out = ctx.fused_decode_step_attention(
                self.layer_number, mixed_qkv=mixed_qkv, num_query_heads=num_query_heads, rotary_pos_emb=emb,
                softmax_scale=self.softmax_scale, **self._norm_args())
            return out.reshape(out.size(0), out.size(1), -1)
        query = ctx.fused_qkv_norm_rope_append(
            self.layer_number, mixed_qkv, num_query_heads=num_query_heads, rotary_pos_emb=emb, config=self.config,
            q_weight=None if self.q_layernorm_weight is None else self.q_layernorm_weight.data,
            k_weight=None if self.k_layernorm_weight is None else self.k_layernorm_weight.data,
            norm=self.qk_norm, eps=self.eps)
        return self._attend(query, ctx)

    def forward(self, query: Tensor, key: Tensor, value: Tensor, inference_context,
                rotary_pos_emb: Optional[Tuple[Tensor, Tensor]] = None) -> Tensor:
        ctx = inference_context
        q_emb = k_emb = None
        if rotary_pos_emb is not None:
            q_emb, k_emb = rotary_pos_emb if isinstance(rotary_pos_emb, tuple) else (rotary_pos_emb,) * 2
        if self.fused:
            assert q_emb is k_emb or q_emb is None or k_emb is None or q_emb.data_ptr() == k_emb.data_ptr(), \
                "the fused path takes one rotary table for query and key"
            if self._step_fusable(ctx, q_emb if q_emb is not None else k_emb):
                out = ctx.fused_decode_step_attention(
                    self.layer_number, query, key, value, rotary_pos_emb=q_emb if q_emb is not None else k_emb,
                    softmax_scale=self.softmax_scale, **self._norm_args())
                return out.reshape(out.size(0), out.size(1), -1)
            ctx.fused_qk_norm_rope_append(
                self.layer_number, query, key, value, rotary_pos_emb=q_emb if q_emb is not None else k_emb,
                config=self.config, q_weight=None if self.q_layernorm_weight is None else self.q_layernorm_weight.data,
                k_weight=None if self.k_layernorm_weight is None else self.k_layernorm_weight.data,
                norm=self.qk_norm, eps=self.eps)
        else:
            from . import ops
            if self.qk_norm is not None:
                n = ctx.padded_active_token_count
                ops.norm_rope_append(query[:n], key[:n], key_out=key[:n], norm=self.qk_norm, eps=self.eps,
                                     q_weight=None if self.q_layernorm_weight is None else self.q_layernorm_weight.data,
                                     k_weight=None if self.k_layernorm_weight is None else self.k_layernorm_weight.data)
            if k_emb is not None:
                key = ctx.apply_rotary_emb_key(key, k_emb, self.config, None)
            ctx.append_key_value_cache(self.layer_number, key, value)
            if q_emb is not None:
                query = ctx.apply_rotary_emb_query(query, q_emb, self.config, None, None)
        return self._attend(query, ctx)

    def _norm_args(self) -> dict:
        return dict(config=self.config, norm=self.qk_norm, eps=self.eps,
                    q_weight=None if self.q_layernorm_weight is None else self.q_layernorm_weight.data,
                    k_weight=None if self.k_layernorm_weight is None else self.k_layernorm_weight.data)

    def _step_fusable(self, ctx, emb: Optional[Tensor]) -> bool:
        """Decode-only steps over 16-bit caches run norm, RoPE, append and attention as one streaming kernel
        (plus its merge) when the shapes allow; a context without that method keeps the separate launches."""
        check = getattr(ctx, "decode_step_fusable", None)
        return check is not None and check(self.head_dim, emb, self.config)

    def _attend(self, query: Tensor, ctx) -> Tensor:
        k_cache, v_cache, block_table = ctx.key_value_cache(self.layer_number)
        if hasattr(ctx, "attention_length_bounds"):
            # the host-side bounds decide which kernel runs and how the keys are split; taking the exact
            # maxima (cu_query_lengths / cu_kv_lengths, as the reference does) would wait for the device
            cu_q, cu_k, kv_lens = ctx.cu_query_seq_lengths, ctx.cu_kv_seq_lengths, ctx.kv_seq_lengths
            max_q, max_k = ctx.attention_length_bounds()
        else:
            cu_q, max_q = ctx.cu_query_lengths()
            cu_k, kv_lens, max_k = ctx.cu_kv_lengths()
        k_scales, v_scales = ctx.key_value_scales(self.layer_number) if hasattr(ctx, "key_value_scales") else (None, None)
        out = flash_decode_and_prefill(query, k_cache, v_cache, max_q, max_k, cu_q, cu_k, kv_lens, block_table,
                                       softmax_scale=self.softmax_scale, k_scales=k_scales, v_scales=v_scales)
        return out.reshape(out.size(0), out.size(1), -1)


class DecodeLinear(torch.nn.Module):
    """``linear_qkv`` / ``linear_proj`` of the attention layer at tensor-parallel size 1, with the reference's call
    contract (megatron/core/tensor_parallel/layers.py:946-1010 ColumnParallelLinear, :1225-1290 RowParallelLinear):
    ``forward(input_) -> (output, output_bias)``, where the bias is added to the output unless ``skip_bias_add`` and
    is handed back instead when it is.  Steps of at most 256 rows run the weight-streaming kernel
    (``ops.linear_decode``); larger (prompt-sized) inputs are plain library GEMMs.
    """

    DECODE_ROWS = 256

    def __init__(self, input_size: int, output_size: int, *, bias: bool = True, skip_bias_add: bool = False,
                 dtype: torch.dtype = torch.bfloat16, device=None):
        super().__init__()
        self.input_size, self.output_size, self.skip_bias_add = input_size, output_size, skip_bias_add
        self.weight = torch.nn.Parameter(torch.empty(output_size, input_size, dtype=dtype, device=device))
        self.bias = torch.nn.Parameter(torch.zeros(output_size, dtype=dtype, device=device)) if bias else None

    def forward(self, input_: Tensor):
        from . import ops
        add = None if (self.bias is None or self.skip_bias_add) else self.bias.data
        rows = input_.numel() // input_.size(-1)
        if rows <= self.DECODE_ROWS:
            output = ops.linear_decode(input_, self.weight.data, add)
        else:
            output = torch.nn.functional.linear(input_, self.weight, add)
        return output, (self.bias if self.skip_bias_add else None)


class PagedSelfAttentionLayer(torch.nn.Module):
    """One attention layer of the dynamic inference path from hidden states to hidden states: what
    ``Attention.forward`` does with a dynamic ``inference_context`` (attention.py:603-847) --
    ``get_query_key_value_tensors`` (:985-1030), ``_adjust_key_value_for_inference`` (:394-414), rotary embedding of
    the query (:740-790), ``flash_decode_and_prefill`` (:470-601) and ``linear_proj`` (:829-845) -- as three launches
    on a decode step: the QKV projection writes the mixed ``[T, Hkv, (G + 2) d]`` tensor, the streaming kernel reads it
    directly (split, head norm, rotary embedding and cache append in its prologue) and the output projection follows
    the merge.  Returns ``(output, bias)`` like the reference.
    """

    def __init__(self, layer_number: int, hidden_size: int, num_query_heads: int, num_kv_heads: int, head_dim: int, *,
                 qk_norm: Optional[str] = None, eps: float = 1e-5, add_qkv_bias: bool = False,
                 add_bias_linear: bool = False, softmax_scale: Optional[float] = None, rotary_interleaved: bool = False,
                 dtype: torch.dtype = torch.bfloat16, device=None):
        super().__init__()
        self.num_query_heads, self.num_kv_heads, self.head_dim = num_query_heads, num_kv_heads, head_dim
        self.linear_qkv = DecodeLinear(hidden_size, (num_query_heads + 2 * num_kv_heads) * head_dim,
                                       bias=add_qkv_bias or add_bias_linear, skip_bias_add=False, dtype=dtype, device=device)
        self.core = PagedSelfAttentionCore(layer_number, head_dim, qk_norm=qk_norm, eps=eps, softmax_scale=softmax_scale,
                                           rotary_interleaved=rotary_interleaved, dtype=dtype, device=device)
        self.linear_proj = DecodeLinear(num_query_heads * head_dim, hidden_size, bias=add_bias_linear,
                                        skip_bias_add=True, dtype=dtype, device=device)

    def forward(self, hidden_states: Tensor, inference_context,
                rotary_pos_emb: Optional[Tuple[Tensor, Tensor]] = None):
        mixed_qkv, _ = self.linear_qkv(hidden_states)
        core_attn_out = self.core.forward_mixed_qkv(mixed_qkv, self.num_query_heads, inference_context, rotary_pos_emb)
        return self.linear_proj(core_attn_out)
