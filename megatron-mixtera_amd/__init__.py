"""MI355X-native decode-step hot path of Megatron-Core's dynamic inference engine.

Public surface (same names as the reference wherever one exists):

* :class:`DynamicInferenceContext`, :class:`ChunkAllocator` and the overflow errors --
  the chunked KV cache and in-flight batching state
  (reference: megatron/core/inference/contexts/).
* :func:`flash_attn_with_kvcache`, :func:`flash_attn_varlen_func` -- the two attention
  calls ``Attention.flash_decode_and_prefill`` makes
  (reference: megatron/core/transformer/attention.py:470-601).
* :mod:`ops` -- thin torch wrappers over the C ABI (KV-append, paged attention,
  fused norm + RoPE, fp8 KV, last-token gather, sampling).
* :mod:`sampling` -- ``sample_from_logits`` and the finished-request mask on one kernel
  (reference: megatron/core/inference/text_generation_controllers/text_generation_controller.py:172-315).
* :mod:`step` -- ``generate_output_tokens_dynamic_batch``: one engine step on a context with the
  model behind a callable (reference: the same file, :411-546).
"""
from . import attention, ops, sampling, step, synthetic  # noqa: F401
from .attention import (  # noqa: F401
    DecodeLinear,
    PagedSelfAttentionCore,
    PagedSelfAttentionLayer,
    adjust_key_value_for_inference,
    flash_decode_and_prefill,
)
from .contexts import (  # noqa: F401
    ActiveRequestCountOverflowError,
    ChunkAllocator,
    ChunkOverflowError,
    ContextOverflowError,
    DynamicInferenceContext,
    MaxSequenceLengthOverflowError,
    RequestOverflowError,
    TokenOverflowError,
    WarmupEngineMode,
)
from .flash_attn_interface import (  # noqa: F401
    _flash_attn_forward,
    flash_attn_varlen_func,
    flash_attn_with_kvcache,
    flash_mla_with_kvcache,
    get_mla_metadata,
)
from .graphs import DecodeLayerGraphs  # noqa: F401

__all__ = [
    "ops",
    "sampling",
    "step",
    "DynamicInferenceContext",
    "ChunkAllocator",
    "WarmupEngineMode",
    "ContextOverflowError",
    "RequestOverflowError",
    "TokenOverflowError",
    "MaxSequenceLengthOverflowError",
    "ChunkOverflowError",
    "ActiveRequestCountOverflowError",
    "flash_attn_with_kvcache",
    "flash_attn_varlen_func",
    "flash_mla_with_kvcache",
    "get_mla_metadata",
    "flash_decode_and_prefill",
    "adjust_key_value_for_inference",
    "PagedSelfAttentionCore",
    "DecodeLayerGraphs",
]
