"""Chunked KV cache + in-flight batching state (mirror of megatron/core/inference/contexts/)."""
from .dynamic_chunk_allocator import ChunkAllocator  # noqa: F401
from .dynamic_context import (  # noqa: F401
    ActiveRequestCountOverflowError,
    ChunkOverflowError,
    ContextOverflowError,
    DynamicInferenceContext,
    MaxSequenceLengthOverflowError,
    RequestOverflowError,
    TokenOverflowError,
    WarmupEngineMode,
)
