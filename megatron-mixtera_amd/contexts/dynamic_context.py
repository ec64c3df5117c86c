"""In-flight batching state and chunked KV cache for dynamic inference on MI355X.

Drop-in for the reference's ``DynamicInferenceContext``
(megatron/core/inference/contexts/dynamic_context.py:94-1365): same constructor keywords,
attribute names, method signatures, tensor dtypes and exceptions, so the controller
(text_generation_controller.py:411-555), the engine (dynamic_engine.py) and
``Attention.forward`` can use it unchanged.  What differs is underneath the per-layer
methods: ``append_key_value_cache`` and ``apply_rotary_emb_*`` enqueue the HIP kernels of
``libmi355_decode.so`` instead of chains of torch indexing kernels, and
:meth:`fused_qk_norm_rope_append` offers the whole norm -> RoPE -> append sequence of a
layer as one launch.

Request rows are laid out ``[paused | active | finished]``; ``paused_request_count`` and
``total_request_count`` mark the boundaries.  Per-request rows are int32, per-token rows
int64, exactly as in the reference, so states can be compared bit for bit.
"""
from __future__ import annotations

import math
import warnings
from enum import Enum
from typing import List, Optional, Tuple, Union

import torch
import torch.nn.functional as F
from torch import Tensor

from .. import ops
from ..flash_attn_interface import note_kv_lengths
from .dynamic_chunk_allocator import ChunkAllocator


class ContextOverflowError(Exception):
    """A request does not fit into the context (reference: dynamic_context.py:30-45).

    ``is_transient`` tells the engine whether retrying later can succeed.
    """

    def __init__(self, request_id: Optional[int], message: Optional[str] = None, *, is_transient: bool = True):
        rid = "--" if request_id is None else str(request_id)
        tail = "" if message is None else f" | {message}"
        super().__init__(f"request {rid}{tail}")
        self.is_transient = is_transient


class RequestOverflowError(ContextOverflowError):
    """No free request row."""


class TokenOverflowError(ContextOverflowError):
    """No room left in the per-token rows."""


class MaxSequenceLengthOverflowError(ContextOverflowError):
    """Prompt + generation budget exceeds ``max_sequence_length`` (never transient)."""

    def __init__(self, request_id, message: Optional[str] = None):
        super().__init__(request_id, message=message, is_transient=False)


class ChunkOverflowError(ContextOverflowError):
    """Not enough free KV chunks."""


class ActiveRequestCountOverflowError(ContextOverflowError):
    """``initialize_attention_state`` was asked to warm up more tokens than ``max_requests``."""

    def __init__(self, max_request_count, active_request_count):
        assert active_request_count > max_request_count
        super().__init__(
            None,
            "active_request_count (%d) > max_request_count (%d)." % (active_request_count, max_request_count),
        )


class WarmupEngineMode(Enum):
    """Which attention path a graph warm-up step should exercise."""

    DECODE = "decode"
    NON_DECODE = "non_decode"


def _ceil_to(value: int, multiple: int) -> int:
    return multiple * int(math.ceil(int(value) / multiple))


class DynamicInferenceContext:
    """Chunked KV cache + batching bookkeeping; see the module docstring.

    Keyword arguments are those of the reference constructor (dynamic_context.py:156-177);
    ``device`` is an addition for host-side testing of the bookkeeping (the kernels need a
    GPU).  ``num_attention_heads`` is the number of KV heads (query groups).
    """

    TOKEN_ROUNDER = 64
    REQUEST_ROUNDER = 4

    # ------------------------------------------------------------------ construction
    def __init__(
        self,
        *,
        params_dtype: torch.dtype,
        num_layers: int,
        kv_channels: int,
        num_attention_heads: int,
        max_sequence_length: int,
        buffer_size_gb: float,
        buffer_guaranteed_fraction: float,
        chunk_size_tokens: int = 256,
        buffer_overflow_factor: Optional[float] = None,
        max_requests_override: Optional[int] = None,
        max_tokens_override: Optional[int] = None,
        tensor_model_parallel_size: Optional[int] = None,
        cache_mla_latent: bool = False,
        kv_lora_rank: Optional[int] = None,
        qk_pos_emb_head_dim: Optional[int] = None,
        num_cuda_graphs: Optional[int] = None,
        materialize_only_last_token_logits: bool = True,
        use_cuda_graphs_for_non_decode_steps: bool = True,
        device: Optional[Union[torch.device, str, int]] = None,
        fused_bookkeeping: Optional[bool] = None,
        kv_cache_dtype: Optional[Union[str, torch.dtype]] = None,
        fp8_append_headroom: float = 2.0,
    ):
        self.materialize_only_last_token_logits = materialize_only_last_token_logits
        self.cache_mla_latent = bool(cache_mla_latent)
        if self.cache_mla_latent:
            assert (
                chunk_size_tokens == 64
            ), "Flash MLA requires a block size of 64. Set --inference-dynamic-batching-chunk-size 64 to fix this assert"
            if kv_lora_rank is None or qk_pos_emb_head_dim is None:
                raise ValueError("cache_mla_latent=True needs kv_lora_rank and qk_pos_emb_head_dim")
            if kv_cache_dtype not in (None, params_dtype):
                raise NotImplementedError("the MLA latent cache is kept in params_dtype (no fp8 variant)")
        self.device = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)

        tp = 1 if tensor_model_parallel_size is None else tensor_model_parallel_size
        if num_attention_heads % tp:
            raise ValueError(f"{num_attention_heads} KV heads are not divisible by tensor parallel size {tp}")
        heads_here = num_attention_heads // tp

        # ---- KV storage format: params_dtype as in the reference, or (an addition) e4m3 bytes with one
        # fp32 scale per (key|value, layer, chunk, head) ----
        if kv_cache_dtype in (None, params_dtype):
            self.kv_cache_fp8 = False
        elif kv_cache_dtype in ("fp8", "fp8_e4m3", "float8_e4m3fn", torch.float8_e4m3fn):
            if params_dtype not in (torch.bfloat16, torch.float16):
                raise ValueError("the fp8 KV cache quantises 16-bit keys and values: params_dtype must be bfloat16 or float16")
            self.kv_cache_fp8 = True
        else:
            raise ValueError(f"unsupported kv_cache_dtype {kv_cache_dtype!r} (None or 'fp8_e4m3')")
        self.fp8_append_headroom = float(fp8_append_headroom)

        # ---- sizing (reference: dynamic_context.py:186-242) ----
        self.chunk_size_tokens = chunk_size_tokens
        kv_itemsize = 1 if self.kv_cache_fp8 else params_dtype.itemsize
        if self.cache_mla_latent:
            # one vector c_t (rank) + the shared RoPE slice per token and layer (reference: :197-203)
            self.kv_reduced_dim = kv_lora_rank + qk_pos_emb_head_dim
            self.chunk_size_bytes = kv_itemsize * num_layers * chunk_size_tokens * self.kv_reduced_dim
        else:
            self.chunk_size_bytes = kv_itemsize * 2 * num_layers * chunk_size_tokens * heads_here * kv_channels
        if self.kv_cache_fp8:
            self.chunk_size_bytes += 4 * 2 * num_layers * heads_here  # its scales
        pool_bytes = int(buffer_size_gb * 1024**3)
        pool_bytes -= pool_bytes % self.chunk_size_bytes
        chunk_count_total = pool_bytes // self.chunk_size_bytes

        token_capacity = pool_bytes / self.chunk_size_bytes * chunk_size_tokens
        self.max_requests = self.round_up_requests(int(token_capacity / max_sequence_length), tp_size=tp)
        self.max_tokens = self.round_up_tokens(int(token_capacity), tp_size=tp)
        if buffer_overflow_factor is not None:
            self.max_requests = self.round_up_requests(int(self.max_requests * buffer_overflow_factor), tp_size=tp)
            self.max_tokens = self.round_up_tokens(int(self.max_tokens * buffer_overflow_factor / 50.0), tp_size=tp)
        if max_requests_override is not None:
            self.max_requests = self.round_up_requests(max_requests_override, tp_size=tp)
        if max_tokens_override is not None:
            self.max_tokens = self.round_up_tokens(max_tokens_override, tp_size=tp)
        self.max_requests = min(self.max_requests, self.max_tokens)

        self.params_dtype = params_dtype
        self.num_layers = num_layers
        self.max_sequence_length = max_sequence_length
        self.num_kv_heads_per_partition = heads_here
        self.kv_channels = kv_channels

        self.total_request_count = 0
        self.active_token_count = 0
        self.paused_request_count = 0
        self.padded_active_token_count = None
        self.padded_active_request_count = None
        self.paused_tokens = None

        dev = self.device

        def req_row(fill=None):
            if fill is None:
                return torch.empty(self.max_requests, dtype=torch.int32, device=dev)
            return torch.full((self.max_requests,), fill, dtype=torch.int32, device=dev)

        def tok_row(fill=None):
            if fill is None:
                return torch.empty(self.max_tokens, dtype=torch.long, device=dev)
            return torch.full((self.max_tokens,), fill, dtype=torch.long, device=dev)

        # ---- per-request rows (int32) ----
        self.request_ids = req_row(-1)
        self.request_query_lengths = req_row()
        self.request_output_lengths = req_row()
        self.request_kv_length_offsets = req_row()
        self.request_kv_chunk_counts = req_row()
        self.request_last_kv_chunk_id = req_row()
        self.request_last_kv_chunk_offset = req_row()

        # ---- per-token rows (int64) ----
        self.token_to_input_ids = tok_row(0)
        self.token_to_pos_ids = tok_row(0)
        self.token_to_request_idx = tok_row()
        self.token_to_chunk_idx = tok_row()
        self.token_to_position_in_request = tok_row()
        self.token_to_local_position_within_kv_chunk = tok_row()

        # ---- the cache: [key|value, layer, chunk, token, head, channel] ----
        if self.cache_mla_latent:
            # [layer, chunk, token, rank + rope]: one row per token, shared by all heads (reference: :288-294)
            self.memory_buffer = torch.full(
                (num_layers, chunk_count_total, chunk_size_tokens, self.kv_reduced_dim),
                -1, dtype=params_dtype, device=dev)
            self.kv_scales = None
        elif self.kv_cache_fp8:
            # bytes (0 = +0.0 in e4m3; the reference's -1 fill would read as NaN here) and their scales
            self.memory_buffer = torch.zeros(
                (2, num_layers, chunk_count_total, chunk_size_tokens, heads_here, kv_channels),
                dtype=torch.uint8, device=dev)
            self.kv_scales = torch.ones((2, num_layers, chunk_count_total, heads_here), dtype=torch.float32, device=dev)
        else:
            self.memory_buffer = torch.full(
                (2, num_layers, chunk_count_total, chunk_size_tokens, heads_here, kv_channels),
                -1, dtype=params_dtype, device=dev)
            self.kv_scales = None

        self.max_kv_chunk_count = math.ceil(max_sequence_length / chunk_size_tokens)
        self.request_to_kv_chunk_ids = torch.full(
            (self.max_requests, self.max_kv_chunk_count), -1, dtype=torch.int, device=dev)

        # ---- graph batch sizes (reference: dynamic_context.py:319-356) ----
        self.cuda_graph_token_counts = None
        if num_cuda_graphs is not None:
            num_cuda_graphs = min(max(num_cuda_graphs, 1), self.max_requests)
            step = math.ceil((self.max_requests / num_cuda_graphs) / 8) * 8
            step = math.ceil(step / tp) * tp
            self.cuda_graph_step_size = step
            if num_cuda_graphs == 1:
                counts = [self.max_requests]
            else:
                counts = list(range(step, self.max_requests, step))
                if counts[-1] != self.max_requests:
                    counts.append(self.max_requests)
                counts.reverse()
            self.cuda_graph_token_counts = counts
            self.cuda_graph_token_counts_set = set(counts)
            self.max_cuda_graph_token_count = max(counts)
        self.cuda_graph_request_counts = self.cuda_graph_token_counts
        self.non_decode_cuda_graphs = use_cuda_graphs_for_non_decode_steps and (num_cuda_graphs is not None)

        # ---- fixed-address mirrors consumed by captured graphs ----
        self.query_seq_lengths_cudagraph_only = torch.zeros(self.max_requests, dtype=torch.int32, device=dev)
        self.cu_query_seq_lengths_cudagraph_only = torch.zeros(self.max_requests + 1, dtype=torch.int32, device=dev)
        self.kv_seq_lengths_cudagraph_only = torch.zeros(self.max_requests, dtype=torch.int32, device=dev)
        self.cu_kv_seq_lengths_cudagraph_only = torch.zeros(self.max_requests + 1, dtype=torch.int32, device=dev)
        self.request_to_kv_chunk_ids_cudagraph_only = torch.zeros(
            (self.max_requests, self.max_kv_chunk_count), dtype=torch.int, device=dev)

        # ---- guaranteed-progress reserve (reference: dynamic_context.py:398-401) ----
        reserve = min(int(buffer_guaranteed_fraction * chunk_count_total), chunk_count_total)
        self.gtd_request_count = max(1, reserve // self.max_kv_chunk_count)
        self.gtd_chunk_count = self.gtd_request_count * self.max_kv_chunk_count

        self.chunk_allocator = ChunkAllocator(
            chunk_count_total=chunk_count_total, gtd_chunk_count=self.gtd_chunk_count, device=dev)
        self.dummy_chunk_idx = self.chunk_allocator.dummy_chunk_idx

        # ---- on-GPU bookkeeping: update_requests / decode attention state as single kernels ----
        # (None = use them whenever the state lives on a GPU; the torch op sequence below is the
        # host-side statement of the same steps and the only one available for device="cpu")
        self.fused_bookkeeping = (dev.type == "cuda") if fused_bookkeeping is None else bool(fused_bookkeeping)
        if self.fused_bookkeeping:
            self._paused_tokens_buf = torch.zeros(self.max_requests, dtype=torch.long, device=dev)
            self._next_tokens_buf = torch.zeros(self.max_requests, dtype=torch.long, device=dev)
            self._update_scratch = torch.zeros(4 * self.max_requests, dtype=torch.int32, device=dev)
            self._newly_paused_buf = torch.zeros(self.max_requests, dtype=torch.int32, device=dev)
            self._finished_ids_buf = torch.zeros(self.max_requests, dtype=torch.int32, device=dev)
            self._counters = torch.zeros(8, dtype=torch.int32, device=dev)
            self._counters_host = torch.zeros(8, dtype=torch.int32, pin_memory=True)
            # largest query / kv length of a prefill or mixed step: written by the attention-state kernel,
            # copied to pinned memory behind an event and only waited for when somebody reads the value
            self._max_lengths = torch.zeros(2, dtype=torch.int32, device=dev)
            self._max_lengths_host = torch.zeros(2, dtype=torch.int32, pin_memory=True)
            self._max_lengths_event = torch.cuda.Event()
        self._max_lengths_pending = False
        # what the host knows without asking the device: the longest prompt admitted since the last
        # update_requests (every other active request has one query token) and a bound on the kv lengths
        self._host_max_query_len = 1
        self._host_kv_len_bound = 0
        # ids of the requests that finished in the last update_requests (fused bookkeeping), else None
        self.last_finished_request_ids = None

        self.reset_attention_state()

    # ------------------------------------------------------------------ rounding helpers
    @classmethod
    def round_up_tokens(cls, value, tp_size=None):
        """Next multiple of ``TOKEN_ROUNDER`` (itself rounded up to a multiple of the TP size)."""
        tp = 1 if tp_size is None else tp_size
        return _ceil_to(value, math.ceil(cls.TOKEN_ROUNDER / tp) * tp)

    @classmethod
    def round_up_requests(cls, value, tp_size=None):
        """Next multiple of ``REQUEST_ROUNDER`` (itself rounded up to a multiple of the TP size)."""
        tp = 1 if tp_size is None else tp_size
        return _ceil_to(value, math.ceil(cls.REQUEST_ROUNDER / tp) * tp)

    @classmethod
    def round_up(cls, value):
        """Deprecated single-rounder form kept for callers that still use it."""
        warnings.warn("`round_up` is deprecated in favor of `round_up_tokens` or `round_up_requests`.")
        return _ceil_to(value, getattr(cls, "ROUNDER", 64))

    # ------------------------------------------------------------------ simple queries
    def is_static_batching(self) -> bool:
        return False

    def is_dynamic_batching(self) -> bool:
        return True

    def increment_sequence_len_offset(self, increment: int) -> None:
        """No-op for dynamic batching (static-context API)."""

    def increment_batch_size_offset(self, increment: int) -> None:
        """No-op for dynamic batching (static-context API)."""

    def reset_batch_size_offset(self) -> None:
        """No-op for dynamic batching (static-context API)."""

    def _active(self) -> slice:
        return slice(self.paused_request_count, self.total_request_count)

    def is_decode_only(self) -> bool:
        """Every active request contributes exactly one token this step."""
        return self.total_request_count - self.paused_request_count == self.active_token_count

    def has_unfinished_requests(self) -> bool:
        return self.total_request_count > 0

    # max_seqlen_q / max_seqlen_k keep the reference's meaning (exact maxima on prefill / mixed steps).  With the
    # fused bookkeeping they are produced on the GPU and fetched lazily: reading one of them waits for the small
    # copy issued by initialize_attention_state; a step that never reads them never waits.
    def _resolve_max_lengths(self) -> None:
        if self._max_lengths_pending:
            self._max_lengths_event.synchronize()
            self._max_seqlen_q, self._max_seqlen_k = self._max_lengths_host.tolist()
            self._max_lengths_pending = False

    @property
    def max_seqlen_q(self):
        self._resolve_max_lengths()
        return self._max_seqlen_q

    @max_seqlen_q.setter
    def max_seqlen_q(self, value) -> None:
        self._max_seqlen_q = value

    @property
    def max_seqlen_k(self):
        self._resolve_max_lengths()
        return self._max_seqlen_k

    @max_seqlen_k.setter
    def max_seqlen_k(self, value) -> None:
        self._max_seqlen_k = value

    def attention_length_bounds(self) -> Tuple[int, int]:
        """``(max query length, upper bound of the kv lengths)`` of this step from what the host already knows,
        without waiting for the device: 1 on decode steps (the padded token count on graph steps), else the
        longest prompt admitted since the last ``update_requests``; kv lengths are bounded by the longest
        prompt so far plus the steps taken, and by ``max_sequence_length``.  The attention kernels only need
        bounds (which kernel, how to split the keys), not the exact maxima."""
        if self.is_decode_only():
            q_max = 1
        elif self.using_cuda_graph_this_step():
            q_max = self.padded_active_token_count
        else:
            q_max = max(1, self._host_max_query_len)
        k_bound = min(self.max_sequence_length, max(1, self._host_kv_len_bound))
        return q_max, k_bound

    def cu_query_lengths(self) -> Tuple[Optional[Tensor], int]:
        return self.cu_query_seq_lengths, self.max_seqlen_q

    def cu_kv_lengths(self) -> Tuple[Optional[Tensor], Tensor, int]:
        return (self.cu_kv_seq_lengths, self.kv_seq_lengths, self.max_seqlen_k)

    def get_active_sequence_lengths(self) -> Tensor:
        return (self.request_kv_length_offsets + self.request_query_lengths)[self._active()]

    def get_max_sequence_lengths(self) -> Tensor:
        return self.request_output_lengths[self._active()]

    def get_active_request_count(self):
        unfinished = torch.less(self.get_active_sequence_lengths(), self.get_max_sequence_lengths())
        return int(unfinished.sum().item())

    # ------------------------------------------------------------------ per-layer hot path
    def append_key_value_cache(self, layer_number: int, key: Tensor, value: Tensor) -> None:
        """Scatter this step's K/V rows into the layer's chunks (bit-exact copy).

        ``layer_number`` is 1-based.  Slots come from ``token_to_chunk_idx`` /
        ``token_to_local_position_within_kv_chunk``; padded tokens land in the dummy chunk.
        """
        n = self.padded_active_token_count
        if self.cache_mla_latent:
            # the caller passes kv_concat as the key; there is no value cache (reference: :533-538)
            latent = key.squeeze(1) if key.dim() == 3 else key
            ops.kv_append(latent[:n].unsqueeze(1), None, self.memory_buffer[layer_number - 1].unsqueeze(2), None,
                          self.token_to_chunk_idx, self.token_to_local_position_within_kv_chunk)
            return
        assert key.size(1) == 1 and value.size(1) == 1
        if self.kv_cache_fp8:
            ops.kv_append_fp8(
                key[:n], value[:n],
                self.memory_buffer[0, layer_number - 1], self.memory_buffer[1, layer_number - 1],
                self.kv_scales[0, layer_number - 1], self.kv_scales[1, layer_number - 1],
                self.token_to_chunk_idx, self.token_to_local_position_within_kv_chunk,
                headroom=self.fp8_append_headroom)
            return
        ops.kv_append(
            key[:n], value[:n],
            self.memory_buffer[0, layer_number - 1], self.memory_buffer[1, layer_number - 1],
            self.token_to_chunk_idx, self.token_to_local_position_within_kv_chunk)

    def key_value_cache(self, layer_number: int) -> Tuple[Tensor, Tensor, Tensor]:
        """Views of the layer's key cache, value cache and this step's block table (latent cache: the
        layer's ``[chunks, tokens, rank + rope]`` buffer and ``None``)."""
        if self.cache_mla_latent:
            return (self.memory_buffer[layer_number - 1], None, self.block_table)
        return (self.memory_buffer[0, layer_number - 1], self.memory_buffer[1, layer_number - 1], self.block_table)

    def key_value_scales(self, layer_number: int) -> Tuple[Optional[Tensor], Optional[Tensor]]:
        """fp8 cache: the layer's key and value scales ``[chunks, heads]``; otherwise ``(None, None)``."""
        if not self.kv_cache_fp8:
            return None, None
        return self.kv_scales[0, layer_number - 1], self.kv_scales[1, layer_number - 1]

    @staticmethod
    def _rope_flags(config) -> bool:
        if getattr(config, "multi_latent_attention", False):
            raise NotImplementedError("multi-latent attention RoPE is not part of the MI355X decode path")
        return bool(getattr(config, "rotary_interleaved", False))

    def apply_rotary_emb_query(self, query: Tensor, query_emb: Tensor, config, cu_seqlens_q: Tensor,
                               cp_group=None, mscale: float = 1.0) -> Tensor:
        """Rotate the first ``padded_active_token_count`` query rows in place; positions = ``token_to_pos_ids``."""
        n = self.padded_active_token_count
        ops.norm_rope_append(query[:n], None, rotary_emb=query_emb, q_positions=self.token_to_pos_ids,
                             rotary_interleaved=self._rope_flags(config), mscale=mscale)
        return query

    def apply_rotary_emb_key(self, key: Tensor, key_emb: Tensor, config, cp_group=None, mscale: float = 1.0) -> Tensor:
        """Rotate key rows; positions = ``token_to_position_in_request``.

        Decode-only steps return a fresh tensor, other steps update ``key[:n]`` in place
        (the reference's behaviour, dynamic_context.py:619-631).
        """
        n = self.padded_active_token_count
        interleaved = self._rope_flags(config)
        if self.is_decode_only():
            assert key.shape[0] == n
            out = torch.empty_like(key)
        else:
            out = key
        ops.norm_rope_append(None, key[:n], key_out=out[:n], rotary_emb=key_emb,
                             k_positions=self.token_to_position_in_request,
                             rotary_interleaved=interleaved, mscale=mscale)
        return out

    def fused_qk_norm_rope_append(self, layer_number: int, query: Tensor, key: Tensor, value: Tensor, *,
                                  rotary_pos_emb: Optional[Tensor], config=None, q_weight: Optional[Tensor] = None,
                                  k_weight: Optional[Tensor] = None, norm: Optional[str] = None, eps: float = 1e-5,
                                  mscale: float = 1.0, faithful_rounding: bool = True) -> Tensor:
        """One launch for q/k norm -> RoPE(q, k) -> append(k, v) of a layer.

        Equivalent to q_layernorm/k_layernorm + ``apply_rotary_emb_key`` +
        ``append_key_value_cache`` + ``apply_rotary_emb_query`` of the reference
        (attention.py:1026-1030, 394-404, 766).  ``query`` is updated in place and returned.
        """
        n = self.padded_active_token_count
        if self.cache_mla_latent:
            raise NotImplementedError("the fused q/k norm + RoPE + append launch serves per-head KV caches, not MLA latents")
        if self.kv_cache_fp8:
            # norm + RoPE in one launch, then the quantising append (the roped key passes through memory)
            key_out = torch.empty_like(key[:n])
            ops.norm_rope_append(
                query[:n], key[:n], key_out=key_out, q_weight=q_weight, k_weight=k_weight, eps=eps, norm=norm,
                rotary_emb=rotary_pos_emb, q_positions=self.token_to_pos_ids,
                k_positions=self.token_to_position_in_request,
                rotary_interleaved=self._rope_flags(config) if config is not None else False, mscale=mscale,
                faithful_rounding=faithful_rounding)
            self.append_key_value_cache(layer_number, key_out, value[:n])
            return query
        ops.norm_rope_append(
            query[:n], key[:n], value=value[:n], q_weight=q_weight, k_weight=k_weight, eps=eps, norm=norm,
            rotary_emb=rotary_pos_emb, q_positions=self.token_to_pos_ids,
            k_positions=self.token_to_position_in_request,
            rotary_interleaved=self._rope_flags(config) if config is not None else False, mscale=mscale,
            k_cache=self.memory_buffer[0, layer_number - 1], v_cache=self.memory_buffer[1, layer_number - 1],
            token_to_chunk_idx=self.token_to_chunk_idx,
            token_to_local_pos=self.token_to_local_position_within_kv_chunk,
            faithful_rounding=faithful_rounding)
        return query

    def decode_step_fusable(self, head_dim: int, rotary_pos_emb: Optional[Tensor], config=None) -> bool:
        """Whether this step can run :meth:`fused_decode_step_attention`: a decode-only step over per-head caches
        (16-bit or fp8) with shapes the fused kernel has (``ops.decode_step_supported``)."""
        if not self.is_decode_only() or self.cache_mla_latent:
            return False
        rot = 0 if rotary_pos_emb is None else rotary_pos_emb.size(-1)
        interleaved = self._rope_flags(config) if config is not None else False
        return ops.decode_step_supported(head_dim, rot, interleaved, self.kv_cache_fp8)

    def fused_decode_step_attention(self, layer_number: int, query: Optional[Tensor] = None,
                                    key: Optional[Tensor] = None, value: Optional[Tensor] = None, *,
                                    mixed_qkv: Optional[Tensor] = None, num_query_heads: int = 0,
                                    rotary_pos_emb: Optional[Tensor] = None, config=None,
                                    q_weight: Optional[Tensor] = None, k_weight: Optional[Tensor] = None,
                                    norm: Optional[str] = None, eps: float = 1e-5, mscale: float = 1.0,
                                    softmax_scale: Optional[float] = None, faithful_rounding: bool = True) -> Tensor:
        """A decode-only step of one layer in two launches: q/k norm, RoPE(q, k), append(k, v) and the attention
        over the layer's cache (attention.py:1026-1030, 394-414, 589-600) -- :meth:`fused_qk_norm_rope_append`
        (or :meth:`fused_qkv_norm_rope_append`) and ``flash_attn_with_kvcache`` in one streaming kernel plus its
        merge.  Takes ``query`` / ``key`` / ``value`` ``[T, 1, H, d]`` or ``mixed_qkv`` ``[T, 1, (Hq + 2 Hkv) d]``;
        returns the attention output ``[T, 1, Hq, d]`` (rows past the padded token count are left unwritten).
        Row i is request i of the step: its token is appended at position ``kv_seq_lengths[i] - 1`` of the
        request's chunks, which is where ``token_to_chunk_idx`` / ``token_to_local_position_within_kv_chunk``
        point on a decode step; query and key rotate by that same position, which is what ``token_to_pos_ids``
        and ``token_to_position_in_request`` hold on a decode step (``update_requests`` sets both to
        ``request_kv_length_offsets``, dynamic_context.py:1248-1254; a one-token prompt starts at 0)."""
        n = self.padded_active_token_count
        k_cache, v_cache, block_table = self.key_value_cache(layer_number)
        _, k_bound = self.attention_length_bounds()
        common = dict(q_weight=q_weight, k_weight=k_weight, eps=eps, norm=norm, rotary_emb=rotary_pos_emb,
                      positions=None,  # = kv_seq_lengths - 1, see the docstring
                      rotary_interleaved=self._rope_flags(config) if config is not None else False, mscale=mscale,
                      softmax_scale=softmax_scale, max_kv_len=k_bound, faithful_rounding=faithful_rounding)
        if self.kv_cache_fp8:  # the quantising append of the step's token rides in the kernel too
            k_scales, v_scales = self.key_value_scales(layer_number)
            common.update(k_scales=k_scales, v_scales=v_scales, headroom=self.fp8_append_headroom)
        if mixed_qkv is not None:
            d = self.kv_channels
            out = torch.empty((mixed_qkv.size(0), 1, num_query_heads, d), dtype=mixed_qkv.dtype, device=mixed_qkv.device)
            ops.decode_step_attention(None, None, None, k_cache, v_cache, self.kv_seq_lengths, block_table,
                                      mixed_qkv=mixed_qkv[:n], num_query_heads=num_query_heads,
                                      num_kv_heads=self.num_kv_heads_per_partition, out=out[:n], **common)
            return out
        out = torch.empty_like(query)
        ops.decode_step_attention(query[:n], key[:n], value[:n], k_cache, v_cache, self.kv_seq_lengths, block_table,
                                  out=out[:n], **common)
        return out

    def fused_qkv_norm_rope_append(self, layer_number: int, mixed_qkv: Tensor, *, num_query_heads: int,
                                   rotary_pos_emb: Optional[Tensor], config=None,
                                   q_weight: Optional[Tensor] = None, k_weight: Optional[Tensor] = None,
                                   norm: Optional[str] = None, eps: float = 1e-5, mscale: float = 1.0,
                                   faithful_rounding: bool = True, query_out: Optional[Tensor] = None) -> Tensor:
        """:meth:`fused_qk_norm_rope_append` starting from the QKV projection's output.

        ``mixed_qkv`` is ``[T, 1, (Hq + 2 Hkv) * d]`` in the per-query-group order that
        ``SelfAttention.get_query_key_value_tensors`` splits (attention.py:985-1030); the split, the
        query reshape (a copy in the reference), both norms, both RoPE calls and the append run as one
        launch.  Returns the query ``[T, 1, Hq, d]`` (``query_out`` if given, else a new tensor).
        """
        n = self.padded_active_token_count
        if self.cache_mla_latent:
            raise NotImplementedError("the fused QKV launch serves per-head KV caches, not MLA latents")
        hkv = self.num_kv_heads_per_partition
        d = self.kv_channels
        if query_out is None:
            query_out = torch.empty((mixed_qkv.size(0), 1, num_query_heads, d), dtype=mixed_qkv.dtype,
                                    device=mixed_qkv.device)
        if self.kv_cache_fp8:
            key_out = torch.empty((n, 1, hkv, d), dtype=mixed_qkv.dtype, device=mixed_qkv.device)
            ops.qkv_norm_rope_append(
                mixed_qkv[:n], num_query_heads=num_query_heads, num_kv_heads=hkv, query_out=query_out[:n],
                key_out=key_out, q_weight=q_weight, k_weight=k_weight, eps=eps, norm=norm, rotary_emb=rotary_pos_emb,
                q_positions=self.token_to_pos_ids, k_positions=self.token_to_position_in_request,
                rotary_interleaved=self._rope_flags(config) if config is not None else False, mscale=mscale,
                faithful_rounding=faithful_rounding)
            group = num_query_heads // hkv
            value = mixed_qkv[:n].reshape(n, hkv, (group + 2) * d)[:, :, (group + 1) * d:].contiguous()
            self.append_key_value_cache(layer_number, key_out, value.unsqueeze(1))
            return query_out
        ops.qkv_norm_rope_append(
            mixed_qkv[:n], num_query_heads=num_query_heads, num_kv_heads=hkv, query_out=query_out[:n],
            q_weight=q_weight, k_weight=k_weight, eps=eps, norm=norm, rotary_emb=rotary_pos_emb,
            q_positions=self.token_to_pos_ids, k_positions=self.token_to_position_in_request,
            rotary_interleaved=self._rope_flags(config) if config is not None else False, mscale=mscale,
            k_cache=self.memory_buffer[0, layer_number - 1], v_cache=self.memory_buffer[1, layer_number - 1],
            token_to_chunk_idx=self.token_to_chunk_idx,
            token_to_local_pos=self.token_to_local_position_within_kv_chunk,
            faithful_rounding=faithful_rounding)
        return query_out

    # ------------------------------------------------------------------ per-step attention state
    def reset_attention_state(self) -> None:
        """Forget the per-step attention metadata (the fixed-address mirrors are zeroed)."""
        self._max_lengths_pending = False
        note_kv_lengths(getattr(self, 'cu_kv_seq_lengths', None), None)
        self.max_seqlen_q = None
        self.max_seqlen_k = None
        self.cu_query_seq_lengths = None
        self.cu_kv_seq_lengths = None
        self.kv_seq_lengths = None
        self.block_table = None
        self.cu_query_seq_lengths_cudagraph_only.fill_(0)
        self.query_seq_lengths_cudagraph_only.fill_(0)
        self.cu_kv_seq_lengths_cudagraph_only.fill_(0)
        self.kv_seq_lengths_cudagraph_only.fill_(0)
        self.request_to_kv_chunk_ids_cudagraph_only.fill_(0)

    def using_cuda_graph_this_step(self) -> bool:
        """Graph sizes exist, the step type may use them, and the batch fits the largest one."""
        if self.cuda_graph_token_counts is None:
            return False
        if not (self.is_decode_only() or self.non_decode_cuda_graphs):
            return False
        return self.active_token_count <= self.max_cuda_graph_token_count

    def initialize_attention_state(self, *, num_warmup_tokens: Optional[int] = None,
                                   warmup_engine_mode: WarmupEngineMode = WarmupEngineMode.DECODE,
                                   num_warmup_requests: Optional[int] = None) -> None:
        """Prepare padding, sequence lengths and the block table for this step's forward pass.

        Reference: dynamic_context.py:656-825.  Decode-only and graph steps publish their
        lengths / block table through the fixed-address ``*_cudagraph_only`` buffers, with
        padded rows holding kv-length 0 and block-table row 0.
        """
        if num_warmup_requests is not None:
            warnings.warn("'num_warmup_requests' is deprecated; use 'num_warmup_tokens'.", DeprecationWarning)
            if num_warmup_tokens is None:
                num_warmup_tokens = num_warmup_requests

        if num_warmup_tokens is not None:
            if num_warmup_tokens > self.max_requests:
                raise ActiveRequestCountOverflowError(self.max_requests, num_warmup_tokens)
            if warmup_engine_mode == WarmupEngineMode.NON_DECODE:
                assert self.non_decode_cuda_graphs, "Set non-decode cuda graphs to True"
                # one request, zero tokens: makes is_decode_only() false for the warm-up
                self.total_request_count = 1

        token_count = self.active_token_count if num_warmup_tokens is None else num_warmup_tokens
        graph_step = self.using_cuda_graph_this_step()
        decode_only = self.is_decode_only()

        if graph_step:
            padded = _ceil_to(token_count, self.cuda_graph_step_size)
            padded = min(padded, self.max_requests)
            assert padded in self.cuda_graph_token_counts_set
            assert padded >= token_count
        else:
            padded = self.round_up_tokens(self.active_token_count)
            if decode_only:
                padded = min(padded, self.max_requests)
        self.padded_active_token_count = padded
        n_active_req = self.total_request_count - self.paused_request_count
        self.padded_active_request_count = padded if (graph_step or decode_only) else n_active_req

        act = self._active()
        if self.fused_bookkeeping and not decode_only:
            # Prefill / mixed step, one kernel and no wait: lengths, their running sums and the block table
            # go into the fixed-address mirrors (as on graph steps; same values as the reference's fresh
            # tensors), the padded token rows are pointed at the dummy chunk, and the two maxima follow
            # through pinned memory for whoever reads max_seqlen_q / max_seqlen_k.
            R = self.padded_active_request_count
            ops.step_attention_state(self, n_active_req, R, padded)
            self.kv_seq_lengths = self.kv_seq_lengths_cudagraph_only[:R]
            self.block_table = self.request_to_kv_chunk_ids_cudagraph_only[:R]
            self.cu_query_seq_lengths = self.cu_query_seq_lengths_cudagraph_only[: R + 1]
            self.cu_kv_seq_lengths = self.cu_kv_seq_lengths_cudagraph_only[: R + 1]
            if graph_step:
                self.max_seqlen_q = padded
                self.max_seqlen_k = self.max_sequence_length
            else:
                self._max_lengths_host.copy_(self._max_lengths, non_blocking=True)
                self._max_lengths_event.record(torch.cuda.current_stream(self.device))
                self._max_lengths_pending = True
            note_kv_lengths(self.cu_kv_seq_lengths, self.kv_seq_lengths)
            return
        if self.fused_bookkeeping and (graph_step or decode_only):
            # one kernel: padded token rows + fixed-address mirrors of lengths and block table
            ops.decode_attention_state(self, n_active_req, padded)
        else:
            # padded token rows: write into the dummy chunk at position 0
            pad = slice(self.active_token_count, padded)
            self.token_to_chunk_idx[pad] = self.dummy_chunk_idx
            self.token_to_local_position_within_kv_chunk[pad] = 0
            self.token_to_position_in_request[pad] = 0

        fused_mirrors = self.fused_bookkeeping and (graph_step or decode_only)
        if not fused_mirrors:
            q_lens = self.request_query_lengths[act]
            kv_lens = (self.request_kv_length_offsets + self.request_query_lengths)[act]
        R = self.padded_active_request_count
        dev = self.device

        if decode_only or graph_step:
            if not self.fused_bookkeeping:
                self.query_seq_lengths_cudagraph_only[:n_active_req] = q_lens
                self.kv_seq_lengths_cudagraph_only[:n_active_req] = kv_lens
                self.request_to_kv_chunk_ids_cudagraph_only[:n_active_req] = self.request_to_kv_chunk_ids[act]
            self.kv_seq_lengths = self.kv_seq_lengths_cudagraph_only[:R]
            self.max_seqlen_k = self.max_sequence_length
            self.block_table = self.request_to_kv_chunk_ids_cudagraph_only[:R]
            if decode_only:
                self.cu_query_seq_lengths = None
                self.cu_kv_seq_lengths = None
                self.max_seqlen_q = 1
            else:
                self.cu_query_seq_lengths_cudagraph_only[1 : R + 1] = torch.cumsum(
                    self.query_seq_lengths_cudagraph_only[:R], dim=0)
                self.cu_query_seq_lengths = self.cu_query_seq_lengths_cudagraph_only[: R + 1]
                self.max_seqlen_q = padded
                cu_kv = torch.cumsum(self.kv_seq_lengths, dim=0)
                self.cu_kv_seq_lengths_cudagraph_only[1 : cu_kv.size(0) + 1] = cu_kv
                self.cu_kv_seq_lengths = self.cu_kv_seq_lengths_cudagraph_only[: R + 1]
        else:
            self.cu_query_seq_lengths = torch.zeros(n_active_req + 1, dtype=torch.int32, device=dev)
            self.cu_query_seq_lengths[1:] = torch.cumsum(q_lens, dim=0)
            self.max_seqlen_q = q_lens.max().item()
            self.kv_seq_lengths = kv_lens
            self.cu_kv_seq_lengths = torch.zeros(n_active_req + 1, dtype=torch.int32, device=dev)
            self.cu_kv_seq_lengths[1:] = torch.cumsum(kv_lens, dim=0)
            self.max_seqlen_k = kv_lens.max().item()
            self.block_table = self.request_to_kv_chunk_ids[act]
        note_kv_lengths(self.cu_kv_seq_lengths, self.kv_seq_lengths)

    def reset(self) -> None:
        """Return to the empty state without reallocating anything (graphs keep the addresses)."""
        self.total_request_count = 0
        self.active_token_count = 0
        self.paused_request_count = 0
        self.padded_active_token_count = 0
        self.padded_active_request_count = 0
        self.paused_tokens = None

        self.request_ids.fill_(-1)
        self.request_query_lengths.fill_(0)
        self.request_output_lengths.fill_(0)
        self.request_kv_length_offsets.fill_(0)
        self.request_kv_chunk_counts.fill_(0)
        self.request_last_kv_chunk_id.fill_(-1)
        self.request_last_kv_chunk_offset.fill_(0)
        self.request_to_kv_chunk_ids.fill_(-1)

        self.token_to_input_ids.fill_(0)
        self.token_to_pos_ids.fill_(0)
        self.token_to_request_idx.fill_(-1)
        self.token_to_position_in_request.fill_(0)
        self.token_to_chunk_idx.fill_(-1)
        self.token_to_local_position_within_kv_chunk.fill_(0)

        self.reset_attention_state()
        self.chunk_allocator.reset()
        self._host_max_query_len = 1
        self._host_kv_len_bound = 0
        self.last_finished_request_ids = None

    def current_input_and_position_ids(self, *, num_warmup_tokens: Optional[int] = None) -> Tuple[Tensor, Tensor]:
        """``[1, T]`` views of this step's input ids and position ids."""
        n = num_warmup_tokens or self.padded_active_token_count
        return (self.token_to_input_ids[:n].unsqueeze(0), self.token_to_pos_ids[:n].unsqueeze(0))

    def last_token_logits(self, logits: Tensor) -> Tensor:
        """Rows of ``logits[0]`` at each active request's last token."""
        assert logits.size(0) == 1
        assert logits.size(1) == self.padded_active_token_count, (
            f"logits.size(1) ({tuple(logits.shape)}) != "
            f"padded_active_token_count ({self.padded_active_token_count}).")
        if logits.device.type == "cuda" and logits.element_size() in (2, 4) and logits.stride(-1) == 1:
            # running sum and row copy in one launch
            return ops.last_token_gather(logits.squeeze(0), self.request_query_lengths[self._active()])
        last = torch.cumsum(self.request_query_lengths[self._active()], dim=0) - 1
        return logits.squeeze(0)[last, :]

    # ------------------------------------------------------------------ request lifecycle
    def add_request(self, request_id: int, tokens: Tensor, num_tokens_to_generate: Optional[int] = None) -> None:
        """Admit a prompt: reserve ``ceil(len/chunk)`` chunks and fill its request / token rows.

        Raises the overflow errors of the reference in the reference's order
        (dynamic_context.py:945-974).
        """
        length = tokens.numel()
        if length > self.max_tokens:
            raise TokenOverflowError(request_id, is_transient=True)
        if self.active_token_count + length > self.max_tokens:
            raise TokenOverflowError(request_id)
        if self.total_request_count >= self.max_requests:
            raise RequestOverflowError(request_id)

        n_chunks = math.ceil(length / self.chunk_size_tokens)
        chunk_ids = self.chunk_allocator.allocate_memory_chunks(n_chunks, safe=True)
        if chunk_ids is None:
            raise ChunkOverflowError(request_id)

        if num_tokens_to_generate is None:
            num_tokens_to_generate = self.max_sequence_length - length
        elif length + num_tokens_to_generate > self.max_sequence_length:
            raise MaxSequenceLengthOverflowError(request_id)

        row = self.total_request_count
        if self.fused_bookkeeping and length > 0:
            # every write below as one launch (the popped ids are read from the allocator's stack on the GPU)
            prompt = tokens.reshape(-1).to(device=self.device, dtype=torch.int64).contiguous()
            ops.add_request(self, row, self.active_token_count, prompt, n_chunks,
                            self.chunk_allocator.chunk_count_avail, request_id, length + num_tokens_to_generate)
            self.total_request_count += 1
            self.active_token_count += length
            self._host_max_query_len = max(self._host_max_query_len, length)
            self._host_kv_len_bound = max(self._host_kv_len_bound, length)
            return
        self.request_ids[row] = request_id
        self.request_query_lengths[row] = length
        self.request_output_lengths[row] = length + num_tokens_to_generate
        self.request_kv_length_offsets[row] = 0
        self.request_to_kv_chunk_ids[row][:n_chunks] = chunk_ids
        self.request_kv_chunk_counts[row] = n_chunks
        self.request_last_kv_chunk_id[row] = chunk_ids[-1]
        self.request_last_kv_chunk_offset[row] = (length - 1) % self.chunk_size_tokens

        span = slice(self.active_token_count, self.active_token_count + length)
        pos = torch.arange(length, device=self.device)
        self.token_to_pos_ids[span] = pos
        self.token_to_input_ids[span] = tokens
        self.token_to_request_idx[span] = row
        self.token_to_position_in_request[span] = pos
        self.token_to_chunk_idx[span] = chunk_ids[pos // self.chunk_size_tokens]
        self.token_to_local_position_within_kv_chunk[span] = pos % self.chunk_size_tokens

        self.total_request_count += 1
        self.active_token_count += length
        self._host_max_query_len = max(self._host_max_query_len, length)
        self._host_kv_len_bound = max(self._host_kv_len_bound, length)

    def _move_book_keeping_tensors(self, src_idxs, dst_idxs, next_tokens):
        """``row[dst] = row[src]`` for every per-request row (right-hand sides gathered first)."""
        for row in (self.request_kv_length_offsets, self.request_query_lengths, self.request_output_lengths,
                    self.request_ids):
            row[dst_idxs] = row[src_idxs]
        next_tokens[dst_idxs] = next_tokens[src_idxs]
        for row in (self.request_to_kv_chunk_ids, self.request_kv_chunk_counts, self.request_last_kv_chunk_id,
                    self.request_last_kv_chunk_offset):
            row[dst_idxs] = row[src_idxs]

    def _release_chunks_of(self, rows: Tensor) -> None:
        owned = self.request_to_kv_chunk_ids[rows]
        self.chunk_allocator.release_memory_chunks(owned[owned != -1])

    def update_requests(self, active_requests_mask: Tensor, new_tokens: Tensor) -> Optional[Tensor]:
        """Advance every request by the token just sampled (reference: dynamic_context.py:1033-1298).

        ``active_requests_mask[i]`` is 1 when active request i continues, 0 when it finished;
        ``new_tokens[i]`` is its sampled token.  Finished requests give their chunks back and
        move to the right; requests whose last chunk is full pause (move left) until a chunk
        can be granted; resumed requests (LIFO) receive a fresh chunk; finally the per-token
        rows are rewritten for a one-token-per-request decode step.  Returns the ids of
        requests that were newly paused and stay paused, or ``None``.
        """
        # after this call every active request has one query token and one more key
        self._host_max_query_len = 1
        self._host_kv_len_bound = min(self._host_kv_len_bound + 1, self.max_sequence_length)
        if self.fused_bookkeeping:
            return self._update_requests_fused(active_requests_mask, new_tokens)
        self.last_finished_request_ids = None
        n_continue = (active_requests_mask == 1).sum().item()
        n_finished = (active_requests_mask == 0).sum().item()
        assert n_continue + n_finished + self.paused_request_count == self.total_request_count

        self.reset_attention_state()
        paused0 = self.paused_request_count

        # nothing left at all: give every chunk back and start over
        if n_continue + paused0 == 0:
            if n_finished > 0:
                done = torch.nonzero(active_requests_mask == 0, as_tuple=True)[0] + paused0
                self._release_chunks_of(done)
            self.request_to_kv_chunk_ids.fill_(-1)
            self.total_request_count = 0
            self.active_token_count = 0
            return None

        if paused0 != 0:
            assert self.paused_tokens is not None
            next_tokens = torch.cat((self.paused_tokens, new_tokens))
        else:
            next_tokens = new_tokens

        # finished requests: release chunks, then fill their holes from the right end
        if n_finished > 0:
            done = torch.nonzero(active_requests_mask == 0, as_tuple=True)[0] + paused0
            self._release_chunks_of(done)
            self.request_to_kv_chunk_ids[done] = -1
            if n_continue > 0:
                holes = torch.nonzero(active_requests_mask[:n_continue] == 0, as_tuple=True)[0] + paused0
                movers = (torch.nonzero(active_requests_mask[n_continue:], as_tuple=True)[0]
                          + n_continue + paused0)
                self._move_book_keeping_tensors(src_idxs=movers, dst_idxs=holes, next_tokens=next_tokens)
                self.request_to_kv_chunk_ids[movers] = -1

        # requests sitting on a full last chunk pause until they get a new one
        newly_paused_request_ids = None
        if n_continue > 0:
            fill = self.request_last_kv_chunk_offset[paused0 : paused0 + n_continue]
            needs_chunk = (fill == self.chunk_size_tokens - 1).byte()
            n_need = (needs_chunk == 1).sum().item()
            if 0 < n_need != n_continue:
                stay_left = torch.nonzero(needs_chunk[:n_need] == 0, as_tuple=True)[0] + paused0
                need_right = torch.nonzero(needs_chunk[n_need:], as_tuple=True)[0] + n_need + paused0
                dst = torch.cat((stay_left, need_right))
                src = torch.cat((need_right, stay_left))
                self._move_book_keeping_tensors(src_idxs=src, dst_idxs=dst, next_tokens=next_tokens)
                newly_paused_request_ids = self.request_ids[dst]
            self.paused_request_count += n_need
            n_continue -= n_need

        # how many paused requests can be given a chunk now
        spare = max(0, self.chunk_allocator.chunk_count_avail - self.gtd_chunk_count)
        if spare:
            n_resume = min(spare, self.paused_request_count)
        else:
            n_resume = min(max(self.gtd_request_count - n_continue, 0), self.paused_request_count)
        self.paused_request_count -= n_resume
        n_continue += n_resume
        assert n_continue > 0, "active_request_count == %d." % n_continue
        if newly_paused_request_ids is not None and n_resume > 0:
            newly_paused_request_ids = newly_paused_request_ids[:-n_resume]

        # next step: one token per active request
        self.total_request_count = n_continue + self.paused_request_count
        self.active_token_count = n_continue
        act = self._active()
        self.token_to_input_ids[:n_continue] = next_tokens[act]
        if self.paused_request_count > 0:
            self.paused_tokens = next_tokens[: self.paused_request_count]

        self.request_kv_length_offsets[act].add_(self.request_query_lengths[act])
        self.request_query_lengths[act].fill_(1)
        self.token_to_pos_ids[:n_continue] = self.request_kv_length_offsets[act]
        self.request_last_kv_chunk_offset[act] = (self.request_last_kv_chunk_offset[act] + 1) % self.chunk_size_tokens

        if n_resume > 0:
            first = self.paused_request_count
            resumed = slice(first, first + n_resume)
            assert torch.all(self.request_last_kv_chunk_offset[resumed] == 0), (
                "The request_last_kv_chunk_offset should be 0 for the requests that just got resumed this step. ")
            chunk_ids = self.chunk_allocator.allocate_memory_chunks(n_resume)
            rows = torch.arange(first, first + n_resume, device=self.device)
            cols = self.request_kv_chunk_counts[resumed]
            self.request_to_kv_chunk_ids[rows, cols] = chunk_ids
            self.request_kv_chunk_counts[resumed] += 1
            self.request_last_kv_chunk_id[resumed] = chunk_ids

        self.token_to_request_idx[:n_continue] = torch.arange(
            self.paused_request_count, self.total_request_count, device=self.device)
        self.token_to_position_in_request[:n_continue] = self.request_kv_length_offsets[act]
        self.token_to_chunk_idx[:n_continue] = self.request_last_kv_chunk_id[act]
        self.token_to_local_position_within_kv_chunk[:n_continue] = self.request_last_kv_chunk_offset[act]
        return newly_paused_request_ids

    def _update_requests_fused(self, active_requests_mask: Tensor, new_tokens: Tensor) -> Optional[Tensor]:
        """``update_requests`` as one kernel + one read-back of the new counters."""
        dev = self.device
        assert active_requests_mask.numel() + self.paused_request_count == self.total_request_count
        mask = active_requests_mask.to(device=dev, dtype=torch.int32).contiguous()
        tokens = new_tokens.to(device=dev, dtype=torch.long).contiguous()
        assert tokens.numel() >= mask.numel()
        if self.paused_request_count:
            assert self.paused_tokens is not None
            if self.paused_tokens.data_ptr() != self._paused_tokens_buf.data_ptr():
                self._paused_tokens_buf[: self.paused_request_count] = self.paused_tokens[: self.paused_request_count]
        ops.update_requests(self, mask, tokens)
        self._counters_host.copy_(self._counters, non_blocking=True)
        torch.cuda.current_stream(dev).synchronize()
        total, paused, active, avail, n_newly, status, was_reset, n_finished = self._counters_host.tolist()
        assert status != 1, "active + finished + paused requests != total_request_count"
        self.last_finished_request_ids = self._finished_ids_buf[:n_finished].clone()
        self.reset_attention_state()
        assert status != 2, "active_request_count == 0."
        assert status != 3, (
            "The request_last_kv_chunk_offset should be 0 for the requests that just got resumed this step. ")
        self.chunk_allocator.chunk_count_avail = avail
        self.total_request_count = total
        self.active_token_count = active
        if was_reset:
            return None
        self.paused_request_count = paused
        if paused > 0:
            self.paused_tokens = self._paused_tokens_buf[:paused]
        return None if n_newly < 0 else self._newly_paused_buf[:n_newly].clone()

    def calculate_log_probs(self, logits: Tensor, new_tokens: Tensor,
                            only_last_token_logits: Optional[bool] = False) -> List[List[float]]:
        """Log-probabilities of the tokens actually chosen, grouped per active request.

        Reference: dynamic_context.py:1300-1365.  For prefill rows the chosen token of position
        p is the prompt token at p+1; the last position of each request takes ``new_tokens``.
        """
        rows = logits.squeeze(0)
        if rows.is_cuda and rows.dtype in (torch.float32, torch.bfloat16, torch.float16) and rows.stride(-1) == 1:
            # one read of every row, no [T, V] fp32 intermediate (other dtypes / layouts: the torch ops below)
            def pick(ids):
                return ops.selected_log_probs(rows[: ids.numel()], ids.to(torch.int64).contiguous())
        else:
            def pick(ids):
                log_probs = F.log_softmax(rows.float(), dim=-1)
                return log_probs[torch.arange(ids.numel(), device=rows.device), ids]
        if only_last_token_logits or self.is_decode_only():
            return [[lp] for lp in pick(new_tokens).flatten().tolist()]

        chosen = self.token_to_input_ids[: self.active_token_count].roll(-1, 0)
        q_lens = self.request_query_lengths[self._active()]
        chosen[q_lens.cumsum(0) - 1] = new_tokens
        picked = pick(chosen)
        return [lp.tolist() for lp in picked.cpu().split(q_lens.tolist(), dim=0)]
