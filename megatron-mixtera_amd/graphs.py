"""HIP-graph capture of the per-layer decode path, one graph per padded decode batch size.

The reference captures its decode step once per entry of
``DynamicInferenceContext.cuda_graph_token_counts`` during engine warm-up
(megatron/core/inference/engines/dynamic_engine.py:143-227, sizes from
megatron/core/inference/contexts/dynamic_context.py:319-382) and replays the graph whose size
``initialize_attention_state`` picked for the step (megatron/core/transformer/cuda_graphs.py:1224-1266
replays per transformer layer).  The part of a layer that lives in this package -- q/k norm, RoPE,
KV-append and paged attention -- is captured here the same way: per layer and per size, with
static q/k/v/out buffers.  Everything a replay reads besides those buffers sits at fixed
addresses inside the context (the ``*_cudagraph_only`` mirrors and the per-token rows), which
``initialize_attention_state`` refreshes before every step.

Nothing in the captured region allocates from the caller's pool, synchronises or memsets.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence, Tuple

import torch
from torch import Tensor

from . import ops
from .contexts.dynamic_context import WarmupEngineMode


class DecodeLayerGraphs:
    """Captured decode graphs for a list of :class:`PagedSelfAttentionCore` layers.

    ``capture()`` must run while the context is empty (as the reference's warm-up does, before
    any request is admitted); it walks ``cuda_graph_token_counts`` from the largest size down and,
    when the context was built with ``use_cuda_graphs_for_non_decode_steps`` (the reference's
    default), captures a second graph per size for prefill / mixed steps
    (``WarmupEngineMode.NON_DECODE``: the varlen attention path over the padded mirrors).
    ``replay(layer_index, query, key, value)`` copies the step's tensors into the static inputs
    of the graph for ``context.padded_active_token_count`` and the step's kind, and returns the
    static output ``[padded, 1, Hq*d]`` (valid until the next replay of the same graph).
    """

    def __init__(self, context, layers: Sequence[torch.nn.Module], *, num_query_heads: int,
                 rotary_pos_emb: Optional[Tuple[Tensor, Tensor]] = None):
        if context.cuda_graph_token_counts is None:
            raise ValueError("the context was built without cuda-graph sizes (num_cuda_graphs=None)")
        self.context = context
        self.layers = list(layers)
        self.num_query_heads = num_query_heads
        self.rotary_pos_emb = rotary_pos_emb
        # (layer index, padded tokens, decode-only?) -> (graph, q, k, v, out)
        self._graphs: Dict[Tuple[int, int, bool], Tuple[torch.cuda.CUDAGraph, Tensor, Tensor, Tensor, Tensor]] = {}
        self._pool = None
        # one workspace for every graph, sized for the largest decode batch and never re-allocated,
        # so no graph is left holding a pointer into freed memory
        ctx = context
        hkv, d = ctx.num_kv_heads_per_partition, ctx.kv_channels
        need = ops.decode_workspace_bytes(ctx.max_requests, num_query_heads, hkv, d, ctx.chunk_size_tokens,
                                          ctx.max_sequence_length, 0)
        if ctx.non_decode_cuda_graphs:  # prefill / mixed steps may split the keys of a request: more scratch
            table_tokens = ctx.request_to_kv_chunk_ids.size(1) * ctx.chunk_size_tokens
            for n in ctx.cuda_graph_token_counts:
                for max_kv in (ctx.max_sequence_length, table_tokens):
                    need = max(need, ops.prefill_workspace_bytes(n, ctx.max_requests, num_query_heads, hkv, d, max_kv, 0))
        self.workspace = torch.empty(max(need, 1), dtype=torch.uint8, device=ctx.device)

    @property
    def sizes(self) -> List[int]:
        return sorted({n for (_, n, _) in self._graphs})

    def capture(self) -> None:
        ctx = self.context
        assert ctx.total_request_count == 0, "capture the graphs before any request is admitted"
        dev = ctx.device
        hkv, d = ctx.num_kv_heads_per_partition, ctx.kv_channels
        dtype = ctx.params_dtype
        side = torch.cuda.Stream(device=dev)
        modes = [WarmupEngineMode.DECODE]
        if ctx.non_decode_cuda_graphs:
            modes.append(WarmupEngineMode.NON_DECODE)
        for mode in modes:
            for n in ctx.cuda_graph_token_counts:  # largest first, as the reference warms up
                ctx.initialize_attention_state(num_warmup_tokens=n, warmup_engine_mode=mode)
                decode = mode == WarmupEngineMode.DECODE
                assert ctx.padded_active_token_count == n and ctx.is_decode_only() == decode
                for li, layer in enumerate(self.layers):
                    q = torch.zeros(n, 1, self.num_query_heads, d, dtype=dtype, device=dev)
                    k = torch.zeros(n, 1, hkv, d, dtype=dtype, device=dev)
                    v = torch.zeros(n, 1, hkv, d, dtype=dtype, device=dev)
                    side.wait_stream(torch.cuda.current_stream(dev))
                    with torch.cuda.stream(side):  # one eager run first (library handles, lazy initialisation)
                        self._run(layer, q, k, v)
                    torch.cuda.current_stream(dev).wait_stream(side)
                    graph = torch.cuda.CUDAGraph()
                    with torch.cuda.graph(graph, pool=self._pool):
                        out = self._run(layer, q, k, v)
                    if self._pool is None:
                        self._pool = graph.pool()
                    self._graphs[(li, n, decode)] = (graph, q, k, v, out)
                ctx.reset()
        ctx.reset()

    def _run(self, layer, q: Tensor, k: Tensor, v: Tensor) -> Tensor:
        with ops.use_workspace(self.workspace):
            return layer(q, k, v, self.context, self.rotary_pos_emb)

    def replay(self, layer_index: int, query: Tensor, key: Tensor, value: Tensor) -> Tensor:
        ctx = self.context
        n = ctx.padded_active_token_count
        decode = ctx.is_decode_only()
        entry = self._graphs.get((layer_index, n, decode)) if ctx.using_cuda_graph_this_step() else None
        if entry is None:
            raise KeyError(f"no {'decode' if decode else 'prefill'} graph for layer {layer_index} and {n} tokens "
                           f"(captured sizes: {self.sizes})")
        graph, q, k, v, out = entry
        q.copy_(query[:n])
        k.copy_(key[:n])
        v.copy_(value[:n])
        graph.replay()
        return out
