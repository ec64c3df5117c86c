"""Scalar-loop restatement of the dynamic context's integer bookkeeping (numpy, CPU).

Restates, one request at a time instead of with vectorised index moves:
* sizing of the chunk pool and of the request / token rows
  (megatron/core/inference/contexts/dynamic_context.py:186-242, 311, 398-401);
* the LIFO chunk allocator with its reserved dummy chunk
  (megatron/core/inference/contexts/dynamic_chunk_allocator.py:23-92);
* ``add_request`` (dynamic_context.py:920-1015);
* ``update_requests`` (dynamic_context.py:1033-1298);
* the padding rules of ``initialize_attention_state`` for decode-only, non-graph steps
  (dynamic_context.py:703-741, 777-821).

Pinned by the constants held in the reference's own tests
(tests/unit_tests/inference/contexts/test_dynamic_context.py:69-87, 263-279, 298-345,
401-515, 535-566, 586-630; tests/unit_tests/inference/engines/test_dynamic_engine.py:381-386,
415-423) -- see tests/test_context_host.py, which checks both this restatement and the
product class against them, and the two against each other on random request streams.
"""
from __future__ import annotations

import math
from typing import List, Optional

import numpy as np


def ceil_to(value: int, multiple: int) -> int:
    return multiple * int(math.ceil(int(value) / multiple))


def sizing(*, itemsize: int, num_layers: int, kv_channels: int, num_heads: int, max_sequence_length: int,
           buffer_size_gb: float, buffer_guaranteed_fraction: float, chunk_size_tokens: int = 256,
           buffer_overflow_factor: Optional[float] = None, max_requests_override: Optional[int] = None,
           max_tokens_override: Optional[int] = None, tp_size: int = 1, token_rounder: int = 64,
           request_rounder: int = 4) -> dict:
    heads = num_heads // tp_size
    chunk_bytes = itemsize * 2 * num_layers * chunk_size_tokens * heads * kv_channels
    pool = int(buffer_size_gb * 1024**3)
    pool -= pool % chunk_bytes
    tr = math.ceil(token_rounder / tp_size) * tp_size
    rr = math.ceil(request_rounder / tp_size) * tp_size
    n_tokens = pool / chunk_bytes * chunk_size_tokens
    max_requests = ceil_to(int(n_tokens / max_sequence_length), rr)
    max_tokens = ceil_to(int(n_tokens), tr)
    if buffer_overflow_factor is not None:
        max_requests = ceil_to(int(max_requests * buffer_overflow_factor), rr)
        max_tokens = ceil_to(int(max_tokens * buffer_overflow_factor / 50.0), tr)
    if max_requests_override is not None:
        max_requests = ceil_to(max_requests_override, rr)
    if max_tokens_override is not None:
        max_tokens = ceil_to(max_tokens_override, tr)
    max_requests = min(max_requests, max_tokens)
    total = pool // chunk_bytes
    max_kv_chunks = math.ceil(max_sequence_length / chunk_size_tokens)
    reserve = min(int(buffer_guaranteed_fraction * total), total)
    gtd_requests = max(1, reserve // max_kv_chunks)
    return dict(chunk_size_bytes=chunk_bytes, chunk_count_total=total, max_requests=max_requests,
                max_tokens=max_tokens, max_kv_chunk_count=max_kv_chunks, gtd_request_count=gtd_requests,
                gtd_chunk_count=gtd_requests * max_kv_chunks)


def cuda_graph_token_counts(max_requests: int, num_cuda_graphs: int, tp_size: int = 1) -> List[int]:
    """Batch sizes captured as graphs (dynamic_context.py:319-344), largest first."""
    n = min(max(num_cuda_graphs, 1), max_requests)
    step = math.ceil((max_requests / n) / 8) * 8
    step = math.ceil(step / tp_size) * tp_size
    if n == 1:
        return [max_requests]
    counts = list(range(step, max_requests, step))
    if counts[-1] != max_requests:
        counts.append(max_requests)
    return counts[::-1]


class RefContext:
    """The bookkeeping state as plain numpy arrays, updated with scalar loops."""

    def __init__(self, *, max_requests: int, max_tokens: int, chunk_count_total: int, chunk_size_tokens: int,
                 max_kv_chunk_count: int, gtd_request_count: int, gtd_chunk_count: int, max_sequence_length: int,
                 token_rounder: int = 64):
        self.max_requests, self.max_tokens = max_requests, max_tokens
        self.C = chunk_size_tokens
        self.M = max_kv_chunk_count
        self.gtd_request_count, self.gtd_chunk_count = gtd_request_count, gtd_chunk_count
        self.max_sequence_length = max_sequence_length
        self.token_rounder = token_rounder
        self.total = chunk_count_total
        self.bag = np.arange(chunk_count_total, dtype=np.int32)
        self.avail = chunk_count_total - 1
        self.dummy = chunk_count_total - 1
        z = lambda n, fill=0: np.full(n, fill, dtype=np.int64)
        self.ids = z(max_requests, -1)
        self.q_len = z(max_requests)
        self.out_len = z(max_requests)
        self.kv_off = z(max_requests)
        self.n_chunks = z(max_requests)
        self.last_chunk = z(max_requests, -1)
        self.last_off = z(max_requests)
        self.table = np.full((max_requests, max_kv_chunk_count), -1, dtype=np.int64)
        self.tok_input = z(max_tokens)
        self.tok_pos = z(max_tokens)
        self.tok_req = z(max_tokens, -1)
        self.tok_chunk = z(max_tokens, -1)
        self.tok_in_req = z(max_tokens)
        self.tok_local = z(max_tokens)
        self.total_requests = 0
        self.paused = 0
        self.active_tokens = 0
        self.paused_tokens: List[int] = []

    # ---- allocator ----
    def alloc(self, n: int, safe: bool = False):
        if self.avail < n + (self.gtd_chunk_count if safe else 0):
            return None
        self.avail -= n
        return [int(x) for x in self.bag[self.avail:self.avail + n]]

    def release(self, chunks) -> None:
        for c in chunks:
            self.bag[self.avail] = c
            self.avail += 1

    # ---- add_request ----
    def add_request(self, request_id: int, tokens, num_tokens_to_generate: Optional[int] = None) -> str:
        """Returns "" on success or the name of the overflow that the reference would raise."""
        n = len(tokens)
        if n > self.max_tokens or self.active_tokens + n > self.max_tokens:
            return "TokenOverflowError"
        if self.total_requests >= self.max_requests:
            return "RequestOverflowError"
        need = math.ceil(n / self.C)
        got = self.alloc(need, safe=True)
        if got is None:
            return "ChunkOverflowError"
        if num_tokens_to_generate is None:
            num_tokens_to_generate = self.max_sequence_length - n
        elif n + num_tokens_to_generate > self.max_sequence_length:
            return "MaxSequenceLengthOverflowError"  # (the reference leaks the chunks here too)
        r = self.total_requests
        self.ids[r], self.q_len[r], self.out_len[r], self.kv_off[r] = request_id, n, n + num_tokens_to_generate, 0
        self.table[r, :need] = got
        self.n_chunks[r], self.last_chunk[r], self.last_off[r] = need, got[-1], (n - 1) % self.C
        for i in range(n):
            t = self.active_tokens + i
            self.tok_pos[t] = self.tok_in_req[t] = i
            self.tok_input[t] = int(tokens[i])
            self.tok_req[t] = r
            self.tok_chunk[t] = got[i // self.C]
            self.tok_local[t] = i % self.C
        self.total_requests += 1
        self.active_tokens += n
        return ""

    # ---- update_requests ----
    def _copy_row(self, dst: int, src_vals) -> None:
        (self.kv_off[dst], self.q_len[dst], self.out_len[dst], self.ids[dst], self.n_chunks[dst],
         self.last_chunk[dst], self.last_off[dst]) = src_vals[:7]
        self.table[dst] = src_vals[7]

    def _row(self, i: int):
        return (self.kv_off[i], self.q_len[i], self.out_len[i], self.ids[i], self.n_chunks[i], self.last_chunk[i],
                self.last_off[i], self.table[i].copy())

    def update_requests(self, mask, new_tokens):
        mask = [int(x) for x in mask]
        n_cont = sum(1 for m in mask if m == 1)
        n_fin = sum(1 for m in mask if m == 0)
        assert n_cont + n_fin + self.paused == self.total_requests
        p0 = self.paused
        if n_cont + p0 == 0:
            for i, m in enumerate(mask):
                if m == 0:
                    self.release([int(c) for c in self.table[p0 + i] if c != -1])
            self.table[:] = -1
            self.total_requests = 0
            self.active_tokens = 0
            return None
        nxt = list(self.paused_tokens[:p0]) + [int(x) for x in new_tokens]
        if n_fin > 0:
            done = [p0 + i for i, m in enumerate(mask) if m == 0]
            for i in done:
                self.release([int(c) for c in self.table[i] if c != -1])
            for i in done:
                self.table[i] = -1
            if n_cont > 0:
                holes = [p0 + i for i in range(n_cont) if mask[i] == 0]
                movers = [p0 + i for i in range(n_cont, len(mask)) if mask[i] == 1]
                rows = [self._row(s) for s in movers]
                toks = [nxt[s] for s in movers]
                for d, vals, tk in zip(holes, rows, toks):
                    self._copy_row(d, vals)
                    nxt[d] = tk
                for s in movers:
                    self.table[s] = -1
        newly_paused = None
        if n_cont > 0:
            need = [1 if self.last_off[p0 + i] == self.C - 1 else 0 for i in range(n_cont)]
            n_need = sum(need)
            if 0 < n_need != n_cont:
                left = [p0 + i for i in range(n_need) if need[i] == 0]
                right = [p0 + i for i in range(n_need, n_cont) if need[i] == 1]
                dst, src = left + right, right + left
                rows = [self._row(s) for s in src]
                toks = [nxt[s] for s in src]
                for d, vals, tk in zip(dst, rows, toks):
                    self._copy_row(d, vals)
                    nxt[d] = tk
                newly_paused = [int(self.ids[d]) for d in dst]
            self.paused += n_need
            n_cont -= n_need
        spare = max(0, self.avail - self.gtd_chunk_count)
        if spare:
            n_resume = min(spare, self.paused)
        else:
            n_resume = min(max(self.gtd_request_count - n_cont, 0), self.paused)
        self.paused -= n_resume
        n_cont += n_resume
        assert n_cont > 0
        if newly_paused is not None and n_resume > 0:
            newly_paused = newly_paused[:-n_resume]
        self.total_requests = n_cont + self.paused
        self.active_tokens = n_cont
        for i in range(n_cont):
            self.tok_input[i] = nxt[self.paused + i]
        if self.paused > 0:
            self.paused_tokens = nxt[: self.paused]
        for r in range(self.paused, self.total_requests):
            self.kv_off[r] += self.q_len[r]
            self.q_len[r] = 1
            self.last_off[r] = (self.last_off[r] + 1) % self.C
        for i in range(n_cont):
            self.tok_pos[i] = self.kv_off[self.paused + i]
        if n_resume > 0:
            got = self.alloc(n_resume)
            for j in range(n_resume):
                r = self.paused + j
                assert self.last_off[r] == 0
                self.table[r, self.n_chunks[r]] = got[j]
                self.n_chunks[r] += 1
                self.last_chunk[r] = got[j]
        for i in range(n_cont):
            r = self.paused + i
            self.tok_req[i] = r
            self.tok_in_req[i] = self.kv_off[r]
            self.tok_chunk[i] = self.last_chunk[r]
            self.tok_local[i] = self.last_off[r]
        return newly_paused

    # ---- decode-step padding (no graphs) ----
    def decode_padding(self):
        """(padded token count, kv lengths incl. padding zeros, block table incl. padding rows of 0)."""
        n_act = self.total_requests - self.paused
        assert n_act == self.active_tokens, "decode-only step expected"
        padded = min(ceil_to(self.active_tokens, self.token_rounder), self.max_requests)
        for t in range(self.active_tokens, padded):
            self.tok_chunk[t], self.tok_local[t], self.tok_in_req[t] = self.dummy, 0, 0
        lens = np.zeros(padded, dtype=np.int64)
        table = np.zeros((padded, self.M), dtype=np.int64)
        for i in range(n_act):
            r = self.paused + i
            lens[i] = self.kv_off[r] + self.q_len[r]
            table[i] = self.table[r]
        return padded, lens, table
