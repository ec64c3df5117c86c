"""Free-list of KV-cache chunk ids.

Same observable behaviour as the reference allocator
(megatron/core/inference/contexts/dynamic_chunk_allocator.py:9-92): a stack of int32
ids kept on the device, handed out from the top, with the highest id set aside as the
"dummy" chunk that padded decode tokens write into.
"""
from __future__ import annotations

from typing import Optional, Union

import torch
from torch import Tensor


class ChunkAllocator:
    """LIFO pool of chunk ids ``0 .. chunk_count_total-2`` (+ one reserved dummy id).

    Args:
        chunk_count_total: chunks in the memory buffer, dummy included.
        gtd_chunk_count: chunks held back for requests that are guaranteed to finish;
            only ``safe=True`` requests respect the reserve.
        device: where the id stack lives (defaults to the current GPU).
    """

    def __init__(self, chunk_count_total: int, gtd_chunk_count: int,
                 device: Optional[Union[torch.device, str, int]] = None):
        if device is None:
            device = torch.cuda.current_device()
        self.chunk_count_total = chunk_count_total
        self.gtd_chunk_count = gtd_chunk_count
        self.dummy_chunk_idx = chunk_count_total - 1
        self.chunk_count_avail = chunk_count_total - 1
        self.chunk_bag = torch.arange(chunk_count_total, dtype=torch.int32, device=device)

    def is_memory_available(self, num_chunks: int, safe: bool = False) -> bool:
        """Can ``num_chunks`` be handed out (leaving the guaranteed reserve alone if ``safe``)?"""
        reserve = self.gtd_chunk_count if safe else 0
        return self.chunk_count_avail >= num_chunks + reserve

    def allocate_memory_chunks(self, num_chunks: int = 1, safe: bool = False) -> Optional[Tensor]:
        """Pop ``num_chunks`` ids off the top of the stack; ``None`` when they do not fit.

        The returned tensor is a view of the stack (ids in ascending stack position).
        """
        if not self.is_memory_available(num_chunks, safe):
            return None
        top = self.chunk_count_avail
        self.chunk_count_avail = top - num_chunks
        return self.chunk_bag[top - num_chunks : top]

    def release_memory_chunks(self, chunks: Tensor) -> None:
        """Push ids back onto the stack in the order given."""
        n = chunks.size(0)
        top = self.chunk_count_avail
        self.chunk_bag[top : top + n] = chunks
        self.chunk_count_avail = top + n

    def reset(self) -> None:
        """Everything but the dummy chunk becomes available again (stack contents kept)."""
        self.chunk_count_avail = self.chunk_count_total - 1
