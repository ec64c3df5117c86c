"""Host side of the decode-step tail: the reference's ``sample_from_logits`` surface on one kernel.

``sample_from_logits`` keeps the argument meaning and the assertions of
``TextGenerationController.sample_from_logits``
(megatron/core/inference/text_generation_controllers/text_generation_controller.py:172-315);
``sample_and_finish_mask`` adds what ``async_generate_output_tokens_dynamic_batch`` computes
right after it (:519-530), so a decode step needs one launch between the logits and
``DynamicInferenceContext.update_requests``.

The reference draws with ``torch.multinomial(probabilities, 1, generator=sampling_rng)``; here
the same generator produces one uniform number per row and the kernel inverts the CDF of the
filtered distribution -- the same distribution from a different stream of random numbers.
``top_n_logprobs`` bookkeeping is not part of this path.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch
from torch import Tensor

from . import ops


def _checked_params(sampling_params) -> Tuple[int, float, float]:
    top_p, top_k, temperature = sampling_params.top_p, sampling_params.top_k, sampling_params.temperature
    assert isinstance(top_p, float)
    assert isinstance(top_k, int)
    assert not (top_k > 0 and top_p > 0.0), "Cannot have top-p and top-k both greater than zero"
    assert top_p <= 1.0, "top-p should be in (0,1]"
    return top_k, top_p, float(temperature)


def _uniform(n: int, device, generator: Optional[torch.Generator]) -> Tensor:
    return torch.rand(n, dtype=torch.float32, device=device, generator=generator)


def sample_from_logits(last_token_logits: Tensor, sampling_params, vocab_size: Optional[int] = None, *,
                       generator: Optional[torch.Generator] = None, uniform: Optional[Tensor] = None) -> Tensor:
    """``[batch]`` int64 samples from ``[batch, vocab]`` logits (not modified)."""
    top_k, top_p, temperature = _checked_params(sampling_params)
    if top_k > 1:
        assert top_k <= last_token_logits.size(1), "top-k is larger than logit size."
        if vocab_size:
            assert top_k < vocab_size, "top-k is larger than vocab size."
    if top_k != 1 and uniform is None:
        uniform = _uniform(last_token_logits.size(0), last_token_logits.device, generator)
    samples, _ = ops.sample_from_logits(last_token_logits, top_k=top_k, top_p=top_p, temperature=temperature,
                                        uniform=uniform, vocab_size=vocab_size if top_k != 1 else None)
    return samples


def sample_and_finish_mask(context, last_token_logits: Tensor, sampling_params, termination_id: int,
                           vocab_size: Optional[int] = None, *, generator: Optional[torch.Generator] = None,
                           uniform: Optional[Tensor] = None) -> Tuple[Tensor, Tensor]:
    """``(new_sample, active_request_mask)`` for the active requests of ``context``: the sample of
    :func:`sample_from_logits` and ``(sample != termination_id) & (sequence length + 1 < maximum)``
    as a uint8 row, ready for ``context.update_requests``."""
    top_k, top_p, temperature = _checked_params(sampling_params)
    if top_k > 1:
        assert top_k <= last_token_logits.size(1), "top-k is larger than logit size."
        if vocab_size:
            assert top_k < vocab_size, "top-k is larger than vocab size."
    active = slice(context.paused_request_count, context.total_request_count)
    n = context.total_request_count - context.paused_request_count
    assert last_token_logits.size(0) == n, "one row of logits per active request"
    if top_k != 1 and uniform is None:
        uniform = _uniform(n, last_token_logits.device, generator)
    samples, mask = ops.sample_from_logits(
        last_token_logits, top_k=top_k, top_p=top_p, temperature=temperature, uniform=uniform,
        vocab_size=vocab_size if top_k != 1 else None, termination_id=termination_id,
        kv_length_offsets=context.request_kv_length_offsets[active],
        query_lengths=context.request_query_lengths[active], output_lengths=context.request_output_lengths[active])
    return samples, mask
