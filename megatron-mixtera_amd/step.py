"""One engine step on a dynamic context: forward -> last-token rows -> sample -> bookkeeping.

The same sequence and the same result dictionary as
``TextGenerationController.async_generate_output_tokens_dynamic_batch``
(megatron/core/inference/text_generation_controllers/text_generation_controller.py:411-546), with
the model behind a callable: ``forward_step(input_ids, position_ids) -> logits``, where ``logits``
is ``[1, padded_active_token_count, vocab]`` or, when the model already gathered the last-token
rows (``materialize_only_last_token_logits``), ``[1, active requests, vocab]``.

Between the logits and ``update_requests`` the reference runs ~25 small torch kernels (cumsum,
index, clone, div, topk / sort, masked_fill, softmax, multinomial, comparisons); here it is two
launches: :func:`ops.last_token_gather` and :func:`ops.sample_from_logits` (sample + finished
mask).  Pipeline-parallel logit broadcast, tokenizer work and top-n log-prob bookkeeping belong
to the controller and are not part of this path.
"""
from __future__ import annotations

from typing import Callable, Dict, Optional

import torch
from torch import Tensor

from . import sampling


@torch.inference_mode()
def generate_output_tokens_dynamic_batch(context, forward_step: Callable[[Tensor, Tensor], Tensor], sampling_params,
                                         termination_id: int, *, vocab_size: Optional[int] = None,
                                         generator: Optional[torch.Generator] = None,
                                         uniform: Optional[Tensor] = None) -> Optional[Dict[str, object]]:
    """Forward step the model and update the inference context.

    Returns ``None`` when the context holds no token, else the reference's dictionary:
    ``active_request_ids`` (int64), ``newly_paused_request_ids``, ``finished_request_ids``,
    ``sample`` (int64), ``log_probs`` and ``cuda_graph_request_count``.
    """
    materialize_only_last = context.materialize_only_last_token_logits
    if getattr(sampling_params, "return_log_probs", False):
        skip_prompt = getattr(sampling_params, "skip_prompt_log_probs_for_dynamic_inference", False)
        assert skip_prompt or materialize_only_last is False, (
            "Materialize only last token logits must be false for returning log probs")

    # No tokens?
    if context.active_token_count == 0:
        return None

    # Initialize attention state.
    context.initialize_attention_state()
    cuda_graph_request_count = context.padded_active_request_count if context.is_decode_only() else None

    # Get flat tokens, position ids; forward pass -> logits.
    input_ids, position_ids = context.current_input_and_position_ids()
    logits = forward_step(input_ids, position_ids)

    # Last token logits.
    n_active = context.total_request_count - context.paused_request_count
    if materialize_only_last:
        last_token_logits = logits.squeeze(0)
        assert last_token_logits.size(0) == n_active, "the model returns one row of logits per active request"
    else:
        last_token_logits = context.last_token_logits(logits)

    # Sample, and test which requests go on: one launch.
    active = slice(context.paused_request_count, context.total_request_count)
    active_request_ids = context.request_ids[active].long()
    new_sample, active_request_mask = sampling.sample_and_finish_mask(
        context, last_token_logits, sampling_params, termination_id, vocab_size, generator=generator, uniform=uniform)
    finished_idxs = torch.nonzero(active_request_mask == 0, as_tuple=True)[0] + context.paused_request_count
    finished_request_ids = context.request_ids[finished_idxs]

    # New sample gets updated in update_requests, so we pass in a clone
    new_sample_copy = new_sample.clone()

    log_probs = None
    if getattr(sampling_params, "return_log_probs", False):
        log_probs = context.calculate_log_probs(logits, new_sample_copy, only_last_token_logits=materialize_only_last)

    # Update requests.
    newly_paused_request_ids = context.update_requests(active_request_mask, new_sample_copy)

    return {
        "active_request_ids": active_request_ids,
        "newly_paused_request_ids": newly_paused_request_ids,
        "finished_request_ids": finished_request_ids,
        "sample": new_sample,
        "log_probs": log_probs,
        "cuda_graph_request_count": cuda_graph_request_count,
    }
