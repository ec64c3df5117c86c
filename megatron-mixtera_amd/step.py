"""One engine step over a dynamic context.

Plays the role of ``TextGenerationController.async_generate_output_tokens_dynamic_batch``
(megatron/core/inference/text_generation_controllers/text_generation_controller.py:411-546) for this
path: the order of the calls on the context and the keys of the returned dictionary are the contract with
the engine and are kept; everything else is arranged for the kernels of this package.  The model sits
behind a callable ``forward_step(input_ids, position_ids) -> logits`` that returns
``[1, padded_active_token_count, vocab]`` or, for a model that gathers the last-token rows itself
(``materialize_only_last_token_logits``), ``[1, active requests, vocab]``.

GPU work between the logits and the next step: one gather launch (``mi_last_token_gather``), one
sampling launch that also writes the finished mask (``mi_sample_from_logits``), optionally one
log-probability launch, and the bookkeeping kernel (``mi_update_requests``), which also lists the ids of
the finished requests -- where the reference issues about 25 small torch kernels plus a ``nonzero`` and an
index for those ids.  Pipeline-parallel broadcast of the logits, tokenizer work and top-n log-probability
bookkeeping stay with the controller.
"""
from __future__ import annotations

from typing import Callable, Dict, Optional

import torch
from torch import Tensor

from . import sampling

ForwardStep = Callable[[Tensor, Tensor], Tensor]


def _wants_log_probs(sampling_params, last_rows_only: bool) -> bool:
    if not getattr(sampling_params, "return_log_probs", False):
        return False
    prompt_skipped = getattr(sampling_params, "skip_prompt_log_probs_for_dynamic_inference", False)
    assert prompt_skipped or not last_rows_only, (
        "Materialize only last token logits must be false for returning log probs")
    return True


def _rows_to_sample(context, logits: Tensor, last_rows_only: bool) -> Tensor:
    """One row of logits per active request: its last token's."""
    if not last_rows_only:
        return context.last_token_logits(logits)
    rows = logits.squeeze(0)
    n_active = context.total_request_count - context.paused_request_count
    assert rows.size(0) == n_active, "the model returns one row of logits per active request"
    return rows


def _finished_ids(context, ids_before: Tensor, keep_mask: Tensor) -> Tensor:
    """Ids of the requests whose mask entry is 0, in row order.  The bookkeeping kernel has already listed
    them; a context that ran the torch op sequence instead (host tensors) has not."""
    listed = getattr(context, "last_finished_request_ids", None)
    if listed is not None:
        return listed
    return ids_before[(keep_mask == 0).to(ids_before.device)].to(torch.int32)


@torch.inference_mode()
def generate_output_tokens_dynamic_batch(context, forward_step: ForwardStep, sampling_params, termination_id: int, *,
                                         vocab_size: Optional[int] = None,
                                         generator: Optional[torch.Generator] = None,
                                         uniform: Optional[Tensor] = None) -> Optional[Dict[str, object]]:
    """Run the model once on the context's current tokens and advance the context by the sampled tokens.

    ``None`` when the context holds no token.  Otherwise a dictionary with ``active_request_ids`` (int64, the
    requests that took part), ``newly_paused_request_ids``, ``finished_request_ids``, ``sample`` (int64, one
    token per active request), ``log_probs`` (``None`` unless asked for) and ``cuda_graph_request_count``
    (the padded batch size of a decode step, else ``None``).
    """
    last_rows_only = context.materialize_only_last_token_logits
    with_log_probs = _wants_log_probs(sampling_params, last_rows_only)
    if context.active_token_count == 0:
        return None

    # the step's padding, lengths and block table; then the model
    context.initialize_attention_state()
    graph_batch = context.padded_active_request_count if context.is_decode_only() else None
    logits = forward_step(*context.current_input_and_position_ids())

    # who took part (the rows move during update_requests, so the ids are taken now)
    ids_before = context.request_ids[context.paused_request_count:context.total_request_count].long()

    # sample + "does this request go on?" in one launch
    sample, keep_mask = sampling.sample_and_finish_mask(
        context, _rows_to_sample(context, logits, last_rows_only), sampling_params, termination_id, vocab_size,
        generator=generator, uniform=uniform)

    log_probs = None
    if with_log_probs:
        log_probs = context.calculate_log_probs(logits, sample, only_last_token_logits=last_rows_only)

    # update_requests works on its own copy of the sample: the caller keeps `sample` as drawn
    newly_paused = context.update_requests(keep_mask, sample.clone())

    return {
        "active_request_ids": ids_before,
        "newly_paused_request_ids": newly_paused,
        "finished_request_ids": _finished_ids(context, ids_before, keep_mask),
        "sample": sample,
        "log_probs": log_probs,
        "cuda_graph_request_count": graph_batch,
    }
