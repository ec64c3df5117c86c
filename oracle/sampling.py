"""Oracle for the tail of a decode step: last-token rows, logit filters, the draw, the finished mask.

TEST INFRASTRUCTURE ONLY -- nothing in the product imports this module.

Restates, on CPU tensors:
* ``DynamicInferenceContext.last_token_logits``: rows ``cumsum(request_query_lengths) - 1``
  (megatron/core/inference/contexts/dynamic_context.py:890-918);
* ``TextGenerationController.sample_from_logits``
  (megatron/core/inference/text_generation_controllers/text_generation_controller.py:172-315):
  greedy argmax (:289-290), division by the temperature (:292-294), the top-k filter
  ``logits < topk(logits, k)[0][..., -1]`` (:216-219), the top-p filter -- descending sort, softmax,
  cumsum, ``cumulative > top_p`` shifted right by one with the first column cleared (:221-240);
* the finished-request test ``(sample != termination_id) & (length + 1 < maximum length)``
  (text_generation_controller.py:519-530);
* ``DynamicInferenceContext.calculate_log_probs`` (dynamic_context.py:1300-1365): which token id each
  logits row is scored on (:1326-1355) and ``log_softmax(logits.float())[row, id]`` (:1317-1322,1357-1359).

The reference then draws with ``torch.multinomial`` from its own generator (:307-309); a stream of
random numbers cannot be reproduced by another implementation, so the draw restated here is the
inverse CDF over the kept probabilities in vocabulary order for a GIVEN uniform number -- the same
distribution.  Temperature: the reference divides in place on the device, where torch evaluates a
division by a host scalar as a multiplication by its fp32 reciprocal and rounds to the tensor's
dtype; :func:`scaled_logits` does exactly that.

Pinned by (tests/test_oracle_sampling.py): ``torch.topk`` / ``torch.sort`` library routines, a
hand-worked top-p example, the set definition "shortest prefix whose mass exceeds p" by brute
force, limiting cases (p -> 0 keeps the argmax, p = 1 keeps all, k = V keeps all),
``numpy.searchsorted`` for the draw, and an empirical-frequency check of the draw; the log-prob
functions by ``torch.log_softmax`` / ``torch.logsumexp`` and by the worked example in the reference's
own comment (dynamic_context.py:1331-1349).
"""
from __future__ import annotations

from typing import Optional

import torch
from torch import Tensor


def last_token_indices(request_query_lengths: Tensor) -> Tensor:
    """Row of each active request's last token in the flattened token dimension."""
    return torch.cumsum(request_query_lengths.long(), dim=0) - 1


def scaled_logits(logits: Tensor, temperature: float) -> Tensor:
    """``logits.div_(temperature)`` as the device evaluates it, returned as fp32 values."""
    if temperature == 1.0:
        return logits.float()
    inv = torch.tensor(1.0, dtype=torch.float32) / torch.tensor(temperature, dtype=torch.float32)
    return (logits.float() * inv).to(logits.dtype).float()


def top_k_keep(x: Tensor, top_k: int) -> Tensor:
    """Boolean ``[R, V]``: entries the top-k filter leaves (everything >= the k-th largest)."""
    kth = torch.topk(x, top_k, dim=-1)[0][..., -1, None]
    return ~(x < kth)


def top_p_keep(x: Tensor, top_p: float) -> Tensor:
    """Boolean ``[R, V]``: entries the top-p filter leaves.  Equal values are ordered by index
    (stable sort); the reference's sort leaves their order open."""
    sorted_x, order = torch.sort(x.double(), dim=-1, descending=True, stable=True)
    cumulative = sorted_x.softmax(dim=-1).cumsum(dim=-1)
    drop = cumulative > top_p
    drop[:, 1:] = drop[:, :-1].clone()
    drop[:, 0] = False
    drop = drop.scatter(1, order, drop)
    return ~drop


def kept_probabilities(x: Tensor, keep: Optional[Tensor]) -> Tensor:
    """fp64 softmax over the kept entries (filtered entries get probability 0)."""
    z = x.double()
    if keep is not None:
        z = z.masked_fill(~keep, float("-inf"))
    return z.softmax(dim=-1)


def draw_inverse_cdf(probabilities: Tensor, uniform: Tensor) -> Tensor:
    """``min{ j : sum_{i<=j} p_i > u }`` per row."""
    cdf = probabilities.double().cumsum(dim=-1)
    want = uniform.double()[:, None] * cdf[:, -1:]
    idx = (cdf > want).to(torch.int8).argmax(dim=-1)
    return idx.long()


def sample_from_logits(logits: Tensor, *, top_k: int = 0, top_p: float = 0.0, temperature: float = 1.0,
                       uniform: Optional[Tensor] = None, vocab_size: Optional[int] = None) -> Tensor:
    """The reference's control flow with the inverse-CDF draw in place of ``torch.multinomial``."""
    assert not (top_k > 0 and top_p > 0.0), "Cannot have top-p and top-k both greater than zero"
    assert top_p <= 1.0, "top-p should be in (0,1]"
    if top_k == 1:
        return torch.argmax(logits.float(), dim=-1)
    x = scaled_logits(logits, temperature)
    keep = None
    if top_k > 1:
        assert top_k <= x.size(1), "top-k is larger than logit size."
        keep = top_k_keep(x, top_k)
    elif top_p > 0.0:
        keep = top_p_keep(x, top_p)
    sample = draw_inverse_cdf(kept_probabilities(x, keep), uniform)
    if vocab_size:
        sample = sample.clamp(0, vocab_size - 1)
    return sample


def active_request_mask(sample: Tensor, termination_id: int, kv_length_offsets: Tensor, query_lengths: Tensor,
                        output_lengths: Tensor) -> Tensor:
    """uint8 mask of the requests that go on generating."""
    lengths = kv_length_offsets.long() + query_lengths.long() + 1
    return ((sample != termination_id).byte() & torch.less(lengths, output_lengths.long()).byte())


def scored_token_ids(token_to_input_ids: Tensor, query_lengths: Tensor, new_tokens: Tensor) -> Tensor:
    """Id each active token row is scored on: the next prompt token inside a request, the newly
    sampled token at its last position (dynamic_context.py:1326-1355), by an explicit loop."""
    ids, row = [], 0
    flat = token_to_input_ids.tolist()
    for n, new in zip(query_lengths.tolist(), new_tokens.tolist()):
        ids += flat[row + 1: row + n] + [new]
        row += n
    return torch.tensor(ids, dtype=torch.int64)


def selected_log_probs(logits: Tensor, token_ids: Tensor) -> Tensor:
    """fp64 ``x[id] - log(sum(exp(x)))`` per row of the fp32-converted logits (:1317, :1357-1359)."""
    x = logits.float().double()
    mx = x.max(dim=-1, keepdim=True).values
    lse = (x - mx).exp().sum(-1).log() + mx.squeeze(-1)
    return x.gather(1, token_ids.view(-1, 1).long()).squeeze(1) - lse
