"""Host-side bookkeeping of DynamicInferenceContext, checked on the CPU (device="cpu").

Three layers of evidence:
1. the constants the reference's own tests hold
   (tests/unit_tests/inference/contexts/test_dynamic_context.py and
   tests/unit_tests/inference/engines/test_dynamic_engine.py in the reference tree),
   applied to the product class AND to the scalar-loop restatement in oracle/context.py;
2. the two implementations against each other on random request streams;
3. invariants (every chunk id is either free or owned exactly once, padded rows, ...).
"""
import json
import math
import os
import random

import numpy as np
import pytest
import torch

from oracle import context as oc

# expected values held by the reference's own tests (data only; each entry names its source)
with open(os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.json")) as _f:
    GOLD = json.load(_f)


@pytest.fixture()
def Ctx(mi):
    cls = mi.DynamicInferenceContext
    saved = (cls.TOKEN_ROUNDER, cls.REQUEST_ROUNDER)
    yield cls
    cls.TOKEN_ROUNDER, cls.REQUEST_ROUNDER = saved


def set_rounder(cls, v):
    cls.ROUNDER = v
    cls.TOKEN_ROUNDER = v
    cls.REQUEST_ROUNDER = v


def small_ctx(Ctx, **over):
    """The fp32 / 4 layers / 2 heads x 8 channels / 0.03 GB / chunk 128 context of the reference tests."""
    set_rounder(Ctx, 64)
    kw = dict(params_dtype=torch.float32, num_layers=4, kv_channels=8, num_attention_heads=2,
              max_sequence_length=512, num_cuda_graphs=None, buffer_size_gb=0.03,
              buffer_guaranteed_fraction=0.1, chunk_size_tokens=128, buffer_overflow_factor=None,
              max_requests_override=None, max_tokens_override=None, device="cpu")
    kw.update(over)
    return Ctx(**kw)


def engine_ctx(Ctx, **over):
    """The bf16 / 4 layers / 4 heads x 8 channels / 0.1 GB / chunk 256 context of the engine tests."""
    set_rounder(Ctx, 4)
    kw = dict(params_dtype=torch.bfloat16, num_layers=4, kv_channels=8, num_attention_heads=4,
              max_sequence_length=20, num_cuda_graphs=None, buffer_size_gb=0.1,
              buffer_guaranteed_fraction=0.01, chunk_size_tokens=256, tensor_model_parallel_size=1, device="cpu")
    kw.update(over)
    return Ctx(**kw)


# --------------------------------------------------------------------------- sizing constants
def test_sizing_constants_of_the_reference_tests(Ctx):
    c = small_ctx(Ctx)
    want = GOLD["sizing_small_context"]["expected"]
    assert c.gtd_chunk_count == want["gtd_chunk_count"] == 48
    assert c.gtd_request_count == want["gtd_request_count"] == 12
    assert c.chunk_allocator.chunk_count_total == want["chunk_count_total"] == 491
    assert c.max_requests == want["max_requests"] == 128
    assert c.max_tokens == want["max_tokens"] == 62848
    assert torch.all(c.request_ids == -1)
    assert c.memory_buffer.shape == (2, 4, 491, 128, 2, 8) and (c.memory_buffer == -1).all()
    assert c.request_to_kv_chunk_ids.shape == (128, 4) and c.request_to_kv_chunk_ids.dtype == torch.int32
    assert c.token_to_chunk_idx.dtype == torch.int64 and c.request_kv_length_offsets.dtype == torch.int32
    ref = oc.sizing(itemsize=4, num_layers=4, kv_channels=8, num_heads=2, max_sequence_length=512,
                    buffer_size_gb=0.03, buffer_guaranteed_fraction=0.1, chunk_size_tokens=128,
                    token_rounder=64, request_rounder=64)
    assert {k: ref[k] for k in want} == want


def test_engine_sizing_constants(Ctx):
    gold = GOLD["sizing_engine_context"]
    c = engine_ctx(Ctx, max_requests_override=32, max_tokens_override=8 * 20)
    assert [c.max_requests, c.max_tokens] == gold["overrides"]["expected"]
    c = engine_ctx(Ctx, buffer_overflow_factor=0.1)
    assert [c.max_requests, c.max_tokens] == gold["overflow_factor"]["expected"]
    ref = oc.sizing(itemsize=2, num_layers=4, kv_channels=8, num_heads=4, max_sequence_length=20,
                    buffer_size_gb=0.1, buffer_guaranteed_fraction=0.01, chunk_size_tokens=256,
                    buffer_overflow_factor=0.1, token_rounder=4, request_rounder=4)
    assert [ref["max_requests"], ref["max_tokens"]] == gold["overflow_factor"]["expected"]
    assert (ref["chunk_size_bytes"], ref["chunk_count_total"]) == (131072, 819)


def test_tensor_parallel_divides_heads_and_rounders(Ctx):
    set_rounder(Ctx, 64)
    assert Ctx.round_up_tokens(65, tp_size=1) == 128
    assert Ctx.round_up_tokens(65, tp_size=3) == 66  # rounder 64 -> 66 (multiple of 3)
    assert Ctx.round_up_requests(1, tp_size=8) == 64
    set_rounder(Ctx, 4)
    assert Ctx.round_up_requests(5) == 8 and Ctx.round_up_requests(5, tp_size=8) == 8
    c = Ctx(params_dtype=torch.bfloat16, num_layers=1, kv_channels=16, num_attention_heads=8,
            max_sequence_length=64, buffer_size_gb=0.001, buffer_guaranteed_fraction=0.1, chunk_size_tokens=16,
            tensor_model_parallel_size=4, device="cpu")
    assert c.memory_buffer.shape[4] == 2
    assert c.chunk_size_bytes == 2 * 2 * 1 * 16 * 2 * 16


@pytest.mark.parametrize("num_cuda_graphs,expected", [tuple(row) for row in GOLD["cuda_graph_token_counts"]["table"]])
def test_cuda_graph_token_counts(Ctx, num_cuda_graphs, expected):
    c = engine_ctx(Ctx, max_requests_override=64, max_tokens_override=64 * 20, num_cuda_graphs=num_cuda_graphs)
    assert c.cuda_graph_token_counts == expected
    assert c.cuda_graph_request_counts == expected
    assert oc.cuda_graph_token_counts(64, num_cuda_graphs) == expected


@pytest.mark.parametrize("mode", ["DECODE", "NON_DECODE"])
@pytest.mark.parametrize("warm,expected", [tuple(row) for row in GOLD["cuda_graph_warmup_padding"]["table"]])
def test_cuda_graph_warmup_padding(mi, Ctx, mode, warm, expected):
    if warm == 1 and mode == "NON_DECODE":
        pytest.skip("not supported by the reference either")
    c = engine_ctx(Ctx, max_sequence_length=17, max_requests_override=32, max_tokens_override=32 * 17,
                   num_cuda_graphs=8)
    assert c.is_decode_only() and c.cuda_graph_token_counts == GOLD["cuda_graph_warmup_padding"]["token_counts"]
    c.initialize_attention_state(num_warmup_tokens=warm, warmup_engine_mode=getattr(mi.WarmupEngineMode, mode))
    assert expected == c.padded_active_request_count == c.padded_active_token_count
    ids, pos = c.current_input_and_position_ids()
    assert ids.shape[1] == pos.shape[1] == expected
    assert c.using_cuda_graph_this_step()
    c.reset()
    for too_many in (64, 128, 1024):
        with pytest.raises(mi.ActiveRequestCountOverflowError):
            c.initialize_attention_state(num_warmup_tokens=too_many,
                                         warmup_engine_mode=getattr(mi.WarmupEngineMode, mode))
    c.reset()
    # more active tokens than max_requests: a non-decode step that cannot use graphs
    for i in range(8):
        c.add_request(i, torch.arange(10), 4)
    c.initialize_attention_state()
    assert not c.is_decode_only() and not c.using_cuda_graph_this_step()


# --------------------------------------------------------------------------- allocator
def test_allocator_vectors(Ctx):
    c = small_ctx(Ctx)
    a = c.chunk_allocator
    gold = GOLD["allocator"]
    assert a.allocate_memory_chunks(4).tolist() == gold["allocate_4"]
    assert a.chunk_count_avail == gold["avail_after_allocate_4"]
    a.release_memory_chunks(torch.tensor(gold["release"], dtype=torch.int32))
    assert a.chunk_count_avail == gold["avail_after_release"]
    assert a.allocate_memory_chunks(1).item() == gold["allocate_1"]
    assert a.chunk_count_avail == gold["avail_after_allocate_1"]
    assert a.allocate_memory_chunks(a.chunk_count_avail + 100) is None
    assert a.dummy_chunk_idx == gold["dummy_chunk_idx"] == c.dummy_chunk_idx
    r = oc.RefContext(max_requests=128, max_tokens=62848, chunk_count_total=491, chunk_size_tokens=128,
                      max_kv_chunk_count=4, gtd_request_count=12, gtd_chunk_count=48, max_sequence_length=512)
    assert r.alloc(4) == gold["allocate_4"] and r.avail == gold["avail_after_allocate_4"]
    r.release(gold["release"])
    assert r.alloc(1) == [gold["allocate_1"]] and r.avail == gold["avail_after_allocate_1"]
    assert r.alloc(r.avail + 100) is None


def test_is_memory_available_truth_table(Ctx):
    c = small_ctx(Ctx)
    a = c.chunk_allocator
    a.chunk_count_avail = 10
    assert a.is_memory_available(10) and not a.is_memory_available(11) and a.is_memory_available(1)
    a.chunk_count_avail = 0
    assert not a.is_memory_available(1)
    a.chunk_count_avail = 10
    a.gtd_chunk_count = 5
    assert a.is_memory_available(6) and not a.is_memory_available(6, safe=True)


# --------------------------------------------------------------------------- overflow errors, reset
def test_overflow_errors(mi, Ctx):
    set_rounder(Ctx, 1)
    c = Ctx(params_dtype=torch.float32, num_layers=2, kv_channels=64, num_attention_heads=8,
            max_sequence_length=128, buffer_size_gb=0.01, buffer_guaranteed_fraction=0.1, chunk_size_tokens=32,
            device="cpu")
    with pytest.raises(mi.RequestOverflowError):
        for i in range(c.max_requests + 1):
            c.add_request(i, torch.zeros(10))
    c = Ctx(params_dtype=torch.float32, num_layers=2, kv_channels=64, num_attention_heads=8,
            max_sequence_length=512, buffer_size_gb=0.1, buffer_guaranteed_fraction=0.1, chunk_size_tokens=128,
            buffer_overflow_factor=1.0, max_requests_override=2, max_tokens_override=20, device="cpu")
    with pytest.raises(mi.TokenOverflowError) as e:
        c.add_request(1, torch.arange(0, 25))
    assert e.value.is_transient and "request 1" in str(e.value)
    with pytest.raises(mi.MaxSequenceLengthOverflowError) as e:
        c.add_request(2, torch.arange(0, 10), num_tokens_to_generate=600)
    assert not e.value.is_transient
    # chunk overflow: ask for more chunks than the non-reserved pool holds
    set_rounder(Ctx, 64)
    c = small_ctx(Ctx)
    c.chunk_allocator.chunk_count_avail = c.gtd_chunk_count + 1
    with pytest.raises(mi.ChunkOverflowError):
        c.add_request(3, torch.arange(0, 300))
    assert issubclass(mi.ChunkOverflowError, mi.ContextOverflowError)


def test_reset_restores_every_row(Ctx):
    c = small_ctx(Ctx, max_sequence_length=128)
    c.total_request_count = 10
    c.active_token_count = 10
    c.paused_request_count = 5
    c.padded_active_token_count = 10
    c.padded_active_request_count = 5
    c.paused_tokens = torch.tensor([1, 2, 3])
    for name in ("request_ids", "request_query_lengths", "request_output_lengths", "request_kv_length_offsets",
                 "request_kv_chunk_counts", "request_last_kv_chunk_id", "request_last_kv_chunk_offset",
                 "token_to_input_ids", "token_to_pos_ids", "token_to_request_idx", "token_to_position_in_request",
                 "token_to_chunk_idx", "token_to_local_position_within_kv_chunk", "request_to_kv_chunk_ids"):
        getattr(c, name).fill_(1)
    c.chunk_allocator.chunk_count_avail = 5
    c.reset()
    assert (c.total_request_count, c.active_token_count, c.paused_request_count) == (0, 0, 0)
    assert (c.padded_active_token_count, c.padded_active_request_count, c.paused_tokens) == (0, 0, None)
    for name, val in (("request_ids", -1), ("request_query_lengths", 0), ("request_kv_length_offsets", 0),
                      ("request_kv_chunk_counts", 0), ("request_last_kv_chunk_id", -1),
                      ("request_last_kv_chunk_offset", 0), ("token_to_input_ids", 0), ("token_to_pos_ids", 0),
                      ("token_to_request_idx", -1), ("token_to_position_in_request", 0), ("token_to_chunk_idx", -1),
                      ("token_to_local_position_within_kv_chunk", 0), ("request_to_kv_chunk_ids", -1)):
        assert torch.all(getattr(c, name) == val), name
    assert c.chunk_allocator.chunk_count_avail == c.chunk_allocator.chunk_count_total - 1


# --------------------------------------------------------------------------- add_request vector
def test_add_request_vector(Ctx):
    c = small_ctx(Ctx)
    gold = GOLD["add_request"]
    n = gold["prompt_length"]
    c.add_request(request_id=0, tokens=torch.arange(0, n, dtype=torch.long))
    assert c.total_request_count == 1 and c.active_token_count == n
    assert c.request_ids[0] == 0 and torch.all(c.request_ids[1:] == -1)
    assert c.request_query_lengths[0] == n and c.request_kv_length_offsets[0] == 0
    assert c.request_to_kv_chunk_ids[0].tolist() == gold["block_row"]
    assert c.request_kv_chunk_counts[0] == gold["chunk_count"] and c.request_last_kv_chunk_id[0] == gold["last_chunk_id"]
    assert c.request_last_kv_chunk_offset[0].item() == gold["last_chunk_offset"]
    ar = torch.arange(0, n)
    assert torch.equal(c.token_to_pos_ids[:n], ar) and torch.equal(c.token_to_input_ids[:n], ar)
    assert torch.equal(c.token_to_position_in_request[:n], ar)
    assert torch.all(c.token_to_chunk_idx[:128] == 488) and torch.all(c.token_to_chunk_idx[128:n] == 489)
    assert torch.equal(c.token_to_local_position_within_kv_chunk[:n], ar % 128)
    assert c.request_output_lengths[0] == 512  # default budget: up to max_sequence_length


# --------------------------------------------------------------------------- update_requests vectors
def _setup_big_scenario(c):
    c.paused_request_count = 2
    c.paused_tokens = torch.tensor([0, 1], dtype=torch.int32)
    c.chunk_allocator.chunk_count_avail -= 11
    avail = c.chunk_allocator.chunk_count_avail
    c.total_request_count = 10
    c.request_to_kv_chunk_ids[0:10, 0] = torch.arange(avail, avail + 10)
    c.request_to_kv_chunk_ids[3][1] = avail
    c.request_kv_length_offsets[0:10] = 10
    c.request_kv_length_offsets[0:2] = c.chunk_size_tokens - 1
    c.request_kv_length_offsets[5:7] = c.chunk_size_tokens - 1
    c.request_kv_length_offsets[3] = c.chunk_size_bytes + 10
    c.request_query_lengths[0:10] = 1
    c.request_ids[0:10] = torch.arange(0, 10)
    c.request_kv_chunk_counts[0:10] = 1
    c.request_kv_chunk_counts[3] = 2
    c.request_last_kv_chunk_id[0:10] = torch.arange(0, 10)
    c.request_last_kv_chunk_id[3] = 11
    c.request_last_kv_chunk_offset[0:10] = 10
    c.request_last_kv_chunk_offset[0:2] = c.chunk_size_tokens - 1
    c.request_last_kv_chunk_offset[5:7] = c.chunk_size_tokens - 1


def test_update_requests_all_finished_resets(Ctx):
    c = small_ctx(Ctx)
    c.paused_request_count = 0
    c.total_request_count = 3
    c.request_kv_chunk_counts[0:3] = 1
    ids = c.chunk_allocator.allocate_memory_chunks(3, safe=True)
    c.request_to_kv_chunk_ids[0:3, 0] = ids
    before = c.chunk_allocator.chunk_count_avail
    c.update_requests(active_requests_mask=torch.Tensor([0, 0, 0]), new_tokens=torch.tensor([0, 1, 2]))
    assert c.total_request_count == 0 and c.chunk_allocator.chunk_count_avail == before + 3
    assert torch.all(c.request_to_kv_chunk_ids == -1)


def test_update_requests_pause_finish_resume_scenario(Ctx):
    """The reference's full scenario: 2 paused, 3 finished, 2 newly paused, 4 resumed (LIFO)."""
    c = small_ctx(Ctx)
    gold = GOLD["update_requests_scenario"]
    mask = torch.tensor(gold["active_requests_mask"], dtype=torch.int32)
    new = torch.tensor(gold["new_tokens"], dtype=torch.int32)
    c.paused_request_count = 2
    c.paused_tokens = torch.tensor([0, 1], dtype=torch.int32)
    c.total_request_count = 5
    with pytest.raises(AssertionError):
        c.update_requests(active_requests_mask=mask, new_tokens=new)

    c = small_ctx(Ctx)
    _setup_big_scenario(c)
    newly = c.update_requests(active_requests_mask=mask, new_tokens=new)
    assert c.request_ids[0:7].tolist() == gold["request_ids"]
    assert (c.paused_request_count, c.total_request_count, c.active_token_count) == (
        gold["paused_request_count"], gold["total_request_count"], gold["active_token_count"])
    assert c.request_last_kv_chunk_offset[0:10].tolist() == gold["request_last_kv_chunk_offset"]
    assert c.token_to_input_ids[:7].tolist() == gold["token_to_input_ids"]
    assert c.token_to_pos_ids[:7].tolist() == gold["token_to_pos_ids"]
    assert c.request_to_kv_chunk_ids[0:10].tolist() == gold["request_to_kv_chunk_ids"]
    assert c.chunk_allocator.chunk_count_avail == gold["chunk_count_avail"]
    # (the scenario stores synthetic last-chunk ids 0..9 for the rows that were not resumed)
    assert c.token_to_chunk_idx[:7].tolist() == [482, 479, 486, 487, 4, 2, 9]
    assert c.token_to_local_position_within_kv_chunk[:7].tolist() == [0, 0, 0, 0, 11, 11, 11]
    assert c.token_to_request_idx[:7].tolist() == list(range(7))
    assert newly is not None and newly.numel() == 0  # both newly paused requests were resumed at once

    # the scalar-loop restatement reaches the same state
    r = oc.RefContext(max_requests=128, max_tokens=62848, chunk_count_total=491, chunk_size_tokens=128,
                      max_kv_chunk_count=4, gtd_request_count=12, gtd_chunk_count=48, max_sequence_length=512)
    r.paused, r.paused_tokens, r.total_requests = 2, [0, 1], 10
    r.avail -= 11
    for i in range(10):
        r.table[i, 0] = r.avail + i
        r.kv_off[i] = r.last_off[i] = 10
        r.q_len[i], r.ids[i], r.n_chunks[i], r.last_chunk[i] = 1, i, 1, i
    r.table[3, 1] = r.avail
    for i in (0, 1, 5, 6):
        r.kv_off[i] = r.last_off[i] = 127
    r.kv_off[3], r.n_chunks[3], r.last_chunk[3] = 16384 + 10, 2, 11
    assert r.update_requests(mask.tolist(), new.tolist()) == []
    assert r.ids[:7].tolist() == gold["request_ids"] and r.avail == gold["chunk_count_avail"]
    assert r.table[:10].tolist() == gold["request_to_kv_chunk_ids"]
    assert r.tok_pos[:7].tolist() == gold["token_to_pos_ids"]


def test_release_chunks_of_finished_requests(Ctx):
    c = small_ctx(Ctx)
    ids = c.chunk_allocator.allocate_memory_chunks(5, safe=True)
    c.total_request_count, c.paused_request_count = 5, 0
    before = c.chunk_allocator.chunk_count_avail
    for i in range(5):
        c.request_to_kv_chunk_ids[i, 0] = ids[i]
        c.request_query_lengths[i] = 1
        c.request_ids[i] = i
    c.update_requests(active_requests_mask=torch.tensor([0, 1, 0, 1, 0]),
                      new_tokens=torch.tensor([10, 11, 12, 13, 14]))
    assert c.total_request_count == 2 and c.active_token_count == 2
    assert c.chunk_allocator.chunk_count_avail == before + 3
    assert c.request_ids[:2].tolist() == [3, 1] and c.token_to_input_ids[:2].tolist() == [13, 11]

    c = small_ctx(Ctx)
    ids = c.chunk_allocator.allocate_memory_chunks(6, safe=True)
    c.total_request_count, c.paused_request_count = 3, 0
    before = c.chunk_allocator.chunk_count_avail
    c.request_to_kv_chunk_ids[0, 0] = ids[0]
    c.request_to_kv_chunk_ids[1, 0:2] = ids[1:3]
    c.request_to_kv_chunk_ids[2, 0:3] = ids[3:6]
    c.request_kv_chunk_counts[0:3] = torch.tensor([1, 2, 3], dtype=torch.int32)
    c.request_query_lengths[0:3] = 1
    c.request_ids[0:3] = torch.arange(3, dtype=torch.int32)
    c.update_requests(active_requests_mask=torch.tensor([0, 0, 0]), new_tokens=torch.tensor([10, 11, 12]))
    assert c.total_request_count == 0 and c.active_token_count == 0
    assert c.chunk_allocator.chunk_count_avail == before + 6


# --------------------------------------------------------------------------- attention-state padding
def test_decode_step_padding_rules(Ctx):
    set_rounder(Ctx, 64)
    c = small_ctx(Ctx)
    for i, n in enumerate((5, 130, 64)):
        c.add_request(i, torch.arange(n))
    c.initialize_attention_state()
    # prefill step: no padded requests, int32 cumulative lengths, exact maxima
    assert not c.is_decode_only()
    assert c.padded_active_token_count == 256 and c.padded_active_request_count == 3
    assert c.cu_query_seq_lengths.tolist() == [0, 5, 135, 199] and c.cu_query_seq_lengths.dtype == torch.int32
    assert c.cu_kv_seq_lengths.tolist() == [0, 5, 135, 199]
    assert (c.max_seqlen_q, c.max_seqlen_k) == (130, 130)
    assert c.kv_seq_lengths.tolist() == [5, 130, 64]
    assert torch.all(c.token_to_chunk_idx[199:256] == c.dummy_chunk_idx)
    assert torch.all(c.token_to_local_position_within_kv_chunk[199:256] == 0)
    assert c.block_table.shape == (3, 4) and c.block_table[1].tolist()[:2] == c.request_to_kv_chunk_ids[1].tolist()[:2]
    logits = torch.arange(256.0).view(1, 256, 1)
    assert c.last_token_logits(logits).flatten().tolist() == [4.0, 134.0, 198.0]
    c.update_requests(torch.tensor([1, 1, 1]), torch.tensor([7, 8, 9]))
    c.initialize_attention_state()
    # decode step: padded to the token rounder (capped by max_requests); padded rows: length 0, table row 0
    assert c.is_decode_only() and c.max_seqlen_q == 1 and c.cu_query_seq_lengths is None
    assert c.padded_active_token_count == c.padded_active_request_count == 64
    assert c.max_seqlen_k == c.max_sequence_length
    assert c.kv_seq_lengths.tolist() == [6, 131, 65] + [0] * 61
    assert torch.all(c.block_table[3:] == 0) and c.block_table.shape == (64, 4)
    assert c.block_table.data_ptr() == c.request_to_kv_chunk_ids_cudagraph_only.data_ptr()
    assert c.token_to_pos_ids[:3].tolist() == [5, 130, 64]
    assert c.token_to_local_position_within_kv_chunk[:3].tolist() == [5, 2, 64]
    assert torch.all(c.token_to_chunk_idx[3:64] == c.dummy_chunk_idx)
    ids, pos = c.current_input_and_position_ids()
    assert ids.shape == (1, 64) and ids[0, :3].tolist() == [7, 8, 9]


def test_calculate_log_probs_mixed_and_decode(Ctx):
    set_rounder(Ctx, 4)
    c = small_ctx(Ctx)
    set_rounder(Ctx, 4)
    c.add_request(0, torch.tensor([3, 1, 2]))
    c.add_request(1, torch.tensor([4, 0]))
    c.initialize_attention_state()
    V = 6
    torch.manual_seed(0)
    logits = torch.randn(1, c.padded_active_token_count, V)
    new = torch.tensor([5, 2])
    got = c.calculate_log_probs(logits[:, :5], new)
    lp = torch.log_softmax(logits[0].float(), -1)
    exp = [[lp[0, 1].item(), lp[1, 2].item(), lp[2, 5].item()], [lp[3, 0].item(), lp[4, 2].item()]]
    assert np.allclose(got[0], exp[0]) and np.allclose(got[1], exp[1])
    got = c.calculate_log_probs(logits[:, :2], new, only_last_token_logits=True)
    assert np.allclose([g[0] for g in got], [lp[0, 5].item(), lp[1, 2].item()])


# --------------------------------------------------------------------------- random streams vs restatement
def _snapshot_product(c):
    n = c.total_request_count
    return dict(
        ids=c.request_ids[:n].tolist(), q=c.request_query_lengths[:n].tolist(),
        off=c.request_kv_length_offsets[:n].tolist(), out=c.request_output_lengths[:n].tolist(),
        nch=c.request_kv_chunk_counts[:n].tolist(), lastc=c.request_last_kv_chunk_id[:n].tolist(),
        lasto=c.request_last_kv_chunk_offset[:n].tolist(), table=c.request_to_kv_chunk_ids.tolist(),
        avail=c.chunk_allocator.chunk_count_avail, bag=c.chunk_allocator.chunk_bag[:c.chunk_allocator.chunk_count_avail].tolist(),
        paused=c.paused_request_count, total=n, act=c.active_token_count,
        tin=c.token_to_input_ids[:c.active_token_count].tolist(), tpos=c.token_to_pos_ids[:c.active_token_count].tolist(),
        treq=c.token_to_request_idx[:c.active_token_count].tolist(), tchunk=c.token_to_chunk_idx[:c.active_token_count].tolist(),
        tloc=c.token_to_local_position_within_kv_chunk[:c.active_token_count].tolist(),
        tinreq=c.token_to_position_in_request[:c.active_token_count].tolist())


def _snapshot_ref(r):
    n = r.total_requests
    a = r.active_tokens
    return dict(
        ids=r.ids[:n].tolist(), q=r.q_len[:n].tolist(), off=r.kv_off[:n].tolist(), out=r.out_len[:n].tolist(),
        nch=r.n_chunks[:n].tolist(), lastc=r.last_chunk[:n].tolist(), lasto=r.last_off[:n].tolist(),
        table=r.table.tolist(), avail=r.avail, bag=r.bag[:r.avail].tolist(), paused=r.paused, total=n, act=a,
        tin=r.tok_input[:a].tolist(), tpos=r.tok_pos[:a].tolist(), treq=r.tok_req[:a].tolist(),
        tchunk=r.tok_chunk[:a].tolist(), tloc=r.tok_local[:a].tolist(), tinreq=r.tok_in_req[:a].tolist())


@pytest.mark.parametrize("seed", [0, 1, 2, 3])
def test_random_request_streams_match_restatement(mi, Ctx, seed):
    """Admit, decode, finish, pause and resume at random with a tiny pool so that every branch runs."""
    rng = random.Random(seed)
    set_rounder(Ctx, 4)
    C, max_seq = 8, 40
    c = Ctx(params_dtype=torch.float32, num_layers=1, kv_channels=4, num_attention_heads=1, max_sequence_length=max_seq,
            buffer_size_gb=30 * (4 * 2 * 1 * C * 1 * 4) / 1024**3, buffer_guaranteed_fraction=0.2,
            chunk_size_tokens=C, max_requests_override=12, max_tokens_override=200, device="cpu")
    s = oc.sizing(itemsize=4, num_layers=1, kv_channels=4, num_heads=1, max_sequence_length=max_seq,
                  buffer_size_gb=30 * (4 * 2 * 1 * C * 1 * 4) / 1024**3, buffer_guaranteed_fraction=0.2,
                  chunk_size_tokens=C, max_requests_override=12, max_tokens_override=200, token_rounder=4,
                  request_rounder=4)
    assert (s["max_requests"], s["max_tokens"], s["chunk_count_total"]) == (
        c.max_requests, c.max_tokens, c.chunk_allocator.chunk_count_total)
    r = oc.RefContext(max_requests=s["max_requests"], max_tokens=s["max_tokens"],
                      chunk_count_total=s["chunk_count_total"], chunk_size_tokens=C,
                      max_kv_chunk_count=s["max_kv_chunk_count"], gtd_request_count=s["gtd_request_count"],
                      gtd_chunk_count=s["gtd_chunk_count"], max_sequence_length=max_seq, token_rounder=4)
    next_id = 0
    events = set()
    for step in range(120):
        # admit a few requests (only between steps, when every active request is in decode phase or new)
        for _ in range(rng.randint(0, 2)):
            n = rng.randint(1, 20)
            toks = [rng.randint(0, 99) for _ in range(n)]
            gen = rng.choice([None, rng.randint(1, max_seq - n + 3)])
            err_ref = r.add_request(next_id, toks, gen)
            try:
                c.add_request(next_id, torch.tensor(toks), gen)
                err = ""
            except mi.ContextOverflowError as e:
                err = type(e).__name__
            assert err == err_ref
            events.add(err or "added")
            if err == "MaxSequenceLengthOverflowError":
                # both implementations have taken chunks they never return (as the reference does)
                pass
            next_id += 1
        assert _snapshot_product(c) == _snapshot_ref(r)
        n_act = c.total_request_count - c.paused_request_count
        if c.total_request_count == 0 or n_act == 0:
            continue
        c.initialize_attention_state()
        if c.is_decode_only():
            padded, lens, table = r.decode_padding()
            assert padded == c.padded_active_token_count
            assert c.kv_seq_lengths.tolist() == lens.tolist() and c.block_table.tolist() == table.tolist()
        # every chunk id is free, owned exactly once, or the dummy
        owned = c.request_to_kv_chunk_ids[c.request_to_kv_chunk_ids >= 0].tolist()
        free = c.chunk_allocator.chunk_bag[: c.chunk_allocator.chunk_count_avail].tolist()
        assert len(set(owned)) == len(owned) and not (set(owned) & set(free))
        assert c.dummy_chunk_idx not in owned and c.dummy_chunk_idx not in free
        # sample: finish by budget or at random
        seq = (c.request_kv_length_offsets + c.request_query_lengths)[c.paused_request_count:c.total_request_count]
        budget = c.request_output_lengths[c.paused_request_count:c.total_request_count]
        mask = [(0 if (int(a) + 1 >= int(b) or rng.random() < 0.08) else 1) for a, b in zip(seq, budget)]
        new = [rng.randint(0, 99) for _ in mask]
        p_before = c.paused_request_count
        got = c.update_requests(torch.tensor(mask, dtype=torch.int32), torch.tensor(new))
        ref = r.update_requests(mask, new)
        assert (None if got is None else got.tolist()) == ref
        if c.paused_request_count > 0:
            events.add("paused")
            assert c.paused_tokens.tolist() == r.paused_tokens
        if c.paused_request_count < p_before:
            events.add("resumed")
        if 0 in mask:
            events.add("finished")
        assert _snapshot_product(c) == _snapshot_ref(r)
    assert {"added", "finished"} <= events
    if seed == 0:
        assert "paused" in events and "resumed" in events


def test_fp8_cache_sizing_counts_bytes_and_scales(mi):
    """An fp8 KV cache (an addition to the reference's constructor) sizes its pool from one byte per
    element plus one fp32 scale per (key|value, layer, chunk, head): 512 KiB + 64 B for the
    Mixtral-shape single-layer chunk of 256 tokens x 8 heads x 128."""
    Ctx = mi.DynamicInferenceContext
    c = Ctx(params_dtype=torch.bfloat16, num_layers=1, kv_channels=128, num_attention_heads=8,
            max_sequence_length=1024, buffer_size_gb=8 * (512 * 1024 + 64) / 1024**3, buffer_guaranteed_fraction=0.1,
            chunk_size_tokens=256, kv_cache_dtype="fp8_e4m3", device="cpu")
    assert c.chunk_size_bytes == 512 * 1024 + 64
    assert c.chunk_allocator.chunk_count_total == 8
    assert c.memory_buffer.dtype == torch.uint8 and c.memory_buffer.numel() == 8 * 512 * 1024
    assert c.kv_scales.shape == (2, 1, 8, 8)
    assert c.key_value_scales(1)[0].shape == (8, 8)
    b = Ctx(params_dtype=torch.bfloat16, num_layers=1, kv_channels=128, num_attention_heads=8,
            max_sequence_length=1024, buffer_size_gb=8 * 1024 * 1024 / 1024**3, buffer_guaranteed_fraction=0.1,
            chunk_size_tokens=256, device="cpu")
    assert b.chunk_size_bytes == 1024 * 1024 and b.kv_scales is None and b.key_value_scales(1) == (None, None)
    with pytest.raises(ValueError, match="kv_cache_dtype"):
        Ctx(params_dtype=torch.bfloat16, num_layers=1, kv_channels=128, num_attention_heads=8,
            max_sequence_length=1024, buffer_size_gb=0.01, buffer_guaranteed_fraction=0.1, kv_cache_dtype="int4",
            device="cpu")


def test_mla_latent_cache_sizing_and_views(mi):
    """cache_mla_latent=True (dynamic_context.py:180-203,288-294,547-557): one row of
    kv_lora_rank + qk_pos_emb_head_dim values per token and layer, no value cache, chunk size 64."""
    Ctx = mi.DynamicInferenceContext
    chunk_bytes = 2 * 3 * 64 * (512 + 64)  # bf16 x layers x tokens x (rank + rope) = 221 184
    c = Ctx(params_dtype=torch.bfloat16, num_layers=3, kv_channels=128, num_attention_heads=16,
            max_sequence_length=256, buffer_size_gb=10 * chunk_bytes / 1024**3, buffer_guaranteed_fraction=0.1,
            chunk_size_tokens=64, cache_mla_latent=True, kv_lora_rank=512, qk_pos_emb_head_dim=64, device="cpu")
    assert c.cache_mla_latent and c.kv_reduced_dim == 576
    assert c.chunk_size_bytes == chunk_bytes == 221184
    assert c.chunk_allocator.chunk_count_total == 10
    assert c.memory_buffer.shape == (3, 10, 64, 576) and bool((c.memory_buffer == -1).all())
    k, v, bt = c.key_value_cache(2)
    assert v is None and k.shape == (10, 64, 576) and k.data_ptr() == c.memory_buffer[1].data_ptr()
    assert c.key_value_scales(1) == (None, None)
    with pytest.raises(AssertionError, match="block size of 64"):
        Ctx(params_dtype=torch.bfloat16, num_layers=1, kv_channels=128, num_attention_heads=16,
            max_sequence_length=256, buffer_size_gb=0.001, buffer_guaranteed_fraction=0.1, chunk_size_tokens=128,
            cache_mla_latent=True, kv_lora_rank=512, qk_pos_emb_head_dim=64, device="cpu")
    with pytest.raises(ValueError, match="kv_lora_rank"):
        Ctx(params_dtype=torch.bfloat16, num_layers=1, kv_channels=128, num_attention_heads=16,
            max_sequence_length=256, buffer_size_gb=0.001, buffer_guaranteed_fraction=0.1, chunk_size_tokens=64,
            cache_mla_latent=True, device="cpu")


def test_synthetic_input_helpers_agree_with_the_checker(mi):
    """The benchmark builds its rotary table and counts its algorithmic bytes with helpers of the package
    (so that its measured leg touches nothing of the checker); both must say what the checker says."""
    from oracle import paged_attention as oa
    from oracle import rope_norm as orn

    for dim, base in ((128, 500000.0), (64, 10000.0)):
        assert torch.equal(mi.synthetic.rotary_angle_table(300, dim, base), orn.rotary_table(300, dim, base=base))
    lens = [5, 700, 0, 256, 257, 8192]
    for kvb, sc in ((2, False), (1, True)):
        assert mi.synthetic.decode_attention_bytes(lens, 32, 8, 128, 256, kv_bytes=kvb, fp8_scales=sc) == \
            oa.decode_attention_bytes(lens, 32, 8, 128, 256, kv_bytes=kvb, fp8_scales=sc)
    # by hand: one request of 3 tokens, 2/1 heads of 8 values, chunk 2 -> 2 chunks
    assert mi.synthetic.decode_attention_bytes([3], 2, 1, 8, 2) == 3 * 1 * 8 * 2 * 2 + 2 * 8 * 4 + 2 * 4 + 4
