"""GPU: update_requests / decode attention state as single kernels (through the C ABI).

The kernels must leave every state tensor exactly as the scalar-loop restatement in
oracle/context.py (and the torch op sequence of the host class) leaves it: integer work, so the
bar is equality.  Cases: the reference's own pause/finish/resume scenario and its constants
(tests/unit_tests/inference/contexts/test_dynamic_context.py in the reference tree), the
all-finished reset, the count-mismatch assertion, and random request streams with a pool small
enough that every branch (finish, pause, LIFO resume, overflow errors) runs.
"""
import random

import pytest
import torch

from oracle import context as oc
from test_context_host import GOLD, _setup_big_scenario, _snapshot_product, _snapshot_ref, set_rounder

pytestmark = pytest.mark.gpu


@pytest.fixture()
def Ctx(mi):
    cls = mi.DynamicInferenceContext
    saved = (cls.TOKEN_ROUNDER, cls.REQUEST_ROUNDER)
    yield cls
    cls.TOKEN_ROUNDER, cls.REQUEST_ROUNDER = saved


def small_ctx(Ctx, dev, **over):
    set_rounder(Ctx, 64)
    kw = dict(params_dtype=torch.float32, num_layers=4, kv_channels=8, num_attention_heads=2,
              max_sequence_length=512, num_cuda_graphs=None, buffer_size_gb=0.03,
              buffer_guaranteed_fraction=0.1, chunk_size_tokens=128, device=dev)
    kw.update(over)
    return Ctx(**kw)


def test_fused_bookkeeping_is_the_default_on_a_gpu(Ctx, dev):
    assert small_ctx(Ctx, dev).fused_bookkeeping is True
    assert small_ctx(Ctx, dev, fused_bookkeeping=False).fused_bookkeeping is False


def test_all_finished_resets(Ctx, dev):
    c = small_ctx(Ctx, dev)
    c.total_request_count = 3
    c.request_kv_chunk_counts[0:3] = 1
    ids = c.chunk_allocator.allocate_memory_chunks(3, safe=True)
    c.request_to_kv_chunk_ids[0:3, 0] = ids
    before = c.chunk_allocator.chunk_count_avail
    bag_before = c.chunk_allocator.chunk_bag.clone()
    c.update_requests(active_requests_mask=torch.Tensor([0, 0, 0]), new_tokens=torch.tensor([0, 1, 2]))
    assert c.total_request_count == 0 and c.active_token_count == 0
    assert c.chunk_allocator.chunk_count_avail == before + 3
    assert torch.all(c.request_to_kv_chunk_ids == -1)
    assert torch.equal(c.chunk_allocator.chunk_bag[: before + 3].cpu()[-3:], ids.cpu().to(torch.int32))
    assert torch.equal(c.chunk_allocator.chunk_bag[:before], bag_before[:before])


def test_count_mismatch_raises_and_changes_nothing(Ctx, dev):
    c = small_ctx(Ctx, dev)
    mask = torch.tensor([1, 0, 1, 1, 1, 0, 0, 1], dtype=torch.int32)
    c.paused_request_count = 2
    c.paused_tokens = torch.tensor([0, 1], dtype=torch.int32, device=dev)
    c.total_request_count = 5
    with pytest.raises(AssertionError):
        c.update_requests(active_requests_mask=mask, new_tokens=torch.arange(2, 10))
    # a mask with a value outside {0, 1} has the right length but the wrong counts
    c = small_ctx(Ctx, dev)
    _setup_big_scenario(c)
    before = _snapshot_product(c)
    bad = mask.clone()
    bad[2] = 2
    with pytest.raises(AssertionError):
        c.update_requests(active_requests_mask=bad, new_tokens=torch.arange(2, 10))
    assert _snapshot_product(c) == before


@pytest.mark.parametrize("fused", [True, False])
def test_pause_finish_resume_scenario(Ctx, dev, fused):
    """2 paused, 3 finished, 2 newly paused, 4 resumed (LIFO): the constants of the reference's test."""
    c = small_ctx(Ctx, dev, fused_bookkeeping=fused)
    gold = GOLD["update_requests_scenario"]          # tests/golden/reference_vectors.json
    mask = torch.tensor(gold["active_requests_mask"], dtype=torch.int32)
    new = torch.tensor(gold["new_tokens"], dtype=torch.int32)
    _setup_big_scenario(c)
    c.paused_tokens = c.paused_tokens.to(dev)
    newly = c.update_requests(active_requests_mask=mask.to(dev), new_tokens=new.to(dev))
    assert c.request_ids[0:7].tolist() == gold["request_ids"]
    assert (c.paused_request_count, c.total_request_count, c.active_token_count) == (
        gold["paused_request_count"], gold["total_request_count"], gold["active_token_count"])
    assert c.request_last_kv_chunk_offset[0:10].tolist() == gold["request_last_kv_chunk_offset"]
    assert c.token_to_input_ids[:7].tolist() == gold["token_to_input_ids"]
    assert c.token_to_pos_ids[:7].tolist() == gold["token_to_pos_ids"]
    assert c.request_to_kv_chunk_ids[0:10].tolist() == gold["request_to_kv_chunk_ids"]
    assert c.chunk_allocator.chunk_count_avail == gold["chunk_count_avail"]
    assert c.token_to_chunk_idx[:7].tolist() == [482, 479, 486, 487, 4, 2, 9]
    assert c.token_to_local_position_within_kv_chunk[:7].tolist() == [0, 0, 0, 0, 11, 11, 11]
    assert c.token_to_request_idx[:7].tolist() == list(range(7))
    assert newly is not None and newly.numel() == 0


def _stream_contexts(Ctx, dev, fused, C=8, max_seq=40):
    set_rounder(Ctx, 4)
    gb = 30 * (4 * 2 * 1 * C * 1 * 4) / 1024**3
    kw = dict(params_dtype=torch.float32, num_layers=1, kv_channels=4, num_attention_heads=1,
              max_sequence_length=max_seq, buffer_size_gb=gb, buffer_guaranteed_fraction=0.2, chunk_size_tokens=C,
              max_requests_override=12, max_tokens_override=200)
    c = Ctx(device=dev, fused_bookkeeping=fused, **kw)
    s = oc.sizing(itemsize=4, num_layers=1, kv_channels=4, num_heads=1, max_sequence_length=max_seq,
                  buffer_size_gb=gb, buffer_guaranteed_fraction=0.2, chunk_size_tokens=C, max_requests_override=12,
                  max_tokens_override=200, token_rounder=4, request_rounder=4)
    r = oc.RefContext(max_requests=s["max_requests"], max_tokens=s["max_tokens"],
                      chunk_count_total=s["chunk_count_total"], chunk_size_tokens=C,
                      max_kv_chunk_count=s["max_kv_chunk_count"], gtd_request_count=s["gtd_request_count"],
                      gtd_chunk_count=s["gtd_chunk_count"], max_sequence_length=max_seq, token_rounder=4)
    return c, r


@pytest.mark.parametrize("seed", [0, 1, 2, 3, 4, 5])
def test_random_request_streams_match_restatement(mi, Ctx, dev, seed):
    rng = random.Random(seed)
    max_seq = 40
    c, r = _stream_contexts(Ctx, dev, True, max_seq=max_seq)
    next_id = 0
    events = set()
    for step in range(120):
        for _ in range(rng.randint(0, 2)):
            n = rng.randint(1, 20)
            toks = [rng.randint(0, 99) for _ in range(n)]
            gen = rng.choice([None, rng.randint(1, max_seq - n + 3)])
            err_ref = r.add_request(next_id, toks, gen)
            try:
                c.add_request(next_id, torch.tensor(toks, device=dev), gen)
                err = ""
            except mi.ContextOverflowError as e:
                err = type(e).__name__
            assert err == err_ref
            events.add(err or "added")
            next_id += 1
        assert _snapshot_product(c) == _snapshot_ref(r), f"seed {seed} step {step} after admission"
        n_act = c.total_request_count - c.paused_request_count
        if c.total_request_count == 0 or n_act == 0:
            continue
        c.initialize_attention_state()
        if c.is_decode_only():
            padded, lens, table = r.decode_padding()
            assert padded == c.padded_active_token_count
            assert c.kv_seq_lengths.tolist() == lens.tolist() and c.block_table.tolist() == table.tolist()
            assert c.query_seq_lengths_cudagraph_only[:padded].tolist() == [1] * n_act + [0] * (padded - n_act)
            pad = slice(c.active_token_count, padded)
            assert c.token_to_chunk_idx[pad].tolist() == [c.dummy_chunk_idx] * (padded - n_act)
            assert not c.token_to_local_position_within_kv_chunk[pad].any()
            assert not c.token_to_position_in_request[pad].any()
            events.add("decode_only")
        seq = (c.request_kv_length_offsets + c.request_query_lengths)[c.paused_request_count:c.total_request_count]
        budget = c.request_output_lengths[c.paused_request_count:c.total_request_count]
        mask = [(0 if (a + 1 >= b or rng.random() < 0.08) else 1) for a, b in zip(seq.tolist(), budget.tolist())]
        new = [rng.randint(0, 99) for _ in mask]
        p_before = c.paused_request_count
        got = c.update_requests(torch.tensor(mask, dtype=torch.int32, device=dev), torch.tensor(new, device=dev))
        ref = r.update_requests(mask, new)
        assert (None if got is None else got.tolist()) == ref, f"seed {seed} step {step}"
        if c.paused_request_count > 0:
            events.add("paused")
            assert c.paused_tokens.tolist() == r.paused_tokens
        if c.paused_request_count < p_before:
            events.add("resumed")
        if 0 in mask:
            events.add("finished")
        assert _snapshot_product(c) == _snapshot_ref(r), f"seed {seed} step {step} after update"
    assert {"added", "finished", "decode_only"} <= events
    if seed == 0:
        assert "paused" in events and "resumed" in events


def test_add_request_kernel_equals_the_indexed_writes(mi, Ctx, dev):
    """Prompts of one token, around the chunk size and over several launch blocks: the one-launch admission leaves
    every state tensor as the reference's sequence of indexed writes does (dynamic_context.py:976-1015)."""
    a = small_ctx(Ctx, dev, fused_bookkeeping=True)
    b = small_ctx(Ctx, dev, fused_bookkeeping=False)
    gen = torch.Generator().manual_seed(4)
    for rid, n in enumerate([1, 127, 128, 129, 300, 512, 5]):
        toks = torch.randint(0, 50000, (n,), generator=gen)
        budget = None if rid % 2 else 3
        for c in (a, b):
            try:
                c.add_request(100 + rid, toks.to(dev), budget)
                err = ""
            except mi.ContextOverflowError as e:
                err = type(e).__name__
            c._last_err = err
        assert a._last_err == b._last_err
        assert _snapshot_product(a) == _snapshot_product(b), f"after request {rid} ({n} tokens)"
    assert a.total_request_count >= 5
    untouched = a.request_to_kv_chunk_ids[a.total_request_count:]
    assert (untouched == -1).all()


def test_kernel_and_torch_op_sequence_agree_on_a_wide_batch(mi, Ctx, dev):
    """More rows than one pass of the workgroup (max_requests > 256): both GPU paths, step by step."""
    set_rounder(Ctx, 4)
    C = 4
    kw = dict(params_dtype=torch.bfloat16, num_layers=1, kv_channels=8, num_attention_heads=1,
              max_sequence_length=24, buffer_size_gb=700 * (2 * 2 * 1 * C * 1 * 8) / 1024**3,
              buffer_guaranteed_fraction=0.05, chunk_size_tokens=C, max_requests_override=600,
              max_tokens_override=4096, device=dev)
    a = Ctx(fused_bookkeeping=True, **kw)
    b = Ctx(fused_bookkeeping=False, **kw)
    rng = random.Random(11)
    next_id = 0
    saw_pause = saw_mixed = saw_finished = False
    widest = 0
    for step in range(40):
        for _ in range(rng.randint(0, 100)):
            toks = torch.tensor([rng.randint(0, 99) for _ in range(rng.randint(1, 6))], device=dev)
            outcome = []
            for c in (a, b):
                try:
                    c.add_request(next_id, toks, 14)
                    outcome.append("")
                except mi.ContextOverflowError as e:
                    outcome.append(type(e).__name__)
            assert outcome[0] == outcome[1]
            next_id += 1
        n_act = a.total_request_count - a.paused_request_count
        if n_act == 0:
            continue
        for c in (a, b):
            c.initialize_attention_state()
        if a.is_decode_only():
            assert torch.equal(a.kv_seq_lengths, b.kv_seq_lengths) and torch.equal(a.block_table, b.block_table)
        else:
            # prefill / mixed step: one launch and no wait on the kernel side, the torch ops and two .item()
            # calls on the other; every published value must be the same
            saw_mixed = True
            assert a._max_lengths_pending, "the kernel path must not have waited for the maxima yet"
            q_bound, k_bound = a.attention_length_bounds()
            for name in ("cu_query_seq_lengths", "cu_kv_seq_lengths", "kv_seq_lengths", "block_table"):
                assert torch.equal(getattr(a, name), getattr(b, name)), name
            pad = slice(a.active_token_count, a.padded_active_token_count)
            for name in ("token_to_chunk_idx", "token_to_local_position_within_kv_chunk", "token_to_position_in_request"):
                assert torch.equal(getattr(a, name)[pad], getattr(b, name)[pad]), name
            assert a.cu_query_lengths()[1] == b.max_seqlen_q and a.cu_kv_lengths()[2] == b.max_seqlen_k
            assert not a._max_lengths_pending
            assert q_bound == b.max_seqlen_q, "the host knows the longest query exactly"
            assert b.max_seqlen_k <= k_bound <= a.max_sequence_length
        seq = (a.request_kv_length_offsets + a.request_query_lengths)[a.paused_request_count:a.total_request_count]
        budget = a.request_output_lengths[a.paused_request_count:a.total_request_count]
        mask = torch.tensor([(0 if (x + 1 >= y or rng.random() < 0.05) else 1)
                             for x, y in zip(seq.tolist(), budget.tolist())], dtype=torch.int32, device=dev)
        new = torch.randint(0, 100, (n_act,), device=dev)
        ids_before = a.request_ids[a.paused_request_count:a.total_request_count].clone()
        ga = a.update_requests(mask, new)
        gb = b.update_requests(mask, new)
        # ids of the finished requests, listed by the kernel in row order; the torch path lists nothing
        assert b.last_finished_request_ids is None
        assert a.last_finished_request_ids.dtype == torch.int32
        assert a.last_finished_request_ids.tolist() == ids_before[mask == 0].tolist()
        saw_finished |= bool((mask == 0).any())
        assert (ga is None) == (gb is None)
        if ga is not None:
            assert ga.tolist() == gb.tolist()
        saw_pause |= a.paused_request_count > 0
        widest = max(widest, a.total_request_count)
        assert _snapshot_product(a) == _snapshot_product(b), f"step {step}"
        if a.paused_request_count:
            assert a.paused_tokens.tolist() == b.paused_tokens.tolist()
    assert widest > 256 and saw_pause and saw_mixed and saw_finished


def test_long_requests_release_many_table_columns(mi, Ctx, dev):
    """Requests that own up to ~190 chunks each (a chunk table 200 columns wide): when they finish, their chunks go
    back to the allocator's stack in the reference's order (rows ascending, columns ascending) -- more columns than
    the 64 lanes that walk a row at a time -- and the survivors' table rows move.  Kernel path against the torch op
    sequence, every state tensor and the stack itself compared after every step."""
    set_rounder(Ctx, 4)
    C = 4
    kw = dict(params_dtype=torch.bfloat16, num_layers=1, kv_channels=8, num_attention_heads=1,
              max_sequence_length=200 * C, buffer_size_gb=3000 * (2 * 2 * 1 * C * 1 * 8) / 1024**3,
              buffer_guaranteed_fraction=0.05, chunk_size_tokens=C, max_requests_override=48,
              max_tokens_override=8192, device=dev)
    a = Ctx(fused_bookkeeping=True, **kw)
    b = Ctx(fused_bookkeeping=False, **kw)
    assert a.request_to_kv_chunk_ids.size(1) == 200
    rng = random.Random(23)
    next_id = 0
    finished_long = 0
    for step in range(30):
        for _ in range(rng.randint(0, 6)):
            n = rng.choice([rng.randint(1, 12), rng.randint(250, 760)])
            toks = torch.tensor([rng.randint(0, 99) for _ in range(n)], device=dev)
            outcome = []
            for c in (a, b):
                try:
                    c.add_request(next_id, toks, 30)
                    outcome.append("")
                except mi.ContextOverflowError as e:
                    outcome.append(type(e).__name__)
            assert outcome[0] == outcome[1]
            next_id += 1
        n_act = a.total_request_count - a.paused_request_count
        if n_act == 0:
            continue
        for c in (a, b):
            c.initialize_attention_state()
        act = slice(a.paused_request_count, a.total_request_count)
        seq = (a.request_kv_length_offsets + a.request_query_lengths)[act]
        budget = a.request_output_lengths[act]
        mask = torch.tensor([(0 if (x + 1 >= y or rng.random() < 0.2) else 1) for x, y in zip(seq.tolist(), budget.tolist())],
                            dtype=torch.int32, device=dev)
        finished_long += int(((mask == 0) & (a.request_kv_chunk_counts[act] > 64)).sum())
        new = torch.randint(0, 100, (n_act,), device=dev)
        ga, gb = a.update_requests(mask, new), b.update_requests(mask, new)
        assert (ga is None) == (gb is None) and (ga is None or ga.tolist() == gb.tolist())
        assert _snapshot_product(a) == _snapshot_product(b), f"step {step}"
        avail = a.chunk_allocator.chunk_count_avail
        assert avail == b.chunk_allocator.chunk_count_avail
        assert torch.equal(a.chunk_allocator.chunk_bag[:avail], b.chunk_allocator.chunk_bag[:avail]), f"stack order, step {step}"
    assert finished_long >= 5, "the case this test is for did not occur"
