"""GPU: the decode layer captured as HIP graphs, one per padded batch size.

Mirrors how the reference uses its CUDA graphs (warm-up capture per
``cuda_graph_token_counts`` entry, replay of the size ``initialize_attention_state`` picks;
dynamic_engine.py:143-227, dynamic_context.py:319-382).  Every replay is checked against an
eager twin (same kernels, same inputs: outputs and caches must be identical bit for bit), with
eager work and synchronisations between replays and each graph replayed several times.
"""
import pytest
import torch

from oracle import rope_norm as orn

pytestmark = pytest.mark.gpu

L, HQ, HKV, D, C = 2, 8, 2, 128, 16


def _ctx(mi, dev, graphs):
    return mi.DynamicInferenceContext(
        params_dtype=torch.bfloat16, num_layers=L, kv_channels=D, num_attention_heads=HKV,
        max_sequence_length=96, buffer_size_gb=200 * (2 * 2 * L * C * HKV * D) / 1024**3,
        buffer_guaranteed_fraction=0.1, chunk_size_tokens=C, max_requests_override=16, max_tokens_override=256,
        num_cuda_graphs=4 if graphs else None, device=dev)


def _layers(mi, dev, gen):
    out = []
    for l in range(L):
        core = mi.PagedSelfAttentionCore(l + 1, D, qk_norm="rms", eps=1e-5, fused=True, device=dev)
        core.q_layernorm_weight.data.copy_((1 + 0.02 * torch.randn(D, generator=gen)).bfloat16())
        core.k_layernorm_weight.data.copy_((1 + 0.02 * torch.randn(D, generator=gen)).bfloat16())
        out.append(core)
    return out


def test_graph_replays_match_eager_steps(mi, dev):
    cls = mi.DynamicInferenceContext
    saved = (cls.TOKEN_ROUNDER, cls.REQUEST_ROUNDER)
    cls.TOKEN_ROUNDER = cls.REQUEST_ROUNDER = 4
    try:
        gen = torch.Generator().manual_seed(21)
        table = orn.rotary_table(96, D, base=10000.0).to(dev)
        ctx_g, ctx_e = _ctx(mi, dev, True), _ctx(mi, dev, False)
        layers = _layers(mi, dev, gen)
        assert ctx_g.cuda_graph_token_counts == [16, 8]  # steps are rounded to multiples of 8
        graphs = mi.DecodeLayerGraphs(ctx_g, layers, num_query_heads=HQ, rotary_pos_emb=(table, table))
        graphs.capture()
        assert graphs.sizes == [8, 16] and ctx_g.total_request_count == 0
        # the warm-up wrote only into the dummy chunk
        assert (ctx_g.memory_buffer[:, :, : ctx_g.dummy_chunk_idx] == -1).all()

        prompts = [5, 16, 17, 9, 3, 22, 4, 6, 2, 1]
        for i, n in enumerate(prompts):
            toks = torch.randint(0, 100, (n,), generator=gen).to(dev)
            for c in (ctx_g, ctx_e):
                c.add_request(i, toks, num_tokens_to_generate=30)
        used = set()
        kinds = set()
        for step in range(14):
            for c in (ctx_g, ctx_e):
                c.initialize_attention_state()
            n = ctx_g.padded_active_token_count
            # step 0 (prefill of the prompts) is too large for any graph; every later step replays
            # one: decode graphs, and the prefill-mode graph for the step after the late admission
            graph_step = ctx_g.using_cuda_graph_this_step()
            assert graph_step == (step != 0), step
            assert ctx_g.is_decode_only() == (step not in (0, 10)), step
            kinds.add((graph_step, ctx_g.is_decode_only()))
            ne = ctx_e.padded_active_token_count
            for l in range(L):
                q = torch.randn(max(n, ne), 1, HQ, D, generator=gen).bfloat16().to(dev)
                k = torch.randn(max(n, ne), 1, HKV, D, generator=gen).bfloat16().to(dev)
                v = torch.randn(max(n, ne), 1, HKV, D, generator=gen).bfloat16().to(dev)
                ref = layers[l](q[:ne].clone(), k[:ne].clone(), v[:ne].clone(), ctx_e, (table, table))
                act = ctx_e.active_token_count
                if graph_step:
                    used.add(n)
                    for rep in range(3):  # replays of one graph with eager work in between
                        if rep:
                            # undo nothing: a replay re-appends the same K/V rows and recomputes the same output
                            torch.cuda.synchronize()
                            _ = (q.float() * 2).sum().item()
                        got = graphs.replay(l, q, k, v)
                        torch.cuda.synchronize()
                        assert torch.equal(got[:act], ref[:act]), f"step {step} layer {l} replay {rep}"
                        assert not got[act:n].any(), "padded rows must come out as zeros"
                else:
                    got = layers[l](q[:n].clone(), k[:n].clone(), v[:n].clone(), ctx_g, (table, table))
                    assert torch.equal(got[:act], ref[:act])
                dummy = ctx_g.dummy_chunk_idx
                assert torch.equal(ctx_g.memory_buffer[:, l, :dummy], ctx_e.memory_buffer[:, l, :dummy])
            n_act = ctx_g.total_request_count - ctx_g.paused_request_count
            mask = torch.ones(n_act, dtype=torch.int32, device=dev)
            if step in (3, 6, 7) and n_act > 1:
                mask[:2] = 0  # shrink the batch so that smaller graphs get used
            if step == 9:
                toks = torch.randint(0, 100, (4,), generator=gen).to(dev)
                new = torch.randint(0, 100, (n_act,), generator=gen).to(dev)
                for c in (ctx_g, ctx_e):
                    c.update_requests(mask, new)
                    c.add_request(100, toks, num_tokens_to_generate=10)  # a prefill step between decode steps
                continue
            new = torch.randint(0, 100, (n_act,), generator=gen).to(dev)
            for c in (ctx_g, ctx_e):
                c.update_requests(mask, new)
        assert len(used) >= 2, used
        assert (True, False) in kinds and (True, True) in kinds  # both kinds of graph were replayed
    finally:
        cls.TOKEN_ROUNDER, cls.REQUEST_ROUNDER = saved


def test_replay_without_a_captured_size_raises(mi, dev):
    ctx = _ctx(mi, dev, True)
    gen = torch.Generator().manual_seed(1)
    graphs = mi.DecodeLayerGraphs(ctx, _layers(mi, dev, gen), num_query_heads=HQ)
    ctx.add_request(0, torch.arange(5, device=dev), num_tokens_to_generate=4)
    ctx.initialize_attention_state()
    q = torch.zeros(ctx.padded_active_token_count, 1, HQ, D, dtype=torch.bfloat16, device=dev)
    k = torch.zeros(ctx.padded_active_token_count, 1, HKV, D, dtype=torch.bfloat16, device=dev)
    with pytest.raises(KeyError):
        graphs.replay(0, q, k, k)
    with pytest.raises(ValueError):
        mi.DecodeLayerGraphs(_ctx(mi, dev, False), [], num_query_heads=HQ)
