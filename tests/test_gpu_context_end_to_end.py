"""GPU: the context + attention glue driven like the reference's controller drives it.

A stand-in "model" produces random q/k/v per layer (the projections are outside the path);
each step runs  initialize_attention_state -> per layer {q/k norm, RoPE(K), append, RoPE(Q),
attention} -> update_requests,  exactly the call sequence of
text_generation_controller.py:440-546 / attention.py:394-414,766,815-828.
A CPU shadow built from the checker's pieces (norm_rope, kv_append, paged attention) follows
the same steps; outputs must agree within 2e-2, the value cache bit for bit.
"""
import pytest
import torch

from oracle import paged_attention as oa
from oracle import rope_norm as orn

pytestmark = pytest.mark.gpu

L, HQ, HKV, D, C = 2, 8, 2, 128, 16


def _make_ctx(mi, dev, dtype=torch.bfloat16):
    mi.DynamicInferenceContext.TOKEN_ROUNDER = 4
    mi.DynamicInferenceContext.REQUEST_ROUNDER = 4
    return mi.DynamicInferenceContext(
        params_dtype=dtype, num_layers=L, kv_channels=D, num_attention_heads=HKV,
        max_sequence_length=96, buffer_size_gb=200 * (2 * 2 * L * C * HKV * D) / 1024**3,
        buffer_guaranteed_fraction=0.1, chunk_size_tokens=C, max_requests_override=16, max_tokens_override=256,
        device=dev)


class Shadow:
    """CPU copy of the KV cache, advanced with the checker's functions."""

    def __init__(self, ctx):
        self.k = [ctx.memory_buffer[0, l].cpu().clone() for l in range(L)]
        self.v = [ctx.memory_buffer[1, l].cpu().clone() for l in range(L)]

    def layer(self, l, ctx, q, k, v, table, weights):
        n = ctx.padded_active_token_count
        act = ctx.active_token_count
        qpos = ctx.token_to_pos_ids[:n].cpu()
        kpos = ctx.token_to_position_in_request[:n].cpu()
        qw, kw = weights
        qr = orn.norm_rope(q.cpu().squeeze(1)[:n], qpos, table, norm="rms", weight=qw, eps=1e-5)
        kr = orn.norm_rope(k.cpu().squeeze(1)[:n], kpos, table, norm="rms", weight=kw, eps=1e-5)
        ci = ctx.token_to_chunk_idx[:act].cpu()
        lo = ctx.token_to_local_position_within_kv_chunk[:act].cpu()
        oa.kv_append(self.k[l], self.v[l], kr[:act], v.cpu().squeeze(1)[:act], ci, lo)
        lens = ctx.kv_seq_lengths.cpu()
        bt = ctx.block_table.cpu()
        if ctx.is_decode_only():
            return oa.paged_decode_attention(qr, self.k[l], self.v[l], lens, bt)
        return oa.paged_varlen_attention(qr[:act], self.k[l], self.v[l], ctx.cu_query_seq_lengths.cpu(), lens, bt)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("fused", [True, False])
def test_prefill_then_decode_steps(mi, dev, fused, dtype):
    """Both 16-bit parameter types of the reference (params_dtype, dynamic_context.py:195,287-308)."""
    saved = (mi.DynamicInferenceContext.TOKEN_ROUNDER, mi.DynamicInferenceContext.REQUEST_ROUNDER)
    try:
        ctx = _make_ctx(mi, dev, dtype)
        assert ctx.memory_buffer.dtype == dtype
        shadow = Shadow(ctx)
        gen = torch.Generator().manual_seed(5)
        table = orn.rotary_table(96, D, base=500000.0)
        table_d = table.to(dev)
        layers = []
        weights = []
        for l in range(L):
            core = mi.PagedSelfAttentionCore(l + 1, D, qk_norm="rms", eps=1e-5, fused=fused, dtype=dtype, device=dev)
            qw = (1 + 0.02 * torch.randn(D, generator=gen)).to(dtype)
            kw = (1 + 0.02 * torch.randn(D, generator=gen)).to(dtype)
            core.q_layernorm_weight.data.copy_(qw)
            core.k_layernorm_weight.data.copy_(kw)
            layers.append(core)
            weights.append((qw, kw))
        prompts = [5, 16, 17, 33, 1]
        for i, n in enumerate(prompts):
            ctx.add_request(i, torch.randint(0, 100, (n,), generator=gen).to(dev), num_tokens_to_generate=20)
        for step in range(8):
            ctx.initialize_attention_state()
            n = ctx.padded_active_token_count
            act = ctx.active_token_count
            for l in range(L):
                q = torch.randn(n, 1, HQ, D, generator=gen).to(dtype)
                k = torch.randn(n, 1, HKV, D, generator=gen).to(dtype)
                v = torch.randn(n, 1, HKV, D, generator=gen).to(dtype)
                ref = shadow.layer(l, ctx, q, k, v, table, weights[l])
                out = layers[l](q.to(dev), k.to(dev), v.to(dev), ctx, (table_d, table_d))
                torch.cuda.synchronize()
                assert out.shape == (n, 1, HQ * D)
                got = out.float().cpu().view(n, HQ, D)[:act]
                err = (got - ref[:act]).abs()
                assert (err <= 2e-2 + 2e-2 * ref[:act].abs()).all(), f"step {step} layer {l}: {err.max().item()}"
                assert torch.isfinite(out).all()
                dummy = ctx.dummy_chunk_idx
                assert torch.equal(ctx.memory_buffer[1, l].cpu()[:dummy], shadow.v[l][:dummy]), "value cache differs"
                kdiff = (ctx.memory_buffer[0, l].cpu()[:dummy].float() - shadow.k[l][:dummy].float()).abs().max()
                assert kdiff.item() <= 4e-2
            n_act = ctx.total_request_count - ctx.paused_request_count
            mask = torch.ones(n_act, dtype=torch.int32, device=dev)
            if step == 3:
                mask[1] = 0  # finish one request mid-way
            ctx.update_requests(mask, torch.randint(0, 100, (n_act,), generator=gen).to(dev))
        assert ctx.total_request_count == 4
    finally:
        mi.DynamicInferenceContext.TOKEN_ROUNDER, mi.DynamicInferenceContext.REQUEST_ROUNDER = saved


def test_fused_and_unfused_paths_write_identical_caches(mi, dev):
    """One launch (norm+RoPE+append) and the reference's call sequence leave the same bits in memory_buffer."""
    saved = (mi.DynamicInferenceContext.TOKEN_ROUNDER, mi.DynamicInferenceContext.REQUEST_ROUNDER)
    try:
        outs, bufs = [], []
        for fused in (True, False):
            gen = torch.Generator().manual_seed(9)
            ctx = _make_ctx(mi, dev)
            table_d = orn.rotary_table(96, D, base=10000.0).to(dev)
            core = mi.PagedSelfAttentionCore(1, D, qk_norm="rms", fused=fused, device=dev)
            core.q_layernorm_weight.data.copy_((1 + 0.02 * torch.randn(D, generator=gen)).bfloat16())
            core.k_layernorm_weight.data.copy_((1 + 0.02 * torch.randn(D, generator=gen)).bfloat16())
            for i, n in enumerate([7, 20]):
                ctx.add_request(i, torch.randint(0, 100, (n,), generator=gen).to(dev), num_tokens_to_generate=8)
            step_out = []
            for step in range(3):
                ctx.initialize_attention_state()
                n = ctx.padded_active_token_count
                q = torch.randn(n, 1, HQ, D, generator=gen).bfloat16().to(dev)
                k = torch.randn(n, 1, HKV, D, generator=gen).bfloat16().to(dev)
                v = torch.randn(n, 1, HKV, D, generator=gen).bfloat16().to(dev)
                step_out.append(core(q, k, v, ctx, (table_d, table_d))[: ctx.active_token_count].clone())
                ctx.update_requests(torch.ones(2, dtype=torch.int32, device=dev),
                                    torch.randint(0, 100, (2,), generator=gen).to(dev))
            torch.cuda.synchronize()
            outs.append(step_out)
            bufs.append(ctx.memory_buffer[:, 0, : ctx.dummy_chunk_idx].clone())
        assert torch.equal(bufs[0], bufs[1])
        for a, b in zip(*outs):
            assert torch.equal(a, b)
    finally:
        mi.DynamicInferenceContext.TOKEN_ROUNDER, mi.DynamicInferenceContext.REQUEST_ROUNDER = saved


def test_mixed_qkv_entry_matches_split_entry(mi, dev):
    """``forward_mixed_qkv`` on the projection output == ``forward`` on the tensors the reference's split
    (attention.py:985-1024) would hand over: same attention output, same cache bits, prefill and decode."""
    saved = (mi.DynamicInferenceContext.TOKEN_ROUNDER, mi.DynamicInferenceContext.REQUEST_ROUNDER)
    try:
        outs, bufs = [], []
        for use_mixed in (True, False):
            gen = torch.Generator().manual_seed(21)
            ctx = _make_ctx(mi, dev)
            table_d = orn.rotary_table(96, D, base=10000.0).to(dev)
            core = mi.PagedSelfAttentionCore(1, D, qk_norm="rms", fused=True, device=dev)
            core.q_layernorm_weight.data.copy_((1 + 0.02 * torch.randn(D, generator=gen)).bfloat16())
            core.k_layernorm_weight.data.copy_((1 + 0.02 * torch.randn(D, generator=gen)).bfloat16())
            for i, n in enumerate([9, 18, 3]):
                ctx.add_request(i, torch.randint(0, 100, (n,), generator=gen).to(dev), num_tokens_to_generate=8)
            step_out = []
            for step in range(3):
                ctx.initialize_attention_state()
                n = ctx.padded_active_token_count
                mixed = torch.randn(n, 1, (HQ + 2 * HKV) * D, generator=gen).bfloat16()
                if use_mixed:
                    out = core.forward_mixed_qkv(mixed.to(dev), HQ, ctx, (table_d, table_d))
                else:
                    q, k, v = orn.split_mixed_qkv(mixed, HQ, HKV)
                    out = core(q.contiguous().to(dev), k.contiguous().to(dev), v.contiguous().to(dev), ctx,
                               (table_d, table_d))
                step_out.append(out[: ctx.active_token_count].clone())
                ctx.update_requests(torch.ones(3, dtype=torch.int32, device=dev),
                                    torch.randint(0, 100, (3,), generator=gen).to(dev))
            torch.cuda.synchronize()
            outs.append(step_out)
            bufs.append(ctx.memory_buffer[:, 0, : ctx.dummy_chunk_idx].clone())
        assert torch.equal(bufs[0], bufs[1])
        for a, b in zip(*outs):
            assert torch.equal(a, b)
    finally:
        mi.DynamicInferenceContext.TOKEN_ROUNDER, mi.DynamicInferenceContext.REQUEST_ROUNDER = saved
