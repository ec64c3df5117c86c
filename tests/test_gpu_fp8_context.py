"""GPU: a context with an fp8-e4m3 KV cache driven through prefill and decode steps.

Same call sequence as tests/test_gpu_context_end_to_end.py (initialize_attention_state -> per layer
{q/k norm, RoPE, quantising append, attention} -> update_requests), with a CPU shadow that applies the
checker's restatement of the append policy and attends over the dequantised bytes.  Value bytes and
value scales must be equal (values are not transformed before quantisation); keys pass through norm
and RoPE first, so their dequantised values are compared within one fp8 step; outputs within 6e-2.
"""
import pytest
import torch

from oracle import paged_attention as oa
from oracle import rope_norm as orn

pytestmark = pytest.mark.gpu

L, HQ, HKV, D, C = 2, 8, 2, 128, 64
DT = torch.bfloat16   # the parameters' type; a test may switch it to fp16


def _make_ctx(mi, dev, **kw):
    mi.DynamicInferenceContext.TOKEN_ROUNDER = 4
    mi.DynamicInferenceContext.REQUEST_ROUNDER = 4
    return mi.DynamicInferenceContext(
        params_dtype=DT, num_layers=L, kv_channels=D, num_attention_heads=HKV,
        max_sequence_length=256, buffer_size_gb=60 * (2 * L * C * HKV * D + 8 * L * HKV) / 1024**3,
        buffer_guaranteed_fraction=0.1, chunk_size_tokens=C, max_requests_override=16, max_tokens_override=512,
        kv_cache_dtype="fp8_e4m3", device=dev, **kw)


def test_fp8_sizing_and_buffers(mi, dev):
    saved = (mi.DynamicInferenceContext.TOKEN_ROUNDER, mi.DynamicInferenceContext.REQUEST_ROUNDER)
    try:
        ctx = _make_ctx(mi, dev)
        assert ctx.chunk_size_bytes == 2 * L * C * HKV * D + 4 * 2 * L * HKV
        assert ctx.chunk_allocator.chunk_count_total == 60
        assert ctx.memory_buffer.dtype == torch.uint8 and ctx.memory_buffer.shape == (2, L, 60, C, HKV, D)
        assert ctx.kv_scales.shape == (2, L, 60, HKV) and ctx.kv_scales.dtype == torch.float32
        k8, v8, _ = ctx.key_value_cache(1)
        assert k8.dtype == torch.uint8 and k8.shape == (60, C, HKV, D)
        ks, vs = ctx.key_value_scales(2)
        assert ks.data_ptr() == ctx.kv_scales[0, 1].data_ptr() and vs.data_ptr() == ctx.kv_scales[1, 1].data_ptr()
        with pytest.raises(ValueError, match="bfloat16 or float16"):
            mi.DynamicInferenceContext(params_dtype=torch.float32, num_layers=1, kv_channels=D, num_attention_heads=1,
                                       max_sequence_length=64, buffer_size_gb=0.001, buffer_guaranteed_fraction=0.1,
                                       chunk_size_tokens=C, kv_cache_dtype="fp8_e4m3", device=dev)
    finally:
        mi.DynamicInferenceContext.TOKEN_ROUNDER, mi.DynamicInferenceContext.REQUEST_ROUNDER = saved


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("head_dim", [128, 64])
@pytest.mark.parametrize("entry", ["fused", "unfused", "mixed_qkv"])
def test_fp8_prefill_then_decode_steps(mi, dev, entry, head_dim, dtype):
    global D, DT
    saved = (mi.DynamicInferenceContext.TOKEN_ROUNDER, mi.DynamicInferenceContext.REQUEST_ROUNDER, D, DT)
    D = head_dim   # (head_dim 64: decode steps take the separate launches, half-split pairs sit in other lanes there)
    DT = dtype
    try:
        ctx = _make_ctx(mi, dev)
        N = ctx.chunk_allocator.chunk_count_total
        sk = [torch.zeros(N, C, HKV, D, dtype=torch.uint8) for _ in range(L)]
        sv = [torch.zeros(N, C, HKV, D, dtype=torch.uint8) for _ in range(L)]
        sks = [torch.ones(N, HKV) for _ in range(L)]
        svs = [torch.ones(N, HKV) for _ in range(L)]
        gen = torch.Generator().manual_seed(5)
        table = orn.rotary_table(256, D, base=500000.0)
        table_d = table.to(dev)
        layers, weights = [], []
        for l in range(L):
            core = mi.PagedSelfAttentionCore(l + 1, D, qk_norm="rms", eps=1e-5, fused=entry != "unfused", dtype=DT, device=dev)
            qw = (1 + 0.02 * torch.randn(D, generator=gen)).to(DT)
            kw = (1 + 0.02 * torch.randn(D, generator=gen)).to(DT)
            core.q_layernorm_weight.data.copy_(qw)
            core.k_layernorm_weight.data.copy_(kw)
            layers.append(core)
            weights.append((qw, kw))
        prompts = [5, 64, 70, 130, 1]  # inside a chunk, exactly one chunk, just over, two chunks and a bit, one token
        for i, n in enumerate(prompts):
            ctx.add_request(i, torch.randint(0, 100, (n,), generator=gen).to(dev), num_tokens_to_generate=20)
        for step in range(7):
            ctx.initialize_attention_state()
            n = ctx.padded_active_token_count
            act = ctx.active_token_count
            qpos = ctx.token_to_pos_ids[:n].cpu()
            kpos = ctx.token_to_position_in_request[:n].cpu()
            ci = ctx.token_to_chunk_idx[:act].cpu()
            lo = ctx.token_to_local_position_within_kv_chunk[:act].cpu()
            lens, bt = ctx.kv_seq_lengths.cpu(), ctx.block_table.cpu()
            for l in range(L):
                mixed = torch.randn(n, 1, (HQ + 2 * HKV) * D, generator=gen).to(DT)
                q, k, v = (t.contiguous() for t in orn.split_mixed_qkv(mixed, HQ, HKV))
                qw, kw = weights[l]
                qr = orn.norm_rope(q.squeeze(1), qpos, table, norm="rms", weight=qw, eps=1e-5)
                kr = orn.norm_rope(k.squeeze(1), kpos, table, norm="rms", weight=kw, eps=1e-5)
                oa.kv_append_fp8(sk[l], sks[l], kr[:act], ci, lo)
                oa.kv_append_fp8(sv[l], svs[l], v.squeeze(1)[:act], ci, lo)
                if ctx.is_decode_only():
                    ref = oa.paged_decode_attention(qr, sk[l], sv[l], lens, bt, k_scales=sks[l], v_scales=svs[l])
                else:
                    ref = oa.paged_varlen_attention(qr[:act], sk[l], sv[l], ctx.cu_query_seq_lengths.cpu(), lens, bt,
                                                    k_scales=sks[l], v_scales=svs[l])
                if entry == "mixed_qkv":
                    out = layers[l].forward_mixed_qkv(mixed.to(dev), HQ, ctx, (table_d, table_d))
                else:
                    out = layers[l](q.to(dev), k.to(dev), v.to(dev), ctx, (table_d, table_d))
                torch.cuda.synchronize()
                got = out.float().cpu().view(n, HQ, D)[:act]
                err = (got - ref[:act]).abs()
                assert (err <= 6e-2 + 6e-2 * ref[:act].abs()).all(), f"step {step} layer {l}: {err.max().item()}"
                dummy = ctx.dummy_chunk_idx
                assert torch.equal(ctx.memory_buffer[1, l].cpu()[:dummy], sv[l][:dummy]), "value bytes differ"
                assert torch.equal(ctx.kv_scales[1, l].cpu()[:dummy], svs[l][:dummy]), "value scales differ"
                kd = oa.dequantize_fp8(ctx.memory_buffer[0, l].cpu()[:dummy], ctx.kv_scales[0, l].cpu()[:dummy])
                ks_ref = oa.dequantize_fp8(sk[l][:dummy], sks[l][:dummy])
                assert ((kd - ks_ref).abs() <= 0.07 * ks_ref.abs() + 0.05).all()  # one e4m3 step (2^-3 relative) at most
            n_act = ctx.total_request_count - ctx.paused_request_count
            mask = torch.ones(n_act, dtype=torch.int32, device=dev)
            if step == 3:
                mask[1] = 0
            ctx.update_requests(mask, torch.randint(0, 100, (n_act,), generator=gen).to(dev))
        assert ctx.total_request_count == 4
    finally:
        mi.DynamicInferenceContext.TOKEN_ROUNDER, mi.DynamicInferenceContext.REQUEST_ROUNDER, D, DT = saved
