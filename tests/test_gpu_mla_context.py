"""GPU: a context with the multi-latent (MLA) latent cache driven through a mixed step and decode steps.

Call sequence of the reference for cache_mla_latents (attention.py:394-414, 561-587;
multi_latent_attention.py:225-300): append kv_concat as the key -> decode steps attend over the latent
cache in absorbed form; prefill / mixed steps decompress the cache (an up-projection, outside this
path: a torch matmul here) and run varlen attention over 192-wide keys and 128-wide values.
The CPU shadow appends with the checker's scatter (bit-exact) and attends with the checker.
"""
import pytest
import torch

from oracle import paged_attention as oa

pytestmark = pytest.mark.gpu

L, H, RANK, ROPE, C = 2, 16, 512, 64, 64


def test_mla_context_mixed_then_decode_steps(mi, dev):
    Ctx = mi.DynamicInferenceContext
    saved = (Ctx.TOKEN_ROUNDER, Ctx.REQUEST_ROUNDER)
    try:
        Ctx.TOKEN_ROUNDER, Ctx.REQUEST_ROUNDER = 4, 4
        ctx = Ctx(params_dtype=torch.bfloat16, num_layers=L, kv_channels=128, num_attention_heads=H,
                  max_sequence_length=256, buffer_size_gb=40 * (2 * L * C * (RANK + ROPE)) / 1024**3,
                  buffer_guaranteed_fraction=0.1, chunk_size_tokens=C, max_requests_override=16,
                  max_tokens_override=512, cache_mla_latent=True, kv_lora_rank=RANK, qk_pos_emb_head_dim=ROPE,
                  device=dev)
        N = ctx.chunk_allocator.chunk_count_total
        shadow = [ctx.memory_buffer[l].cpu().clone() for l in range(L)]
        g = torch.Generator().manual_seed(8)
        w_k = (torch.randn(RANK, H * 128, generator=g) / RANK ** 0.5).bfloat16().to(dev)
        w_v = (torch.randn(RANK, H * 128, generator=g) / RANK ** 0.5).bfloat16().to(dev)
        for i, n in enumerate([5, 64, 70, 130, 1]):
            ctx.add_request(i, torch.randint(0, 100, (n,), generator=g).to(dev), num_tokens_to_generate=20)
        scale = (128 + ROPE) ** -0.5
        for step in range(5):
            ctx.initialize_attention_state()
            n, act = ctx.padded_active_token_count, ctx.active_token_count
            ci = ctx.token_to_chunk_idx[:act].cpu()
            lo = ctx.token_to_local_position_within_kv_chunk[:act].cpu()
            lens, bt = ctx.kv_seq_lengths.cpu(), ctx.block_table.cpu()
            cu_q, max_q = ctx.cu_query_lengths()
            cu_k, kv_lens, max_k = ctx.cu_kv_lengths()
            for l in range(L):
                kv_concat = (torch.randn(n, 1, RANK + ROPE, generator=g) * 0.5).bfloat16()
                ctx.append_key_value_cache(l + 1, kv_concat.to(dev), None)
                shadow[l][ci.long(), lo.long()] = kv_concat.squeeze(1)[:act]
                latent, none, table = ctx.key_value_cache(l + 1)
                assert none is None
                dummy = ctx.dummy_chunk_idx
                assert torch.equal(latent.cpu()[:dummy], shadow[l][:dummy]), "latent rows differ"
                if ctx.is_decode_only():
                    q = torch.randn(n, 1, H, RANK + ROPE, generator=g).bfloat16()
                    out = mi.flash_decode_and_prefill(q.to(dev), latent, None, max_q, max_k, cu_q, cu_k, kv_lens, table,
                                                      softmax_scale=scale, mla_head_dim_v=RANK)
                    ref = oa.mla_decode_attention(q.squeeze(1), shadow[l], lens, bt, scale, RANK)
                    got = out.float().cpu().squeeze(1)
                    assert got.shape == (n, H, RANK)
                else:
                    # decompression of the whole cache, as MLASelfAttention.uncompress_kv_from_cache does
                    k_nope = (latent[..., :RANK] @ w_k).view(N, C, H, 128)
                    value = (latent[..., :RANK] @ w_v).view(N, C, H, 128)
                    key = torch.cat([k_nope, latent[..., RANK:].unsqueeze(-2).expand(-1, -1, H, -1)], dim=-1)
                    q = torch.randn(n, 1, H, 128 + ROPE, generator=g).bfloat16()
                    out = mi.flash_decode_and_prefill(q.to(dev), key, value, max_q, max_k, cu_q, cu_k, kv_lens, table,
                                                      softmax_scale=scale)
                    ref = oa.paged_varlen_attention(q.squeeze(1)[:act], key.cpu(), value.cpu(), cu_q.cpu(), lens, bt,
                                                    softmax_scale=scale)
                    got = out.float().cpu().squeeze(1)
                    assert got.shape == (n, H, 128)
                torch.cuda.synchronize()
                err = (got[:act] - ref[:act]).abs()
                assert torch.isfinite(got).all()
                assert (err <= 2e-2 + 2e-2 * ref[:act].abs()).all(), f"step {step} layer {l}: {err.max().item()}"
            n_act = ctx.total_request_count - ctx.paused_request_count
            ctx.update_requests(torch.ones(n_act, dtype=torch.int32, device=dev),
                                torch.randint(0, 100, (n_act,), generator=g).to(dev))
        assert ctx.total_request_count == 5
    finally:
        Ctx.TOKEN_ROUNDER, Ctx.REQUEST_ROUNDER = saved
