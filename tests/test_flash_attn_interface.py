"""The flash-attn call shapes of the reference's dynamic path (attention.py:507-600): what the adapters accept and
what they refuse.  The refusals need no GPU; the GPU cases check that the flash-attention-3 forms
(`_flash_attn_forward(..., seqused_k=, page_table=)`, `flash_attn_with_kvcache(..., page_table=)`) give the results
of the flash-attention-2 forms."""
import pytest
import torch


def _fa3_kwargs(**over):
    """The keyword set of the reference's call (attention.py:510-544), every optional argument at the value it has there."""
    kw = dict(k_new=None, v_new=None, qv=None, out=None, cu_seqlens_k=None, cu_seqlens_k_new=None, seqused_q=None,
              kv_batch_idx=None, leftpad_k=None, rotary_cos=None, rotary_sin=None, seqlens_rotary=None, q_descale=None,
              k_descale=None, v_descale=None, causal=True, window_size=(-1, -1), attention_chunk=0, softcap=0.0,
              rotary_interleaved=True, scheduler_metadata=None, num_splits=0, pack_gqa=None, sm_margin=0)
    kw.update(over)
    return kw


@pytest.mark.parametrize("bad", [dict(window_size=(128, 0)), dict(softcap=30.0), dict(attention_chunk=64),
                                 dict(k_new=torch.zeros(1)), dict(q_descale=torch.ones(1)), dict(leftpad_k=torch.zeros(1))])
def test_fa3_form_refuses_what_would_change_the_result(mi, bad):
    q = torch.zeros(4, 2, 64)
    cache = torch.zeros(1, 16, 2, 64)
    with pytest.raises(NotImplementedError):
        mi._flash_attn_forward(q=q, k=cache, v=cache, cu_seqlens_q=torch.tensor([0, 4], dtype=torch.int32),
                               seqused_k=torch.tensor([4], dtype=torch.int32), max_seqlen_q=4, max_seqlen_k=4,
                               page_table=torch.zeros(1, 1, dtype=torch.int32), softmax_scale=0.125, **_fa3_kwargs(**bad))


def test_fa3_form_needs_the_varlen_arguments(mi):
    q = torch.zeros(4, 2, 64)
    cache = torch.zeros(1, 16, 2, 64)
    with pytest.raises(NotImplementedError):
        mi._flash_attn_forward(q=q, k=cache, v=cache, cu_seqlens_q=None, seqused_k=torch.tensor([4], dtype=torch.int32),
                               max_seqlen_q=4, max_seqlen_k=4, page_table=torch.zeros(1, 1, dtype=torch.int32),
                               softmax_scale=0.125, **_fa3_kwargs())
    with pytest.raises(NotImplementedError):  # no block table: the dense form does not exist on this path
        mi._flash_attn_forward(q=q, k=cache, v=cache, cu_seqlens_q=torch.tensor([0, 4], dtype=torch.int32),
                               seqused_k=torch.tensor([4], dtype=torch.int32), max_seqlen_q=4, max_seqlen_k=4,
                               page_table=None, softmax_scale=0.125, **_fa3_kwargs())


@pytest.mark.gpu
@pytest.mark.parametrize("d", [64, 128])
def test_fa3_prefill_form_equals_the_fa2_form(mi, dev, d):
    q, kc, vc, cu_q, lens, bt = mi.synthetic.make_prefill_case(
        dev, n_prefill=3, new_tokens=150, ctx_lo=0, ctx_hi=400, n_decode=5, dec_lo=1, dec_hi=700,
        Hq=16, Hkv=4, d=d, chunk=64, seed=d)
    cu_k = torch.zeros(lens.numel() + 1, dtype=torch.int32, device=dev)
    cu_k[1:] = torch.cumsum(lens, 0)
    max_q, max_k = int((cu_q[1:] - cu_q[:-1]).max()), int(lens.max())
    ref = mi.flash_attn_varlen_func(q, kc, vc, cu_q, cu_k, max_q, max_k, softmax_scale=d ** -0.5, causal=True,
                                    block_table=bt)
    got, *unused = mi._flash_attn_forward(q=q, k=kc, v=vc, cu_seqlens_q=cu_q, seqused_k=lens, max_seqlen_q=max_q,
                                          max_seqlen_k=max_k, page_table=bt, softmax_scale=d ** -0.5, **_fa3_kwargs())
    torch.cuda.synchronize()
    assert torch.equal(got, ref)
    out = torch.empty_like(q)
    got2, _ = mi._flash_attn_forward(q=q, k=kc, v=vc, cu_seqlens_q=cu_q, seqused_k=lens, max_seqlen_q=max_q,
                                     max_seqlen_k=max_k, page_table=bt, softmax_scale=d ** -0.5,
                                     **_fa3_kwargs(out=out))
    torch.cuda.synchronize()
    assert got2 is out and torch.equal(out, ref)


@pytest.mark.gpu
def test_fa3_decode_form_equals_the_fa2_form(mi, dev):
    cfg = mi.synthetic.DecodeConfig("fa3", 9, 32, 8, 128, 1, 900, chunk=128, seed=33)
    case = mi.synthetic.make_decode_case(cfg, dev)
    a = mi.flash_attn_with_kvcache(q=case.q, k_cache=case.k_cache, v_cache=case.v_cache, cache_seqlens=case.kv_lens,
                                   causal=True, block_table=case.block_table)
    b = mi.flash_attn_with_kvcache(q=case.q, k_cache=case.k_cache, v_cache=case.v_cache, cache_seqlens=case.kv_lens,
                                   causal=True, page_table=case.block_table)
    torch.cuda.synchronize()
    assert torch.equal(a, b)
