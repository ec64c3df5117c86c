"""GPU parity: varlen causal attention over the decompressed caches of multi-latent attention
(key width 192, value width 128, separate strides), against the fp32 checker: 2e-2 abs/rel."""
import pytest
import torch

from oracle import paged_attention as oa

pytestmark = pytest.mark.gpu


def _case(mi, q_lens, ctx, H, chunk, seed):
    kv_lens = torch.tensor([a + b for a, b in zip(q_lens, ctx)], dtype=torch.int32)
    cu_q = torch.zeros(len(q_lens) + 1, dtype=torch.int32)
    cu_q[1:] = torch.cumsum(torch.tensor(q_lens), 0)
    g = torch.Generator().manual_seed(seed)
    bt, N = mi.synthetic.build_block_table(kv_lens, chunk, g)
    q = torch.randn(int(cu_q[-1]), H, 192, generator=g).bfloat16()
    kc = torch.randn(N, chunk, H, 192, generator=g).bfloat16()
    vc = torch.randn(N, chunk, H, 128, generator=g).bfloat16()
    return q, kc, vc, cu_q, kv_lens, bt


@pytest.mark.parametrize("H", [1, 4, 16])
@pytest.mark.parametrize("chunk", [16, 64, 256])
def test_mla_prefill_matches_checker(mi, dev, H, chunk):
    q_lens = [1, 2, 15, 16, 17, 63, 64, 65, 200, 1, 97]
    ctx = [0, 5, 0, 16, 31, 0, 100, 1, 333, 70, 40]
    q, kc, vc, cu_q, lens, bt = _case(mi, q_lens, ctx, H, chunk, seed=H + chunk)
    scale = 192 ** -0.5
    out = mi.ops.paged_prefill_attention_mla(q.to(dev), kc.to(dev), vc.to(dev), cu_q.to(dev), lens.to(dev),
                                             bt.to(dev), softmax_scale=scale)
    torch.cuda.synchronize()
    ref = oa.paged_varlen_attention(q, kc, vc, cu_q, lens, bt, softmax_scale=scale)
    got = out.float().cpu()
    assert got.shape == ref.shape == (q.size(0), H, 128) and torch.isfinite(got).all()
    err = (got - ref).abs()
    assert (err <= 2e-2 + 2e-2 * ref.abs()).all(), f"max err {err.max().item():.4e}"


@pytest.mark.parametrize("pingpong", [-1, 1, 2])  # register-only kernel, two-phase, two-phase in lock-step
@pytest.mark.parametrize("Hq,Hkv", [(8, 8), (8, 2), (16, 1), (20, 1), (64, 2)])
def test_mla_prefill_kernel_choice_and_grouped_heads(mi, dev, pingpong, Hq, Hkv):
    """The two-phase tile kernel (both wave schedules) and the register kernel, with several query heads
    per key head, over lengths either side of the 64-key tiles and the chunk size."""
    chunk = 128
    q_lens = [1, 64, 65, 300, 2, 127, 1, 513]
    ctx = [700, 0, 63, 129, 1000, 1, 0, 256]
    kv_lens = torch.tensor([a + b for a, b in zip(q_lens, ctx)], dtype=torch.int32)
    cu_q = torch.zeros(len(q_lens) + 1, dtype=torch.int32)
    cu_q[1:] = torch.cumsum(torch.tensor(q_lens), 0)
    g = torch.Generator().manual_seed(100 + Hq + Hkv)
    bt, N = mi.synthetic.build_block_table(kv_lens, chunk, g)
    q = torch.randn(int(cu_q[-1]), Hq, 192, generator=g).bfloat16()
    kc = torch.randn(N, chunk, Hkv, 192, generator=g).bfloat16()
    vc = torch.randn(N, chunk, Hkv, 128, generator=g).bfloat16()
    mi.ops.set_tuning("prefill_two_phase", pingpong)
    try:
        out = mi.ops.paged_prefill_attention_mla(q.to(dev), kc.to(dev), vc.to(dev), cu_q.to(dev), kv_lens.to(dev),
                                                 bt.to(dev), softmax_scale=0.07)
        torch.cuda.synchronize()
    finally:
        mi.ops.set_tuning("prefill_two_phase", 0)
    ref = oa.paged_varlen_attention(q, kc, vc, cu_q, kv_lens, bt, softmax_scale=0.07)
    got = out.float().cpu()
    err = (got - ref).abs()
    assert torch.isfinite(got).all() and (err <= 2e-2 + 2e-2 * ref.abs()).all(), f"max err {err.max().item():.4e}"


@pytest.mark.parametrize("forced", [0, 3, 16])
def test_mla_prefill_few_rows_over_long_contexts_split_the_keys(mi, dev, forced):
    """A chunk of a prompt over a long history: the keys of a request are cut into ranges (automatic count,
    or forced ones -- also more ranges than short requests have tiles), partials merged by a second kernel."""
    H, chunk = 4, 64
    q_lens, ctx = [40, 1, 17, 3], [3000, 2500, 0, 70]
    q, kc, vc, cu_q, lens, bt = _case(mi, q_lens, ctx, H, chunk, seed=40 + forced)
    q_pad = torch.cat([q, torch.randn(2, H, 192).bfloat16()])
    mi.ops.set_tuning("prefill_kv_split", forced)
    try:
        out = mi.ops.paged_prefill_attention_mla(q_pad.to(dev), kc.to(dev), vc.to(dev), cu_q.to(dev), lens.to(dev),
                                                 bt.to(dev), softmax_scale=0.07, max_kv_len=int(lens.max()))
        torch.cuda.synchronize()
    finally:
        mi.ops.set_tuning("prefill_kv_split", 0)
    ref = oa.paged_varlen_attention(q, kc, vc, cu_q, lens, bt, softmax_scale=0.07)
    got = out.float().cpu()
    T = q.size(0)
    assert torch.isfinite(got).all() and (got[T:] == 0).all()
    err = (got[:T] - ref).abs()
    assert (err <= 2e-2 + 2e-2 * ref.abs()).all(), f"max err {err.max().item():.4e}"


def test_mla_prefill_strided_caches_and_padding_rows(mi, dev):
    """Key and value caches as views of one wider buffer (as a split of the up-projection output gives
    them), token padding after the last request, trailing zero-length requests."""
    H, chunk = 4, 64
    q, kc, vc, cu_q, lens, bt = _case(mi, [40, 1, 130], [10, 99, 0], H, chunk, seed=7)
    N = kc.size(0)
    both = torch.zeros(N, chunk, H, 192 + 128, dtype=torch.bfloat16)
    both[..., :192], both[..., 192:] = kc, vc
    both_d = both.to(dev)
    T = q.size(0)
    q_pad = torch.cat([q, torch.randn(5, H, 192).bfloat16()])
    cu_pad = torch.cat([cu_q, cu_q[-1:].repeat(2)])
    lens_pad = torch.cat([lens, torch.zeros(2, dtype=torch.int32)])
    bt_pad = torch.cat([bt, torch.zeros(2, bt.size(1), dtype=torch.int32)])
    out = mi.ops.paged_prefill_attention_mla(q_pad.to(dev), both_d[..., :192], both_d[..., 192:], cu_pad.to(dev),
                                             lens_pad.to(dev), bt_pad.to(dev), softmax_scale=0.07)
    torch.cuda.synchronize()
    ref = oa.paged_varlen_attention(q, kc, vc, cu_q, lens, bt, softmax_scale=0.07)
    got = out.float().cpu()
    assert (got[:T] - ref).abs().max().item() < 2e-2
    assert (got[T:] == 0).all()


def test_mla_prefill_argument_errors(mi, dev):
    q, kc, vc, cu_q, lens, bt = _case(mi, [5], [0], 2, 16, seed=1)
    with pytest.raises(mi._lib.KernelError, match="192"):
        mi.ops.paged_prefill_attention_mla(q.to(dev)[..., :128].contiguous(), kc.to(dev)[..., :128].contiguous(),
                                           vc.to(dev), cu_q.to(dev), lens.to(dev), bt.to(dev), softmax_scale=0.1)
    with pytest.raises(ValueError, match="widths differ"):
        mi.ops.paged_prefill_attention_mla(q.to(dev)[..., :128].contiguous(), kc.to(dev), vc.to(dev), cu_q.to(dev),
                                           lens.to(dev), bt.to(dev), softmax_scale=0.1)
