"""GPU parity: paged varlen causal attention (prefill / mixed batches) against the CPU checker."""
import pytest
import torch

from oracle import paged_attention as oa

pytestmark = pytest.mark.gpu


def _check(mi, q, kc, vc, cu_q, lens, bt, tol=2e-2):
    out = mi.ops.paged_prefill_attention(q, kc, vc, cu_q, lens, bt, max_kv_len=int(lens.max()))
    torch.cuda.synchronize()
    ref = oa.paged_varlen_attention(q.cpu(), kc.cpu(), vc.cpu(), cu_q.cpu(), lens.cpu(), bt.cpu())
    got = out.float().cpu()
    assert torch.isfinite(got).all()
    err = (got - ref).abs()
    assert (err <= tol + tol * ref.abs()).all(), f"max err {err.max().item():.4e}"


@pytest.mark.parametrize("Hq,Hkv,d", [(8, 8, 64), (32, 8, 128), (8, 1, 128), (16, 8, 64), (32, 2, 128)])
def test_mixed_prefill_and_decode(mi, dev, Hq, Hkv, d):
    q, kc, vc, cu_q, lens, bt = mi.synthetic.make_prefill_case(
        dev, n_prefill=3, new_tokens=150, ctx_lo=0, ctx_hi=400, n_decode=5, dec_lo=1, dec_hi=700,
        Hq=Hq, Hkv=Hkv, d=d, chunk=64, seed=Hq + Hkv + d)
    _check(mi, q, kc, vc, cu_q, lens, bt)


@pytest.mark.parametrize("subtiles,lds_rows", [(1, 0), (2, 0), (2, 2), (2, 3), (4, 2), (4, 3)])
def test_ragged_prefill_lengths(mi, dev, subtiles, lds_rows):
    """New-token counts around every block boundary, with and without existing context."""
    torch.manual_seed(0)
    q_lens = [1, 2, 15, 16, 17, 63, 64, 65, 128, 200, 1, 97, 500]
    ctx = [0, 5, 0, 16, 31, 0, 100, 1, 0, 333, 0, 40, 7]
    Hq, Hkv, d, chunk = 32, 8, 128, 32
    kv_lens = torch.tensor([a + b for a, b in zip(q_lens, ctx)], dtype=torch.int32)
    cu_q = torch.zeros(len(q_lens) + 1, dtype=torch.int32)
    cu_q[1:] = torch.cumsum(torch.tensor(q_lens), 0)
    gen = torch.Generator().manual_seed(1)
    bt, N = mi.synthetic.build_block_table(kv_lens, chunk, gen)
    q = torch.randn(int(cu_q[-1]), Hq, d, generator=gen).bfloat16().to(dev)
    kc = torch.randn(N, chunk, Hkv, d, generator=gen).bfloat16().to(dev)
    vc = torch.randn(N, chunk, Hkv, d, generator=gen).bfloat16().to(dev)
    mi.ops.set_tuning("prefill_tile_subtiles", subtiles)
    mi.ops.set_tuning("prefill_lds_row_tiles", lds_rows)  # 0 = register-only kernel
    try:
        _check(mi, q, kc, vc, cu_q.to(dev), kv_lens.to(dev), bt.to(dev))
    finally:
        mi.ops.set_tuning("prefill_tile_subtiles", 4)
        mi.ops.set_tuning("prefill_lds_row_tiles", 2)


def test_prefill_equals_decode_for_single_tokens(mi, dev):
    """A varlen batch of one-token requests is a decode batch: both kernels agree."""
    cfg = mi.synthetic.DecodeConfig("pd", 7, 32, 8, 128, 1, 900, chunk=128, seed=21)
    case = mi.synthetic.make_decode_case(cfg, dev)
    cu_q = torch.arange(8, dtype=torch.int32, device=dev)
    a = mi.ops.paged_prefill_attention(case.q.squeeze(1), case.k_cache, case.v_cache, cu_q, case.kv_lens,
                                       case.block_table)
    b = mi.ops.paged_decode_attention(case.q, case.k_cache, case.v_cache, case.kv_lens, case.block_table)
    torch.cuda.synchronize()
    assert (a.float() - b.squeeze(1).float()).abs().max().item() < 8e-3


def test_padded_requests_with_zero_lengths(mi, dev):
    """Graph-mode padding: trailing requests with q-len 0 and kv-len 0 are skipped."""
    q, kc, vc, cu_q, lens, bt = mi.synthetic.make_prefill_case(
        dev, n_prefill=2, new_tokens=40, ctx_lo=10, ctx_hi=90, n_decode=2, dec_lo=5, dec_hi=99,
        Hq=8, Hkv=2, d=128, chunk=64, seed=3)
    R = lens.numel()
    cu_pad = torch.cat([cu_q, cu_q[-1:].repeat(3)])
    lens_pad = torch.cat([lens, torch.zeros(3, dtype=torch.int32, device=dev)])
    bt_pad = torch.cat([bt, torch.zeros(3, bt.size(1), dtype=torch.int32, device=dev)])
    out = mi.ops.paged_prefill_attention(q, kc, vc, cu_pad, lens_pad, bt_pad)
    torch.cuda.synchronize()
    ref = oa.paged_varlen_attention(q.cpu(), kc.cpu(), vc.cpu(), cu_q.cpu(), lens.cpu(), bt.cpu())
    assert (out.float().cpu() - ref).abs().max().item() < 2e-2
