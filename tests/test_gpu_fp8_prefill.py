"""GPU parity: fp8-e4m3 KV in prefill / mixed steps -- the quantising append of many tokens and the
varlen attention over byte caches (through the C ABI).

Bars: appended bytes and scales equal the checker's restatement of the library's policy (integer /
byte work); attention within 6e-2 abs/rel of the fp32 checker run on the dequantised cache.
"""
import pytest
import torch

from oracle import paged_attention as oa

pytestmark = pytest.mark.gpu


def _fp8_case(mi, dev, **kw):
    q, kc, vc, cu_q, lens, bt = mi.synthetic.make_prefill_case(dev, **kw)
    k8 = torch.empty(kc.shape, dtype=torch.uint8, device=dev)
    v8 = torch.empty_like(k8)
    ks = torch.empty(kc.size(0), kc.size(2), dtype=torch.float32, device=dev)
    vs = torch.empty_like(ks)
    mi.ops.quantize_chunks_fp8(kc, k8, ks)
    mi.ops.quantize_chunks_fp8(vc, v8, vs)
    return q, k8, v8, ks, vs, cu_q, lens, bt


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("d", [128, 64])
@pytest.mark.parametrize("pingpong", [1, 2])
@pytest.mark.parametrize("Hq,Hkv,chunk", [(32, 8, 64), (8, 1, 128), (32, 2, 256), (16, 16, 64)])
def test_fp8_mixed_prefill_and_decode(mi, dev, Hq, Hkv, chunk, pingpong, d, dtype):
    q, k8, v8, ks, vs, cu_q, lens, bt = _fp8_case(
        mi, dev, n_prefill=3, new_tokens=150, ctx_lo=0, ctx_hi=400, n_decode=5, dec_lo=1, dec_hi=700,
        Hq=Hq, Hkv=Hkv, d=d, chunk=chunk, seed=Hq + Hkv + chunk, dtype=dtype)
    mi.ops.set_tuning("prefill_two_phase", pingpong)
    try:
        out = mi.ops.paged_prefill_attention(q, k8, v8, cu_q, lens, bt, max_kv_len=int(lens.max()),
                                             k_scales=ks, v_scales=vs)
        torch.cuda.synchronize()
    finally:
        mi.ops.set_tuning("prefill_two_phase", 0)
    ref = oa.paged_varlen_attention(q.cpu(), k8.cpu(), v8.cpu(), cu_q.cpu(), lens.cpu(), bt.cpu(),
                                    k_scales=ks.cpu(), v_scales=vs.cpu())
    got = out.float().cpu()
    assert torch.isfinite(got).all()
    err = (got - ref).abs()
    assert (err <= 6e-2 + 6e-2 * ref.abs()).all(), f"max err {err.max().item():.4e}"
    # the quantisation itself is not what the tolerance absorbs: against the same bytes the error is small
    assert err.max().item() < 2.5e-2


def test_fp8_prefill_boundaries_and_scale_spread(mi, dev):
    """Lengths around tile / chunk boundaries; scales that differ by two orders of magnitude between chunks."""
    q_lens = [1, 2, 63, 64, 65, 128, 200, 1, 97, 300]
    ctx = [0, 5, 0, 16, 31, 100, 333, 70, 40, 7]
    Hq, Hkv, d, chunk = 32, 8, 128, 64
    kv_lens = torch.tensor([a + b for a, b in zip(q_lens, ctx)], dtype=torch.int32)
    cu_q = torch.zeros(len(q_lens) + 1, dtype=torch.int32)
    cu_q[1:] = torch.cumsum(torch.tensor(q_lens), 0)
    gen = torch.Generator().manual_seed(11)
    bt, N = mi.synthetic.build_block_table(kv_lens, chunk, gen)
    q = torch.randn(int(cu_q[-1]), Hq, d, generator=gen).bfloat16().to(dev)
    # (magnitudes at most ~1: the bar is absolute, and 30x keys would turn the softmax into an argmax
    # whose near-ties any rounding flips)
    kmag = torch.tensor([0.05, 0.5, 1.5])[torch.randint(0, 3, (N, 1, Hkv, 1), generator=gen)]
    vmag = torch.tensor([0.01, 0.1, 1.0])[torch.randint(0, 3, (N, 1, Hkv, 1), generator=gen)]
    kc = (torch.randn(N, chunk, Hkv, d, generator=gen) * kmag).bfloat16()
    vc = (torch.randn(N, chunk, Hkv, d, generator=gen) * vmag).bfloat16()
    k8, ks = oa.quantize_chunks_fp8(kc)
    v8, vs = oa.quantize_chunks_fp8(vc)
    out = mi.ops.paged_prefill_attention(q, k8.to(dev), v8.to(dev), cu_q.to(dev), kv_lens.to(dev), bt.to(dev),
                                         k_scales=ks.to(dev), v_scales=vs.to(dev))
    torch.cuda.synchronize()
    ref = oa.paged_varlen_attention(q.cpu(), k8, v8, cu_q, kv_lens, bt, k_scales=ks, v_scales=vs)
    err = (out.float().cpu() - ref).abs()
    assert (err <= 6e-2 + 6e-2 * ref.abs()).all(), f"max err {err.max().item():.4e}"


def test_fp8_prefill_rejects_what_it_cannot_run(mi, dev):
    q, k8, v8, ks, vs, cu_q, lens, bt = _fp8_case(
        mi, dev, n_prefill=1, new_tokens=20, ctx_lo=0, ctx_hi=10, n_decode=0, dec_lo=1, dec_hi=2,
        Hq=8, Hkv=2, d=128, chunk=16, seed=1)
    with pytest.raises(mi._lib.KernelError, match="multiple of 64"):
        mi.ops.paged_prefill_attention(q, k8, v8, cu_q, lens, bt, k_scales=ks, v_scales=vs)
    with pytest.raises(ValueError, match="scales"):
        mi.ops.paged_prefill_attention(q, k8, v8, cu_q, lens, bt, k_scales=ks)
    with pytest.raises(ValueError, match="16-bit type"):
        mi.ops.paged_prefill_attention(q, k8, v8, cu_q, lens, bt)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("headroom", [2.0, 1.5])
def test_fp8_append_many_tokens_matches_the_policy(mi, dev, headroom, dtype):
    """Prompts that fill chunks, end inside a chunk, continue a partly filled chunk, plus padded rows
    that all point at one slot of the dummy chunk."""
    Hkv, d, chunk, N = 4, 128, 64, 24
    gen = torch.Generator().manual_seed(5)
    # (first position, number of new tokens, physical chunks of the request)
    reqs = [(0, 64, [3]), (0, 150, [7, 1, 12]), (40, 60, [5, 9]), (64, 10, [2, 14]), (0, 1, [20]), (63, 2, [6, 8])]
    rows_c, rows_l = [], []
    for first, n, chunks in reqs:
        for pos in range(first, first + n):
            rows_c.append(chunks[pos // chunk])
            rows_l.append(pos % chunk)
    pad = 5
    rows_c += [N - 1] * pad
    rows_l += [0] * pad
    T = len(rows_c)
    tc, tl = torch.tensor(rows_c), torch.tensor(rows_l)
    key = (torch.randn(T, Hkv, d, generator=gen) * 3).to(dtype)
    val = torch.randn(T, Hkv, d, generator=gen).to(dtype)
    key[5:9, 1] = 0  # a few all-zero head rows
    k8 = torch.randint(0, 255, (N, chunk, Hkv, d), generator=gen, dtype=torch.uint8)
    v8 = torch.randint(0, 255, (N, chunk, Hkv, d), generator=gen, dtype=torch.uint8)
    ks = torch.rand(N, Hkv, generator=gen) + 0.5   # chunks 5 and 6 are continued: their scales are reused
    vs = torch.rand(N, Hkv, generator=gen) + 0.5
    k8d, v8d, ksd, vsd = k8.to(dev), v8.to(dev), ks.to(dev), vs.to(dev)
    mi.ops.kv_append_fp8(key.to(dev), val.to(dev), k8d, v8d, ksd, vsd, tc.to(dev), tl.to(dev), headroom=headroom)
    torch.cuda.synchronize()
    real = T - pad
    for cache, scales, rows, got_c, got_s in ((k8, ks, key, k8d, ksd), (v8, vs, val, v8d, vsd)):
        want_c, want_s = cache.clone(), scales.clone()
        oa.kv_append_fp8(want_c, want_s, rows[:real], tc[:real], tl[:real], headroom=headroom)
        assert torch.equal(got_s.cpu()[: N - 1], want_s[: N - 1])
        assert torch.equal(got_c.cpu()[: N - 1], want_c[: N - 1])
    assert torch.equal(ksd.cpu()[5], ks[5]) and torch.equal(ksd.cpu()[6], ks[6])  # continued chunks keep their scale
    # a chunk filled by one call gets the same bytes and scale as the whole-chunk quantiser
    full = torch.full((1, chunk, Hkv, d), 0, dtype=dtype)
    full[0] = key[:64]
    b, s_ = oa.quantize_chunks_fp8(full)
    assert torch.equal(k8d.cpu()[3], b[0]) and torch.equal(ksd.cpu()[3], s_[0])
