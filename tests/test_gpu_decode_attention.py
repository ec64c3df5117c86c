"""GPU parity: paged decode attention (C ABI -> HIP) against the fp32 CPU checker.

Tolerance: |out - ref| <= 2e-2 + 2e-2 * |ref| for a bf16 cache, 6e-2 for an fp8 cache.
"""
import pytest
import torch

from oracle import paged_attention as oa

pytestmark = pytest.mark.gpu


def _close(out, ref, tol):
    out = out.float().cpu().reshape(ref.shape)
    err = (out - ref).abs()
    bound = tol + tol * ref.abs()
    worst = (err - bound).max().item()
    assert torch.isfinite(out).all(), "non-finite output"
    assert worst <= 0, f"max abs err {err.max().item():.4e} exceeds {tol} abs/rel (excess {worst:.3e})"


def _run_case(mi, case, **kw):
    out = mi.ops.paged_decode_attention(case.q, case.k_cache, case.v_cache, case.kv_lens, case.block_table, **kw)
    torch.cuda.synchronize()
    return out


def _ref(case):
    return oa.paged_decode_attention(case.q.cpu().squeeze(1), case.k_cache.cpu(), case.v_cache.cpu(),
                                     case.kv_lens.cpu(), case.block_table.cpu())


def test_cfg1_reference_size(mi, dev):
    """Batch 4, 8/8 heads, d 64, chunk 256, len U[64,1024], 64 physical chunks."""
    case = mi.synthetic.make_decode_case(mi.synthetic.CONFIGS["cfg1"], dev, pool_chunks=64)
    assert case.k_cache.size(0) == 64
    _close(_run_case(mi, case), _ref(case), 2e-2)


def test_cfg2_shape_reduced_batch(mi, dev):
    """Llama-3-8B shape (32/8 heads, d 128, len U[512,8192]) at batch 8 so the CPU checker stays fast."""
    case = mi.synthetic.make_decode_case(mi.synthetic.CONFIGS["cfg2"], dev, batch=8)
    _close(_run_case(mi, case), _ref(case), 2e-2)


@pytest.mark.parametrize("Hq,Hkv", [(8, 8), (8, 4), (32, 8), (64, 8), (16, 1), (6, 2)])
@pytest.mark.parametrize("d", [64, 128])
def test_head_grouping(mi, dev, Hq, Hkv, d):
    cfg = mi.synthetic.DecodeConfig("g", 5, Hq, Hkv, d, 1, 700, chunk=64, seed=Hq * 131 + Hkv * 7 + d)
    case = mi.synthetic.make_decode_case(cfg, dev)
    _close(_run_case(mi, case), _ref(case), 2e-2)


@pytest.mark.parametrize("chunk", [16, 48, 128, 256])
@pytest.mark.parametrize("subtiles", [1, 2])
@pytest.mark.parametrize("grid", [0, 1, 7, 4096])
def test_ragged_lengths_and_edges(mi, dev, chunk, subtiles, grid):
    """Lengths around every tile / chunk boundary, plus zero-length (padded) rows, for several
    ways of cutting the flattened tile sequence into workgroup spans (grid 0 = the default)."""
    lens = torch.tensor([0, 1, 2, 15, 16, 17, 31, 32, 33, chunk - 1, chunk, chunk + 1, 2 * chunk, 3 * chunk + 5, 0, 777],
                        dtype=torch.int32)
    cfg = mi.synthetic.DecodeConfig("edges", lens.numel(), 8, 2, 128, 0, 0, chunk=chunk, seed=chunk + subtiles)
    case = mi.synthetic.make_decode_case(cfg, dev, lens=lens)
    mi.ops.set_tuning("decode_tile_subtiles", subtiles)
    mi.ops.set_tuning("decode_grid", grid)
    try:
        for split in (0, 16, 64, 512):  # minimum tokens per workgroup span
            out = _run_case(mi, case, split_tokens=split, max_kv_len=int(lens.max()))
            _close(out, _ref(case), 2e-2)
            assert (out[case.kv_lens == 0] == 0).all(), "zero-length rows must be zeros"
    finally:
        mi.ops.set_tuning("decode_tile_subtiles", 0)
        mi.ops.set_tuning("decode_grid", 0)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("d", [96, 192, 256])
@pytest.mark.parametrize("Hq,Hkv", [(8, 8), (32, 8), (12, 4), (16, 1)])
def test_head_widths_96_192_256(mi, dev, d, Hq, Hkv, dtype):
    """Head widths beside 64 and 128 (Phi-3-small / Gemma use 96 and 256, decompressed multi-latent keys 192):
    ragged lengths around the tile and chunk edges, several chunk sizes and span cuts."""
    for chunk in (16, 64, 256):
        lens = torch.tensor([0, 1, 15, 16, 17, 33, chunk - 1, chunk, chunk + 1, 3 * chunk + 5, 1999], dtype=torch.int32)
        cfg = mi.synthetic.DecodeConfig("w", lens.numel(), Hq, Hkv, d, 0, 0, chunk=chunk, seed=d + Hq + chunk)
        case = mi.synthetic.make_decode_case(cfg, dev, lens=lens, dtype=dtype)
        ref = _ref(case)
        for split, grid in ((0, 0), (16, 4096), (512, 7)):
            with mi.ops.tuning(decode_grid=grid):
                out = _run_case(mi, case, split_tokens=split, max_kv_len=int(lens.max()))
            _close(out, ref, 2e-2)
            assert (out[case.kv_lens == 0] == 0).all(), "zero-length rows must be zeros"


@pytest.mark.parametrize("Hq,Hkv", [(32, 1), (64, 2), (17, 1), (48, 2), (40, 2), (64, 1)])
@pytest.mark.parametrize("d", [64, 128, 256])
def test_more_than_16_query_heads_per_kv_head(mi, dev, Hq, Hkv, d):
    """Up to 64 query heads share a KV head (multi-query models: Falcon-7B 71 -> 1 is beyond, Gemma-2B 8 -> 1 and
    StarCoder 48 -> 1 within): every 16 of them take a wavefront of their own."""
    lens = torch.tensor([0, 1, 17, 64, 65, 700, 2500], dtype=torch.int32)
    cfg = mi.synthetic.DecodeConfig("mq", lens.numel(), Hq, Hkv, d, 0, 0, chunk=64, seed=Hq * 3 + d)
    case = mi.synthetic.make_decode_case(cfg, dev, lens=lens)
    ref = _ref(case)
    for split, grid in ((0, 0), (64, 9), (16, 4096)):
        with mi.ops.tuning(decode_grid=grid):
            out = _run_case(mi, case, split_tokens=split, max_kv_len=int(lens.max()))
        _close(out, ref, 2e-2)
    # fp8 cache, width 128
    if d == 128:
        k8, ks = oa.quantize_chunks_fp8(case.k_cache.cpu())
        v8, vs = oa.quantize_chunks_fp8(case.v_cache.cpu())
        out = mi.ops.paged_decode_attention(case.q, k8.to(dev), v8.to(dev), case.kv_lens, case.block_table,
                                            k_scales=ks.to(dev), v_scales=vs.to(dev))
        torch.cuda.synchronize()
        ref8 = oa.paged_decode_attention(case.q.cpu().squeeze(1), k8, v8, lens, case.block_table.cpu(), k_scales=ks,
                                         v_scales=vs)
        _close(out, ref8, 2e-2)


def test_more_requests_than_one_launch_takes(mi, dev):
    """The streaming kernels keep 8 bytes per request in LDS, 7 680 requests per launch; the reference has no
    such limit (a decode step without a graph pads to max_requests), so larger batches run in slices."""
    R = 7680 + 7680 + 300
    gen = torch.Generator().manual_seed(5)
    lens = torch.randint(0, 70, (R,), generator=gen, dtype=torch.int32)
    cfg = mi.synthetic.DecodeConfig("many", R, 8, 2, 64, 0, 0, chunk=16, seed=2)
    case = mi.synthetic.make_decode_case(cfg, dev, lens=lens)
    out = _run_case(mi, case, max_kv_len=70)
    _close(out, _ref(case), 2e-2)
    assert (out[case.kv_lens == 0] == 0).all()
    # a mixed batch whose one-row requests exceed the limit: 3 prompts + R one-token requests
    q_lens = [40, 1, 130] + [1] * R
    kv = torch.cat([torch.tensor([100, 9, 130], dtype=torch.int32), lens.clamp(min=1)])
    cu_q = torch.zeros(len(q_lens) + 1, dtype=torch.int32)
    cu_q[1:] = torch.cumsum(torch.tensor(q_lens), 0)
    bt, N = mi.synthetic.build_block_table(kv, 16, gen)
    q = torch.randn(int(cu_q[-1]), 8, 64, generator=gen).bfloat16()
    kc = torch.randn(N, 16, 2, 64, generator=gen).bfloat16()
    vc = torch.randn(N, 16, 2, 64, generator=gen).bfloat16()
    got = mi.ops.paged_prefill_attention(q.to(dev), kc.to(dev), vc.to(dev), cu_q.to(dev), kv.to(dev), bt.to(dev),
                                         max_kv_len=int(kv.max()))
    torch.cuda.synchronize()
    _close(got, oa.paged_varlen_attention(q, kc, vc, cu_q, kv, bt), 2e-2)


def test_block_table_width_and_padding_rows(mi, dev):
    """Block table wider than needed (graph mode passes max_sequence_length) with -1 / 0 padding."""
    cfg = mi.synthetic.DecodeConfig("wide", 6, 32, 8, 128, 100, 2000, chunk=256, seed=5)
    case = mi.synthetic.make_decode_case(cfg, dev)
    wide = torch.zeros(8, 40, dtype=torch.int32, device=dev)  # two padded rows: table row 0, length 0
    wide[:6, : case.block_table.size(1)] = case.block_table
    lens = torch.zeros(8, dtype=torch.int32, device=dev)
    lens[:6] = case.kv_lens
    q = torch.cat([case.q, torch.randn(2, 1, 32, 128, device=dev).bfloat16()])
    out = mi.ops.paged_decode_attention(q, case.k_cache, case.v_cache, lens, wide, max_kv_len=40 * 256)
    torch.cuda.synchronize()
    _close(out[:6], _ref(case), 2e-2)
    assert (out[6:] == 0).all()


def test_chunk_permutation_invariance(mi, dev):
    """Moving the data to other physical chunks (and updating the table) must not change a single bit."""
    cfg = mi.synthetic.DecodeConfig("perm", 6, 32, 8, 128, 300, 3000, seed=9)
    case = mi.synthetic.make_decode_case(cfg, dev)
    out1 = _run_case(mi, case)
    N = case.k_cache.size(0)
    perm = torch.randperm(N, generator=torch.Generator().manual_seed(1)).to(dev)  # new id of old chunk i
    k2, v2 = torch.empty_like(case.k_cache), torch.empty_like(case.v_cache)
    k2[perm] = case.k_cache
    v2[perm] = case.v_cache
    bt2 = torch.where(case.block_table >= 0, perm[case.block_table.clamp(min=0).long()].int(), case.block_table)
    out2 = mi.ops.paged_decode_attention(case.q, k2, v2, case.kv_lens, bt2)
    torch.cuda.synchronize()
    assert torch.equal(out1, out2)


def test_all_equal_keys_give_mean_of_values(mi, dev):
    cfg = mi.synthetic.DecodeConfig("mean", 3, 16, 4, 128, 200, 1200, seed=3)
    case = mi.synthetic.make_decode_case(cfg, dev)
    case.k_cache[:] = case.k_cache[0, 0]  # every token's key row identical -> uniform softmax
    out = _run_case(mi, case).cpu().float().squeeze(1)
    for r in range(3):
        L = int(case.kv_lens[r])
        v = oa.gather_request_kv(case.v_cache.cpu(), case.block_table[r].cpu(), L).mean(0)  # [Hkv, d]
        ref = v.repeat_interleave(4, dim=0)
        assert (out[r] - ref).abs().max().item() < 1e-2


def test_split_invariance_cfg2_full_size(mi, dev):
    """Full Llama-3-8B batch-64 size: different span sizes agree with each other (merge == single pass)."""
    case = mi.synthetic.make_decode_case(mi.synthetic.CONFIGS["cfg2"], dev, on_device_rng=True)
    mx = int(case.kv_lens.max())
    base = _run_case(mi, case, max_kv_len=mx).float()
    for split, grid in ((512, 4096), (2048, 0), (8192, 0), (1 << 20, 0)):  # the last one: no splitting at all
        mi.ops.set_tuning("decode_grid", grid)
        try:
            other = _run_case(mi, case, split_tokens=split, max_kv_len=mx).float()
        finally:
            mi.ops.set_tuning("decode_grid", 0)
        assert (base - other).abs().max().item() < 8e-3
    # and a sample of rows against the checker
    rows = [0, 17, 63]
    ref = oa.paged_decode_attention(case.q[rows].cpu().squeeze(1), case.k_cache.cpu(), case.v_cache.cpu(),
                                    case.kv_lens[rows].cpu(), case.block_table[rows].cpu())
    _close(base[rows], ref, 2e-2)


def test_long_context_split_merge(mi, dev):
    """cfg4 shape (64/8 heads, 131072-token context, hundreds of partials per request) at batch 2."""
    case = mi.synthetic.make_decode_case(mi.synthetic.CONFIGS["cfg4"], dev, batch=2, on_device_rng=True)
    out = _run_case(mi, case).float()
    out2 = _run_case(mi, case, split_tokens=65536).float()
    assert (out - out2).abs().max().item() < 5e-3
    ref = oa.paged_decode_attention(case.q[:1].cpu().squeeze(1), case.k_cache.cpu(), case.v_cache.cpu(),
                                    case.kv_lens[:1].cpu(), case.block_table[:1].cpu())
    _close(out[:1], ref, 2e-2)


@pytest.mark.parametrize("d", [128, 64])
def test_fp8_kv_cache(mi, dev, d):
    """cfg5 shape at batch 6 / shorter contexts (and the same at head_dim 64): quantiser is bit-exact, attention
    within 6e-2."""
    cfg = mi.synthetic.DecodeConfig("fp8", 6, 32, 8, d, 1024, 6000, fp8=True, seed=1005)
    case = mi.synthetic.make_decode_case(cfg, dev)
    N = case.k_cache.size(0)
    k8 = torch.empty(case.k_cache.shape, dtype=torch.uint8, device=dev)
    v8 = torch.empty_like(k8)
    ks = torch.empty(N, cfg.Hkv, dtype=torch.float32, device=dev)
    vs = torch.empty_like(ks)
    mi.ops.quantize_chunks_fp8(case.k_cache, k8, ks)
    mi.ops.quantize_chunks_fp8(case.v_cache, v8, vs)
    torch.cuda.synchronize()
    k8_ref, ks_ref = oa.quantize_chunks_fp8(case.k_cache.cpu())
    v8_ref, vs_ref = oa.quantize_chunks_fp8(case.v_cache.cpu())
    assert torch.equal(ks.cpu(), ks_ref) and torch.equal(vs.cpu(), vs_ref), "scales differ"
    assert torch.equal(k8.cpu(), k8_ref) and torch.equal(v8.cpu(), v8_ref), "e4m3 bytes differ"

    out = mi.ops.paged_decode_attention(case.q, k8, v8, case.kv_lens, case.block_table, k_scales=ks, v_scales=vs)
    torch.cuda.synchronize()
    # reference of record: fp32 attention over the ORIGINAL (unquantised) K/V, tolerance 6e-2
    _close(out, _ref(case), 6e-2)
    # and tighter against the checker run on the dequantised cache
    ref_q = oa.paged_decode_attention(case.q.cpu().squeeze(1), k8_ref, v8_ref, case.kv_lens.cpu(),
                                      case.block_table.cpu(), k_scales=ks_ref, v_scales=vs_ref)
    _close(out, ref_q, 2e-2)


def test_fp8_decode_append(mi, dev):
    """New-token quantise+append: bytes and scales equal the checker's, for chunk-opening and mid-chunk tokens."""
    lens = torch.tensor([1, 257, 300, 512, 513, 0, 77], dtype=torch.int32)
    cfg = mi.synthetic.DecodeConfig("fp8app", lens.numel(), 32, 8, 128, 0, 0, fp8=True, seed=77)
    case = mi.synthetic.make_decode_case(cfg, dev, lens=lens)
    k8_ref, ks_ref = oa.quantize_chunks_fp8(case.k_cache.cpu())
    v8_ref, vs_ref = oa.quantize_chunks_fp8(case.v_cache.cpu())
    k8, v8, ks, vs = k8_ref.to(dev), v8_ref.to(dev), ks_ref.to(dev), vs_ref.to(dev)
    mi.ops.kv_append_decode_fp8(case.k_new, case.v_new, k8, v8, ks, vs, case.block_table, case.kv_lens, headroom=2.0)
    torch.cuda.synchronize()
    rows, ids, loc = oa.decode_slots(case.block_table.cpu(), lens, cfg.chunk)
    for src, c8, cs in ((case.k_new, k8_ref, ks_ref), (case.v_new, v8_ref, vs_ref)):
        src = src.cpu().squeeze(1)
        for r, c, l in zip(rows.tolist(), ids.tolist(), loc.tolist()):
            if l == 0:
                amax = src[r].float().abs().amax(dim=-1)
                cs[c] = torch.where(amax > 0, 2.0 * amax / 448.0, torch.ones_like(amax))
            c8[c, l] = oa.quantize_token_fp8(src[r], cs[c])
    assert torch.equal(ks.cpu(), ks_ref) and torch.equal(vs.cpu(), vs_ref)
    assert torch.equal(k8.cpu(), k8_ref) and torch.equal(v8.cpu(), v8_ref)


def test_rejects_bad_arguments(mi, dev):
    cfg = mi.synthetic.DecodeConfig("bad", 2, 8, 2, 128, 10, 100, chunk=64, seed=1)
    case = mi.synthetic.make_decode_case(cfg, dev)
    with pytest.raises(mi._lib.KernelError):
        mi.ops.paged_decode_attention(case.q, case.k_cache, case.v_cache, case.kv_lens, case.block_table,
                                      split_tokens=24)  # not a multiple of 16
    with pytest.raises(mi._lib.KernelError):
        mi.ops.paged_decode_attention(case.q, case.k_cache, case.v_cache, case.kv_lens, case.block_table,
                                      workspace=torch.empty(16, dtype=torch.uint8, device=dev), split_tokens=16)
    q80 = torch.randn(2, 1, 8, 80, device=dev).bfloat16()
    kc80 = torch.randn(4, 64, 2, 80, device=dev).bfloat16()
    with pytest.raises(mi._lib.KernelError):
        mi.ops.paged_decode_attention(q80, kc80, kc80, case.kv_lens, case.block_table)
