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


@pytest.mark.parametrize("subtiles,row_tiles", [(1, 2), (2, 2), (1, 4), (2, 4)])
def test_ragged_prefill_lengths(mi, dev, subtiles, row_tiles):
    """New-token counts around every block boundary, with and without existing context, at a chunk size (32) that
    is no multiple of the 64-key staged tiles: the register-only kernel, 16 or 32 keys per iteration, 32 or 64 rows
    per wavefront."""
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
    with mi.ops.tuning(prefill_tile_subtiles=subtiles, prefill_row_tiles=row_tiles):
        _check(mi, q, kc, vc, cu_q.to(dev), kv_lens.to(dev), bt.to(dev))


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


@pytest.mark.parametrize("pingpong", [1, 2, 3])
@pytest.mark.parametrize("chunk", [64, 128, 256])
@pytest.mark.parametrize("Hq,Hkv", [(32, 8), (8, 8), (16, 1), (16, 2)])
@pytest.mark.parametrize("d", [128, 64, 96])
def test_two_phase_kernel_ragged_lengths(mi, dev, pingpong, chunk, Hq, Hkv, d):
    """The tile kernels (head_dim 128, 96 or 64, chunk a multiple of 64): new-token counts and cached
    contexts around every tile (64 keys), workgroup (256 rows) and chunk boundary, for 1, 2, 4, 8
    and 16 query heads per KV head; the two-phase kernel staggered (1) and in lock-step (2), and the one-stream
    kernel that serves head_dim 128 by default (3; other widths fall back to the two-phase kernel)."""
    q_lens = [1, 2, 15, 16, 17, 63, 64, 65, 128, 200, 1, 97, 500, 256, 257, 3]
    ctx = [0, 5, 0, 16, 31, 0, 100, 1, 0, 333, 0, 40, 7, 64, 63, 1020]
    kv_lens = torch.tensor([a + b for a, b in zip(q_lens, ctx)], dtype=torch.int32)
    cu_q = torch.zeros(len(q_lens) + 1, dtype=torch.int32)
    cu_q[1:] = torch.cumsum(torch.tensor(q_lens), 0)
    gen = torch.Generator().manual_seed(chunk + Hq)
    bt, N = mi.synthetic.build_block_table(kv_lens, chunk, gen)
    q = torch.randn(int(cu_q[-1]), Hq, d, generator=gen).bfloat16().to(dev)
    kc = torch.randn(N, chunk, Hkv, d, generator=gen).bfloat16().to(dev)
    vc = torch.randn(N, chunk, Hkv, d, generator=gen).bfloat16().to(dev)
    mi.ops.set_tuning("prefill_two_phase", pingpong)
    try:
        _check(mi, q, kc, vc, cu_q.to(dev), kv_lens.to(dev), bt.to(dev))
    finally:
        mi.ops.set_tuning("prefill_two_phase", 0)


def _ragged_case(mi, dev, Hq, Hkv, d, chunk, dtype, seed, pad_rows=0):
    q_lens = [1, 2, 15, 16, 17, 63, 64, 65, 128, 200, 1, 97, 300, 3]
    ctx = [0, 5, 0, 16, 31, 0, 100, 1, 0, 333, 0, 40, 7, 1020]
    kv_lens = torch.tensor([a + b for a, b in zip(q_lens, ctx)], dtype=torch.int32)
    cu_q = torch.zeros(len(q_lens) + 1, dtype=torch.int32)
    cu_q[1:] = torch.cumsum(torch.tensor(q_lens), 0)
    gen = torch.Generator().manual_seed(seed)
    bt, N = mi.synthetic.build_block_table(kv_lens, chunk, gen)
    q = torch.randn(int(cu_q[-1]) + pad_rows, Hq, d, generator=gen).to(dtype).to(dev)
    kc = torch.randn(N, chunk, Hkv, d, generator=gen).to(dtype).to(dev)
    vc = torch.randn(N, chunk, Hkv, d, generator=gen).to(dtype).to(dev)
    return q, kc, vc, cu_q.to(dev), kv_lens.to(dev), bt.to(dev)


def _check_padded(mi, q, kc, vc, cu_q, lens, bt, tol=2e-2):
    out = mi.ops.paged_prefill_attention(q, kc, vc, cu_q, lens, bt, max_kv_len=int(lens.max()))
    torch.cuda.synchronize()
    T = int(cu_q[-1])
    assert (out[T:] == 0).all(), "padding rows must be zeros"
    ref = oa.paged_varlen_attention(q[:T].cpu(), kc.cpu(), vc.cpu(), cu_q.cpu(), lens.cpu(), bt.cpu())
    got = out[:T].float().cpu()
    assert torch.isfinite(got).all()
    err = (got - ref).abs()
    assert (err <= tol + tol * ref.abs()).all(), f"max err {err.max().item():.4e}"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("chunk", [16, 64, 256])
@pytest.mark.parametrize("Hq,Hkv", [(8, 8), (32, 8), (12, 4), (16, 1)])
@pytest.mark.parametrize("d", [96, 192, 256])
def test_head_widths_96_192_256(mi, dev, d, Hq, Hkv, chunk, dtype):
    """Head widths beside 64 and 128 in prefill and mixed batches (the two-phase tile kernel when the chunk size
    allows -- 16 rows per wavefront at 192 and 256, 32-key tiles at 256 -- split keys, the lock-step schedule and the
    register-only kernel included): ragged new-token counts and contexts, one-row requests through the decode
    kernels, padding rows."""
    q, kc, vc, cu_q, lens, bt = _ragged_case(mi, dev, Hq, Hkv, d, chunk, dtype, seed=d + Hq + chunk, pad_rows=3)
    _check_padded(mi, q, kc, vc, cu_q, lens, bt)
    if chunk % 64 == 0:
        for knobs in ({"prefill_kv_split": 3}, {"prefill_two_phase": 2}, {"prefill_two_phase": -1}):
            with mi.ops.tuning(**knobs):
                _check_padded(mi, q, kc, vc, cu_q, lens, bt)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("kernel", ["two_phase", "two_phase_staggered", "registers", "split_keys", "split_keys_staggered"])
@pytest.mark.parametrize("d", [64, 96, 128, 192, 256])
def test_scores_that_keep_growing_along_the_context(mi, dev, d, kernel, dtype):
    """Keys grow with their position (x52 at token 1 020), so a row's largest score moves up by far more than any
    window a kernel takes its exponentials within (2^8 for fp16 operands, 2^30 for bf16), tile after tile; rows
    whose query points the other way see it fall instead."""
    knobs = {"two_phase": {}, "two_phase_staggered": {"prefill_two_phase": 1}, "registers": {"prefill_two_phase": -1},
             "split_keys": {"prefill_kv_split": 3},
             "split_keys_staggered": {"prefill_kv_split": 3, "prefill_two_phase": 1}}[kernel]
    chunk = 64
    q, kc, vc, cu_q, lens, bt = _ragged_case(mi, dev, 16, 4, d, chunk, dtype, seed=700 + d)
    pos = torch.arange(chunk, device=dev)
    kf = kc.float()
    for r in range(bt.size(0)):
        for ci in range((int(lens[r]) + chunk - 1) // chunk):
            kf[int(bt[r, ci])] *= (1 + 0.05 * (ci * chunk + pos)).view(-1, 1, 1)
    kc = kf.to(dtype)
    with mi.ops.tuning(**knobs):
        _check(mi, q, kc, vc, cu_q, lens, bt)


@pytest.mark.parametrize("kernel", ["two_phase", "registers", "split_keys"])
@pytest.mark.parametrize("Hq,Hkv", [(32, 1), (64, 2), (17, 1), (48, 2), (40, 2), (64, 1)])
@pytest.mark.parametrize("d", [64, 96, 128, 192, 256])
def test_more_than_16_query_heads_per_kv_head(mi, dev, kernel, Hq, Hkv, d):
    """Up to 64 query heads per KV head: every 16 of them (the last group: the rest) take workgroups of their own."""
    knobs = {"two_phase": {}, "registers": {"prefill_two_phase": -1}, "split_keys": {"prefill_kv_split": 3}}[kernel]
    q, kc, vc, cu_q, lens, bt = _ragged_case(mi, dev, Hq, Hkv, d, 64, torch.bfloat16, seed=Hq + d, pad_rows=2)
    with mi.ops.tuning(**knobs):
        _check_padded(mi, q, kc, vc, cu_q, lens, bt)


def test_stale_cache_rows_beyond_the_length_do_not_leak(mi, dev):
    """Slots past a request's last token may hold anything (NaN patterns included): the staged tiles
    re-read the last valid row instead of them."""
    q, kc, vc, cu_q, lens, bt = mi.synthetic.make_prefill_case(
        dev, n_prefill=3, new_tokens=70, ctx_lo=3, ctx_hi=200, n_decode=0, dec_lo=1, dec_hi=2,
        Hq=16, Hkv=4, d=128, chunk=64, seed=11)
    ref = mi.ops.paged_prefill_attention(q, kc, vc, cu_q, lens, bt).clone()
    kc2, vc2 = kc.clone(), vc.clone()
    lens_h, bt_h = lens.cpu(), bt.cpu()
    for r in range(lens.numel()):
        L = int(lens_h[r])
        ci, off = divmod(L, 64)
        if off:  # poison the unused tail of the last chunk
            pc = int(bt_h[r, ci])
            kc2[pc, off:] = float("nan")
            vc2[pc, off:] = float("nan")
    out = mi.ops.paged_prefill_attention(q, kc2, vc2, cu_q, lens, bt)
    torch.cuda.synchronize()
    assert torch.equal(out, ref)


@pytest.mark.parametrize("d", [128, 96, 192, 256])
def test_chunked_prefill_is_consistent_at_full_size(mi, dev, d):
    """Size-independent property on the cfg3-sized prompts (8 x 2048 tokens over U[0,4096] cached), at head_dim 128
    and at the widths whose tile kernel has a shape of its own (96: 208-byte rows; 192 / 256: 16 rows per wavefront,
    32-key tiles at 256):
    the rows of the second half of every prompt, computed with the first half already counted as
    cached context, equal the same rows of the single full call bit for bit (same tiles, same order),
    and the block table can be permuted without changing a bit.  The last 48 rows of the first and the last
    prompt are also checked against the fp32 checker."""
    q, kc, vc, cu_q, lens, bt = mi.synthetic.make_prefill_case(
        dev, n_prefill=8, new_tokens=2048, ctx_lo=0, ctx_hi=4096, n_decode=0, dec_lo=1, dec_hi=2,
        Hq=32, Hkv=8, d=d, chunk=256, seed=1003 + d, on_device_rng=True)
    full = mi.ops.paged_prefill_attention(q, kc, vc, cu_q, lens, bt, max_kv_len=int(lens.max()))
    torch.cuda.synchronize()
    assert torch.isfinite(full).all()
    for r in (0, 7):
        # the request's chunks alone, compacted, so that only a few megabytes travel to the host
        L = int(lens[r])
        nch = (L + 255) // 256
        ids = bt[r, :nch].long()
        end = int(cu_q[r + 1])
        ref = oa.paged_varlen_attention(q[end - 48:end].cpu(), kc[ids].cpu(), vc[ids].cpu(),
                                        torch.tensor([0, 48], dtype=torch.int32), torch.tensor([L], dtype=torch.int32),
                                        torch.arange(nch, dtype=torch.int32)[None])
        err = (full[end - 48:end].float().cpu() - ref).abs()
        assert (err <= 2e-2 + 2e-2 * ref.abs()).all(), f"request {r}: max err {err.max().item():.3e}"
    # second halves only: 1024 new tokens per request, same kv lengths
    rows = torch.cat([torch.arange(int(cu_q[r]) + 1024, int(cu_q[r + 1]), device=dev) for r in range(8)])
    cu_half = torch.arange(0, 8 * 1024 + 1, 1024, dtype=torch.int32, device=dev)
    half = mi.ops.paged_prefill_attention(q[rows].contiguous(), kc, vc, cu_half, lens, bt, max_kv_len=int(lens.max()))
    torch.cuda.synchronize()
    assert torch.equal(half, full[rows])
    # move every chunk to another physical slot
    N = kc.size(0)
    perm = torch.randperm(N, generator=torch.Generator().manual_seed(5)).to(dev)
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(N, device=dev)
    kc_p, vc_p = kc[perm], vc[perm]          # chunk i of the new pool is old chunk perm[i]
    bt_p = inv[bt.long().clamp(min=0)].to(torch.int32)
    moved = mi.ops.paged_prefill_attention(q, kc_p, vc_p, cu_q, lens, bt_p, max_kv_len=int(lens.max()))
    torch.cuda.synchronize()
    assert torch.equal(moved, full)


@pytest.mark.parametrize("d", [128, 64])
@pytest.mark.parametrize("forced", [0, 2, 7, 64])
def test_few_rows_over_long_contexts_split_the_keys(mi, dev, forced, d):
    """A chunk of a prompt (or a short turn) over a long cached context: the tile kernel cuts the keys of
    every request into ranges (automatic = knob 0, or a forced count), writes partials and merges them.
    Requests shorter than the number of ranges get empty ranges; one-token requests go the decode way."""
    q_lens = [96, 1, 40, 1, 7]
    ctx = [9000, 4000, 130, 0, 63]
    Hq, Hkv, chunk = 32, 8, 64
    kv_lens = torch.tensor([a + b for a, b in zip(q_lens, ctx)], dtype=torch.int32)
    cu_q = torch.zeros(len(q_lens) + 1, dtype=torch.int32)
    cu_q[1:] = torch.cumsum(torch.tensor(q_lens), 0)
    gen = torch.Generator().manual_seed(31)
    bt, N = mi.synthetic.build_block_table(kv_lens, chunk, gen)
    q = torch.randn(int(cu_q[-1]), Hq, d, generator=gen).bfloat16().to(dev)
    kc = torch.randn(N, chunk, Hkv, d, generator=gen).bfloat16().to(dev)
    vc = torch.randn(N, chunk, Hkv, d, generator=gen).bfloat16().to(dev)
    mi.ops.set_tuning("prefill_kv_split", forced)
    try:
        _check(mi, q, kc, vc, cu_q.to(dev), kv_lens.to(dev), bt.to(dev))
        split = mi.ops.paged_prefill_attention(q, kc, vc, cu_q.to(dev), kv_lens.to(dev), bt.to(dev),
                                               max_kv_len=int(kv_lens.max()))
        mi.ops.set_tuning("prefill_kv_split", -1)
        whole = mi.ops.paged_prefill_attention(q, kc, vc, cu_q.to(dev), kv_lens.to(dev), bt.to(dev),
                                               max_kv_len=int(kv_lens.max()))
        torch.cuda.synchronize()
        assert (split.float() - whole.float()).abs().max().item() <= 1e-2   # same arithmetic, another summation order
    finally:
        mi.ops.set_tuning("prefill_kv_split", 0)


def test_split_keys_with_padding_rows_and_fp8(mi, dev):
    """Padding rows behind the last request stay zero; the fp8 cache takes the same split path."""
    q_lens, ctx = [50, 3], [5000, 2000]
    Hq, Hkv, d, chunk = 16, 2, 128, 128
    kv_lens = torch.tensor([a + b for a, b in zip(q_lens, ctx)], dtype=torch.int32)
    cu_q = torch.tensor([0, 50, 53], dtype=torch.int32)
    gen = torch.Generator().manual_seed(32)
    bt, N = mi.synthetic.build_block_table(kv_lens, chunk, gen)
    T = 53 + 11                                                   # 11 padding rows
    q = torch.randn(T, Hq, d, generator=gen).bfloat16().to(dev)
    kc = (torch.randn(N, chunk, Hkv, d, generator=gen) * 0.7).bfloat16().to(dev)
    vc = (torch.randn(N, chunk, Hkv, d, generator=gen) * 0.7).bfloat16().to(dev)
    out = mi.ops.paged_prefill_attention(q, kc, vc, cu_q.to(dev), kv_lens.to(dev), bt.to(dev), max_kv_len=int(kv_lens.max()))
    torch.cuda.synchronize()
    assert (out[53:] == 0).all()
    ref = oa.paged_varlen_attention(q[:53].cpu(), kc.cpu(), vc.cpu(), cu_q, kv_lens, bt)
    err = (out[:53].float().cpu() - ref).abs()
    assert (err <= 2e-2 + 2e-2 * ref.abs()).all()
    k8 = torch.empty(kc.shape, dtype=torch.uint8, device=dev)
    v8 = torch.empty_like(k8)
    ks = torch.empty(N, Hkv, dtype=torch.float32, device=dev)
    vs = torch.empty_like(ks)
    mi.ops.quantize_chunks_fp8(kc, k8, ks)
    mi.ops.quantize_chunks_fp8(vc, v8, vs)
    out8 = mi.ops.paged_prefill_attention(q, k8, v8, cu_q.to(dev), kv_lens.to(dev), bt.to(dev), max_kv_len=int(kv_lens.max()),
                                          k_scales=ks, v_scales=vs)
    torch.cuda.synchronize()
    ref8 = oa.paged_varlen_attention(q[:53].cpu(), k8.cpu(), v8.cpu(), cu_q, kv_lens, bt, k_scales=ks.cpu(), v_scales=vs.cpu())
    err8 = (out8[:53].float().cpu() - ref8).abs()
    assert (err8 <= 2.5e-2 + 2.5e-2 * ref8.abs()).all() and (out8[53:] == 0).all()


@pytest.mark.parametrize("kernel", ["two_phase", "two_phase_staggered", "two_phase_no_offset", "registers", "registers_64_rows", "split_keys"])
@pytest.mark.parametrize("Hq,Hkv", [(12, 4), (10, 2), (28, 4), (6, 1), (12, 1), (15, 1)])
@pytest.mark.parametrize("d", [128, 64])
def test_query_head_groups_that_are_not_powers_of_two(mi, dev, kernel, Hq, Hkv, d):
    """3, 5, 6, 7, 12 or 15 query heads per KV head (Llama-3.2-3B, Qwen2.5-14B, Qwen2-7B ... have such groups):
    a wavefront's 32 (64) rows then hold as many whole tokens as fit, the rest are padding rows.  Every
    prefill kernel, lengths either side of the per-workgroup token counts (48 tokens at a group of 5)."""
    knobs = {"two_phase": {}, "two_phase_staggered": {"prefill_two_phase": 1}, "two_phase_no_offset": {"prefill_two_phase": 2},
             "registers": {"prefill_two_phase": -1},
             "registers_64_rows": {"prefill_two_phase": -1, "prefill_row_tiles": 4},
             "split_keys": {"prefill_kv_split": 3}}[kernel]
    G = Hq // Hkv
    per_wg = 8 * (32 // G)
    q_lens = [1, per_wg - 1, per_wg, per_wg + 1, 2 * per_wg + 3, 1, 301, 5]
    ctx = [300, 0, 64, 7, 500, 0, 129, 1000]
    kv_lens = torch.tensor([a + b for a, b in zip(q_lens, ctx)], dtype=torch.int32)
    cu_q = torch.zeros(len(q_lens) + 1, dtype=torch.int32)
    cu_q[1:] = torch.cumsum(torch.tensor(q_lens), 0)
    gen = torch.Generator().manual_seed(Hq * 100 + Hkv + d)
    bt, N = mi.synthetic.build_block_table(kv_lens, 64, gen)
    q = torch.randn(int(cu_q[-1]) + 3, Hq, d, generator=gen).bfloat16().to(dev)   # three padding rows
    kc = torch.randn(N, 64, Hkv, d, generator=gen).bfloat16().to(dev)
    vc = torch.randn(N, 64, Hkv, d, generator=gen).bfloat16().to(dev)
    with mi.ops.tuning(**knobs):
        out = mi.ops.paged_prefill_attention(q, kc, vc, cu_q.to(dev), kv_lens.to(dev), bt.to(dev), max_kv_len=int(kv_lens.max()))
        torch.cuda.synchronize()
    T = int(cu_q[-1])
    ref = oa.paged_varlen_attention(q[:T].cpu(), kc.cpu(), vc.cpu(), cu_q, kv_lens, bt)
    got = out.float().cpu()
    assert torch.isfinite(got).all() and (got[T:] == 0).all()
    err = (got[:T] - ref).abs()
    assert (err <= 2e-2 + 2e-2 * ref.abs()).all(), f"max err {err.max().item():.4e}"


@pytest.mark.parametrize("fault", ["short", "misaligned"])
def test_a_bad_workspace_is_refused_before_anything_is_launched(mi, dev, fault):
    """A mixed batch hands its one-row requests to the decode kernels after the tile kernel; a workspace those cannot
    use must be refused before the tile kernel is enqueued (a negative return = nothing launched)."""
    lib = mi._lib.load()
    q, kc, vc, cu_q, lens, bt = mi.synthetic.make_prefill_case(
        dev, n_prefill=2, new_tokens=100, ctx_lo=0, ctx_hi=200, n_decode=4, dec_lo=1, dec_hi=500,
        Hq=32, Hkv=8, d=128, chunk=64, seed=5)
    T, R = q.shape[0], lens.numel()
    need = lib.mi_prefill_workspace_bytes(T, R, 32, 8, 128, int(lens.max()), 0, None)
    buf = torch.empty(need + 64, dtype=torch.uint8, device=dev)
    ws_ptr, ws_bytes = (buf.data_ptr(), 1024) if fault == "short" else (buf.data_ptr() + 4, need)
    out = torch.full_like(q, float("nan"))
    ks = kc.stride()
    rc = lib.mi_paged_prefill_attention(
        q.data_ptr(), q.stride(0), q.stride(1), kc.data_ptr(), vc.data_ptr(), ks[0], ks[1], ks[2], bt.data_ptr(),
        bt.stride(0), cu_q.data_ptr(), lens.data_ptr(), out.data_ptr(), out.stride(0), out.stride(1), ws_ptr, ws_bytes,
        T, R, 32, 8, 128, 64, int(lens.max()), 0, 128 ** -0.5, 0, None, None)
    torch.cuda.synchronize()
    assert rc < 0 and b"workspace" in lib.mi_last_error()
    assert torch.isnan(out.float()).all(), "rows were written although the call was refused"


@pytest.mark.parametrize("R", [64, 65, 150, 4096, 4097, 4200])
@pytest.mark.parametrize("kernel", [1, 3])
def test_batches_of_many_requests(mi, dev, R, kernel):
    """More requests than a wavefront has lanes: a workgroup of the one-stream tile kernel finds its request in
    passes of 64 candidates (one pass up to 64 requests, two up to 4 096, three beyond), the two-phase kernel by bisection;
    every request has a few new tokens behind a short context."""
    gen = torch.Generator().manual_seed(R)
    q_lens = torch.randint(2, 7, (R,), generator=gen)
    ctx = torch.randint(0, 71, (R,), generator=gen)
    Hq, Hkv, d, chunk = 8, 2, 128, 64
    kv_lens = (q_lens + ctx).to(torch.int32)
    cu_q = torch.zeros(R + 1, dtype=torch.int32)
    cu_q[1:] = torch.cumsum(q_lens, 0)
    bt, N = mi.synthetic.build_block_table(kv_lens, chunk, gen)
    q = torch.randn(int(cu_q[-1]), Hq, d, generator=gen).bfloat16().to(dev)
    kc = torch.randn(N, chunk, Hkv, d, generator=gen).bfloat16().to(dev)
    vc = torch.randn(N, chunk, Hkv, d, generator=gen).bfloat16().to(dev)
    with mi.ops.tuning(prefill_two_phase=kernel):
        _check(mi, q, kc, vc, cu_q.to(dev), kv_lens.to(dev), bt.to(dev))
