"""GPU parity at the FULL size of the benchmark configurations 3, 4 and 5 (configuration 2 has its own in
tests/test_gpu_decode_attention.py).

The CPU checker cannot run these sizes in seconds, so each test combines
  * a size-independent property over the whole batch: the result does not depend on how the flattened tile
    sequence is cut into workgroup spans (split + log-sum-exp merge == single pass), and
  * the fp32 checker on a few sampled rows, whose chunks are copied to the CPU and renumbered (the checker then
    sees a small cache with the same logical contents).
Tolerance: 2e-2 abs/rel for a bf16 cache, 6e-2 for an fp8 cache against the unquantised values.
A test is skipped only when the device has too little free memory for its pool.
"""
import pytest
import torch

from oracle import paged_attention as oa

pytestmark = pytest.mark.gpu


def _need_free(gib):
    free, _ = torch.cuda.mem_get_info()
    if free < gib * 2**30:
        pytest.skip(f"needs {gib} GiB of free device memory")


def _close(got, ref, tol, what=""):
    got = got.float().cpu().reshape(ref.shape)
    assert torch.isfinite(got).all(), f"{what}: non-finite output"
    err = (got - ref).abs()
    assert (err <= tol + tol * ref.abs()).all(), f"{what}: max err {err.max().item():.4e} exceeds {tol} abs/rel"


def _compact(table_rows, n_pool, *tensors):
    """Chunks the given block-table rows use, copied to the CPU and renumbered 0..n-1: returns the remapped rows
    and, per tensor (indexed by chunk in dimension 0), its used slices on the CPU."""
    rows = table_rows.cpu()
    used = rows[rows >= 0].unique().long()
    remap = torch.full((n_pool,), -1, dtype=torch.int32)
    remap[used] = torch.arange(used.numel(), dtype=torch.int32)
    new_rows = torch.where(rows >= 0, remap[rows.clamp(min=0).long()], rows)
    return new_rows, [t[used.to(t.device)].cpu() for t in tensors]


def _span_variants(mi, run, base, bound):
    """The same call with other ways of cutting the tile sequence: minimum span, forced grid sizes."""
    for split, grid in ((4096, 0), (0, 64), (0, 1000), (1 << 20, 4096)):
        mi.ops.set_tuning("decode_grid", grid)
        try:
            other = run(split).float()
        finally:
            mi.ops.set_tuning("decode_grid", 0)
        diff = (base - other).abs().max().item()
        assert diff < bound, f"split_tokens {split}, grid {grid}: differs from the default cut by {diff:.3e}"


def test_cfg4_long_context_full_size(mi, dev):
    """Batch 16, 64 query / 8 KV heads, head_dim 128, 131 072 tokens each (8 GiB of keys and values)."""
    _need_free(20)
    case = mi.synthetic.make_decode_case(mi.synthetic.CONFIGS["cfg4"], dev, on_device_rng=True)
    assert case.q.size(0) == 16 and int(case.kv_lens.min()) == 131072

    def run(split):
        out = mi.ops.paged_decode_attention(case.q, case.k_cache, case.v_cache, case.kv_lens, case.block_table,
                                            split_tokens=split, max_kv_len=131072)
        torch.cuda.synchronize()
        return out

    base = run(0).float()
    _span_variants(mi, run, base, 5e-3)
    for r in (0, 7, 15):  # one request at a time: 512 chunks = 1 GiB of fp32 on the host
        rows, (kc, vc) = _compact(case.block_table[r:r + 1], case.k_cache.size(0), case.k_cache, case.v_cache)
        ref = oa.paged_decode_attention(case.q[r:r + 1].cpu().squeeze(1), kc, vc, case.kv_lens[r:r + 1].cpu(), rows)
        _close(base[r:r + 1], ref, 2e-2, f"cfg4 row {r}")


def test_cfg5_fp8_cache_full_size(mi, dev):
    """Batch 256, 32 / 8 heads, head_dim 128, contexts U[1024, 32768] over an fp8-e4m3 cache with one fp32
    scale per (chunk, KV head): quantiser bytes of sampled chunks equal the checker's, attention within 6e-2 of the
    fp32 checker on the unquantised values and 2e-2 on the dequantised ones."""
    _need_free(40)
    cfg = mi.synthetic.CONFIGS["cfg5"]
    case = mi.synthetic.make_decode_case(cfg, dev, on_device_rng=True)
    assert case.q.size(0) == 256 and int(case.kv_lens.max()) > 30000
    N = case.k_cache.size(0)
    k8 = torch.empty(case.k_cache.shape, dtype=torch.uint8, device=dev)
    v8 = torch.empty_like(k8)
    ks = torch.empty(N, cfg.Hkv, dtype=torch.float32, device=dev)
    vs = torch.empty_like(ks)
    mi.ops.quantize_chunks_fp8(case.k_cache, k8, ks)
    mi.ops.quantize_chunks_fp8(case.v_cache, v8, vs)
    torch.cuda.synchronize()
    mx = int(case.kv_lens.max())

    def run(split):
        out = mi.ops.paged_decode_attention(case.q, k8, v8, case.kv_lens, case.block_table, split_tokens=split,
                                            max_kv_len=mx, k_scales=ks, v_scales=vs)
        torch.cuda.synchronize()
        return out

    base = run(0).float()
    _span_variants(mi, run, base, 8e-3)
    lens = case.kv_lens.cpu()
    sample = sorted({0, 255, int(lens.argmax()), int(lens.argmin())})
    for r in sample:
        rows, (kc, vc, kq, vq, ksc, vsc) = _compact(case.block_table[r:r + 1], N, case.k_cache, case.v_cache,
                                                    k8, v8, ks, vs)
        kq_ref, ks_ref = oa.quantize_chunks_fp8(kc)
        vq_ref, vs_ref = oa.quantize_chunks_fp8(vc)
        assert torch.equal(ksc, ks_ref) and torch.equal(vsc, vs_ref), f"row {r}: scales differ from the checker's"
        assert torch.equal(kq, kq_ref) and torch.equal(vq, vq_ref), f"row {r}: e4m3 bytes differ from the checker's"
        q = case.q[r:r + 1].cpu().squeeze(1)
        ref_unq = oa.paged_decode_attention(q, kc, vc, lens[r:r + 1], rows)
        ref_deq = oa.paged_decode_attention(q, kq, vq, lens[r:r + 1], rows, k_scales=ksc, v_scales=vsc)
        _close(base[r:r + 1], ref_unq, 6e-2, f"cfg5 row {r} vs unquantised")
        _close(base[r:r + 1], ref_deq, 2e-2, f"cfg5 row {r} vs dequantised")


def test_cfg3_mixed_batch_full_size(mi, dev):
    """The one varlen call of configuration 3: 8 prefill requests of 2048 new tokens over U[0, 4096] cached ones
    plus 120 one-token requests with U[512, 8192] tokens, 32 / 8 heads, head_dim 128, chunk 256.
    Decode rows: equal to the decode entry point on the same 120 requests (the same streaming kernel cut into other
    spans) and, for three of them, to the checker.  Prefill rows: the last 64 rows of two prompts against the
    checker (rows Lq-64 .. Lq-1 of a request are a request of 64 new tokens over the same keys)."""
    _need_free(12)
    Hq, Hkv, d, chunk = 32, 8, 128, 256
    q, kc, vc, cu_q, lens, bt = mi.synthetic.make_prefill_case(
        dev, n_prefill=8, new_tokens=2048, ctx_lo=0, ctx_hi=4096, n_decode=120, dec_lo=512, dec_hi=8192,
        Hq=Hq, Hkv=Hkv, d=d, chunk=chunk, seed=1003, on_device_rng=True)
    assert q.size(0) == 8 * 2048 + 120 and lens.numel() == 128
    mx = int(lens.max())
    out = mi.ops.paged_prefill_attention(q, kc, vc, cu_q, lens, bt, max_kv_len=mx)
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all()

    # the 120 one-token requests through the decode entry point
    dec_rows = cu_q[8:128].long()
    dec = mi.ops.paged_decode_attention(q[dec_rows].unsqueeze(1).contiguous(), kc, vc, lens[8:].contiguous(),
                                        bt[8:].contiguous(), max_kv_len=mx)
    torch.cuda.synchronize()
    diff = (out[dec_rows].float() - dec.squeeze(1).float()).abs().max().item()
    assert diff < 8e-3, f"decode rows of the mixed call differ from the decode entry point by {diff:.3e}"
    for r in (8, 60, 127):
        rows, (kcc, vcc) = _compact(bt[r:r + 1], kc.size(0), kc, vc)
        row = int(cu_q[r])
        ref = oa.paged_decode_attention(q[row:row + 1].cpu(), kcc, vcc, lens[r:r + 1].cpu(), rows)
        _close(out[row:row + 1], ref, 2e-2, f"cfg3 decode request {r}")

    # the last 64 rows of two prompts (the shortest and the longest cached context)
    ctx = (lens[:8] - 2048).cpu()
    for r in sorted({int(ctx.argmin()), int(ctx.argmax())}):
        rows, (kcc, vcc) = _compact(bt[r:r + 1], kc.size(0), kc, vc)
        b = int(cu_q[r + 1])
        ref = oa.paged_varlen_attention(q[b - 64:b].cpu(), kcc, vcc, torch.tensor([0, 64], dtype=torch.int32),
                                        lens[r:r + 1].cpu(), rows)
        _close(out[b - 64:b], ref, 2e-2, f"cfg3 prompt {r}, last 64 rows")
    # and the first 64 rows of one prompt: a request of 64 new tokens over the cached context alone
    r = 3
    a = int(cu_q[r])
    rows, (kcc, vcc) = _compact(bt[r:r + 1], kc.size(0), kc, vc)
    ref = oa.paged_varlen_attention(q[a:a + 64].cpu(), kcc, vcc, torch.tensor([0, 64], dtype=torch.int32),
                                    (lens[r:r + 1] - 2048 + 64).cpu(), rows)
    _close(out[a:a + 64], ref, 2e-2, f"cfg3 prompt {r}, first 64 rows")


@pytest.mark.parametrize("name,need", [("cfg2", 6), ("cfg4", 24)])
def test_one_kernel_decode_step_full_size(mi, dev, name, need):
    """The benchmark's default step at full size (configuration 2: batch 64, U[512, 8192]; configuration 4: batch 16
    x 131 072): RMSNorm + RoPE + append + attention in the streaming kernel against the separate launches -- the
    appended cache rows bit for bit, the outputs within 8e-3 -- and three sampled rows against the checker's chain."""
    from oracle import rope_norm as orn
    _need_free(need)
    cfg = mi.synthetic.CONFIGS[name]
    case = mi.synthetic.make_decode_case(cfg, dev, on_device_rng=True)
    R, d = case.q.size(0), cfg.d
    mx = int(case.kv_lens.max())
    gen = torch.Generator().manual_seed(11)
    qw = (1 + 0.02 * torch.randn(d, generator=gen)).bfloat16()
    kw = (1 + 0.02 * torch.randn(d, generator=gen)).bfloat16()
    table = mi.synthetic.rotary_angle_table(mx + 1, d, base=500000.0)
    pos = (case.kv_lens.long() - 1).contiguous()
    common = dict(q_weight=qw.to(dev), k_weight=kw.to(dev), eps=1e-5, norm="rms", rotary_emb=table.to(dev))
    # where the step's token lands: the caches are too large to clone, so the appended rows are compared by slot
    lens_h, bt_h = case.kv_lens.cpu().long(), case.block_table.cpu().long()
    slot_chunk = bt_h[torch.arange(R), (lens_h - 1) // cfg.chunk].to(dev)
    slot_pos = ((lens_h - 1) % cfg.chunk).to(dev)

    out_a = mi.ops.decode_step_attention(case.q, case.k_new, case.v_new, case.k_cache, case.v_cache, case.kv_lens,
                                         case.block_table, positions=None, max_kv_len=mx, **common)
    torch.cuda.synchronize()
    k_rows_a = case.k_cache[slot_chunk, slot_pos].clone()
    v_rows_a = case.v_cache[slot_chunk, slot_pos].clone()
    case.k_cache[slot_chunk, slot_pos] = 0   # make sure the second path writes them again
    case.v_cache[slot_chunk, slot_pos] = 0
    q_b = torch.empty_like(case.q)
    with mi.ops.tuning(norm_rope_vectorised=-1):
        mi.ops.norm_rope_append(case.q, case.k_new, value=case.v_new, query_out=q_b, q_positions=pos, k_positions=pos,
                                k_cache=case.k_cache, v_cache=case.v_cache, block_table=case.block_table,
                                kv_lens=case.kv_lens, **common)
    out_b = mi.ops.paged_decode_attention(q_b, case.k_cache, case.v_cache, case.kv_lens, case.block_table, max_kv_len=mx)
    torch.cuda.synchronize()
    assert torch.equal(case.k_cache[slot_chunk, slot_pos], k_rows_a), "appended key rows differ from the separate launch"
    assert torch.equal(case.v_cache[slot_chunk, slot_pos], v_rows_a)
    assert torch.equal(v_rows_a, case.v_new.squeeze(1))
    diff = (out_a.float() - out_b.float()).abs().max().item()
    assert diff <= 8e-3, f"one-kernel step and separate launches differ by {diff:.3e}"
    for r in (0, R // 2, R - 1):
        rows, (kc, vc) = _compact(case.block_table[r:r + 1], case.k_cache.size(0), case.k_cache, case.v_cache)
        q_ref = orn.norm_rope(case.q[r:r + 1].cpu().squeeze(1), pos[r:r + 1].cpu(), table, norm="rms", weight=qw, eps=1e-5)
        ref = oa.paged_decode_attention(q_ref, kc, vc, case.kv_lens[r:r + 1].cpu(), rows)
        _close(out_a[r:r + 1], ref, 2e-2, f"{name} row {r}")


def test_one_kernel_decode_step_over_the_fp8_cache_full_size(mi, dev):
    """Configuration 5 at full size (batch 256, U[1024, 32768], fp8-e4m3 cache): the one-kernel decode step --
    RMSNorm + RoPE + quantising append + attention -- against the separate launches: the appended bytes and every
    scale bit for bit, the outputs within 8e-3."""
    _need_free(40)
    cfg = mi.synthetic.CONFIGS["cfg5"]
    case = mi.synthetic.make_decode_case(cfg, dev, on_device_rng=True)
    R, d = case.q.size(0), cfg.d
    N = case.k_cache.size(0)
    k8 = torch.empty(case.k_cache.shape, dtype=torch.uint8, device=dev)
    v8 = torch.empty_like(k8)
    ks = torch.empty(N, cfg.Hkv, dtype=torch.float32, device=dev)
    vs = torch.empty_like(ks)
    mi.ops.quantize_chunks_fp8(case.k_cache, k8, ks)
    mi.ops.quantize_chunks_fp8(case.v_cache, v8, vs)
    del case.k_cache, case.v_cache
    torch.cuda.empty_cache()
    # a few requests whose step token opens a chunk: shorten them to one token past a chunk boundary
    lens = case.kv_lens.clone()
    lens[::37] = (lens[::37] // cfg.chunk) * cfg.chunk + 1
    mx = int(lens.max())
    gen = torch.Generator().manual_seed(12)
    qw = (1 + 0.02 * torch.randn(d, generator=gen)).bfloat16().to(dev)
    kw = (1 + 0.02 * torch.randn(d, generator=gen)).bfloat16().to(dev)
    table = mi.synthetic.rotary_angle_table(mx + 1, d, base=500000.0).to(dev)
    pos = (lens.long() - 1).contiguous()
    common = dict(q_weight=qw, k_weight=kw, eps=1e-5, norm="rms", rotary_emb=table)
    lens_h, bt_h = lens.cpu().long(), case.block_table.cpu().long()
    slot_chunk = bt_h[torch.arange(R), (lens_h - 1) // cfg.chunk].to(dev)
    slot_pos = ((lens_h - 1) % cfg.chunk).to(dev)
    ks0, vs0 = ks.clone(), vs.clone()

    out_a = mi.ops.decode_step_attention(case.q, case.k_new, case.v_new, k8, v8, lens, case.block_table,
                                         positions=None, max_kv_len=mx, k_scales=ks, v_scales=vs, headroom=2.0, **common)
    torch.cuda.synchronize()
    k_rows_a, v_rows_a = k8[slot_chunk, slot_pos].clone(), v8[slot_chunk, slot_pos].clone()
    ks_a, vs_a = ks.clone(), vs.clone()
    assert not torch.equal(ks_a, ks0), "no token opened a chunk: the case does not test the scale path"
    k8[slot_chunk, slot_pos] = 0
    v8[slot_chunk, slot_pos] = 0
    ks.copy_(ks0); vs.copy_(vs0)
    q_b, k_b = torch.empty_like(case.q), torch.empty_like(case.k_new)
    with mi.ops.tuning(norm_rope_vectorised=-1):
        mi.ops.norm_rope_append(case.q, case.k_new, query_out=q_b, key_out=k_b, q_positions=pos, k_positions=pos, **common)
    mi.ops.kv_append_decode_fp8(k_b, case.v_new, k8, v8, ks, vs, case.block_table, lens, headroom=2.0)
    out_b = mi.ops.paged_decode_attention(q_b, k8, v8, lens, case.block_table, max_kv_len=mx, k_scales=ks, v_scales=vs)
    torch.cuda.synchronize()
    assert torch.equal(k8[slot_chunk, slot_pos], k_rows_a) and torch.equal(v8[slot_chunk, slot_pos], v_rows_a), \
        "appended bytes differ from the separate launches"
    assert torch.equal(ks, ks_a) and torch.equal(vs, vs_a), "scales differ from the separate launches"
    diff = (out_a.float() - out_b.float()).abs().max().item()
    assert diff <= 8e-3, f"one-kernel step and separate launches differ by {diff:.3e}"
