"""GPU parity with fp16 queries, caches and weights (the reference's ``params_dtype`` is fp16 as often as bf16,
dynamic_context.py:195,287-308): every attention and norm / rotary kernel has an fp16 instantiation, selected by
the ``dtype`` argument of its entry point.  The checker is dtype-generic (it lifts its inputs to fp32, and
evaluates the norm / rotary chain op by op in the tensors' type); tolerance 2e-2 abs/rel as for bf16.
The cases mirror the bf16 tests: head groupings, ragged lengths, both prefill kernels, split keys, mixed batches,
multi-latent decode and prefill, the fused append, logits in fp16.
"""
import pytest
import torch

from oracle import paged_attention as oa
from oracle import rope_norm as orn
from oracle import sampling as osm

pytestmark = pytest.mark.gpu
F16 = torch.float16


def _close(got, ref, tol=2e-2, what=""):
    got = got.float().cpu().reshape(ref.shape)
    assert torch.isfinite(got).all(), f"{what}: non-finite output"
    err = (got - ref).abs()
    assert (err <= tol + tol * ref.abs()).all(), f"{what}: max err {err.max().item():.4e}"


@pytest.mark.parametrize("Hq,Hkv", [(8, 8), (32, 8), (64, 8), (6, 2), (16, 1)])
@pytest.mark.parametrize("d", [64, 128])
def test_decode_head_groupings(mi, dev, Hq, Hkv, d):
    cfg = mi.synthetic.DecodeConfig("g16", 5, Hq, Hkv, d, 1, 700, chunk=64, seed=Hq * 131 + Hkv * 7 + d)
    case = mi.synthetic.make_decode_case(cfg, dev, dtype=F16)
    out = mi.ops.paged_decode_attention(case.q, case.k_cache, case.v_cache, case.kv_lens, case.block_table)
    torch.cuda.synchronize()
    assert out.dtype == F16
    ref = oa.paged_decode_attention(case.q.cpu().squeeze(1), case.k_cache.cpu(), case.v_cache.cpu(), case.kv_lens.cpu(),
                                    case.block_table.cpu())
    _close(out, ref, what="decode")


@pytest.mark.parametrize("chunk", [16, 128, 256])
@pytest.mark.parametrize("grid", [0, 1, 7, 4096])
def test_decode_ragged_lengths_splits_and_merge(mi, dev, chunk, grid):
    lens = torch.tensor([0, 1, 2, 15, 16, 17, 31, 32, 33, chunk - 1, chunk, chunk + 1, 2 * chunk, 3 * chunk + 5, 0, 4777],
                        dtype=torch.int32)
    cfg = mi.synthetic.DecodeConfig("edges16", lens.numel(), 8, 2, 128, 0, 0, chunk=chunk, seed=chunk)
    case = mi.synthetic.make_decode_case(cfg, dev, lens=lens, dtype=F16)
    ref = oa.paged_decode_attention(case.q.cpu().squeeze(1), case.k_cache.cpu(), case.v_cache.cpu(), lens,
                                    case.block_table.cpu())
    with mi.ops.tuning(decode_grid=grid):
        for split in (0, 64, 512):
            out = mi.ops.paged_decode_attention(case.q, case.k_cache, case.v_cache, case.kv_lens, case.block_table,
                                                split_tokens=split, max_kv_len=int(lens.max()))
            torch.cuda.synchronize()
            _close(out, ref, what=f"decode split {split}")
            assert (out[case.kv_lens == 0] == 0).all()


def test_decode_cfg2_shape_and_the_no_alloc_entry(mi, dev):
    case = mi.synthetic.make_decode_case(mi.synthetic.CONFIGS["cfg2"], dev, batch=8, dtype=F16)
    out = mi.ops.paged_decode_attention(case.q, case.k_cache, case.v_cache, case.kv_lens, case.block_table)
    out2 = mi.ops.paged_decode_attention_noalloc(case.q, case.k_cache, case.v_cache, case.kv_lens, case.block_table,
                                                 torch.empty_like(case.q))
    torch.cuda.synchronize()
    ref = oa.paged_decode_attention(case.q.cpu().squeeze(1), case.k_cache.cpu(), case.v_cache.cpu(), case.kv_lens.cpu(),
                                    case.block_table.cpu())
    _close(out, ref, what="cfg2 shape")
    assert torch.equal(out, out2)


def test_mismatched_types_are_rejected(mi, dev):
    case = mi.synthetic.make_decode_case(mi.synthetic.DecodeConfig("mm", 2, 8, 2, 128, 10, 100, chunk=64, seed=1), dev, dtype=F16)
    with pytest.raises(ValueError, match="16-bit type"):
        mi.ops.paged_decode_attention(case.q.bfloat16(), case.k_cache, case.v_cache, case.kv_lens, case.block_table)
    with pytest.raises(ValueError, match="bf16 or fp16"):
        mi.ops.paged_decode_attention(case.q.float(), case.k_cache, case.v_cache, case.kv_lens, case.block_table)


@pytest.mark.parametrize("d", [128, 64])
def test_fp16_queries_over_an_fp8_cache(mi, dev, d):
    """fp16 rows quantised to e4m3 (bytes and scales equal to the checker's), then decode attention with fp16
    queries over the bytes: 2e-2 against the checker on the dequantised cache, 6e-2 against the unquantised one."""
    cfg = mi.synthetic.DecodeConfig("fp8h", 6, 32, 8, d, 600, 5000, fp8=True, seed=1007)
    case = mi.synthetic.make_decode_case(cfg, dev, dtype=F16)
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
    assert out.dtype == F16
    ref_q = oa.paged_decode_attention(case.q.cpu().squeeze(1), k8_ref, v8_ref, case.kv_lens.cpu(), case.block_table.cpu(),
                                      k_scales=ks_ref, v_scales=vs_ref)
    _close(out, ref_q, what="fp16 over fp8, dequantised cache")
    ref = oa.paged_decode_attention(case.q.cpu().squeeze(1), case.k_cache.cpu(), case.v_cache.cpu(), case.kv_lens.cpu(),
                                    case.block_table.cpu())
    err = (out.float().cpu().squeeze(1) - ref).abs()
    assert (err <= 6e-2 + 6e-2 * ref.abs()).all()
    # the step's token, appended by the quantising decode append with fp16 rows
    k8a, v8a, ksa, vsa = k8.clone(), v8.clone(), ks.clone(), vs.clone()
    mi.ops.kv_append_decode_fp8(case.k_new, case.v_new, k8a, v8a, ksa, vsa, case.block_table, case.kv_lens, headroom=2.0)
    torch.cuda.synchronize()
    lens, bt = case.kv_lens.cpu(), case.block_table.cpu()
    for r in range(lens.numel()):
        pos = int(lens[r]) - 1
        c, l = int(bt[r, pos // cfg.chunk]), pos % cfg.chunk
        for src, c8, cs in ((case.k_new, k8a, ksa), (case.v_new, v8a, vsa)):
            row = src.cpu()[r].view(cfg.Hkv, d)
            scale = (2.0 * row.float().abs().amax(dim=1) / 448.0) if l == 0 else cs.cpu()[c]
            if l == 0:
                assert torch.equal(cs.cpu()[c], scale)
            assert torch.equal(c8.cpu()[c, l], oa.quantize_token_fp8(row, scale))


@pytest.mark.parametrize("kernel", ["two_phase", "two_phase_staggered", "two_phase_lock_step", "registers", "split_keys"])
@pytest.mark.parametrize("Hq,Hkv,d", [(32, 8, 128), (8, 8, 64), (12, 4, 128), (16, 1, 64), (32, 8, 96)])
def test_prefill_and_mixed_batches(mi, dev, kernel, Hq, Hkv, d):
    knobs = {"two_phase": {}, "two_phase_staggered": {"prefill_two_phase": 1}, "two_phase_lock_step": {"prefill_two_phase": 2},
             "registers": {"prefill_two_phase": -1},
             "split_keys": {"prefill_kv_split": 3}}[kernel]
    q_lens = [1, 2, 15, 16, 17, 63, 64, 65, 128, 200, 1, 97, 500, 256, 257, 3]
    ctx = [700, 5, 0, 16, 31, 0, 100, 1, 0, 333, 0, 40, 7, 64, 63, 1020]
    kv_lens = torch.tensor([a + b for a, b in zip(q_lens, ctx)], dtype=torch.int32)
    cu_q = torch.zeros(len(q_lens) + 1, dtype=torch.int32)
    cu_q[1:] = torch.cumsum(torch.tensor(q_lens), 0)
    gen = torch.Generator().manual_seed(Hq + d)
    bt, N = mi.synthetic.build_block_table(kv_lens, 64, gen)
    q = torch.randn(int(cu_q[-1]) + 2, Hq, d, generator=gen).to(F16)      # two padding rows
    kc = torch.randn(N, 64, Hkv, d, generator=gen).to(F16)
    vc = torch.randn(N, 64, Hkv, d, generator=gen).to(F16)
    with mi.ops.tuning(**knobs):
        out = mi.ops.paged_prefill_attention(q.to(dev), kc.to(dev), vc.to(dev), cu_q.to(dev), kv_lens.to(dev), bt.to(dev),
                                             max_kv_len=int(kv_lens.max()))
        torch.cuda.synchronize()
    T = int(cu_q[-1])
    assert out.dtype == F16 and (out[T:] == 0).all()
    ref = oa.paged_varlen_attention(q[:T], kc, vc, cu_q, kv_lens, bt)
    _close(out[:T], ref, what=f"prefill {kernel}")


@pytest.mark.parametrize("Hq", [8, 16, 64])
@pytest.mark.parametrize("lds", [0, -1])
def test_mla_decode(mi, dev, Hq, lds):
    gen = torch.Generator().manual_seed(Hq)
    lens = torch.tensor([0, 1, 63, 64, 65, 700, 2049, 5000], dtype=torch.int32)
    bt, N = mi.synthetic.build_block_table(lens, 64, gen)
    cache = (torch.randn(N + 1, 64, 576, generator=gen) * 0.5).to(F16)
    q = torch.randn(lens.numel(), 1, Hq, 576, generator=gen).to(F16)
    with mi.ops.tuning(mla_decode_lds=lds):
        out = mi.ops.paged_mla_decode_attention(q.to(dev), cache.to(dev), lens.to(dev), bt.to(dev), softmax_scale=0.07)
        torch.cuda.synchronize()
    ref = oa.mla_decode_attention(q.squeeze(1), cache, lens, bt, 0.07, 512)
    _close(out.squeeze(1), ref, what="mla decode")


@pytest.mark.parametrize("two_phase", [0, -1])
def test_mla_prefill(mi, dev, two_phase):
    H, chunk = 4, 64
    q_lens, ctx = [40, 1, 170, 3], [300, 250, 0, 70]
    kv_lens = torch.tensor([a + b for a, b in zip(q_lens, ctx)], dtype=torch.int32)
    cu_q = torch.zeros(len(q_lens) + 1, dtype=torch.int32)
    cu_q[1:] = torch.cumsum(torch.tensor(q_lens), 0)
    gen = torch.Generator().manual_seed(17)
    bt, N = mi.synthetic.build_block_table(kv_lens, chunk, gen)
    q = torch.randn(int(cu_q[-1]), H, 192, generator=gen).to(F16)
    kc = torch.randn(N, chunk, H, 192, generator=gen).to(F16)
    vc = torch.randn(N, chunk, H, 128, generator=gen).to(F16)
    with mi.ops.tuning(prefill_two_phase=two_phase):
        out = mi.ops.paged_prefill_attention_mla(q.to(dev), kc.to(dev), vc.to(dev), cu_q.to(dev), kv_lens.to(dev),
                                                 bt.to(dev), softmax_scale=0.07)
        torch.cuda.synchronize()
    ref = oa.paged_varlen_attention(q, kc, vc, cu_q, kv_lens, bt, softmax_scale=0.07)
    _close(out, ref, what="mla prefill")


def _ulp_diff_f16(a, b):
    ia, ib = a.view(torch.int16).int(), b.view(torch.int16).int()
    ka = torch.where(ia < 0, -(ia & 0x7FFF), ia)
    kb = torch.where(ib < 0, -(ib & 0x7FFF), ib)
    return (ka - kb).abs()


@pytest.mark.parametrize("norm", [None, "rms", "l2"])
@pytest.mark.parametrize("interleaved", [False, True])
@pytest.mark.parametrize("d,rot", [(128, 128), (64, 64), (128, 64), (128, 40), (96, 96), (192, 64), (256, 256)])
@pytest.mark.parametrize("vectorised", [1, -1])
def test_norm_rope_follows_the_fp16_op_chain(mi, dev, norm, interleaved, d, rot, vectorised):
    """With faithful rounding the kernel rounds to fp16 wherever the unfused fp16 chain does: under 1 % of the
    elements differ at all (the device's rsqrt / cos / sin differ from the host's in the last bit), and those by at
    most 2 ulp of the head vector's largest element -- a rotation whose two products nearly cancel turns one ulp of
    a product into many ulp of the small difference, so the bound is on the operands' scale.  Otherwise 2e-2."""
    gen = torch.Generator().manual_seed(d + rot + (7 if interleaved else 0))
    T, Hq, Hkv = 37, 8, 2
    q = torch.randn(T, 1, Hq, d, generator=gen).to(F16)
    k = torch.randn(T, 1, Hkv, d, generator=gen).to(F16)
    qw = (1 + 0.02 * torch.randn(d, generator=gen)).to(F16)
    kw = (1 + 0.02 * torch.randn(d, generator=gen)).to(F16)
    table = orn.rotary_table(9000, rot, base=500000.0, interleaved=interleaved)
    qpos = torch.randint(0, 9000, (T,), generator=gen)
    kpos = torch.randint(0, 9000, (T,), generator=gen)
    eps = 1e-5 if norm == "rms" else 1e-6
    q_ref = orn.norm_rope(q.squeeze(1), qpos, table, norm=norm, weight=qw if norm == "rms" else None, eps=eps,
                          interleaved=interleaved)
    k_ref = orn.norm_rope(k.squeeze(1), kpos, table, norm=norm, weight=kw if norm == "rms" else None, eps=eps,
                          interleaved=interleaved)
    with mi.ops.tuning(norm_rope_vectorised=vectorised):
        for faithful in (True, False):
            qd, kd = q.to(dev).clone(), k.to(dev)
            k_out = torch.empty_like(kd)
            mi.ops.norm_rope_append(qd, kd, key_out=k_out, q_weight=qw.to(dev), k_weight=kw.to(dev), eps=eps, norm=norm,
                                    rotary_emb=table.to(dev), q_positions=qpos.to(dev), k_positions=kpos.to(dev),
                                    rotary_interleaved=interleaved, faithful_rounding=faithful)
            torch.cuda.synchronize()
            for got, ref in ((qd.cpu().squeeze(1), q_ref), (k_out.cpu().squeeze(1), k_ref)):
                err = (got.float() - ref.float()).abs()
                assert (err <= 2e-2 + 2e-2 * ref.float().abs()).all(), f"max err {err.max().item()}"
                if faithful:
                    assert (_ulp_diff_f16(got, ref) > 0).float().mean().item() < 0.01
                    scale = ref.float().abs().amax(-1, keepdim=True)
                    assert (err <= 2 * 2.0 ** -10 * scale).all()


@pytest.mark.parametrize("mixed", [False, True])
def test_fused_norm_rope_append_then_attention(mi, dev, mixed):
    """One decode step in fp16: fused RMSNorm + RoPE + append (from split tensors or from the QKV projection's
    output), then attention -- value rows land bit for bit, key rows and the output within tolerance."""
    lens = torch.tensor([5, 256, 257, 1000, 0, 31], dtype=torch.int32)
    cfg = mi.synthetic.DecodeConfig("fa16", lens.numel(), 32, 8, 128, 0, 0, seed=4)
    case = mi.synthetic.make_decode_case(cfg, dev, lens=lens, dtype=F16)
    kc0, vc0 = case.k_cache.cpu().clone(), case.v_cache.cpu().clone()
    table = orn.rotary_table(2048, 128, base=500000.0)
    pos = (lens.long() - 1).clamp(min=0)
    gen = torch.Generator().manual_seed(3)
    qw = (1 + 0.02 * torch.randn(128, generator=gen)).to(F16)
    kw = (1 + 0.02 * torch.randn(128, generator=gen)).to(F16)
    R = lens.numel()
    q_out = torch.empty_like(case.q)
    common = dict(q_weight=qw.to(dev), k_weight=kw.to(dev), norm="rms", eps=1e-5, rotary_emb=table.to(dev),
                  q_positions=pos.to(dev), k_positions=pos.to(dev), k_cache=case.k_cache, v_cache=case.v_cache,
                  block_table=case.block_table, kv_lens=case.kv_lens)
    if mixed:
        G = 4
        grouped = torch.cat([case.q.view(R, 8, G * 128), case.k_new.view(R, 8, 128), case.v_new.view(R, 8, 128)], dim=-1)
        mi.ops.qkv_norm_rope_append(grouped.reshape(R, 1, -1).contiguous(), num_query_heads=32, num_kv_heads=8,
                                    query_out=q_out, **common)
    else:
        mi.ops.norm_rope_append(case.q, case.k_new, value=case.v_new, query_out=q_out, **common)
    out = mi.ops.paged_decode_attention(q_out, case.k_cache, case.v_cache, case.kv_lens, case.block_table)
    torch.cuda.synchronize()
    q_ref = orn.norm_rope(case.q.cpu().squeeze(1), pos, table, norm="rms", weight=qw, eps=1e-5)
    k_ref = orn.norm_rope(case.k_new.cpu().squeeze(1), pos, table, norm="rms", weight=kw, eps=1e-5)
    rows, ids, loc = oa.decode_slots(case.block_table.cpu(), lens, cfg.chunk)
    oa.kv_append(kc0, vc0, k_ref[rows], case.v_new.cpu().squeeze(1)[rows], ids, loc)
    dummy = case.k_cache.size(0) - 1
    assert torch.equal(case.v_cache.cpu()[:dummy], vc0[:dummy]), "value append is not bit-exact"
    assert (case.k_cache.cpu()[:dummy].float() - kc0[:dummy].float()).abs().max().item() <= 2e-2
    ref = oa.paged_decode_attention(q_ref, kc0, vc0, lens, case.block_table.cpu())
    _close(out, ref, what="decode step")


def test_fp16_logits_sampling_and_log_probs(mi, dev):
    gen = torch.Generator().manual_seed(8)
    R, V = 9, 5003
    logits = (torch.randn(R, V, generator=gen) * 3).to(F16)
    u = torch.rand(R, generator=gen)
    greedy, _ = mi.ops.sample_from_logits(logits.to(dev), top_k=1)
    assert torch.equal(greedy.cpu(), logits.float().argmax(-1))
    got, _ = mi.ops.sample_from_logits(logits.to(dev), top_k=7, temperature=0.8, uniform=u.to(dev))
    want = osm.sample_from_logits(logits, top_k=7, temperature=0.8, uniform=u)
    assert torch.equal(got.cpu(), want)
    ids = torch.randint(0, V, (R,), generator=gen)
    lp = mi.ops.selected_log_probs(logits.to(dev), ids.to(dev))
    torch.cuda.synchronize()
    ref = torch.log_softmax(logits.double(), -1)[torch.arange(R), ids]
    assert (lp.cpu().double() - ref).abs().max().item() <= 2e-5
