"""GPU parity: the fused decode step (head norm + RoPE + append of the step's token + attention in the streaming
kernel, `mi_decode_step_attention`) against the separate launches and against the CPU checker.

* cache rows: bit-identical to what `mi_norm_rope_append` (element-wise kernel) writes -- same arithmetic, same
  order of the reductions; untouched slots keep their contents;
* attention output: 2e-2 abs/rel against the fp32 checker fed with the checker's own norm / RoPE chain, and
  within 8e-3 of the separate launches (the queries' sum of squares is reduced in another order, so a query
  element can differ by one 16-bit ulp).
"""
import pytest
import torch

from oracle import paged_attention as oa
from oracle import rope_norm as orn

pytestmark = pytest.mark.gpu


def _close(got, ref, tol, what):
    got = got.float().cpu().reshape(ref.shape)
    assert torch.isfinite(got).all(), f"{what}: non-finite output"
    err = (got - ref.float()).abs()
    assert (err <= tol + tol * ref.float().abs()).all(), f"{what}: max err {err.max().item():.4e}"


def _step_case(mi, dev, *, Hq, Hkv, d, chunk, lens, dtype, seed):
    lens = torch.tensor(lens, dtype=torch.int32)
    cfg = mi.synthetic.DecodeConfig("step", lens.numel(), Hq, Hkv, d, 0, 0, chunk=chunk, seed=seed)
    case = mi.synthetic.make_decode_case(cfg, dev, lens=lens, dtype=dtype)
    gen = torch.Generator().manual_seed(seed + 1)
    qw = (1 + 0.05 * torch.randn(d, generator=gen)).to(dtype)
    kw = (1 + 0.05 * torch.randn(d, generator=gen)).to(dtype)
    pos = torch.randint(0, 4000, (lens.numel(),), generator=gen)
    return case, lens, qw, kw, pos


def _run_both(mi, dev, case, lens, qw, kw, pos, *, norm, table, interleaved, mixed, faithful=True, **attn_kw):
    """(fused output, fused caches), (separate output, separate caches)."""
    R, _, Hq, d = case.q.shape
    Hkv = case.k_new.size(2)
    G = Hq // Hkv
    common = dict(q_weight=qw.to(dev) if norm == "rms" else None, k_weight=kw.to(dev) if norm == "rms" else None,
                  norm=norm, eps=1e-5, rotary_emb=None if table is None else table.to(dev),
                  rotary_interleaved=interleaved, faithful_rounding=faithful)
    kc_a, vc_a = case.k_cache.clone(), case.v_cache.clone()
    kc_b, vc_b = case.k_cache.clone(), case.v_cache.clone()
    posd = pos.to(dev)
    if mixed:
        grouped = torch.cat([case.q.view(R, Hkv, G * d), case.k_new.view(R, Hkv, d), case.v_new.view(R, Hkv, d)], -1)
        grouped = grouped.reshape(R, 1, -1).contiguous()
        out_a = mi.ops.decode_step_attention(None, None, None, kc_a, vc_a, case.kv_lens, case.block_table,
                                             mixed_qkv=grouped, num_query_heads=Hq, num_kv_heads=Hkv, positions=posd,
                                             **common, **attn_kw)
    else:
        out_a = mi.ops.decode_step_attention(case.q, case.k_new, case.v_new, kc_a, vc_a, case.kv_lens,
                                             case.block_table, positions=posd, **common, **attn_kw)
    q_b = torch.empty_like(case.q)
    with mi.ops.tuning(norm_rope_vectorised=-1):
        mi.ops.norm_rope_append(case.q, case.k_new, value=case.v_new, query_out=q_b, q_positions=posd, k_positions=posd,
                                k_cache=kc_b, v_cache=vc_b, block_table=case.block_table, kv_lens=case.kv_lens, **common)
    out_b = mi.ops.paged_decode_attention(q_b, kc_b, vc_b, case.kv_lens, case.block_table, **attn_kw)
    torch.cuda.synchronize()
    return (out_a, kc_a, vc_a), (out_b, kc_b, vc_b)


def _oracle(case, lens, qw, kw, pos, *, norm, table, interleaved):
    kc, vc = case.k_cache.cpu().clone(), case.v_cache.cpu().clone()
    q, k, v = case.q.cpu().squeeze(1), case.k_new.cpu().squeeze(1), case.v_new.cpu().squeeze(1)
    w = dict(norm=norm, eps=1e-5, interleaved=interleaved)
    q_ref = orn.norm_rope(q, pos, table, weight=qw if norm == "rms" else None, **w)
    k_ref = orn.norm_rope(k, pos, table, weight=kw if norm == "rms" else None, **w)
    rows, ids, loc = oa.decode_slots(case.block_table.cpu(), lens, case.k_cache.size(1))
    oa.kv_append(kc, vc, k_ref[rows], v[rows], ids, loc)
    return oa.paged_decode_attention(q_ref, kc, vc, lens, case.block_table.cpu()), kc, vc


LENS = [0, 1, 2, 15, 16, 17, 31, 32, 33, 63, 64, 65, 129, 700, 0, 2049]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("norm", [None, "rms", "l2"])
@pytest.mark.parametrize("rotary", ["none", "half", "half64", "interleaved", "interleaved40"])
@pytest.mark.parametrize("Hq,Hkv,d", [(32, 8, 128), (8, 8, 64), (6, 2, 128), (16, 1, 64), (20, 1, 128)])
def test_fused_step_equals_the_separate_launches(mi, dev, Hq, Hkv, d, rotary, norm, dtype):
    if rotary == "half64" and d == 64:
        pytest.skip("rot_dim 64 is the full width at head_dim 64")
    rot = {"none": 0, "half": d, "half64": 64, "interleaved": d, "interleaved40": 40}[rotary]
    interleaved = rotary.startswith("interleaved")
    table = orn.rotary_table(4096, rot, base=500000.0, interleaved=interleaved) if rot else None
    case, lens, qw, kw, pos = _step_case(mi, dev, Hq=Hq, Hkv=Hkv, d=d, chunk=64, lens=LENS, dtype=dtype, seed=Hq + d)
    (out_a, kc_a, vc_a), (out_b, kc_b, vc_b) = _run_both(mi, dev, case, lens, qw, kw, pos, norm=norm, table=table,
                                                         interleaved=interleaved, mixed=False,
                                                         max_kv_len=int(lens.max()))
    dummy = case.k_cache.size(0) - 1   # (rows of length 0 are padding: nothing is appended for them)
    assert torch.equal(kc_a[:dummy], kc_b[:dummy]), "key cache differs from the separate launch"
    assert torch.equal(vc_a[:dummy], vc_b[:dummy]), "value cache differs from the separate launch"
    diff = (out_a.float() - out_b.float()).abs().max().item()
    assert diff <= 8e-3, f"fused and separate outputs differ by {diff:.3e}"
    assert (out_a[case.kv_lens == 0] == 0).all()
    ref, kc_ref, vc_ref = _oracle(case, lens, qw, kw, pos, norm=norm, table=table, interleaved=interleaved)
    _close(out_a, ref, 2e-2, "fused step vs checker")
    assert torch.equal(vc_a.cpu()[:dummy], vc_ref[:dummy])
    _close(kc_a[:dummy], kc_ref[:dummy], 2e-2, "key cache vs checker")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("mixed", [False, True])
@pytest.mark.parametrize("Hq,Hkv,d,rot,interleaved", [
    (12, 4, 96, 0, False), (12, 4, 96, 64, False), (12, 4, 96, 96, True), (24, 1, 96, 64, False),
    (8, 2, 192, 192, False), (8, 2, 192, 128, False), (8, 2, 192, 64, False), (8, 2, 192, 192, True),
    (16, 2, 256, 256, False), (16, 2, 256, 128, False), (16, 2, 256, 64, False), (16, 2, 256, 0, False),
    (4, 4, 256, 200, True)])
def test_fused_step_at_head_widths_96_192_256(mi, dev, Hq, Hkv, d, rot, interleaved, mixed, dtype):
    """The one-kernel decode step at the other head widths (two wavefronts per SIMD at 192 and 256): half-split
    rotary pairs a whole number of 32-element fragments apart (rot_dim 64, 128, 192 or 256), interleaved pairs of
    any even width, no rotary embedding; per-head and mixed (projection-output) inputs."""
    table = orn.rotary_table(4096, rot, base=500000.0, interleaved=interleaved) if rot else None
    case, lens, qw, kw, pos = _step_case(mi, dev, Hq=Hq, Hkv=Hkv, d=d, chunk=64, lens=LENS, dtype=dtype, seed=Hq + d + rot)
    (out_a, kc_a, vc_a), (out_b, kc_b, vc_b) = _run_both(mi, dev, case, lens, qw, kw, pos, norm="rms", table=table,
                                                         interleaved=interleaved, mixed=mixed,
                                                         max_kv_len=int(lens.max()))
    dummy = case.k_cache.size(0) - 1
    assert torch.equal(kc_a[:dummy], kc_b[:dummy]), "key cache differs from the separate launch"
    assert torch.equal(vc_a[:dummy], vc_b[:dummy]), "value cache differs from the separate launch"
    diff = (out_a.float() - out_b.float()).abs().max().item()
    assert diff <= 8e-3, f"fused and separate outputs differ by {diff:.3e}"
    ref, kc_ref, vc_ref = _oracle(case, lens, qw, kw, pos, norm="rms", table=table, interleaved=interleaved)
    _close(out_a, ref, 2e-2, "fused step vs checker")
    _close(kc_a[:dummy], kc_ref[:dummy], 2e-2, "key cache vs checker")


@pytest.mark.parametrize("mixed", [False, True])
@pytest.mark.parametrize("chunk", [16, 128, 256])
@pytest.mark.parametrize("grid,split", [(0, 0), (1, 0), (7, 64), (4096, 16)])
def test_fused_step_span_cuts_and_mixed_qkv_input(mi, dev, mixed, chunk, grid, split):
    """However the tile sequence is cut into spans, exactly one span (the one that ends the request) appends the
    token, before it reads it; the QKV projection's output is read in place."""
    lens = [1, 5, chunk - 1, chunk, chunk + 1, 3 * chunk, 3 * chunk + 1, 1999, 0, 16, 17, 4097]
    table = orn.rotary_table(4096, 128, base=10000.0)
    case, lens, qw, kw, pos = _step_case(mi, dev, Hq=32, Hkv=8, d=128, chunk=chunk, lens=lens, dtype=torch.bfloat16,
                                         seed=chunk + grid)
    with mi.ops.tuning(decode_grid=grid):
        (out_a, kc_a, vc_a), (out_b, kc_b, vc_b) = _run_both(mi, dev, case, lens, qw, kw, pos, norm="rms", table=table,
                                                             interleaved=False, mixed=mixed, split_tokens=split,
                                                             max_kv_len=int(lens.max()))
    dummy = case.k_cache.size(0) - 1
    assert torch.equal(kc_a[:dummy], kc_b[:dummy]) and torch.equal(vc_a[:dummy], vc_b[:dummy])
    assert (out_a.float() - out_b.float()).abs().max().item() <= 8e-3
    ref, _, _ = _oracle(case, lens, qw, kw, pos, norm="rms", table=table, interleaved=False)
    _close(out_a, ref, 2e-2, "fused step vs checker")


def test_fused_step_without_faithful_rounding_and_repeated_steps(mi, dev):
    """Three steps in a row on the same caches (each appends one token per request), fp32 evaluation of the chain."""
    table = orn.rotary_table(4096, 128, base=10000.0)
    lens0 = [1, 63, 64, 255, 256, 700]
    case, lens, qw, kw, pos = _step_case(mi, dev, Hq=16, Hkv=4, d=128, chunk=64, lens=[n + 3 for n in lens0],
                                         dtype=torch.bfloat16, seed=3)
    kc, vc = case.k_cache, case.v_cache
    kc_ref, vc_ref = kc.cpu().clone(), vc.cpu().clone()
    gen = torch.Generator().manual_seed(9)
    for step in range(3):
        cur = torch.tensor([n + step + 1 for n in lens0], dtype=torch.int32)
        q = torch.randn(cur.numel(), 1, 16, 128, generator=gen).bfloat16()
        k = torch.randn(cur.numel(), 1, 4, 128, generator=gen).bfloat16()
        v = torch.randn(cur.numel(), 1, 4, 128, generator=gen).bfloat16()
        p = (cur - 1).long()
        out = mi.ops.decode_step_attention(q.to(dev), k.to(dev), v.to(dev), kc, vc, cur.to(dev), case.block_table,
                                           q_weight=qw.to(dev), k_weight=kw.to(dev), norm="rms", rotary_emb=table.to(dev),
                                           positions=None if step == 1 else p.to(dev),  # None: kv_lens - 1
                                           faithful_rounding=False)
        torch.cuda.synchronize()
        q_ref = orn.norm_rope(q.squeeze(1), p, table, norm="rms", weight=qw, eps=1e-5)
        k_ref = orn.norm_rope(k.squeeze(1), p, table, norm="rms", weight=kw, eps=1e-5)
        rows, ids, loc = oa.decode_slots(case.block_table.cpu(), cur, 64)
        oa.kv_append(kc_ref, vc_ref, k_ref[rows], v.squeeze(1)[rows], ids, loc)
        ref = oa.paged_decode_attention(q_ref, kc_ref, vc_ref, cur, case.block_table.cpu())
        _close(out, ref, 2e-2, f"step {step}")
    dummy = kc.size(0) - 1
    assert torch.equal(vc.cpu()[:dummy], vc_ref[:dummy])
    _close(kc[:dummy], kc_ref[:dummy], 2e-2, "key cache after three steps")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("mixed", [False, True])
@pytest.mark.parametrize("rotary", ["none", "half", "interleaved", "interleaved40"])
@pytest.mark.parametrize("norm", [None, "rms"])
@pytest.mark.parametrize("Hq,Hkv", [(32, 8), (6, 2), (20, 1)])
def test_fused_step_over_an_fp8_cache(mi, dev, Hq, Hkv, norm, rotary, mixed, dtype):
    """The one-kernel step over an fp8-e4m3 cache: bytes and scales equal to the separate launches (norm / rotary
    with key_out, then the quantising append), tokens that open a chunk (lengths 1, 65, 129: they set the scale) and
    tokens that reuse a stored scale; output within 8e-3 of the separate launches and 6e-2 of the unquantised checker."""
    d, chunk = 128, 64
    rot = {"none": 0, "half": d, "interleaved": d, "interleaved40": 40}[rotary]
    interleaved = rotary.startswith("interleaved")
    table = orn.rotary_table(4096, rot, base=500000.0, interleaved=interleaved) if rot else None
    lens_l = [0, 1, 2, 63, 64, 65, 66, 128, 129, 130, 700, 2049, 0, 193]
    case, lens, qw, kw, pos = _step_case(mi, dev, Hq=Hq, Hkv=Hkv, d=d, chunk=chunk, lens=lens_l, dtype=dtype,
                                         seed=Hq + rot)
    R = lens.numel()
    G = Hq // Hkv
    k8 = torch.empty(case.k_cache.shape, dtype=torch.uint8, device=dev)
    v8 = torch.empty_like(k8)
    ks = torch.empty(case.k_cache.size(0), Hkv, dtype=torch.float32, device=dev)
    vs = torch.empty_like(ks)
    mi.ops.quantize_chunks_fp8(case.k_cache, k8, ks)
    mi.ops.quantize_chunks_fp8(case.v_cache, v8, vs)
    # chunks the step's token is about to open hold no token yet: whatever they held must not matter
    for r in range(R):
        L = int(lens[r])
        if L > 0 and (L - 1) % chunk == 0:
            c = int(case.block_table[r, (L - 1) // chunk])
            k8[c] = 0x7e; v8[c] = 0x7e; ks[c] = 1e30; vs[c] = -5.0
    common = dict(q_weight=qw.to(dev) if norm == "rms" else None, k_weight=kw.to(dev) if norm == "rms" else None,
                  norm=norm, eps=1e-5, rotary_emb=None if table is None else table.to(dev),
                  rotary_interleaved=interleaved)
    posd = pos.to(dev)
    k8a, v8a, ksa, vsa = k8.clone(), v8.clone(), ks.clone(), vs.clone()
    k8b, v8b, ksb, vsb = k8.clone(), v8.clone(), ks.clone(), vs.clone()
    if mixed:
        grouped = torch.cat([case.q.view(R, Hkv, G * d), case.k_new.view(R, Hkv, d), case.v_new.view(R, Hkv, d)], -1)
        out_a = mi.ops.decode_step_attention(None, None, None, k8a, v8a, case.kv_lens, case.block_table,
                                             mixed_qkv=grouped.reshape(R, 1, -1).contiguous(), num_query_heads=Hq,
                                             num_kv_heads=Hkv, positions=posd, k_scales=ksa, v_scales=vsa, headroom=1.5,
                                             max_kv_len=int(lens.max()), **common)
    else:
        out_a = mi.ops.decode_step_attention(case.q, case.k_new, case.v_new, k8a, v8a, case.kv_lens, case.block_table,
                                             positions=posd, k_scales=ksa, v_scales=vsa, headroom=1.5,
                                             max_kv_len=int(lens.max()), **common)
    q_b, k_b = torch.empty_like(case.q), torch.empty_like(case.k_new)
    with mi.ops.tuning(norm_rope_vectorised=-1):
        mi.ops.norm_rope_append(case.q, case.k_new, query_out=q_b, key_out=k_b, q_positions=posd, k_positions=posd, **common)
    mi.ops.kv_append_decode_fp8(k_b, case.v_new, k8b, v8b, ksb, vsb, case.block_table, case.kv_lens, headroom=1.5)
    out_b = mi.ops.paged_decode_attention(q_b, k8b, v8b, case.kv_lens, case.block_table, k_scales=ksb, v_scales=vsb,
                                          max_kv_len=int(lens.max()))
    torch.cuda.synchronize()
    assert torch.equal(k8a, k8b) and torch.equal(v8a, v8b), "cache bytes differ from the separate launches"
    assert torch.equal(ksa, ksb) and torch.equal(vsa, vsb), "scales differ from the separate launches"
    diff = (out_a.float() - out_b.float()).abs().max().item()
    assert diff <= 8e-3, f"fused and separate outputs differ by {diff:.3e}"
    assert (out_a[case.kv_lens == 0] == 0).all()
    # against the checker: its own norm / rotary chain for the queries, attention over the dequantised cache the
    # step left behind (2e-2); single values of short rows carry the full e4m3 rounding, so the unquantised
    # checker is only held to 6e-2 where at least 64 keys average it out
    w = dict(norm=norm, eps=1e-5, interleaved=interleaved)
    q_ref = orn.norm_rope(case.q.cpu().squeeze(1), pos, table, weight=qw if norm == "rms" else None, **w)
    ref8 = oa.paged_decode_attention(q_ref, k8a.cpu(), v8a.cpu(), lens, case.block_table.cpu(), k_scales=ksa.cpu(),
                                     v_scales=vsa.cpu())
    _close(out_a, ref8, 2e-2, "fused fp8 step vs the checker over the dequantised cache")
    ref, _, _ = _oracle(case, lens, qw, kw, pos, norm=norm, table=table, interleaved=interleaved)
    long_rows = lens >= 64
    _close(out_a[long_rows.to(dev)], ref[long_rows], 6e-2, "fused fp8 step vs the unquantised checker")


def test_fused_step_rejects_what_it_has_no_kernel_for(mi, dev):
    case, lens, qw, kw, pos = _step_case(mi, dev, Hq=8, Hkv=2, d=128, chunk=64, lens=[5, 9], dtype=torch.bfloat16, seed=1)
    table = orn.rotary_table(64, 40, base=10000.0)  # half-split pairs 20 elements apart
    assert not mi.ops.decode_step_supported(128, 40, False, False)
    assert mi.ops.decode_step_supported(128, 40, True, False) and mi.ops.decode_step_supported(64, 64, False, False)
    assert not mi.ops.decode_step_supported(96, 96, False, False) and mi.ops.decode_step_supported(128, 128, False, True)
    assert not mi.ops.decode_step_supported(128, 64, False, True) and not mi.ops.decode_step_supported(64, 64, False, True)
    assert mi.ops.decode_step_supported(96, 64, False, False) and mi.ops.decode_step_supported(256, 256, False, False)
    assert not mi.ops.decode_step_supported(80, 0, False, False)
    with pytest.raises(mi._lib.KernelError, match="rot_dim / 2"):
        mi.ops.decode_step_attention(case.q, case.k_new, case.v_new, case.k_cache, case.v_cache, case.kv_lens,
                                     case.block_table, rotary_emb=table.to(dev), positions=pos.to(dev))
    q80 = torch.zeros(2, 1, 8, 80, dtype=torch.bfloat16, device=dev)
    k80 = torch.zeros(2, 1, 2, 80, dtype=torch.bfloat16, device=dev)
    c80 = torch.zeros(4, 64, 2, 80, dtype=torch.bfloat16, device=dev)
    with pytest.raises(mi._lib.KernelError, match="head_dim"):
        mi.ops.decode_step_attention(q80, k80, k80, c80, c80, case.kv_lens, case.block_table)


def test_fused_step_more_requests_than_one_launch_takes(mi, dev):
    """Beyond 7 680 requests the step runs in slices: queries, new rows, positions, lengths and table rows of a
    slice all start at the slice's first request."""
    R = 7680 + 900
    gen = torch.Generator().manual_seed(6)
    lens = torch.randint(0, 50, (R,), generator=gen).tolist()
    table = orn.rotary_table(64, 64, base=10000.0)
    case, lens, qw, kw, pos = _step_case(mi, dev, Hq=4, Hkv=2, d=64, chunk=16, lens=lens, dtype=torch.bfloat16, seed=8)
    pos = (lens.long() - 1).clamp(min=0)
    (out_a, kc_a, vc_a), (out_b, kc_b, vc_b) = _run_both(mi, dev, case, lens, qw, kw, pos, norm="rms", table=table,
                                                         interleaved=False, mixed=False, max_kv_len=50)
    dummy = case.k_cache.size(0) - 1
    assert torch.equal(kc_a[:dummy], kc_b[:dummy]) and torch.equal(vc_a[:dummy], vc_b[:dummy])
    assert (out_a.float() - out_b.float()).abs().max().item() <= 8e-3
    ref, _, _ = _oracle(case, lens, qw, kw, pos, norm="rms", table=table, interleaved=False)
    _close(out_a, ref, 2e-2, "sliced fused step vs checker")
