"""GPU parity: fused head norm + rotary embedding (+ append) against the op-by-op CPU chain.

Floating point: bf16 results within 2e-2 abs/rel of the fp32 formula; in the faithful
rounding mode the kernel reproduces the bf16 op chain up to the last-place effects of
cos/sin/rsqrt implementations (a tiny fraction of elements, by at most 2 ulps of the head vector's largest element).
"""
import pytest
import torch

from oracle import paged_attention as oa
from oracle import rope_norm as orn

pytestmark = pytest.mark.gpu


def _ulp_diff(a, b):
    a = a.view(torch.int16).to(torch.int32)
    b = b.view(torch.int16).to(torch.int32)
    # map sign-magnitude bf16 bit patterns to a monotone integer line
    a = torch.where(a < 0, -(a & 0x7FFF), a)
    b = torch.where(b < 0, -(b & 0x7FFF), b)
    return (a - b).abs()


@pytest.mark.parametrize("norm", [None, "rms", "l2"])
@pytest.mark.parametrize("interleaved", [False, True])
@pytest.mark.parametrize("d,rot", [(128, 128), (64, 64), (128, 64), (128, 96), (64, 32), (128, 40),
                                   (96, 96), (96, 48), (96, 32), (192, 192), (192, 64), (256, 256), (256, 128), (256, 90)])
@pytest.mark.parametrize("vectorised", [1, -1])
def test_norm_rope_matches_unfused_chain(mi, dev, norm, interleaved, d, rot, vectorised):
    """Both kernels: 16 bytes per lane (taken when every rotary partner is a whole number of lanes
    away; rot 40 falls back for half-split pairs by itself) and the element-wise one."""
    mi.ops.set_tuning("norm_rope_vectorised", vectorised)
    try:
        _norm_rope_case(mi, dev, norm, interleaved, d, rot)
    finally:
        mi.ops.set_tuning("norm_rope_vectorised", 0)


def _norm_rope_case(mi, dev, norm, interleaved, d, rot):
    gen = torch.Generator().manual_seed(d + rot + (7 if interleaved else 0))
    T, Hq, Hkv = 37, 8, 2
    q = torch.randn(T, 1, Hq, d, generator=gen).bfloat16()
    k = torch.randn(T, 1, Hkv, d, generator=gen).bfloat16()
    qw = (1 + 0.02 * torch.randn(d, generator=gen)).bfloat16()
    kw = (1 + 0.02 * torch.randn(d, generator=gen)).bfloat16()
    table = orn.rotary_table(9000, rot, base=500000.0, interleaved=interleaved)
    qpos = torch.randint(0, 9000, (T,), generator=gen)
    kpos = torch.randint(0, 9000, (T,), generator=gen)
    eps = 1e-5 if norm == "rms" else 1e-6
    q_ref = orn.norm_rope(q.squeeze(1), qpos, table, norm=norm, weight=qw if norm == "rms" else None, eps=eps,
                          interleaved=interleaved)
    k_ref = orn.norm_rope(k.squeeze(1), kpos, table, norm=norm, weight=kw if norm == "rms" else None, eps=eps,
                          interleaved=interleaved)
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
                # under 1 % of the elements differ at all (the device's rsqrt / cos / sin differ from the host's in
                # the last bit), and those by at most 2 ulp of the head vector's largest element: a rotation whose
                # two products nearly cancel turns one ulp of a product into many ulp of the small difference
                assert (_ulp_diff(got, ref) > 0).float().mean().item() < 0.01
                scale = ref.float().abs().amax(-1, keepdim=True)
                assert (err <= 2 * 2.0 ** -7 * scale).all()
        assert torch.equal(kd.cpu(), k), "the key input must not be modified"


@pytest.mark.parametrize("vectorised", [1, -1])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
def test_large_rotary_angles(mi, dev, vectorised, dtype):
    """Angles far beyond one turn: rows of the table reach 1e3, 1e5, 1e6 (the kernels' own range reduction) and 3e7 rad
    (the library functions behind it); the result still equals the op-by-op chain, whose cos / sin are the host's."""
    gen = torch.Generator().manual_seed(5)
    T, Hq, Hkv, d = 64, 4, 2, 128
    tops = [1e3, 1e5, 1e6, 3e7]
    table = torch.stack([torch.rand(d, generator=gen) * tops[i % 4] for i in range(T)]).float()
    table[:, d // 2:] = table[:, :d // 2]  # half-split pairs share an angle
    pos = torch.randperm(T, generator=gen)
    q = torch.randn(T, 1, Hq, d, generator=gen).to(dtype)
    k = torch.randn(T, 1, Hkv, d, generator=gen).to(dtype)
    q_ref = orn.norm_rope(q.squeeze(1), pos, table, norm=None)
    k_ref = orn.norm_rope(k.squeeze(1), pos, table, norm=None)
    with mi.ops.tuning(norm_rope_vectorised=vectorised):
        qd, kd = q.to(dev).clone(), k.to(dev)
        k_out = torch.empty_like(kd)
        mi.ops.norm_rope_append(qd, kd, key_out=k_out, rotary_emb=table.to(dev), q_positions=pos.to(dev),
                                k_positions=pos.to(dev), faithful_rounding=True)
        torch.cuda.synchronize()
    ulp = 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10
    for got, ref in ((qd.cpu().squeeze(1), q_ref), (k_out.cpu().squeeze(1), k_ref)):
        err = (got.float() - ref.float()).abs()
        assert (got != ref).float().mean().item() < 0.01
        assert (err <= 2 * ulp * ref.float().abs().amax(-1, keepdim=True)).all(), f"max err {err.max().item()}"


def test_position_zero_is_identity_and_passthrough_tail(mi, dev):
    T, H, d, rot = 5, 4, 128, 64
    x = torch.randn(T, 1, H, d).bfloat16().to(dev)
    table = orn.rotary_table(16, rot).to(dev)
    y = x.clone()
    pos = torch.zeros(T, dtype=torch.int64, device=dev)
    mi.ops.norm_rope_append(y, None, rotary_emb=table, q_positions=pos)
    torch.cuda.synchronize()
    assert torch.equal(x, y)
    pos = torch.arange(T, dtype=torch.int64, device=dev) + 3
    mi.ops.norm_rope_append(y, None, rotary_emb=table, q_positions=pos)
    torch.cuda.synchronize()
    assert torch.equal(x[..., rot:], y[..., rot:]) and not torch.equal(x[..., :rot], y[..., :rot])


@pytest.mark.parametrize("mode", ["token_rows", "block_table"])
def test_fused_append_writes_rotated_key_and_raw_value(mi, dev, mode):
    lens = torch.tensor([5, 256, 257, 1000, 0, 31], dtype=torch.int32)
    cfg = mi.synthetic.DecodeConfig("fa", lens.numel(), 32, 8, 128, 0, 0, seed=4)
    case = mi.synthetic.make_decode_case(cfg, dev, lens=lens)
    kc0, vc0 = case.k_cache.cpu().clone(), case.v_cache.cpu().clone()
    table = orn.rotary_table(2048, 128, base=500000.0)
    pos = (lens.long() - 1).clamp(min=0)
    w = (1 + 0.02 * torch.randn(128)).bfloat16()
    q = case.q.clone()
    k_out = torch.empty_like(case.k_new)
    rows, ids, loc = oa.decode_slots(case.block_table.cpu(), lens, cfg.chunk)
    kwargs = {}
    if mode == "token_rows":
        ci = torch.full((lens.numel(),), case.k_cache.size(0) - 1, dtype=torch.int64)
        lo = torch.zeros(lens.numel(), dtype=torch.int64)
        ci[rows], lo[rows] = ids, loc
        kwargs = dict(token_to_chunk_idx=ci.to(dev), token_to_local_pos=lo.to(dev))
    else:
        kwargs = dict(block_table=case.block_table, kv_lens=case.kv_lens)
    mi.ops.norm_rope_append(q, case.k_new, value=case.v_new, key_out=k_out, q_weight=w.to(dev), k_weight=w.to(dev),
                            norm="rms", eps=1e-5, rotary_emb=table.to(dev), q_positions=pos.to(dev),
                            k_positions=pos.to(dev), k_cache=case.k_cache, v_cache=case.v_cache, **kwargs)
    torch.cuda.synchronize()
    # append is bit-exact given the rotated key the kernel itself produced
    oa.kv_append(kc0, vc0, k_out.cpu().squeeze(1)[rows], case.v_new.cpu().squeeze(1)[rows], ids, loc)
    dummy = case.k_cache.size(0) - 1
    assert torch.equal(case.k_cache.cpu()[:dummy], kc0[:dummy])
    assert torch.equal(case.v_cache.cpu()[:dummy], vc0[:dummy])
    k_ref = orn.norm_rope(case.k_new.cpu().squeeze(1), pos, table, norm="rms", weight=w, eps=1e-5)
    assert (k_out.cpu().squeeze(1).float() - k_ref.float()).abs().max().item() <= 4e-2


@pytest.mark.parametrize("d,hq,hkv", [(128, 32, 8), (128, 8, 8), (64, 12, 4), (128, 5, 1), (96, 32, 8), (192, 6, 2), (256, 16, 1)])
@pytest.mark.parametrize("vectorised", [1, -1])
@pytest.mark.parametrize("interleaved", [False, True])
def test_mixed_qkv_input_equals_split_inputs(mi, dev, d, hq, hkv, vectorised, interleaved):
    """Reading the QKV projection's output directly gives the bits the same launch produces from the
    split tensors (attention.py:985-1024), for query, key output, key cache and value cache, and
    agrees with the op-by-op chain on the checker's split."""
    mi.ops.set_tuning("norm_rope_vectorised", vectorised)
    try:
        gen = torch.Generator().manual_seed(11 + d + hq)
        T, C = 45, 16
        mixed = torch.randn(T, 1, (hq + 2 * hkv) * d, generator=gen).bfloat16()
        q, k, v = orn.split_mixed_qkv(mixed, hq, hkv)
        qw = (1 + 0.02 * torch.randn(d, generator=gen)).bfloat16().to(dev)
        kw = (1 + 0.02 * torch.randn(d, generator=gen)).bfloat16().to(dev)
        table = orn.rotary_table(500, d, base=10000.0, interleaved=interleaved)
        pos = torch.randint(0, 500, (T,), generator=gen)
        n_chunks = (T + C - 1) // C + 1
        ci = (torch.randperm(T, generator=gen) // C).long()
        lo = torch.empty(T, dtype=torch.int64)
        for c in range(n_chunks):  # distinct slots inside each chunk
            idx = (ci == c).nonzero().flatten()
            lo[idx] = torch.randperm(C, generator=gen)[: idx.numel()]
        common = dict(q_weight=qw, k_weight=kw, norm="rms", eps=1e-5, rotary_emb=table.to(dev), q_positions=pos.to(dev),
                      k_positions=pos.to(dev), rotary_interleaved=interleaved, token_to_chunk_idx=ci.to(dev),
                      token_to_local_pos=lo.to(dev))
        res = []
        for use_mixed in (True, False):
            kc = torch.full((n_chunks, C, hkv, d), -1.0, dtype=torch.bfloat16, device=dev)
            vc = torch.full_like(kc, -1.0)
            qo = torch.empty(T, 1, hq, d, dtype=torch.bfloat16, device=dev)
            ko = torch.empty(T, 1, hkv, d, dtype=torch.bfloat16, device=dev)
            if use_mixed:
                md = mixed.to(dev)
                mi.ops.qkv_norm_rope_append(md, num_query_heads=hq, num_kv_heads=hkv, query_out=qo, key_out=ko,
                                            k_cache=kc, v_cache=vc, **common)
                torch.cuda.synchronize()
                assert torch.equal(md.cpu(), mixed), "the projection output must not be modified"
            else:
                mi.ops.norm_rope_append(q.contiguous().to(dev), k.contiguous().to(dev), value=v.contiguous().to(dev),
                                        query_out=qo, key_out=ko, k_cache=kc, v_cache=vc, **common)
                torch.cuda.synchronize()
            res.append((qo.cpu(), ko.cpu(), kc.cpu(), vc.cpu()))
        for a, b in zip(*res):
            assert torch.equal(a, b)
        qo, ko, kc, vc = res[0]
        # value rows are copied bit for bit into their slots, other slots keep the fill
        vc_ref = torch.full_like(vc, -1.0)
        vc_ref[ci, lo] = v.squeeze(1)
        assert torch.equal(vc, vc_ref)
        assert torch.equal(kc[ci, lo], ko.squeeze(1))
        q_ref = orn.norm_rope(q.squeeze(1), pos, table, norm="rms", weight=qw.cpu(), eps=1e-5, interleaved=interleaved)
        k_ref = orn.norm_rope(k.squeeze(1), pos, table, norm="rms", weight=kw.cpu(), eps=1e-5, interleaved=interleaved)
        for got, ref in ((qo.squeeze(1), q_ref), (ko.squeeze(1), k_ref)):
            # a last-place difference in cos / sin is many ulps of a result that nearly cancels, so
            # bound the error absolutely and the number of differing elements
            err = (got.float() - ref.float()).abs()
            assert (err <= 2e-2 + 2e-2 * ref.float().abs()).all(), f"max err {err.max().item()}"
            assert (_ulp_diff(got, ref) > 0).float().mean().item() < 0.01
    finally:
        mi.ops.set_tuning("norm_rope_vectorised", 0)


def test_mixed_qkv_argument_errors(mi, dev):
    mixed = torch.zeros(4, 1, (8 + 4) * 128, dtype=torch.bfloat16, device=dev)
    qo = torch.empty(4, 1, 8, 128, dtype=torch.bfloat16, device=dev)
    with pytest.raises(ValueError):  # no destination for the key
        mi.ops.qkv_norm_rope_append(mixed, num_query_heads=8, num_kv_heads=2, query_out=qo)
    with pytest.raises(ValueError):  # width does not match the head counts
        mi.ops.qkv_norm_rope_append(mixed, num_query_heads=7, num_kv_heads=2, query_out=qo,
                                    key_out=torch.empty(4, 1, 2, 128, dtype=torch.bfloat16, device=dev))
