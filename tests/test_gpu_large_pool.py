"""GPU parity at pool sizes where byte offsets no longer fit 32 bits: caches of 5 GiB per tensor (the
benchmark configurations run on 8-16 GiB pools), requests whose chunks sit at the very end of the pool and
either side of the 2 GiB and 4 GiB marks.  The CPU checker sees only the chunks in use (copied out and
renumbered), so the comparison costs what a small case costs.

Covers decode (bf16 and fp8), the mixed prefill path, the scatter append and the fused norm + rotary
append into high chunks, and the multi-latent decode over a latent cache above 4 GiB.
"""
import pytest
import torch

from oracle import paged_attention as oa
from oracle import rope_norm as orn

pytestmark = pytest.mark.gpu

C, HKV, D = 256, 8, 128
CHUNK_BYTES = C * HKV * D * 2            # 512 KiB per chunk and tensor
N_POOL = 5 * 2048 + 3                    # 5 GiB and a bit


def _chunk_ids(need, gen):
    """`need` chunk ids: the last ones of the pool, the ones either side of the 2 GiB and 4 GiB marks, the rest random."""
    special = [N_POOL - 2, N_POOL - 3, 0, 4095, 4096, 4097, 8191, 8192, 8193, N_POOL - 4]
    rest = torch.randperm(N_POOL - 1, generator=gen).tolist()
    ids = []
    for c in special + rest:
        if c not in ids:
            ids.append(c)
        if len(ids) == need:
            break
    perm = torch.randperm(need, generator=gen).tolist()
    return [ids[i] for i in perm]


def _table(lens, gen):
    need = [(int(l) + C - 1) // C for l in lens]
    ids = _chunk_ids(sum(need), gen)
    table = torch.full((len(need), max(need)), -1, dtype=torch.int32)
    at = 0
    for r, n in enumerate(need):
        table[r, :n] = torch.tensor(ids[at:at + n], dtype=torch.int32)
        at += n
    return table


def _compact(table, *caches):
    """Chunks in use copied to the CPU and renumbered 0..n-1; returns (remapped table, cpu caches)."""
    used = table[table >= 0].unique().long()
    remap = torch.full((N_POOL,), -1, dtype=torch.int32)
    remap[used] = torch.arange(used.numel(), dtype=torch.int32)
    new_table = torch.where(table >= 0, remap[table.clamp(min=0).long()], table)
    return new_table, [c[used.to(c.device)].cpu() for c in caches]


@pytest.fixture(scope="module")
def pool(mi, dev):
    free, _ = torch.cuda.mem_get_info()
    if free < 14 * 2**30:
        pytest.skip("needs 14 GiB of free device memory")
    gen = torch.Generator(device=dev).manual_seed(77)
    kc = mi.synthetic.randn_fill_(torch.empty(N_POOL, C, HKV, D, dtype=torch.bfloat16, device=dev), gen)
    vc = mi.synthetic.randn_fill_(torch.empty(N_POOL, C, HKV, D, dtype=torch.bfloat16, device=dev), gen)
    assert kc.numel() * 2 > 5 * 2**30
    yield kc, vc
    del kc, vc
    torch.cuda.empty_cache()


def _close(got, ref, tol):
    got = got.float().cpu().reshape(ref.shape)
    assert torch.isfinite(got).all()
    err = (got - ref).abs()
    assert (err <= tol + tol * ref.abs()).all(), f"max err {err.max().item():.4e}"


def test_decode_over_chunks_beyond_4_gib(mi, dev, pool):
    kc, vc = pool
    gen = torch.Generator().manual_seed(1)
    lens = torch.tensor([700, 3000, 1, 256, 257, 5000, 0, 1900], dtype=torch.int32)
    table = _table(lens, gen)
    assert int(table.max()) == N_POOL - 2 and (table.long() * CHUNK_BYTES).max() > 2**32
    q = torch.randn(lens.numel(), 1, 32, D, generator=gen).bfloat16()
    out = mi.ops.paged_decode_attention(q.to(dev), kc, vc, lens.to(dev), table.to(dev))
    torch.cuda.synchronize()
    small_table, (kcs, vcs) = _compact(table, kc, vc)
    _close(out, oa.paged_decode_attention(q.squeeze(1), kcs, vcs, lens, small_table), 2e-2)


def test_fp8_decode_over_chunks_beyond_2_gib(mi, dev, pool):
    kc, vc = pool
    k8 = torch.empty(kc.shape, dtype=torch.uint8, device=dev)     # 2.5 GiB per tensor
    v8 = torch.empty_like(k8)
    ks = torch.empty(N_POOL, HKV, dtype=torch.float32, device=dev)
    vs = torch.empty_like(ks)
    mi.ops.quantize_chunks_fp8(kc, k8, ks)
    mi.ops.quantize_chunks_fp8(vc, v8, vs)
    gen = torch.Generator().manual_seed(2)
    lens = torch.tensor([900, 2500, 64, 4000], dtype=torch.int32)
    table = _table(lens, gen)
    q = torch.randn(lens.numel(), 1, 32, D, generator=gen).bfloat16()
    out = mi.ops.paged_decode_attention(q.to(dev), k8, v8, lens.to(dev), table.to(dev), k_scales=ks, v_scales=vs)
    torch.cuda.synchronize()
    small_table, (k8s, v8s, kss, vss) = _compact(table, k8, v8, ks, vs)
    ref = oa.paged_decode_attention(q.squeeze(1), k8s, v8s, lens, small_table, k_scales=kss, v_scales=vss)
    _close(out, ref, 2.5e-2)
    # the quantiser itself on the high chunks: bytes and scales equal the checker's
    used = table[table >= 0].unique().long()
    hi = used[used > 8192][:3]
    ref8, refs = oa.quantize_chunks_fp8(kc[hi.to(dev)].cpu())
    assert torch.equal(k8[hi.to(dev)].cpu(), ref8) and torch.equal(ks[hi.to(dev)].cpu(), refs)


def test_mixed_prefill_over_chunks_beyond_4_gib(mi, dev, pool):
    kc, vc = pool
    gen = torch.Generator().manual_seed(3)
    q_lens = [300, 1, 700, 1, 64]
    ctx = [100, 2000, 0, 511, 3000]
    lens = torch.tensor([a + b for a, b in zip(q_lens, ctx)], dtype=torch.int32)
    cu_q = torch.zeros(len(q_lens) + 1, dtype=torch.int32)
    cu_q[1:] = torch.cumsum(torch.tensor(q_lens), 0)
    table = _table(lens, gen)
    q = torch.randn(int(cu_q[-1]), 32, D, generator=gen).bfloat16()
    out = mi.ops.paged_prefill_attention(q.to(dev), kc, vc, cu_q.to(dev), lens.to(dev), table.to(dev))
    torch.cuda.synchronize()
    small_table, (kcs, vcs) = _compact(table, kc, vc)
    _close(out, oa.paged_varlen_attention(q, kcs, vcs, cu_q, lens, small_table), 2e-2)


def test_appends_into_high_chunks(mi, dev, pool):
    kc, vc = pool
    gen = torch.Generator().manual_seed(4)
    q_lens = [5, 1, 300]
    ctx = [250, 1023, 0]
    lens = torch.tensor([a + b for a, b in zip(q_lens, ctx)], dtype=torch.int32)
    cu_q = torch.zeros(len(q_lens) + 1, dtype=torch.int32)
    cu_q[1:] = torch.cumsum(torch.tensor(q_lens), 0)
    table = _table(lens, gen)
    pos, ci, lo = mi.synthetic.prefill_token_rows(cu_q, lens, table, C)
    T = int(cu_q[-1])
    k = torch.randn(T, 1, HKV, D, generator=gen).bfloat16()
    v = torch.randn(T, 1, HKV, D, generator=gen).bfloat16()
    used = table[table >= 0].unique().long()
    before_k, before_v = kc[used.to(dev)].cpu(), vc[used.to(dev)].cpu()
    # plain scatter
    mi.ops.kv_append(k.to(dev), v.to(dev), kc, vc, ci.to(dev), lo.to(dev))
    torch.cuda.synchronize()
    small_table, (kcs, vcs) = _compact(table, kc, vc)
    _, sci, slo = mi.synthetic.prefill_token_rows(cu_q, lens, small_table, C)
    oa.kv_append(before_k, before_v, k.squeeze(1), v.squeeze(1), sci, slo)
    assert torch.equal(kcs.view(torch.int16), before_k.view(torch.int16))
    assert torch.equal(vcs.view(torch.int16), before_v.view(torch.int16))
    # fused norm + rotary + append: the raw value rows land bit-exact, the rotated keys within tolerance
    q = torch.randn(T, 1, 32, D, generator=gen).bfloat16()
    w = (1 + 0.02 * torch.randn(D, generator=gen)).bfloat16()
    table_rot = orn.rotary_table(int(lens.max()) + 1, D, base=500000.0)
    k2 = torch.randn(T, 1, HKV, D, generator=gen).bfloat16()
    v2 = torch.randn(T, 1, HKV, D, generator=gen).bfloat16()
    mi.ops.norm_rope_append(q.to(dev), k2.to(dev), value=v2.to(dev), q_weight=w.to(dev), k_weight=w.to(dev), eps=1e-5,
                            norm="rms", rotary_emb=table_rot.to(dev), q_positions=pos.to(dev), k_positions=pos.to(dev),
                            k_cache=kc, v_cache=vc, token_to_chunk_idx=ci.to(dev), token_to_local_pos=lo.to(dev))
    torch.cuda.synchronize()
    _, (kcs, vcs) = _compact(table, kc, vc)
    k_ref = orn.norm_rope(k2.squeeze(1), pos, table_rot, norm="rms", weight=w, eps=1e-5)
    oa.kv_append(before_k, before_v, k_ref, v2.squeeze(1), sci, slo)
    assert torch.equal(vcs.view(torch.int16), before_v.view(torch.int16))
    err = (kcs.float() - before_k.float()).abs()
    assert (err <= 2e-2 + 2e-2 * before_k.float().abs()).all()


def test_mla_decode_over_a_latent_cache_beyond_4_gib(mi, dev, pool):
    del pool  # (only to run after the tests that need it; this cache is its own allocation)
    free, _ = torch.cuda.mem_get_info()
    n = 15000                                   # 15000 x 256 x 576 x 2 B = 4.1 GiB
    if free < 6 * 2**30:
        pytest.skip("needs 6 GiB of free device memory")
    gen_d = torch.Generator(device=dev).manual_seed(5)
    cache = mi.synthetic.randn_fill_(torch.empty(n, C, 576, dtype=torch.bfloat16, device=dev), gen_d)
    cache.mul_(0.5)
    gen = torch.Generator().manual_seed(6)
    lens = torch.tensor([2000, 300, 5000, 1], dtype=torch.int32)
    need = [(int(l) + C - 1) // C for l in lens]
    ids = [n - 2, n - 3, 0, 14563, 14564, 7281, 7282] + torch.randperm(n - 4, generator=gen).tolist()
    ids = list(dict.fromkeys(ids))[:sum(need)]
    table = torch.full((len(need), max(need)), -1, dtype=torch.int32)
    at = 0
    for r, k in enumerate(need):
        table[r, :k] = torch.tensor(ids[at:at + k], dtype=torch.int32)
        at += k
    assert (table.long() * C * 576 * 2).max() > 2**32
    for Hq in (16, 128):
        q = torch.randn(lens.numel(), 1, Hq, 576, generator=gen).bfloat16()
        out = mi.ops.paged_mla_decode_attention(q.to(dev), cache, lens.to(dev), table.to(dev), softmax_scale=0.07)
        torch.cuda.synchronize()
        used = table[table >= 0].unique().long()
        remap = torch.full((n,), -1, dtype=torch.int32)
        remap[used] = torch.arange(used.numel(), dtype=torch.int32)
        small = torch.where(table >= 0, remap[table.clamp(min=0).long()], table)
        ref = oa.mla_decode_attention(q.squeeze(1), cache[used.to(dev)].cpu(), lens, small, 0.07, 512)
        _close(out.squeeze(1), ref, 2e-2)
