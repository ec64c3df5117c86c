"""Pins for the CPU checker of paged attention / KV append / fp8 storage (no GPU needed).

Each test is chosen so that a plausible mistake in the checker (wrong head pairing, mask off by
one, wrong chunk addressing, dropped scale, wrong merge weight) fails at least one of them.
"""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import paged_attention as oa


def _paged(B, Hq, Hkv, d, chunk, lens, seed):
    g = torch.Generator().manual_seed(seed)
    need = [(l + chunk - 1) // chunk for l in lens]
    N = sum(need) + 3
    perm = torch.randperm(N - 1, generator=g)
    M = max(need + [1])
    bt = torch.full((B, M), -1, dtype=torch.int32)
    at = 0
    for r, n in enumerate(need):
        bt[r, :n] = perm[at:at + n].int()
        at += n
    kc = torch.randn(N, chunk, Hkv, d, generator=g)
    vc = torch.randn(N, chunk, Hkv, d, generator=g)
    q = torch.randn(B, Hq, d, generator=g)
    return q, kc, vc, torch.tensor(lens, dtype=torch.int32), bt


def _brute_force(q, kc, vc, lens, bt, chunk, shift_for=None):
    """fp64 scalar loops straight from the definition."""
    B, Hq, d = q.shape
    Hkv = kc.size(2)
    G = Hq // Hkv
    out = torch.zeros(B, Hq, d, dtype=torch.float64)
    for r in range(B):
        for h in range(Hq):
            L = int(lens[r])
            if L == 0:
                continue
            s = []
            for j in range(L):
                krow = kc[int(bt[r, j // chunk]), j % chunk, h // G].double()
                s.append(float((q[r, h].double() * krow).sum()) / math.sqrt(d))
            m = max(s)
            w = [math.exp(x - m) for x in s]
            z = sum(w)
            for j in range(L):
                out[r, h] += (w[j] / z) * vc[int(bt[r, j // chunk]), j % chunk, h // G].double()
    return out


def test_decode_matches_fp64_brute_force():
    q, kc, vc, lens, bt = _paged(3, 4, 2, 8, 4, [1, 6, 9], seed=0)
    ref = _brute_force(q, kc, vc, lens, bt, 4)
    got = oa.paged_decode_attention(q, kc, vc, lens, bt)
    assert (got.double() - ref).abs().max() < 1e-5


def test_decode_matches_library_sdpa_with_repeated_kv_heads():
    """Gather, repeat every KV head G times (the reference's GQA expansion), library SDPA."""
    chunk = 16
    q, kc, vc, lens, bt = _paged(4, 8, 2, 32, chunk, [5, 16, 17, 70], seed=1)
    got = oa.paged_decode_attention(q, kc, vc, lens, bt)
    for r in range(4):
        L = int(lens[r])
        k = oa.gather_request_kv(kc, bt[r], L).repeat_interleave(4, dim=1)  # [L, Hq, d]
        v = oa.gather_request_kv(vc, bt[r], L).repeat_interleave(4, dim=1)
        ref = F.scaled_dot_product_attention(q[r].unsqueeze(1), k.transpose(0, 1), v.transpose(0, 1))  # [Hq,1,d]
        assert (got[r] - ref.squeeze(1)).abs().max() < 1e-5


def test_varlen_bottom_right_causal_mask_matches_sdpa_with_explicit_mask():
    chunk, Hq, Hkv, d = 8, 4, 2, 16
    q_lens, ctx = [1, 3, 7, 5], [9, 0, 4, 11]
    kv = [a + b for a, b in zip(q_lens, ctx)]
    _, kc, vc, lens, bt = _paged(4, Hq, Hkv, d, chunk, kv, seed=2)
    cu = torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32)
    q = torch.randn(int(cu[-1]), Hq, d, generator=torch.Generator().manual_seed(3))
    got = oa.paged_varlen_attention(q, kc, vc, cu, lens, bt)
    for r in range(4):
        a, b, L = int(cu[r]), int(cu[r + 1]), kv[r]
        k = oa.gather_request_kv(kc, bt[r], L).repeat_interleave(2, dim=1).transpose(0, 1)
        v = oa.gather_request_kv(vc, bt[r], L).repeat_interleave(2, dim=1).transpose(0, 1)
        Lq = b - a
        mask = torch.arange(L).view(1, L) <= torch.arange(Lq).view(Lq, 1) + (L - Lq)
        ref = F.scaled_dot_product_attention(q[a:b].transpose(0, 1), k, v, attn_mask=mask).transpose(0, 1)
        assert (got[a:b] - ref).abs().max() < 1e-5
    # the last new token sees everything, the first sees exactly ctx+1 keys
    r = 2
    a = int(cu[r])
    k = oa.gather_request_kv(kc, bt[r], ctx[r] + 1)
    v = oa.gather_request_kv(vc, bt[r], ctx[r] + 1)
    first = oa.attention_one_request(q[a:a + 1], k, v, d ** -0.5, None)
    assert (got[a] - first[0]).abs().max() < 1e-5


def test_special_cases_single_key_and_equal_keys_and_zero_length():
    q, kc, vc, lens, bt = _paged(3, 4, 2, 8, 4, [1, 7, 0], seed=4)
    kc[:] = kc[0, 0, 0]  # all keys equal -> uniform weights
    got = oa.paged_decode_attention(q, kc, vc, lens, bt)
    v0 = oa.gather_request_kv(vc, bt[0], 1)[0].repeat_interleave(2, dim=0)  # single key -> V itself
    assert (got[0] - v0).abs().max() < 1e-6
    v1 = oa.gather_request_kv(vc, bt[1], 7).mean(0).repeat_interleave(2, dim=0)
    assert (got[1] - v1).abs().max() < 1e-6
    assert (got[2] == 0).all()


def test_invariant_under_physical_chunk_permutation():
    chunk = 8
    q, kc, vc, lens, bt = _paged(3, 4, 4, 16, chunk, [20, 3, 33], seed=5)
    a = oa.paged_decode_attention(q, kc, vc, lens, bt)
    N = kc.size(0)
    perm = torch.randperm(N, generator=torch.Generator().manual_seed(6))
    k2, v2 = torch.empty_like(kc), torch.empty_like(vc)
    k2[perm], v2[perm] = kc, vc
    bt2 = torch.where(bt >= 0, perm[bt.clamp(min=0).long()].int(), bt)
    b = oa.paged_decode_attention(q, k2, v2, lens, bt2)
    assert torch.equal(a, b)


def test_lse_merge_equals_single_pass():
    g = torch.Generator().manual_seed(7)
    q = torch.randn(1, 8, 16, generator=g)
    k = torch.randn(50, 2, 16, generator=g)
    v = torch.randn(50, 2, 16, generator=g)
    full, _ = oa.attention_with_lse(q, k, v, 0.25)
    parts, lses = [], []
    for a, b in ((0, 7), (7, 8), (8, 40), (40, 50)):
        o, l = oa.attention_with_lse(q, k[a:b], v[a:b], 0.25)
        parts.append(o)
        lses.append(l)
    merged = oa.lse_merge(parts, lses)
    assert (merged - full).abs().max() < 1e-5
    # weights are e^{lse}: doubling one partial's lse weight must change the result
    lses2 = [lses[0] + 1.0] + lses[1:]
    assert (oa.lse_merge(parts, lses2) - full).abs().max() > 1e-3


def test_kv_append_and_decode_slots():
    chunk = 4
    kc = torch.full((6, chunk, 2, 3), -1.0)
    vc = torch.full((6, chunk, 2, 3), -1.0)
    bt = torch.tensor([[4, 1, -1], [2, -1, -1], [0, 3, 5]], dtype=torch.int32)
    lens = torch.tensor([5, 0, 12], dtype=torch.int32)
    rows, ids, loc = oa.decode_slots(bt, lens, chunk)
    assert rows.tolist() == [0, 2] and ids.tolist() == [1, 5] and loc.tolist() == [0, 3]
    key = torch.arange(3 * 2 * 3, dtype=torch.float32).view(3, 2, 3)
    oa.kv_append(kc, vc, key[rows], -key[rows], ids, loc)
    assert torch.equal(kc[1, 0], key[0]) and torch.equal(vc[5, 3], -key[2])
    untouched = torch.ones(6, chunk, dtype=torch.bool)
    untouched[1, 0] = untouched[5, 3] = False
    assert (kc[untouched] == -1).all() and (vc[untouched] == -1).all()


def test_fp8_quantiser_against_known_e4m3_values():
    """OCP e4m3fn: max 448, 3 mantissa bits, round to nearest even, scale = amax/448 per (chunk, head)."""
    x = torch.zeros(1, 4, 2, 4)
    x[0, 0, 0] = torch.tensor([448.0, -224.0, 1.0, 0.0])      # head 0: amax 448 -> scale 1
    x[0, 1, 0] = torch.tensor([17.0, 19.0, 0.001, -447.0])     # 17 -> 16 (tie to even), 19 -> 20, tiny -> subnormal/0
    x[0, 0, 1] = torch.tensor([2.0, -1.0, 0.5, 0.25])          # head 1: amax 2 -> scale 2/448
    q, s = oa.quantize_chunks_fp8(x.bfloat16())
    assert s[0, 0].item() == 1.0 and abs(s[0, 1].item() - 2.0 / 448.0) < 1e-9
    deq = oa.dequantize_fp8(q, s)
    assert deq[0, 0, 0].tolist() == [448.0, -224.0, 1.0, 0.0]
    assert deq[0, 1, 0, 0].item() == 16.0 and deq[0, 1, 0, 1].item() == 20.0 and deq[0, 1, 0, 3].item() == -448.0
    assert torch.allclose(deq[0, 0, 1], torch.tensor([2.0, -1.0, 0.5, 0.25]))
    assert q[0, 0, 0, 0].item() == 0x7E  # 448 = 0b0.1111.110
    # relative error of a normal value is at most 2^-4
    y = torch.randn(3, 8, 2, 16).bfloat16()
    q, s = oa.quantize_chunks_fp8(y)
    d = oa.dequantize_fp8(q, s)
    big = y.float().abs() > 0.1
    assert ((d - y.float()).abs()[big] / y.float().abs()[big]).max() <= 2 ** -4 + 1e-6


def test_decode_attention_bytes_formula():
    # 2 requests of 300 and 256 tokens, 8 KV heads, d 128, bf16: KV rows + q/out + table + lengths
    n = oa.decode_attention_bytes([300, 256], 32, 8, 128, 256)
    assert n == (300 + 256) * 8 * 128 * 2 * 2 + 2 * 32 * 128 * 4 + (2 + 1) * 4 + 2 * 4
    n8 = oa.decode_attention_bytes([300, 256], 32, 8, 128, 256, kv_bytes=1, fp8_scales=True)
    assert n8 == (300 + 256) * 8 * 128 * 2 + 2 * 32 * 128 * 4 + 3 * 4 + 2 * 4 + 3 * 8 * 2 * 4


def test_fp8_append_policy_pins():
    """The many-token append policy: a run that fills a chunk is the whole-chunk quantiser; a run that
    stops short gets headroom; a run that continues a chunk keeps the stored scale and saturates."""
    g = torch.Generator().manual_seed(12)
    C, Hkv, d = 16, 2, 8
    rows = (torch.randn(40, Hkv, d, generator=g) * 2).bfloat16()
    cache = torch.zeros(4, C, Hkv, d, dtype=torch.uint8)
    scales = torch.full((4, Hkv), 0.125)
    chunk_idx = torch.tensor([2] * 16 + [0] * 10 + [3] * 14)
    local = torch.tensor(list(range(16)) + list(range(10)) + list(range(2, 16)))
    oa.kv_append_fp8(cache, scales, rows, chunk_idx, local, headroom=2.0)
    full = rows[:16].reshape(1, C, Hkv, d)
    b, s = oa.quantize_chunks_fp8(full)
    assert torch.equal(cache[2], b[0]) and torch.equal(scales[2], s[0])
    amax = rows[16:26].float().abs().amax(dim=(0, 2))
    assert torch.equal(scales[0], 2.0 * amax / 448.0)            # opened but not filled: headroom 2
    assert (cache[0, 10:] == 0).all()                            # slots after the run untouched
    assert torch.equal(scales[3], torch.full((Hkv,), 0.125))     # continued chunk: scale kept
    want = oa.quantize_token_fp8(rows[26], scales[3])
    assert torch.equal(cache[3, 2], want) and (cache[3, :2] == 0).all()
    # 448 * 0.125 = 56 is the largest magnitude the kept scale can hold: larger values saturate to 0x7e / 0xfe
    big = torch.full((1, Hkv, d), 100.0).bfloat16()
    oa.kv_append_fp8(cache, scales, big, torch.tensor([3]), torch.tensor([0 + 1]), headroom=2.0)
    assert (cache[3, 1] == 0x7E).all()


def test_mla_decode_checker_against_library_attention_and_brute_force():
    """Latent-cache decode: scores over the whole shared row, values = its first dv columns.  Pinned by the
    library's scaled_dot_product_attention (which takes a narrower value) and by fp64 loops."""
    g = torch.Generator().manual_seed(31)
    R, Hq, dk, dv, C = 3, 5, 24, 16, 8
    lens = torch.tensor([13, 1, 0], dtype=torch.int32)
    N = 6
    cache = torch.randn(N, C, dk, generator=g)
    bt = torch.tensor([[4, 1, -1], [2, -1, -1], [-1, -1, -1]], dtype=torch.int32)
    q = torch.randn(R, Hq, dk, generator=g)
    scale = 0.37
    out = oa.mla_decode_attention(q, cache, lens, bt, scale, dv)
    assert out.shape == (R, Hq, dv) and (out[2] == 0).all()
    for r in range(2):
        L = int(lens[r])
        rows = torch.cat([cache[int(c)] for c in bt[r, : (L + C - 1) // C]])[:L]
        want = F.scaled_dot_product_attention(q[r][None, :, None, :], rows[None, None].expand(1, Hq, L, dk),
                                              rows[None, None, :, :dv].expand(1, Hq, L, dv), scale=scale)[0, :, 0]
        assert torch.allclose(out[r], want, atol=1e-5)
        for h in range(Hq):  # brute force
            s = [sum(float(q[r, h, i]) * float(rows[j, i]) for i in range(dk)) * scale for j in range(L)]
            m = max(s)
            w = [math.exp(x - m) for x in s]
            for e in (0, dv - 1):
                ref = sum(w[j] * float(rows[j, e]) for j in range(L)) / sum(w)
                assert abs(float(out[r, h, e]) - ref) < 1e-5
