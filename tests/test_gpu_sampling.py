"""GPU: last-token gather, sampling and the finished-request mask (through the C ABI).

Bars.  The gather, the argmax, the top-k cut and the mask are integer / selection work: equality
with the checker.  The top-p cut and the draw depend on sums of exponentials, which the kernel
carries as 2^-32 fixed point and the checker in fp64: a result must equal the checker's whenever
the checker's decision has a margin (2e-6 of the total mass: the
kernel's exponentials are fp32), and must in every case satisfy the definition within that margin
(mass strictly above the cut <= top_p < mass down to the cut; CDF bracket of the drawn index).
"""
from types import SimpleNamespace

import pytest
import torch

from oracle import sampling as osm

pytestmark = pytest.mark.gpu

TOL = 2e-6        # top-p cut: distance of the kept mass from top_p
DRAW_TOL = 2e-6   # draw: distance of u from the CDF steps either side of the drawn index


def _logits(R, V, seed, dtype=torch.float32, spread=3.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(R, V, generator=g) * spread).to(dtype)


# ----------------------------------------------------------------------------------------------
# last-token gather
# ----------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype,E", [(torch.bfloat16, 4096), (torch.float32, 1000), (torch.bfloat16, 37),
                                     (torch.float32, 128256), (torch.bfloat16, 3)])
def test_last_token_gather_bit_exact(mi, dev, dtype, E):
    g = torch.Generator().manual_seed(E)
    q_lens = torch.randint(1, 40, (300,), generator=g, dtype=torch.int32)
    q_lens[5:150] = 1
    if E > 100000:
        q_lens = q_lens[:12]
    T = int(q_lens.sum()) + 7  # padding rows at the end
    rows = torch.randn(T, E, generator=g).to(dtype).to(dev)
    got = mi.ops.last_token_gather(rows, q_lens.to(dev))
    want = rows.cpu()[osm.last_token_indices(q_lens)]
    assert got.dtype == dtype and torch.equal(got.cpu(), want)


def test_last_token_gather_strided_source(mi, dev):
    g = torch.Generator().manual_seed(3)
    q_lens = torch.tensor([4, 1, 9, 2], dtype=torch.int32)
    big = torch.randn(16, 96, generator=g).bfloat16().to(dev)
    rows = big[:, 8:72]  # row stride 96, offset 16 bytes
    got = mi.ops.last_token_gather(rows, q_lens.to(dev))
    assert torch.equal(got.cpu(), rows.cpu()[osm.last_token_indices(q_lens)])
    assert mi.ops.last_token_gather(rows, q_lens[:0].to(dev)).shape == (0, 64)


# ----------------------------------------------------------------------------------------------
# greedy
# ----------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("V", [1, 63, 1000, 32000, 128256])
def test_greedy_is_first_argmax(mi, dev, dtype, V):
    x = _logits(9, V, V, dtype)
    if V >= 63:
        x[1, :] = 0.5                      # all equal -> index 0
        x[2, 40] = x[2].max()              # two equal maxima -> the lower index
        x[2, 7] = x[2, 40]
        x[3, 10] = 0.0
        x[3, 20] = -0.0                    # signed zeros compare equal
        x[3] = torch.where(x[3] > 0, -x[3], x[3])
        x[3, 10], x[3, 20] = -0.0, 0.0
        x[4, V - 1] = 1e4                  # last element
        x[5, 5] = float("inf")
        x[6, :] = float("-inf")
    s, mask = mi.ops.sample_from_logits(x.to(dev), top_k=1)
    assert mask is None and s.dtype == torch.int64
    assert torch.equal(s.cpu(), osm.sample_from_logits(x, top_k=1))


# ----------------------------------------------------------------------------------------------
# filters
# ----------------------------------------------------------------------------------------------
def _check_draw(x_scaled, cut, u, s):
    """CDF bracket of every drawn index for the kept set {x >= cut}; returns the fp64 probabilities."""
    keep = x_scaled >= cut[:, None]
    pr = osm.kept_probabilities(x_scaled, keep)
    cdf = pr.cumsum(-1)
    R = x_scaled.size(0)
    idx = torch.arange(R)
    assert keep[idx, s].all(), "a filtered entry was drawn"
    assert (pr[idx, s] > 0).all()
    hi = cdf[idx, s]
    lo = hi - pr[idx, s]
    want = u.double()
    assert ((lo - DRAW_TOL <= want) & (want <= hi + DRAW_TOL)).all()
    exact = osm.draw_inverse_cdf(pr, u)
    clear = ((want - lo).abs() > DRAW_TOL) & ((hi - want).abs() > DRAW_TOL)
    assert clear.any() and torch.equal(s[clear], exact[clear])
    return pr


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("V,k", [(64, 2), (1000, 50), (32000, 40), (128256, 2), (128256, 50), (128256, 5000),
                                 (777, 777)])
@pytest.mark.parametrize("temperature", [1.0, 0.7])
def test_top_k_cut_is_exact_and_draw_brackets(mi, dev, dtype, V, k, temperature):
    R = 16
    x = _logits(R, V, 7 * V + k, dtype)
    if V > 100:
        x[3, 100:100 + min(60, V - 100)] = x[3].float().topk(k).values[-1]  # many ties at the k-th value
        x[4, V // 2:] = float("-inf")  # pre-masked entries
    if k > V // 2:
        x[4] = _logits(1, V, 5, dtype)[0]
    u = torch.rand(R, generator=torch.Generator().manual_seed(k))
    s, _, cut = mi.ops.sample_from_logits(x.to(dev), top_k=k, temperature=temperature, uniform=u.to(dev),
                                          return_cut=True)
    xs = osm.scaled_logits(x, temperature)
    kth = torch.topk(xs, k, dim=-1).values[:, -1]
    assert torch.equal(cut.cpu(), kth)
    _check_draw(xs, kth, u, s.cpu())
    # the same call again gives the same tokens (integer sums)
    s2, _ = mi.ops.sample_from_logits(x.to(dev), top_k=k, temperature=temperature, uniform=u.to(dev))
    assert torch.equal(s, s2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("V", [50, 1000, 32000, 128256])
@pytest.mark.parametrize("top_p", [0.05, 0.5, 0.9, 0.999])
def test_top_p_cut_meets_the_definition(mi, dev, dtype, V, top_p):
    R = 16
    spread = 3.0 if V < 100000 else 4.0
    x = _logits(R, V, 11 * V + int(top_p * 1000), dtype, spread)
    x[2] *= 0.05           # nearly flat row: the prefix is long
    x[5, V // 3:] = float("-inf")
    u = torch.rand(R, generator=torch.Generator().manual_seed(V))
    _check_top_p(mi, dev, x, top_p, 0.9, u)


def _check_top_p(mi, dev, x, top_p, temperature, u):
    s, _, cut = mi.ops.sample_from_logits(x.to(dev), top_p=top_p, temperature=temperature, uniform=u.to(dev),
                                          return_cut=True)
    cut = cut.cpu()
    xs = osm.scaled_logits(x, temperature)
    pr = xs.double().softmax(-1)
    above = (pr * (xs > cut[:, None])).sum(-1)          # mass strictly above the cut value
    down_to = (pr * (xs >= cut[:, None])).sum(-1)       # ... including it
    assert (above <= top_p + TOL).all() and (down_to > top_p - TOL).all()
    # equality with the checker's kept set wherever its decision is not within the margin
    keep = osm.top_p_keep(xs, top_p)
    want_cut = xs.masked_fill(~keep, float("inf")).min(-1).values
    clear = ((above - top_p).abs() > TOL) & ((down_to - top_p).abs() > TOL)
    assert torch.equal(cut[clear], want_cut[clear])
    _check_draw(xs, cut, u, s.cpu())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("top_p", [0.3, 0.9])
def test_top_p_one_pass_form_and_its_fallbacks(mi, dev, dtype, top_p):
    """Top-p on rows of 32 768: peaked rows find their cut among the listed candidates, the others (flat, nearly
    flat, a few finite values, half the row tied at the top) go through the general path; both must meet the
    definition."""
    V = 32768
    x = _logits(10, V, 1200 + int(10 * top_p), dtype, spread=5.0)   # rows 7-9: peaked random rows
    x[0, :] = -0.75
    x[1, :] = float("-inf"); x[1, [5, 17000, 32767]] = torch.tensor([0.5, 1.5, 1.0], dtype=dtype)
    x[2, :] = 0.25; x[2, 12345] = 9.0
    x[3, : V // 2] = 3.0
    x[4, ::2] = float("-inf")
    x[5] = (torch.arange(V).float() / V * 30).to(dtype)
    x[6] *= 0.02
    u = torch.rand(10, generator=torch.Generator().manual_seed(int(100 * top_p)))
    _check_top_p(mi, dev, x, top_p, 1.0, u)


def test_no_filter_draws_from_the_full_softmax(mi, dev):
    x = _logits(32, 5000, 21)
    u = torch.rand(32, generator=torch.Generator().manual_seed(22))
    s, _, cut = mi.ops.sample_from_logits(x.to(dev), temperature=1.3, uniform=u.to(dev), return_cut=True)
    assert torch.isinf(cut).all() and (cut < 0).all()
    _check_draw(osm.scaled_logits(x, 1.3), cut.cpu(), u, s.cpu())
    # top_p = 1 filters nothing either
    s1, _ = mi.ops.sample_from_logits(x.to(dev), top_p=1.0, temperature=1.3, uniform=u.to(dev))
    assert torch.equal(s1, s)


@pytest.mark.parametrize("mode", [dict(top_k=6), dict(top_p=0.8), dict()])
def test_draw_frequencies_follow_the_kept_probabilities(mi, dev, mode):
    V, n = 48, 1 << 16
    row = _logits(1, V, 31)[0]
    x = row.expand(n, V).contiguous()
    u = torch.rand(n, generator=torch.Generator().manual_seed(32))
    s, _ = mi.ops.sample_from_logits(x.to(dev), uniform=u.to(dev), **mode)
    if "top_k" in mode:
        keep = osm.top_k_keep(row[None], mode["top_k"])
    elif "top_p" in mode:
        keep = osm.top_p_keep(row[None], mode["top_p"])
    else:
        keep = torch.ones(1, V, dtype=torch.bool)
    pr = osm.kept_probabilities(row[None], keep)[0]
    freq = torch.bincount(s.cpu(), minlength=V).double() / n
    assert (freq[~keep[0]] == 0).all()
    sigma = (pr * (1 - pr) / n).sqrt()
    assert ((freq - pr).abs() <= 5 * sigma + 1e-6).all()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("k", [2, 10, 200, 256, 257, 768, 769])
def test_top_k_one_pass_form_and_its_fallbacks(mi, dev, dtype, k):
    """Rows of 32 768 and a small k take the form that lists candidates above a sampled threshold in one pass; rows
    where the estimate cannot work -- flat (every value a candidate), a few finite values (fewer candidates than k),
    a spike in an otherwise flat row, half the row tied at the maximum -- must come out the same through the general
    path.  k = 769 never takes the one-pass form."""
    V = 32768
    x = _logits(10, V, 900 + k, dtype)
    x[0, :] = -0.75                                             # flat: every entry equals the cut
    x[1, :] = float("-inf"); x[1, [5, 17000, 32767]] = torch.tensor([0.5, 1.5, 1.0], dtype=dtype)  # three finite values
    x[2, :] = 0.25; x[2, 12345] = 9.0                           # one spike over a flat row
    x[3, : V // 2] = 3.0                                        # half the row tied at the top
    x[4, ::2] = float("-inf")                                   # every other entry pre-masked
    x[5] = (torch.arange(V).float() / V).to(dtype)              # sorted ascending: the sample sees every level
    x[6] = (torch.arange(V, 0, -1).float() / V).to(dtype)
    u = torch.rand(10, generator=torch.Generator().manual_seed(k))
    s, _, cut = mi.ops.sample_from_logits(x.to(dev), top_k=k, uniform=u.to(dev), return_cut=True)
    xs = osm.scaled_logits(x, 1.0)
    kth = torch.topk(xs, k, dim=-1).values[:, -1]
    assert torch.equal(cut.cpu(), kth)
    _check_draw(xs, kth, u, s.cpu())
    assert s[1].item() in (5, 17000, 32767) and (k > 1 and s[2].item() >= 0)
    s2, _ = mi.ops.sample_from_logits(x.to(dev), top_k=k, uniform=u.to(dev))
    assert torch.equal(s, s2)


def test_extreme_rows(mi, dev):
    V = 4096
    x = _logits(6, V, 41)
    x[0, :] = 1.25                       # flat row: every entry equals the cut, all are kept
    x[1, 9] = float("inf")               # no distribution: argmax
    x[2, 100] = 80.0                     # one entry holds all the mass
    x[3, :] = float("-inf"); x[3, 77] = 0.0
    x[4, 5] = float("nan")               # NaN counts as the maximum, as in torch.argmax
    u = torch.tensor([0.5, 0.3, 0.9999, 0.2, 0.1, 0.7])
    for mode in (dict(top_k=10), dict(top_p=0.9), dict()):
        s, _ = mi.ops.sample_from_logits(x.to(dev), uniform=u.to(dev), **mode)
        s = s.cpu()
        assert s[0].item() == int(0.5 * V) or abs(s[0].item() - 0.5 * V) <= 1
        assert s[1].item() == 9 and s[2].item() == 100 and s[3].item() == 77 and s[4].item() == 5
        assert 0 <= s[5].item() < V
    # clamp to the tokenizer's vocabulary (sampling path only)
    x = _logits(64, 300, 42)
    u = torch.rand(64, generator=torch.Generator().manual_seed(43))
    s, _ = mi.ops.sample_from_logits(x.to(dev), uniform=u.to(dev))
    sc, _ = mi.ops.sample_from_logits(x.to(dev), uniform=u.to(dev), vocab_size=100)
    assert torch.equal(sc, s.clamp(0, 99)) and (s > 99).any()


def test_argument_errors(mi, dev):
    x = _logits(4, 100, 51).to(dev)
    u = torch.rand(4).to(dev)
    with pytest.raises(mi._lib.KernelError, match="top-k is larger"):
        mi.ops.sample_from_logits(x, top_k=101, uniform=u)
    with pytest.raises(mi._lib.KernelError, match="both greater than zero"):
        mi.ops.sample_from_logits(x, top_k=5, top_p=0.5, uniform=u)
    with pytest.raises(mi._lib.KernelError, match="temperature"):
        mi.ops.sample_from_logits(x, temperature=0.0, uniform=u)
    with pytest.raises(ValueError, match="uniform"):
        mi.ops.sample_from_logits(x, top_k=5)
    with pytest.raises(ValueError):
        mi.ops.sample_from_logits(x.double(), top_k=1)
    with pytest.raises(RuntimeError, match="no CPU path"):
        mi.ops.sample_from_logits(x.cpu(), top_k=1)
    s, m = mi.ops.sample_from_logits(x[:0], top_k=1)
    assert s.numel() == 0


# ----------------------------------------------------------------------------------------------
# the reference's surface and the finished-request mask
# ----------------------------------------------------------------------------------------------
def test_sample_from_logits_surface(mi, dev):
    x = _logits(8, 2000, 61).to(dev)
    params = SimpleNamespace(top_k=1, top_p=0.0, temperature=1.0)
    assert torch.equal(mi.sampling.sample_from_logits(x, params).cpu(), x.cpu().argmax(-1))
    before = x.clone()
    params = SimpleNamespace(top_k=0, top_p=0.9, temperature=0.8)
    g = torch.Generator(device=dev).manual_seed(5)
    a = mi.sampling.sample_from_logits(x, params, vocab_size=2000, generator=g)
    g.manual_seed(5)
    b = mi.sampling.sample_from_logits(x, params, vocab_size=2000, generator=g)
    assert torch.equal(a, b) and torch.equal(x, before)
    with pytest.raises(AssertionError, match="both greater than zero"):
        mi.sampling.sample_from_logits(x, SimpleNamespace(top_k=2, top_p=0.5, temperature=1.0))
    with pytest.raises(AssertionError, match="larger than vocab size"):
        mi.sampling.sample_from_logits(x, SimpleNamespace(top_k=50, top_p=0.0, temperature=1.0), vocab_size=50)
    with pytest.raises(AssertionError):
        mi.sampling.sample_from_logits(x, SimpleNamespace(top_k=2.0, top_p=0.0, temperature=1.0))


def test_decode_step_tail_on_a_context(mi, dev):
    """logits -> last-token rows -> sample + mask -> update_requests, against the checker."""
    Ctx = mi.DynamicInferenceContext
    c = Ctx(params_dtype=torch.bfloat16, num_layers=1, kv_channels=16, num_attention_heads=2,
            max_sequence_length=128, buffer_size_gb=0.01, buffer_guaranteed_fraction=0.1, chunk_size_tokens=16,
            device=dev)
    g = torch.Generator().manual_seed(71)
    V, term = 500, 3
    prompts = [5, 17, 1, 30, 9, 2]
    budgets = [3, 50, 2, 40, 1, 60]   # requests 0, 2 and 4 run out of length soon
    for i, (n, b) in enumerate(zip(prompts, budgets)):
        c.add_request(i, torch.randint(10, V, (n,), generator=g).to(dev), num_tokens_to_generate=b)
    for step in range(3):
        c.initialize_attention_state()
        T = c.padded_active_token_count
        logits = (torch.randn(1, T, V, generator=g) * 3).bfloat16().to(dev)
        if step == 1:
            logits[0, :, term] = 50.0  # everyone draws the termination id
        n = c.total_request_count - c.paused_request_count
        act = slice(c.paused_request_count, c.total_request_count)
        q_lens = c.request_query_lengths[act].cpu()
        last = c.last_token_logits(logits)
        assert torch.equal(last.cpu(), logits[0].cpu()[osm.last_token_indices(q_lens)])
        u = torch.rand(n, generator=g)
        params = SimpleNamespace(top_k=4, top_p=0.0, temperature=1.0)
        sample, mask = mi.sampling.sample_and_finish_mask(c, last, params, term, vocab_size=V, uniform=u.to(dev))
        want = osm.sample_from_logits(last.cpu(), top_k=4, uniform=u, vocab_size=V)
        assert torch.equal(sample.cpu(), want)
        want_mask = osm.active_request_mask(want, term, c.request_kv_length_offsets[act].cpu(), q_lens,
                                            c.request_output_lengths[act].cpu())
        assert mask.dtype == torch.uint8 and torch.equal(mask.cpu(), want_mask)
        if step == 0:
            assert want_mask.tolist().count(0) >= 1  # the one-token budget ends here
        c.update_requests(mask, sample.clone())
        if step == 1:
            assert not c.has_unfinished_requests()
            break


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("V", [1, 7, 4096, 32003, 131072])
def test_selected_log_probs_match_fp64_checker(mi, dev, dtype, V):
    """log_softmax(row)[id] with one read of the row: 2e-5 absolute against fp64 (fp32 sums of up to
    131 072 terms, hardware exp2 / log)."""
    g = torch.Generator().manual_seed(V)
    T = 37
    x = (torch.randn(T, V, generator=g) * 5).to(dtype)
    if V > 64:
        x[1, 10:40] = float("-inf")
        x[2, :] = 3.0                         # uniform row: -log V
        x[3, V // 2] = 60.0                   # one dominant entry
    ids = torch.randint(0, V, (T,), generator=g)
    if V > 64:
        ids[3] = V // 2
    got = mi.ops.selected_log_probs(x.to(dev), ids.to(dev)).cpu()
    want = osm.selected_log_probs(x, ids)
    assert torch.isfinite(got).all()
    assert (got.double() - want).abs().max().item() <= 2e-5
    if V > 64:
        assert abs(got[2].item() + float(torch.tensor(float(V)).log())) <= 2e-5
        assert abs(got[3].item()) <= 2e-5


def test_selected_log_probs_unaligned_rows_and_bad_ids(mi, dev):
    g = torch.Generator().manual_seed(5)
    big = torch.randn(6, 1003, generator=g)
    x = big[:, 1:1002]                         # rows neither 16-byte aligned nor a multiple of 4 wide
    ids = torch.randint(0, 1001, (6,), generator=g)
    got = mi.ops.selected_log_probs(x.to(dev)[:, :], ids.to(dev)).cpu()
    xd = big.to(dev)[:, 1:1002]
    got2 = mi.ops.selected_log_probs(xd, ids.to(dev)).cpu()
    want = osm.selected_log_probs(x, ids)
    assert (got.double() - want).abs().max().item() <= 2e-5
    assert (got2.double() - want).abs().max().item() <= 2e-5
    ids[4] = 1001
    ids[5] = -1
    bad = mi.ops.selected_log_probs(xd, ids.to(dev)).cpu()
    assert torch.isnan(bad[4]) and torch.isnan(bad[5]) and torch.isfinite(bad[:4]).all()


def test_context_log_probs_through_the_kernel(mi, dev):
    """calculate_log_probs on a mixed step: ids from the shifted prompt, grouped per request."""
    Ctx = mi.DynamicInferenceContext
    saved = (Ctx.TOKEN_ROUNDER, Ctx.REQUEST_ROUNDER)
    try:
        Ctx.TOKEN_ROUNDER, Ctx.REQUEST_ROUNDER = 4, 4
        ctx = Ctx(params_dtype=torch.bfloat16, num_layers=1, kv_channels=64, num_attention_heads=2,
                  max_sequence_length=64, buffer_size_gb=0.01, buffer_guaranteed_fraction=0.1, chunk_size_tokens=16,
                  max_requests_override=16, max_tokens_override=256, device=dev)
        g = torch.Generator().manual_seed(8)
        V = 300
        prompts = [torch.randint(0, V, (n,), generator=g) for n in (5, 1, 9)]
        for rid, pr in enumerate(prompts):
            ctx.add_request(rid, pr.to(dev), num_tokens_to_generate=4)
        ctx.initialize_attention_state()
        T = ctx.padded_active_token_count        # 15 active rows padded to 16
        logits = torch.randn(1, T, V, generator=g)
        new = torch.randint(0, V, (3,), generator=g)
        got = ctx.calculate_log_probs(logits.to(dev), new.to(dev))
        ids = osm.scored_token_ids(torch.cat(prompts), torch.tensor([5, 1, 9]), new)
        want = osm.selected_log_probs(logits[0][: ctx.active_token_count], ids)
        assert [len(r) for r in got] == [5, 1, 9]
        flat = torch.tensor([v for r in got for v in r], dtype=torch.float64)
        assert (flat - want).abs().max().item() <= 2e-5
        # last-token rows only
        rows = ctx.last_token_logits(logits.to(dev))
        got_last = ctx.calculate_log_probs(rows.unsqueeze(0), new.to(dev), only_last_token_logits=True)
        want_last = osm.selected_log_probs(logits[0][osm.last_token_indices(torch.tensor([5, 1, 9]))], new)
        assert (torch.tensor(got_last, dtype=torch.float64).flatten() - want_last).abs().max().item() <= 2e-5
    finally:
        Ctx.TOKEN_ROUNDER, Ctx.REQUEST_ROUNDER = saved
