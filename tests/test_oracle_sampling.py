"""Pins for the sampling checker (no GPU needed): library routines, a hand-worked example, the set
definition by brute force, limiting cases and the empirical frequencies of the draw."""
import numpy as np
import pytest
import torch

from oracle import sampling as osm


def test_last_token_indices_vector():
    # prompt lengths 3, 1, 5 flattened: last tokens sit at rows 2, 3, 8
    assert osm.last_token_indices(torch.tensor([3, 1, 5], dtype=torch.int32)).tolist() == [2, 3, 8]


def test_top_k_keep_matches_topk_and_keeps_ties():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(5, 200, generator=g)
    for k in (2, 7, 200):
        keep = osm.top_k_keep(x, k)
        assert (keep.sum(-1) == k).all()
        idx = torch.topk(x, k, dim=-1).indices
        assert keep.gather(1, idx).all()
    # the k-th value appears three times: all of them stay (`logits < kth` drops none of them)
    row = torch.tensor([[0.0, 5.0, 3.0, 3.0, 1.0, 3.0]])
    assert osm.top_k_keep(row, 2).tolist() == [[False, True, True, True, False, True]]


def test_top_p_hand_example():
    # probabilities 0.5, 0.3, 0.15, 0.05 given in shuffled order; cumulative 0.5, 0.8, 0.95, 1.0.
    # top_p 0.7: cumulative > 0.7 -> [F, T, T, T], shifted right -> [F, F, T, T]: two entries stay.
    probs = torch.tensor([[0.15, 0.5, 0.05, 0.3]], dtype=torch.float64)
    keep = osm.top_p_keep(probs.log(), 0.7)
    assert keep.tolist() == [[False, True, False, True]]
    # top_p 0.5: cumulative > 0.5 is false at the first entry (0.5 > 0.5 is false) -> second stays too
    assert osm.top_p_keep(probs.log(), 0.5).tolist() == [[False, True, False, True]]
    assert osm.top_p_keep(probs.log(), 0.49).tolist() == [[False, True, False, False]]


def test_top_p_is_shortest_prefix_with_mass_above_p():
    g = torch.Generator().manual_seed(2)
    x = torch.randn(6, 50, generator=g, dtype=torch.float64) * 2
    for p in (0.1, 0.5, 0.9, 0.999):
        keep = osm.top_p_keep(x, p)
        pr = x.softmax(-1)
        for r in range(x.size(0)):
            order = sorted(range(50), key=lambda j: -pr[r, j].item())
            mass, expect = 0.0, set()
            for j in order:  # brute force: add entries until the mass exceeds p
                expect.add(j)
                mass += pr[r, j].item()
                if mass > p:
                    break
            assert set(torch.nonzero(keep[r]).flatten().tolist()) == expect


def test_top_p_limits():
    g = torch.Generator().manual_seed(3)
    x = torch.randn(4, 64, generator=g)
    tiny = osm.top_p_keep(x, 1e-9)
    assert (tiny.sum(-1) == 1).all() and (tiny.float().argmax(-1) == x.argmax(-1)).all()
    assert osm.top_p_keep(x, 1.0).all()


def test_scaled_logits_rounds_like_the_tensor_dtype():
    x = torch.tensor([1.0, 2.5, -3.0]).bfloat16()
    y = osm.scaled_logits(x, 0.7)
    assert torch.equal(y, y.bfloat16().float())  # representable in bf16
    inv = torch.tensor(1.0) / torch.tensor(0.7)
    assert torch.equal(y, (x.float() * inv).bfloat16().float())
    assert torch.equal(osm.scaled_logits(x, 1.0), x.float())


def test_draw_matches_searchsorted_and_hand_case():
    p = torch.tensor([[0.1, 0.0, 0.4, 0.5]], dtype=torch.float64)
    # CDF 0.1, 0.1, 0.5, 1.0: u = 0.05 -> 0; u = 0.1 -> 2 (0.1 > 0.1 fails, zero-mass entry skipped)
    for u, want in ((0.05, 0), (0.1, 2), (0.4999, 2), (0.5, 3), (0.999, 3)):
        assert osm.draw_inverse_cdf(p, torch.tensor([u])).item() == want
    g = torch.Generator().manual_seed(4)
    pr = torch.rand(8, 300, generator=g, dtype=torch.float64)
    u = torch.rand(8, generator=g, dtype=torch.float64)
    got = osm.draw_inverse_cdf(pr, u)
    for r in range(8):
        cdf = np.cumsum(pr[r].numpy())
        assert got[r].item() == int(np.searchsorted(cdf, u[r].item() * cdf[-1], side="right"))


def test_draw_reproduces_the_probabilities():
    g = torch.Generator().manual_seed(5)
    logits = torch.randn(1, 12, generator=g)
    n = 200_000
    u = torch.rand(n, generator=g)
    keep = osm.top_k_keep(logits, 5)
    pr = osm.kept_probabilities(logits, keep)
    draws = osm.draw_inverse_cdf(pr.expand(n, -1), u)
    freq = torch.bincount(draws, minlength=12).double() / n
    assert (freq[~keep[0]] == 0).all()
    assert (freq - pr[0]).abs().max() < 4e-3  # ~4 sigma at p = 0.5


def test_sample_from_logits_control_flow():
    g = torch.Generator().manual_seed(6)
    logits = torch.randn(3, 40, generator=g)
    assert torch.equal(osm.sample_from_logits(logits, top_k=1), logits.argmax(-1))
    with pytest.raises(AssertionError):
        osm.sample_from_logits(logits, top_k=2, top_p=0.5, uniform=torch.zeros(3))
    # u = 0 picks the first kept entry in vocabulary order
    s = osm.sample_from_logits(logits, top_k=3, uniform=torch.zeros(3))
    assert torch.equal(s, osm.top_k_keep(logits, 3).float().argmax(-1))
    assert (osm.sample_from_logits(logits, top_p=0.9, uniform=torch.full((3,), 0.999), vocab_size=10) <= 9).all()


def test_active_request_mask_vector():
    sample = torch.tensor([7, 2, 9, 2])
    # lengths after this token: 5, 5, 10, 10 against maxima 10, 10, 10, 11; termination id 2
    m = osm.active_request_mask(sample, 2, torch.tensor([3, 3, 8, 8]), torch.tensor([1, 1, 1, 1]),
                                torch.tensor([10, 10, 10, 11]))
    assert m.dtype == torch.uint8 and m.tolist() == [1, 0, 0, 0]


def test_scored_token_ids_reference_comment_example():
    # the worked example in the reference's comment (dynamic_context.py:1331-1349), kept as data
    import json, os
    with open(os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.json")) as f:
        gold = json.load(f)["log_probs_token_shift"]
    ids = osm.scored_token_ids(torch.tensor(gold["active_token_ids"]), torch.tensor(gold["active_query_lengths"]),
                               torch.tensor(gold["new_tokens"]))
    assert ids.tolist() == gold["scored_token_ids"] == [52, 12, 16, 3, 12, 72, 24, 88, 86]
    # and the roll / index-assign formulation the reference uses (:1350-1355)
    g = torch.Generator().manual_seed(11)
    q = torch.randint(1, 9, (13,), generator=g)
    tok = torch.randint(0, 1000, (int(q.sum()),), generator=g)
    new = torch.randint(0, 1000, (13,), generator=g)
    rolled = tok.roll(-1, 0)
    rolled[q.cumsum(0) - 1] = new
    assert torch.equal(osm.scored_token_ids(tok, q, new), rolled)


def test_selected_log_probs_matches_library_log_softmax():
    g = torch.Generator().manual_seed(12)
    for dtype in (torch.float32, torch.bfloat16):
        x = (torch.randn(9, 777, generator=g) * 6).to(dtype)
        x[2, 5:50] = float("-inf")      # masked entries carry no mass
        ids = torch.randint(0, 777, (9,), generator=g)
        ids[2] = 3
        want = torch.log_softmax(x.float().double(), dim=-1)[torch.arange(9), ids]
        got = osm.selected_log_probs(x, ids)
        assert torch.allclose(got, want, rtol=0, atol=1e-12)
        lse = torch.logsumexp(x.float().double(), dim=-1)
        assert torch.allclose(got, x.float().double()[torch.arange(9), ids] - lse, rtol=0, atol=1e-12)
    # probabilities of a row sum to one
    row = torch.randn(1, 50, generator=g).expand(50, 50)
    assert abs(osm.selected_log_probs(row, torch.arange(50)).exp().sum().item() - 1.0) < 1e-12
