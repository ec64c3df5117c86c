"""GPU: whole engine steps -- forward, last-token rows, sampling, finished mask, bookkeeping.

A two-layer toy transformer (embedding, per layer QKV projection -> this package's attention core
-> output projection with a residual, then a vocabulary projection) is driven by
``step.generate_output_tokens_dynamic_batch`` the way the reference's controller drives a model
(text_generation_controller.py:411-546).  The projections are plain torch matmuls (they are outside
the path); everything between them is the HIP path.

The checker recomputes every step from scratch on the CPU in fp32 with DENSE causal attention over
each request's full token history (no cache, no paging; the history is the tokens the GPU run
sampled, so one near-tie cannot derail the comparison): last-token logits must agree within 3e-2,
the sampled token must be the argmax of the GPU's own logits, and finished / active ids and the
context's counters must follow the reference's rules.
"""
from types import SimpleNamespace

import pytest
import torch

from oracle import rope_norm as orn
from oracle import sampling as osm

pytestmark = pytest.mark.gpu

V, H, HQ, HKV, D, L = 96, 64, 4, 2, 64, 2
TERM = 7


class ToyModel:
    def __init__(self, mi, dev, seed):
        g = torch.Generator().manual_seed(seed)
        r = lambda *s: (torch.randn(*s, generator=g) / (s[0] ** 0.5))
        self.emb = torch.randn(V, H, generator=g)
        self.wqkv = [r(H, (HQ + 2 * HKV) * D) for _ in range(L)]
        self.wo = [r(HQ * D, H) for _ in range(L)]
        self.head = r(H, V)
        self.table = orn.rotary_table(256, D, base=10000.0)
        self.dev = dev
        self.cores = [mi.PagedSelfAttentionCore(l + 1, D, fused=True, device=dev) for l in range(L)]
        self.d = {k: [w.to(dev) for w in getattr(self, k)] for k in ("wqkv", "wo")}
        self.emb_d, self.head_d, self.table_d = self.emb.to(dev), self.head.to(dev), self.table.to(dev)
        self.last_logits = None

    def forward_step(self, ctx):
        def fwd(input_ids, position_ids):
            x = self.emb_d[input_ids[0]]
            for l in range(L):
                mixed = (x @ self.d["wqkv"][l]).bfloat16().unsqueeze(1)
                a = self.cores[l].forward_mixed_qkv(mixed, HQ, ctx, (self.table_d, self.table_d))
                x = x + a.squeeze(1).float() @ self.d["wo"][l]
            self.last_logits = (x @ self.head_d).unsqueeze(0)
            return self.last_logits
        return fwd

    def dense_last_logits(self, tokens):
        """fp32, dense causal attention over the whole history of one request; last position's logits."""
        n = len(tokens)
        x = self.emb[torch.tensor(tokens)]
        pos = torch.arange(n)
        for l in range(L):
            mixed = (x @ self.wqkv[l]).bfloat16().view(n, 1, -1)
            q, k, v = orn.split_mixed_qkv(mixed, HQ, HKV)
            q = orn.norm_rope(q.squeeze(1), pos, self.table).float()   # rotary in bf16, like the path
            k = orn.norm_rope(k.squeeze(1), pos, self.table).float()
            v = v.squeeze(1).float()
            k = k.repeat_interleave(HQ // HKV, dim=1)
            v = v.repeat_interleave(HQ // HKV, dim=1)
            s = torch.einsum("ihd,jhd->hij", q, k) * D ** -0.5
            s = s.masked_fill(torch.ones(n, n).triu(1).bool(), float("-inf"))
            a = torch.einsum("hij,jhd->ihd", s.softmax(-1), v).reshape(n, HQ * D)
            x = x + a @ self.wo[l]
        return x[-1] @ self.head


def test_steps_follow_the_dense_model_and_the_bookkeeping_rules(mi, dev):
    Ctx = mi.DynamicInferenceContext
    saved = (Ctx.TOKEN_ROUNDER, Ctx.REQUEST_ROUNDER)
    try:
        Ctx.TOKEN_ROUNDER, Ctx.REQUEST_ROUNDER = 4, 4
        C = 16
        ctx = Ctx(params_dtype=torch.bfloat16, num_layers=L, kv_channels=D, num_attention_heads=HKV,
                  max_sequence_length=64, buffer_size_gb=300 * (2 * 2 * L * C * HKV * D) / 1024**3,
                  buffer_guaranteed_fraction=0.1, chunk_size_tokens=C, max_requests_override=16,
                  max_tokens_override=256, materialize_only_last_token_logits=False, device=dev)
        model = ToyModel(mi, dev, seed=3)
        g = torch.Generator().manual_seed(4)
        prompts = {rid: torch.randint(8, V, (n,), generator=g).tolist() for rid, n in enumerate([3, 17, 1, 30, 9])}
        budget = {0: 2, 1: 12, 2: 5, 3: 12, 4: 1}
        history = {rid: list(p) for rid, p in prompts.items()}
        for rid, p in prompts.items():
            ctx.add_request(rid, torch.tensor(p, device=dev), num_tokens_to_generate=budget[rid])
        params = SimpleNamespace(top_k=1, top_p=0.0, temperature=1.0, return_log_probs=False)
        live = set(prompts)
        finished_all = []
        for step in range(14):
            if not ctx.has_unfinished_requests():
                break
            ids_before = ctx.request_ids[ctx.paused_request_count: ctx.total_request_count].tolist()
            assert set(ids_before) == live
            result = mi.step.generate_output_tokens_dynamic_batch(ctx, model.forward_step(ctx), params, TERM,
                                                                  vocab_size=V)
            assert result["active_request_ids"].tolist() == ids_before
            assert result["log_probs"] is None
            sample = result["sample"].cpu()
            # logits of this step, gathered at the last token of every request, against the dense model
            logits = model.last_logits[0].cpu()
            q_lens = [len(history[rid]) if step_is_prefill(history, prompts, rid) else 1 for rid in ids_before]
            last = osm.last_token_indices(torch.tensor(q_lens))
            got = logits[last]
            want = torch.stack([model.dense_last_logits(history[rid]) for rid in ids_before])
            assert (got - want).abs().max().item() <= 3e-2, f"step {step}: {(got - want).abs().max().item()}"
            assert torch.equal(sample, got.argmax(-1))
            # bookkeeping rules
            finished = []
            for rid, tok in zip(ids_before, sample.tolist()):
                history[rid].append(tok)
                if tok == TERM or len(history[rid]) >= len(prompts[rid]) + budget[rid]:
                    finished.append(rid)
            # (listed by the bookkeeping kernel, in the row order the reference's nonzero + index gives)
            assert result["finished_request_ids"].tolist() == finished
            live -= set(finished)
            finished_all += finished
            assert ctx.total_request_count == len(live)
            if live:
                assert result["cuda_graph_request_count"] is None or step > 0
                assert ctx.active_token_count == len(live) and ctx.is_decode_only()
        assert not live and sorted(finished_all) == sorted(prompts)
        assert ctx.chunk_allocator.chunk_count_avail == ctx.chunk_allocator.chunk_count_total - 1
        assert mi.step.generate_output_tokens_dynamic_batch(ctx, model.forward_step(ctx), params, TERM) is None
    finally:
        Ctx.TOKEN_ROUNDER, Ctx.REQUEST_ROUNDER = saved


def step_is_prefill(history, prompts, rid):
    return len(history[rid]) == len(prompts[rid])


def test_sampled_steps_and_last_token_materialisation(mi, dev):
    """Top-k sampling through the driver with a model that returns only the last-token rows."""
    Ctx = mi.DynamicInferenceContext
    saved = (Ctx.TOKEN_ROUNDER, Ctx.REQUEST_ROUNDER)
    try:
        Ctx.TOKEN_ROUNDER, Ctx.REQUEST_ROUNDER = 4, 4
        C = 16
        ctx = Ctx(params_dtype=torch.bfloat16, num_layers=L, kv_channels=D, num_attention_heads=HKV,
                  max_sequence_length=64, buffer_size_gb=300 * (2 * 2 * L * C * HKV * D) / 1024**3,
                  buffer_guaranteed_fraction=0.1, chunk_size_tokens=C, max_requests_override=16,
                  max_tokens_override=256, materialize_only_last_token_logits=True, device=dev)
        model = ToyModel(mi, dev, seed=5)
        g = torch.Generator().manual_seed(6)
        for rid, n in enumerate([6, 21, 2]):
            ctx.add_request(rid, torch.randint(8, V, (n,), generator=g).to(dev), num_tokens_to_generate=6)
        full = model.forward_step(ctx)
        seen = {}

        def last_rows_only(input_ids, position_ids):
            seen["rows"] = ctx.last_token_logits(full(input_ids, position_ids))
            return seen["rows"].unsqueeze(0)

        params = SimpleNamespace(top_k=5, top_p=0.0, temperature=0.8, return_log_probs=False)
        for step in range(4):
            n = ctx.total_request_count - ctx.paused_request_count
            u = torch.rand(n, generator=g)
            result = mi.step.generate_output_tokens_dynamic_batch(ctx, last_rows_only, params, TERM, vocab_size=V,
                                                                  uniform=u.to(dev))
            rows = seen["rows"].cpu()
            assert rows.shape == (n, V) and result["sample"].shape == (n,)
            want = osm.sample_from_logits(rows, top_k=5, temperature=0.8, uniform=u, vocab_size=V)
            assert torch.equal(result["sample"].cpu(), want)
    finally:
        Ctx.TOKEN_ROUNDER, Ctx.REQUEST_ROUNDER = saved
