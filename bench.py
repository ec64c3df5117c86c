#!/usr/bin/env python3
"""Benchmark of the paged decode step on one MI355X.

One "step" is one pass of the decode hot path of a single layer over one batch:
fused q/k RMSNorm + RoPE + KV-append (one launch), then paged GQA decode attention
(split kernel + merge kernel).  The default workload is the Llama-3-8B shape:
batch 64, 32 query / 8 KV heads, head dim 128, context lengths U[512, 8192], chunk 256,
bf16, all inputs resident in HBM before timing starts.

Prints ONE JSON line.  ``value`` is algorithmic decode-attention bytes divided by the step
time; ``roofline`` prices the KV-streaming kernel alone, timed with HIP events recorded on
the launch stream inside the same timed region; ``cpu_baseline`` is the CPU checker
(``oracle/``) timed on the host cores on a bounded sample of the same workload.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published peak
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16 matrix peak, published

# HBM bytes per launch of the streaming kernel, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of
# this same script, each counter scaled by what it reads for a plain 1 GiB device copy
# (profiles/decode_stream_kernels_hbm_traffic_cfg2_cfg4_cfg5.md).  Hardware counters cannot be
# read from inside the benchmark, so the figure is recorded here per workload; None = not collected.
MEASURED_HBM_TRAFFIC_BYTES = {
    # decode workloads: "<cfg>" = the attention-only streaming kernel, "<cfg>_step" = the one-kernel decode step
    "cfg2": 1_226_700_000, "cfg2_step": 1_215_000_000, "cfg4": 8_724_700_000, "cfg4_step": 8_634_800_000,
    "cfg5": 9_070_200_000, "cfg5_step": 9_050_500_000,
    # the mixed step: tile kernel, stream kernel
    "cfg3_tile": 401_700_000, "cfg3_stream": 2_195_700_000,
    # multi-latent decode at 128 heads (reads + the partial results it writes)
    "mla_decode_h128": 454_500_000, "mla_decode_h128_long": 1_305_000_000}
# Where each figure above was read, so that a reader of the JSON line can tell a stale constant from a fresh one:
# the summary file and the last commit that touched the kernel when the counters were collected.
_DECODE_TRAFFIC = ("profiles/decode_stream_kernels_hbm_traffic_cfg2_cfg4_cfg5.md (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, "
                   "library as of commit b54c9eb)")
_MIXED_TRAFFIC = ("profiles/paged_prefill_woven_kernel_cfg3_mfma.md (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, kernels as of "
                  "commit e60638b; the one later change of the tile kernel, e3f1ea0, masks two base addresses at its set-up)")
_MLA_HEADS_TRAFFIC = ("profiles/paged_mla_decode_heads_kernel_h128_counters.md (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, "
                      "kernel as of commit c8e09ff; the row pitch changed since, the traffic does not depend on it)")
TRAFFIC_SOURCE = {"mla_decode_h128": _MLA_HEADS_TRAFFIC, "mla_decode_h128_long": _MLA_HEADS_TRAFFIC, "cfg2": _DECODE_TRAFFIC, "cfg2_step": _DECODE_TRAFFIC, "cfg4": _DECODE_TRAFFIC,
                  "cfg4_step": _DECODE_TRAFFIC, "cfg5": _DECODE_TRAFFIC, "cfg5_step": _DECODE_TRAFFIC, "cfg3_tile": _MIXED_TRAFFIC,
                  "cfg3_stream": _MIXED_TRAFFIC}


# Single-kernel workloads for the rows built around the path (multi-latent decode, the tail of a step).
SECONDARY_WORKLOADS = {
    # name: (kind, parameters)
    "mla_decode_h16": ("mla", dict(Hq=16, B=64, lo=512, hi=8192)),
    "mla_decode_h128": ("mla", dict(Hq=128, B=64, lo=512, hi=8192)),
    "mla_decode_h16_long": ("mla", dict(Hq=16, B=16, lo=65536, hi=65536)),
    "mla_decode_h128_long": ("mla", dict(Hq=128, B=16, lo=65536, hi=65536)),
    "mla_prefill_h16": ("mla_prefill", dict(H=16, n=8, new=2048, ctx=2048)),
    "mla_prefill_h128": ("mla_prefill", dict(H=128, n=2, new=2048, ctx=2048)),
    "prefill_d64": ("prefill", dict(Hq=32, Hkv=8, d=64, n=8, new=2048, ctx=2048)),
    "prefill_d96": ("prefill", dict(Hq=32, Hkv=8, d=96, n=8, new=2048, ctx=2048)),
    "prefill_d128": ("prefill", dict(Hq=32, Hkv=8, d=128, n=8, new=2048, ctx=2048)),
    "prefill_d192": ("prefill", dict(Hq=32, Hkv=8, d=192, n=8, new=2048, ctx=2048)),
    "prefill_d256": ("prefill", dict(Hq=32, Hkv=8, d=256, n=8, new=2048, ctx=2048)),
    "prefill_d128_mqa": ("prefill", dict(Hq=64, Hkv=2, d=128, n=8, new=2048, ctx=2048)),
    # the projections either side of the path at decode size (cfg2's layer: hidden 4096, 32 / 8 heads of 128)
    "qkv_proj_decode": ("linear", dict(T=64, N=6144, K=4096, bias=True)),
    "out_proj_decode": ("linear", dict(T=64, N=4096, K=4096, bias=False)),
    "sampling_top_k": ("sampling", dict(R=64, V=128256, top_k=50, top_p=0.0)),
    "sampling_top_p": ("sampling", dict(R=64, V=128256, top_k=0, top_p=0.9)),
    "sampling_top_p_peaked": ("sampling", dict(R=64, V=128256, top_k=0, top_p=0.9, peaked=True)),
    "sampling_greedy": ("sampling", dict(R=64, V=128256, top_k=1, top_p=0.0)),
    "log_probs_bf16": ("log_probs", dict(T=4096, V=131072, bf16=True)),
    "log_probs_fp32": ("log_probs", dict(T=4096, V=131072, bf16=False)),
}


def run_secondary(args, mi, lib, torch, dev):
    """One kernel per step; HIP events on the launch stream around every call give the kernel time."""
    kind, prm = SECONDARY_WORKLOADS[args.workload]
    gen = torch.Generator().manual_seed(7)
    flops = None
    if kind == "mla":
        Hq, B = prm["Hq"], prm["B"]
        lens = torch.randint(prm["lo"], prm["hi"] + 1, (B,), generator=gen, dtype=torch.int32)
        bt, N = mi.synthetic.build_block_table(lens, 256, gen)
        cache = torch.empty(N + 1, 256, 576, dtype=torch.bfloat16, device=dev).normal_(0, 0.5)
        q = torch.randn(B, 1, Hq, 576, device=dev).bfloat16()
        lens_d, bt_d = lens.to(dev), bt.to(dev)
        out = torch.empty(B, 1, Hq, 512, dtype=torch.bfloat16, device=dev)
        step = lambda: mi.ops.paged_mla_decode_attention(q, cache, lens_d, bt_d, softmax_scale=0.072, out=out)
        nbytes = int(lens.sum()) * 576 * 2 + B * Hq * (576 + 512) * 2 + int(((lens + 255) // 256).sum()) * 4 + B * 4
        flops = int(lens.sum()) * Hq * (576 + 512) * 2
        kernel = "paged_mla_decode_heads_kernel" if Hq % 128 == 0 else "paged_mla_decode_lds_kernel"
        what = (f"absorbed multi-latent decode attention, {Hq} query heads, batch {B}, latent rows of 576 bf16, "
                f"context U[{prm['lo']},{prm['hi']}], chunk 256")
        dtype = "bf16 (fp32 accumulate)"
        timed_by_library = True
    elif kind in ("mla_prefill", "prefill"):
        mla = kind == "mla_prefill"
        Hq, Hkv = (prm["H"], prm["H"]) if mla else (prm["Hq"], prm["Hkv"])
        dk, dv = (192, 128) if mla else (prm["d"], prm["d"])
        n, new, ctx = prm["n"], prm["new"], prm["ctx"]
        lens = torch.full((n,), new + ctx, dtype=torch.int32)
        cu_q = torch.arange(n + 1, dtype=torch.int32) * new
        bt, N = mi.synthetic.build_block_table(lens, 256, gen)
        kc = torch.empty(N + 1, 256, Hkv, dk, dtype=torch.bfloat16, device=dev).normal_(0, 0.5)
        vc = torch.empty(N + 1, 256, Hkv, dv, dtype=torch.bfloat16, device=dev).normal_(0, 0.5)
        q = torch.randn(n * new, Hq, dk, device=dev).bfloat16()
        out = torch.empty(n * new, Hq, dv, dtype=torch.bfloat16, device=dev)
        cu_d, lens_d, bt_d = cu_q.to(dev), lens.to(dev), bt.to(dev)
        if mla:
            step = lambda: mi.ops.paged_prefill_attention_mla(q, kc, vc, cu_d, lens_d, bt_d, softmax_scale=0.072, out=out)
        else:
            step = lambda: mi.ops.paged_prefill_attention(q, kc, vc, cu_d, lens_d, bt_d, max_kv_len=new + ctx, out=out)
        pairs = n * (new * ctx + new * (new + 1) // 2)          # (query row, visible key) pairs per head
        flops = 2 * Hq * (dk + dv) * pairs
        nbytes = n * (new + ctx) * Hkv * (dk + dv) * 2 + n * new * Hq * (dk + dv) * 2
        kernel = ("paged_prefill_woven_kernel" if (not mla and dk == 128 and args.prefill_kernel in (0, 3))
                  else "paged_prefill_pp_kernel")
        what = (f"paged varlen causal attention, {n} x {new} new tokens over {ctx} cached, {Hq}/{Hkv} heads, "
                f"keys {dk} / values {dv} wide, chunk 256")
        dtype = "bf16 (fp32 accumulate)"
        timed_by_library = True
    elif kind == "linear":
        T, N, K = prm["T"], prm["N"], prm["K"]
        x = (torch.randn(T, K, generator=gen) * 0.5).bfloat16().to(dev)
        # a model's layers each bring their own matrix from HBM: the step walks a ring of matrices larger than the
        # 256 MB last-level cache, so that no call finds its weights cached from the call before
        n_w = max(2, -(-320 * 1024 * 1024 // (N * K * 2)))
        ws = [torch.empty(N, K, dtype=torch.bfloat16, device=dev).normal_(0, K ** -0.5) for _ in range(n_w)]
        w = ws[0]
        bias_t = torch.randn(N, generator=gen).bfloat16().to(dev) if prm["bias"] else None
        out = torch.empty(T, N, dtype=torch.bfloat16, device=dev)
        ring = {"i": 0}

        def step():
            ring["i"] = (ring["i"] + 1) % n_w
            mi.ops.linear_decode(x, ws[ring["i"]], bias_t, out=out)
        nbytes = N * K * 2 + T * K * 2 + T * N * 2 + (N * 2 if prm["bias"] else 0)
        flops = 2 * T * N * K
        kernel = "linear_decode_kernel"
        what = (f"y[{T}, {N}] = x[{T}, {K}] . W[{N}, {K}]^T{' + bias' if prm['bias'] else ''}: the weight matrix streamed "
                f"once (a ring of {n_w} matrices, so every call reads its weights from HBM), fp32 partial sums over slices "
                f"of K and their reduction launch included in the step")
        dtype = "bf16 (fp32 accumulate)"
        timed_by_library = True
    elif kind == "sampling":
        R, V = prm["R"], prm["V"]
        logits = torch.randn(R, V, generator=gen) * 3
        if prm.get("peaked"):  # a language model's rows: a few dozen tokens far above the rest
            logits *= 2.0 / 3.0
            for r in range(R):
                logits[r, torch.randperm(V, generator=gen)[:32]] += torch.rand(32, generator=gen) * 6 + 9
        logits = logits.to(dev)
        u = torch.rand(R, generator=gen).to(dev)
        step = lambda: mi.ops.sample_from_logits(logits, top_k=prm["top_k"], top_p=prm["top_p"], temperature=0.8,
                                                 uniform=u)
        nbytes = R * V * 4 + R * 12
        kernel = "sample_kernel"
        what = (f"sampling of {R} rows of {V} fp32 logits ({'32 tokens 9-15 above a N(0, 2) bulk' if prm.get('peaked') else 'N(0, 3)'}), "
                f"top_k {prm['top_k']}, top_p {prm['top_p']}, temperature 0.8")
        dtype = "fp32 logits, 2^-32 fixed-point mass"
        timed_by_library = False
    else:
        T, V = prm["T"], prm["V"]
        logits = torch.empty(T, V, dtype=torch.bfloat16 if prm["bf16"] else torch.float32, device=dev).normal_(0, 3)
        ids = torch.randint(0, V, (T,), generator=gen).to(dev)
        step = lambda: mi.ops.selected_log_probs(logits, ids)
        nbytes = T * V * logits.element_size() + T * 12
        kernel = "selected_log_probs_kernel"
        what = f"log-probabilities of the chosen tokens, {T} rows of {V} {'bf16' if prm['bf16'] else 'fp32'} logits"
        dtype = "fp32 accumulation"
        timed_by_library = False

    # (untimed steps until the clocks have settled after the set-up, as for the decode workloads)
    t_settle = time.perf_counter()
    while time.perf_counter() - t_settle < args.settle_s:
        for _ in range(10):
            step()
        torch.cuda.synchronize()
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    if timed_by_library:
        lib.mi_profile_enable(1)
    events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    t0 = time.perf_counter()
    for a, b in events:
        a.record()   # (these ops launch on torch's current stream, which is the stream the events see)
        step()
        b.record()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    call_ms = sum(a.elapsed_time(b) for a, b in events) / args.steps
    kernel_ms = call_ms
    if timed_by_library:
        # (the two-width-equal prefill call times two launches per step: the tile kernel, then the decode
        # kernel that serves one-row requests -- none here; the first of each pair is the tile kernel)
        per_step = 2 if kind == "prefill" else 1
        buf = (ctypes.c_float * (args.steps * per_step))()
        n_ev = lib.mi_profile_collect(buf, args.steps * per_step)
        lib.mi_profile_enable(0)
        mine = [buf[i] for i in range(0, n_ev, per_step)]
        kernel_ms = sum(mine) / max(1, len(mine))
    ms_per_step = elapsed * 1e3 / args.steps
    mfma_bound = (kind == "mla" and prm["Hq"] >= 64) or kind in ("mla_prefill", "prefill")
    roofline = ({"bound": "mfma", "kernel": kernel, "achieved": round(flops / kernel_ms / 1e9, 1),
                 "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                 "frac": round(flops / kernel_ms / 1e9 / MFMA_BF16_PEAK_TFLOPS, 4)} if mfma_bound else
                {"bound": "hbm", "kernel": kernel, "achieved": round(nbytes / kernel_ms / 1e6, 1), "peak": HBM_PEAK_GBPS,
                 "unit": "GB/s", "frac": round(nbytes / kernel_ms / 1e6 / HBM_PEAK_GBPS, 4)})
    roofline.update({"kernel_ms": round(kernel_ms, 5), "traffic": MEASURED_HBM_TRAFFIC_BYTES.get(args.workload)})
    if kind == "linear":
        # the library's GEMM on the same operands, timed the same way (what the reference's linear layers call)
        def lin():
            ring["i"] = (ring["i"] + 1) % n_w
            torch.nn.functional.linear(x, ws[ring["i"]], bias_t)
        for _ in range(args.warmup):
            lin()
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
        for a, b2 in ev:
            a.record()
            lin()
            b2.record()
        torch.cuda.synchronize()
        roofline["library_gemm_ms"] = round(sum(a.elapsed_time(b2) for a, b2 in ev) / args.steps, 5)
        roofline["call_ms"] = round(call_ms, 5)
        # both again as 3 x n_w calls captured in a HIP graph and replayed: GPU time per call without the host's
        # launch cost (the eager figures above are bound by it: two launches here, one in the library)
        nbytes_ws = lib.mi_linear_decode_workspace_bytes(T, N, K)
        fixed_ws = torch.empty(max(nbytes_ws, 16), dtype=torch.uint8, device=dev)

        def replayed(fn):
            graph = torch.cuda.CUDAGraph()
            with mi.ops.use_workspace(fixed_ws), torch.cuda.graph(graph):
                for _ in range(3 * n_w):
                    fn()
            for _ in range(3):
                graph.replay()
            torch.cuda.synchronize()
            a, b2 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            for _ in range(10):
                graph.replay()
            b2.record()
            torch.cuda.synchronize()
            return round(a.elapsed_time(b2) / (30 * n_w), 5)
        roofline["call_ms_graph"] = replayed(step)
        roofline["library_gemm_ms_graph"] = replayed(lin)
    if args.workload in TRAFFIC_SOURCE:
        roofline["traffic_source"] = TRAFFIC_SOURCE[args.workload]
    return ({
        "metric": f"{args.workload}_GBps", "value": round(nbytes / (ms_per_step * 1e-3) / 1e9, 1), "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": dtype, "data": "synthetic",
        "config": {"workload": what, "algorithmic_bytes_per_step": nbytes, "flops_per_step": flops,
                   "call_ms_by_events": round(call_ms, 5)},
        "roofline": roofline})


def run_bookkeeping(args, mi, lib, torch, dev):
    """The host-visible bookkeeping of a decode step at serving sizes: mi_add_request per admitted prompt,
    mi_step_attention_state for the first (prefill) step, then per decode step mi_decode_attention_state and
    mi_update_requests with its read-back of the new counters.  R requests, a chunk table M columns wide."""
    from importlib import import_module
    ops = mi.ops
    ctx_mod = import_module(mi.__name__ + ".contexts.dynamic_context")
    chunk = 256
    timed = {}

    def timing(name):
        inner = getattr(ops, name)

        def wrapper(*a, **k):
            ev = (torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
            ev[0].record()
            r = inner(*a, **k)
            ev[1].record()
            timed.setdefault(name, []).append(ev)
            return r
        return inner, wrapper

    names = ("add_request", "step_attention_state", "decode_attention_state", "update_requests")
    saved = {}
    for n in names:
        saved[n], w = timing(n)
        setattr(ops, n, w)
    rows = []
    try:
        for R in (64, 256, 1024):
            for M in (32, 128, 512):
                timed.clear()
                gen = torch.Generator().manual_seed(R * 1000 + M)
                ctx = ctx_mod.DynamicInferenceContext(
                    params_dtype=torch.bfloat16, num_layers=1, kv_channels=64, num_attention_heads=1,
                    max_sequence_length=M * chunk, buffer_size_gb=0.75, buffer_guaranteed_fraction=0.1,
                    chunk_size_tokens=chunk, max_requests_override=R, max_tokens_override=R * 512, device=dev,
                    fused_bookkeeping=True)
                assert ctx.request_to_kv_chunk_ids.size(1) == M and ctx.max_requests >= R
                # prompts end a few tokens before a chunk edge for a share of the requests, so the timed decode steps
                # cross chunk boundaries (the allocating branch of the update) as well as the plain one
                lens = torch.randint(100, 500, (R,), generator=gen)
                lens[::4] = chunk - torch.randint(1, max(2, args.steps), (len(lens[::4]),), generator=gen)
                prompts = [torch.randint(0, 32000, (int(n),), generator=gen).to(dev) for n in lens]
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for i, pr in enumerate(prompts):
                    ctx.add_request(i, pr, 4096)
                torch.cuda.synchronize()
                add_wall_us = (time.perf_counter() - t0) * 1e6 / R
                ctx.initialize_attention_state()            # the prefill step's state
                for _ in range(args.warmup + args.steps - 1):
                    ops.step_attention_state(ctx, R, ctx.padded_active_request_count, ctx.padded_active_token_count)
                mask = torch.ones(R, dtype=torch.int32, device=dev)
                tokens = torch.randint(0, 32000, (R,), generator=gen).to(dev)
                ctx.update_requests(mask, tokens)
                wall = []
                for i in range(args.warmup + args.steps):
                    torch.cuda.synchronize()
                    t0 = time.perf_counter()
                    ctx.initialize_attention_state()
                    ctx.update_requests(mask, tokens)
                    wall.append((time.perf_counter() - t0) * 1e6)
                torch.cuda.synchronize()
                assert ctx.total_request_count == R and ctx.paused_request_count == 0
                # churn: 8 requests finish in a decode step (their chunks go back, rows from the right fill the holes),
                # 8 prompts are admitted, and the next step is a mixed one
                fin, fin_wall, mixed = [], [], []
                next_id = R
                for i in range(min(args.steps, 20)):
                    ctx.initialize_attention_state()
                    mask_f = mask.clone()
                    mask_f[torch.randperm(R, generator=gen)[:8].to(dev)] = 0
                    torch.cuda.synchronize()
                    t0 = time.perf_counter()
                    ctx.update_requests(mask_f, tokens)
                    fin_wall.append((time.perf_counter() - t0) * 1e6)
                    fin.append(timed["update_requests"][-1])
                    for k in range(8):
                        ctx.add_request(next_id, prompts[(next_id * 7) % R], 4096)
                        next_id += 1
                    ctx.initialize_attention_state()
                    mixed.append(timed["step_attention_state"][-1])
                    ctx.update_requests(mask, tokens)
                torch.cuda.synchronize()
                assert ctx.total_request_count == R
                mean_us = lambda evs: round(sum(a.elapsed_time(b) for a, b in evs) * 1e3 / max(1, len(evs)), 2)
                w = args.warmup
                rows.append({
                    "requests": R, "table_columns": M,
                    "add_request_us": mean_us(timed["add_request"]), "add_request_wall_us": round(add_wall_us, 2),
                    "step_attention_state_us": mean_us(timed["step_attention_state"][w:w + args.steps]),
                    "decode_attention_state_us": mean_us(timed["decode_attention_state"][w:w + args.steps]),
                    "update_requests_us": mean_us(timed["update_requests"][1 + w:1 + w + args.steps]),
                    "decode_step_wall_us": round(sum(wall[w:]) / max(1, len(wall[w:])), 2),
                    "update_requests_8_finished_us": mean_us(fin[2:]),
                    "update_requests_8_finished_wall_us": round(sum(fin_wall[2:]) / max(1, len(fin_wall[2:])), 2),
                    "step_attention_state_after_admission_us": mean_us(mixed[2:]),
                })
                del ctx
                torch.cuda.empty_cache()
    finally:
        for n in names:
            setattr(ops, n, saved[n])
    head = rows[-1]
    step_us = head["decode_attention_state_us"] + head["update_requests_us"]
    # what one decode step's two launches must move at the largest size: the block table copied into its mirror
    # (read + write), 7 request rows read and written, 6 token rows written
    R, M = head["requests"], head["table_columns"]
    nbytes = R * M * 4 * 2 + R * 7 * 4 * 2 + R * 6 * 8
    return {
        "metric": "bookkeeping_decode_step_us", "value": head["decode_step_wall_us"], "unit": "us", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(head["decode_step_wall_us"] / 1e3, 5),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "int32 / int64", "data": "synthetic",
        "config": {"workload": "request / token bookkeeping of the dynamic context: value = host-visible time of one "
                               "decode step's initialize_attention_state + update_requests (two launches, one 32-byte "
                               "read-back) at 1024 requests and a 512-column chunk table; *_us = HIP events around each "
                               "launch", "sizes": rows},
        "roofline": {"bound": "hbm", "kernel": "decode_attention_state_kernel + update_requests_kernel",
                     "achieved": round(nbytes / step_us / 1e3, 2), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(nbytes / step_us / 1e3 / HBM_PEAK_GBPS, 5), "kernel_ms": round(step_us / 1e3, 5),
                     "traffic": None,
                     "note": "launch- and dependency-bound integer work: a few MB per step, so the bandwidth fraction "
                             "only says that these launches cost microseconds, not how well they stream"}}


def run_stream_read(args, mi, torch, dev):
    """Calibration leg: a plain read-only streaming kernel (csrc/bench/stream_read.hip, built into
    libmi355_bench.so) over a buffer of ``--read-mib`` MiB -- what a kernel that does nothing but read reaches
    on this box, i.e. the practical ceiling under the published 8 TB/s that the KV-streaming kernel is held against."""
    path = mi._lib.PKG_DIR / "libmi355_bench.so"
    if not path.exists():
        print(f"{path} not found: build first (python megatron-mixtera_amd/build.py)", file=sys.stderr)
        sys.exit(2)
    blib = ctypes.CDLL(str(path))
    blib.mi_bench_stream_read.restype = ctypes.c_int
    blib.mi_bench_stream_read.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p, ctypes.c_int32,
                                          ctypes.c_int32, ctypes.c_void_p]
    nbytes = args.read_mib << 20
    src = torch.empty(nbytes, dtype=torch.uint8, device=dev).random_()
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    wgs = cus * args.read_wgs_per_cu
    sink = torch.zeros(wgs, dtype=torch.int32, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    results = {}
    for name, nt in (("nontemporal", 1), ("cacheable", 0)):
        def step():
            rc = blib.mi_bench_stream_read(src.data_ptr(), nbytes, sink.data_ptr(), wgs, nt, stream)
            assert rc == 0
        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
        t0 = time.perf_counter()
        for a, b in events:
            a.record()
            step()
            b.record()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
        ms = sorted(a.elapsed_time(b) for a, b in events)
        results[name] = {"kernel_ms_mean": sum(ms) / len(ms), "kernel_ms_min": ms[0], "ms_per_step": elapsed * 1e3 / args.steps}
    best = results["nontemporal"]
    achieved = nbytes / best["kernel_ms_mean"] / 1e6
    return ({
        "metric": "stream_read_GBps", "value": round(nbytes / (best["ms_per_step"] * 1e-3) / 1e9, 1), "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(best["ms_per_step"], 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "u8", "data": "synthetic",
        "config": {"workload": f"read-only streaming kernel over {args.read_mib} MiB, {wgs} workgroups of 512 threads, "
                               f"four 16-byte loads per thread per iteration, non-temporal loads",
                   "algorithmic_bytes_per_step": nbytes,
                   "cacheable_loads_GBps": round(nbytes / results["cacheable"]["kernel_ms_mean"] / 1e6, 1),
                   "best_launch_GBps": round(nbytes / best["kernel_ms_min"] / 1e6, 1)},
        "roofline": {"bound": "hbm", "kernel": "stream_read_kernel", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "kernel_ms": round(best["kernel_ms_mean"], 5), "traffic": None}})


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="cfg2",
                    choices=["cfg1", "cfg2", "cfg3", "cfg3_decode", "cfg4", "cfg5", "stream_read", "bookkeeping",
                             *SECONDARY_WORKLOADS],
                    help="cfg2 (default) is the headline decode step; cfg3 is the mixed prefill+decode batch; the "
                         "mla_* / prefill_d* / sampling_* / log_probs_* workloads time one kernel of the rows built around the path")
    ap.add_argument("--split-tokens", type=int, default=0)
    ap.add_argument("--subtiles", type=int, default=0, help="16-token sub-tiles per loop iteration (1, 2 or 4)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--hip-graph", action="store_true", help="replay the step as one captured HIP graph")
    ap.add_argument("--attention-only", action="store_true", help="time the attention call alone")
    ap.add_argument("--separate-launches", action="store_true",
                    help="decode workloads: norm / RoPE / append as a launch of its own before the attention call")
    ap.add_argument("--fp8-kv", action="store_true", help="cfg3 only: run the mixed batch over an fp8-e4m3 KV cache")
    ap.add_argument("--read-mib", type=int, default=1146,
                    help="stream_read only: buffer size (default: the 1.2 GB one cfg2 launch streams)")
    ap.add_argument("--read-wgs-per-cu", type=int, default=2, help="stream_read only: workgroups per CU")
    ap.add_argument("--cpu-budget-s", type=float, default=12.0, help="seconds of CPU work for the cpu_baseline leg")
    ap.add_argument("--prefill-kernel", type=int, default=0, choices=[0, 1, 2, 3, -1],
                    help="MiTuning.prefill_two_phase for this run: 0 = the default (3), 1 = the two-phase tile kernel at "
                         "every width, 2 = the same with its wave groups in lock-step, 3 = the one-stream kernel at "
                         "head_dim 128, -1 = the register-only kernel")
    ap.add_argument("--settle-s", type=float, default=0.25,
                    help="seconds of untimed steps before the warm-up steps (clock settling; 0 = none)")
    ap.add_argument("--sustained-launches", type=int, default=1000,
                    help="cfg3: back-to-back launches of the tile kernel for the power-capped figure (0 = skip)")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="default cfg2 run only: do not append the cfg3 / cfg4 / cfg5 legs (other_configs)")
    ap.add_argument("--calibrate-copy-mib", type=int, default=0,
                    help="also run a plain device copy of this many MiB (a known-size reference for "
                         "scaling hardware traffic counters collected by an external profiler)")
    return ap.parse_args()


def _compact_chunks(torch, table_rows, n_pool, *tensors):
    """The chunks some block-table rows use, copied to the CPU and renumbered 0..n-1 (same logical contents)."""
    rows = table_rows.cpu()
    used = rows[rows >= 0].unique().long()
    remap = torch.full((n_pool,), -1, dtype=torch.int32)
    remap[used] = torch.arange(used.numel(), dtype=torch.int32)
    new_rows = torch.where(rows >= 0, remap[rows.clamp(min=0).long()], rows)
    return new_rows, [None if t is None else t[used.to(t.device)].cpu() for t in tensors]


class BoardPower:
    """Board power while a leg runs: a thread reads the amdgpu hwmon files (the driver's running average, which
    follows the load with a lag of a few hundred milliseconds, so only legs of about a second say anything)."""

    def __init__(self):
        import glob
        inp = sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_input")
                     + glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_average"))
        cap = sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_cap"))
        self.path = inp[0] if inp else None
        self.cap_w = self._read(cap[0]) if cap else None
        clk = sorted(glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk"))
        self.clk_path = clk[0] if clk else None   # the line marked '*' is the core clock right now
        self.samples = []
        self.clk_samples = []
        self._stop = False
        self._thread = None

    @staticmethod
    def _read(path):
        try:
            with open(path) as f:
                return int(f.read().strip()) / 1e6
        except (OSError, ValueError):
            return None

    @staticmethod
    def _read_clock(path):
        try:
            with open(path) as f:
                for line in f:
                    if "*" in line:
                        return float(line.split(":")[1].lower().replace("mhz", "").replace("*", "").strip())
        except (OSError, ValueError, IndexError):
            pass
        return None

    def __enter__(self):
        import threading
        if self.path:
            def loop():
                while not self._stop:
                    now = time.perf_counter()
                    self.samples.append((now, self._read(self.path)))
                    if self.clk_path:
                        self.clk_samples.append((now, self._read_clock(self.clk_path)))
                    time.sleep(0.01)
            self._thread = threading.Thread(target=loop, daemon=True)
            self._thread.start()
        return self

    def __exit__(self, *exc):
        self._stop = True
        if self._thread:
            self._thread.join()

    def mean_w(self, t_from: float, t_to: float):
        vals = [w for t, w in self.samples if w is not None and t_from <= t <= t_to]
        return round(sum(vals) / len(vals), 1) if vals else None

    def mean_clock_mhz(self, t_from: float, t_to: float):
        vals = [c for t, c in self.clk_samples if c is not None and t_from <= t <= t_to]
        return round(sum(vals) / len(vals), 0) if vals else None


def _time_cpu(torch, one_pass, budget_s: float = 12.0):
    """Median pass time after one warm-up: at least 3 timed passes, about ``budget_s`` seconds of CPU work."""
    torch.set_num_threads(os.cpu_count() or 1)
    times = []
    budget = time.perf_counter() + budget_s
    while len(times) < 4 or (time.perf_counter() < budget and len(times) < 200):
        t0 = time.perf_counter()
        one_pass()
        times.append(time.perf_counter() - t0)
    return sorted(times[1:])[len(times[1:]) // 2], len(times) - 1


def cpu_baseline(case, cfg, sample_requests: int, qw, kw, table, attention_only: bool, budget_s: float = 12.0):
    """Time the CPU checker on the first ``sample_requests`` requests of the same seeded batch, doing what the GPU
    step does: unfused q/k RMSNorm + RoPE (op by op in bf16), the scatter append of the new key / value rows
    (quantising for an fp8 cache), then gather through the block table + fp32 attention."""
    import torch

    from oracle import paged_attention as oa
    from oracle import rope_norm as orn

    n = min(sample_requests, case.q.size(0))
    q = case.q[:n].cpu().squeeze(1)
    k_new = case.k_new[:n].cpu().squeeze(1)
    v_new = case.v_new[:n].cpu().squeeze(1)
    lens = case.kv_lens[:n].cpu()
    bt, (kc, vc, ks, vs) = _compact_chunks(torch, case.block_table[:n], case.k_cache.size(0), case.k_cache,
                                           case.v_cache, case.k_scales, case.v_scales)
    pos = lens.long() - 1
    qw_c, kw_c, table_c = qw.cpu(), kw.cpu(), table.cpu()
    rows, ids, loc = oa.decode_slots(bt, lens, cfg.chunk)

    def one_pass():
        qn = q
        if not attention_only:
            qn = orn.norm_rope(q, pos, table_c, norm="rms", weight=qw_c, eps=1e-5)
            kn = orn.norm_rope(k_new, pos, table_c, norm="rms", weight=kw_c, eps=1e-5)
            if cfg.fp8:
                oa.kv_append_fp8(kc, ks, kn[rows], ids, loc)
                oa.kv_append_fp8(vc, vs, v_new[rows], ids, loc)
            else:
                oa.kv_append(kc, vc, kn[rows], v_new[rows], ids, loc)
        return oa.paged_decode_attention(qn, kc, vc, lens, bt, k_scales=ks, v_scales=vs)

    t, passes = _time_cpu(torch, one_pass, budget_s)
    nbytes = oa.decode_attention_bytes(lens.tolist(), cfg.Hq, cfg.Hkv, cfg.d, cfg.chunk,
                                       kv_bytes=1 if cfg.fp8 else 2, fp8_scales=cfg.fp8)
    what = ("fp32 gather + softmax checker" if attention_only else
            "unfused RMSNorm + RoPE, scatter append, then fp32 gather + softmax (oracle/rope_norm.py, oracle/paged_attention.py)")
    return {"value": nbytes / t / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"first {n} of {case.q.size(0)} requests of the same seeded batch: {what}; attention bytes of "
                      f"the sample / pass time, median of {passes} passes after 1 warm-up, {t * 1e3:.1f} ms/pass"}


def cpu_baseline_mixed(q, k_new, v_new, kc, vc, cu_q, lens, bt, qw, kw, table, n_prefill: int, n_decode: int,
                       Hq: int, Hkv: int, d: int, chunk: int, budget_s: float = 12.0):
    """The mixed step on the CPU checker for a bounded sample of the batch: the first ``n_prefill`` prefill
    requests and the first ``n_decode`` one-token requests -- unfused RMSNorm + RoPE of their new tokens, scatter
    append, varlen causal attention through the block table."""
    import torch

    from oracle import paged_attention as oa
    from oracle import rope_norm as orn

    lq_all = (cu_q[1:] - cu_q[:-1]).cpu()
    pre = [r for r in range(lens.numel()) if int(lq_all[r]) > 1][:n_prefill]
    dec = [r for r in range(lens.numel()) if int(lq_all[r]) == 1][:n_decode]
    reqs = pre + dec
    cu = cu_q.cpu()
    tok = torch.cat([torch.arange(int(cu[r]), int(cu[r + 1])) for r in reqs])
    qs, ks_new, vs_new = q[tok.to(q.device)].cpu(), k_new[tok.to(q.device)].cpu(), v_new[tok.to(q.device)].cpu()
    lens_s = lens.cpu()[reqs]
    lq = lq_all[reqs]
    cu_s = torch.zeros(len(reqs) + 1, dtype=torch.int32)
    cu_s[1:] = torch.cumsum(lq, 0)
    bt_s, (kcc, vcc) = _compact_chunks(torch, bt[reqs], kc.size(0), kc, vc)
    # per-token position, chunk and slot, as the context lays them out
    req_of = torch.repeat_interleave(torch.arange(len(reqs)), lq.long())
    pos = torch.arange(tok.numel()) - cu_s[req_of].long() + (lens_s.long() - lq.long())[req_of]
    ids = bt_s.long()[req_of, pos // chunk]
    loc = pos % chunk
    qw_c, kw_c, table_c = qw.cpu(), kw.cpu(), table.cpu()

    def one_pass():
        qn = orn.norm_rope(qs, pos, table_c, norm="rms", weight=qw_c, eps=1e-5)
        kn = orn.norm_rope(ks_new, pos, table_c, norm="rms", weight=kw_c, eps=1e-5)
        oa.kv_append(kcc, vcc, kn, vs_new, ids, loc)
        return oa.paged_varlen_attention(qn, kcc, vcc, cu_s, lens_s, bt_s)

    t, passes = _time_cpu(torch, one_pass, budget_s)
    lk = lens_s.long()
    is_pre = lq > 1
    dec_bytes = oa.decode_attention_bytes(lk[~is_pre].tolist(), Hq, Hkv, d, chunk)
    pre_bytes = int(lk[is_pre].sum()) * Hkv * d * 2 * 2 + int(lq[is_pre].sum()) * Hq * d * 4
    return {"value": (dec_bytes + pre_bytes) / t / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"{len(pre)} of the prefill requests ({int(lq[is_pre].sum())} new tokens) and {len(dec)} of the "
                      f"one-token requests of the same seeded batch: unfused RMSNorm + RoPE, scatter append, varlen "
                      f"causal attention through the block table (oracle/); the sample's algorithmic bytes / pass time, "
                      f"median of {passes} passes after 1 warm-up, {t * 1e3:.1f} ms/pass"}


def run_mixed_batch(args, mi, lib, torch, dev):
    """cfg3: 8 prefill requests x 2048 new tokens over U[0,4096] cached tokens + 120 decode requests
    with U[512,8192] tokens, one varlen call.  Step = fused RMSNorm+RoPE+append of all new tokens,
    then paged varlen attention (tile kernel for the prefill requests, streaming + merge kernels for
    the one-token requests).  Two roofline objects: MFMA for the tile kernel, HBM for the stream."""
    Hq, Hkv, d, chunk = 32, 8, 128, 256
    q, kc, vc, cu_q, lens, bt = mi.synthetic.make_prefill_case(
        dev, n_prefill=8, new_tokens=2048, ctx_lo=0, ctx_hi=4096, n_decode=120, dec_lo=512, dec_hi=8192,
        Hq=Hq, Hkv=Hkv, d=d, chunk=chunk, seed=1003, on_device_rng=True)
    T = q.size(0)
    gen = torch.Generator().manual_seed(2003)
    k_new = torch.randn(T, Hkv, d, generator=gen).bfloat16().to(dev)
    v_new = torch.randn(T, Hkv, d, generator=gen).bfloat16().to(dev)
    qw = (1 + 0.02 * torch.randn(d, generator=gen)).bfloat16().to(dev)
    kw = (1 + 0.02 * torch.randn(d, generator=gen)).bfloat16().to(dev)
    pos, tok_chunk, tok_local = mi.synthetic.prefill_token_rows(cu_q, lens, bt, chunk)
    max_len = int(lens.max())
    table = mi.synthetic.rotary_angle_table(max_len + 1, d, base=500000.0).to(dev)
    q_rot = torch.empty_like(q)
    out = torch.empty_like(q)
    ks = vs = None
    if args.fp8_kv:
        k8, v8 = torch.empty(kc.shape, dtype=torch.uint8, device=dev), torch.empty(kc.shape, dtype=torch.uint8, device=dev)
        ks = torch.empty(kc.size(0), Hkv, dtype=torch.float32, device=dev)
        vs = torch.empty_like(ks)
        mi.ops.quantize_chunks_fp8(kc, k8, ks)
        mi.ops.quantize_chunks_fp8(vc, v8, vs)
        kc, vc = k8, v8
        k_rot = torch.empty_like(k_new)

    def step():
        if args.fp8_kv:
            mi.ops.norm_rope_append(q, k_new, query_out=q_rot, key_out=k_rot, q_weight=qw, k_weight=kw, eps=1e-5,
                                    norm="rms", rotary_emb=table, q_positions=pos, k_positions=pos)
            mi.ops.kv_append_fp8(k_rot, v_new, kc, vc, ks, vs, tok_chunk, tok_local)
        else:
            mi.ops.norm_rope_append(q, k_new, query_out=q_rot, value=v_new, q_weight=qw, k_weight=kw, eps=1e-5,
                                    norm="rms", rotary_emb=table, q_positions=pos, k_positions=pos, k_cache=kc,
                                    v_cache=vc, token_to_chunk_idx=tok_chunk, token_to_local_pos=tok_local)
        mi.ops.paged_prefill_attention(q_rot, kc, vc, cu_q, lens, bt, max_kv_len=max_len, out=out,
                                       k_scales=ks, v_scales=vs)

    if args.calibrate_copy_mib:  # a copy of known size for scaling an external profiler's traffic counters
        src = torch.empty(args.calibrate_copy_mib << 20, dtype=torch.uint8, device=dev).random_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    lib.mi_profile_enable(1)
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    buf = (ctypes.c_float * (2 * args.steps))()
    n_ev = lib.mi_profile_collect(buf, 2 * args.steps)
    lib.mi_profile_enable(0)
    tile_ms = sum(buf[i] for i in range(0, n_ev, 2)) / max(1, n_ev // 2)
    stream_ms = sum(buf[i] for i in range(1, n_ev, 2)) / max(1, n_ev // 2)

    # The tile kernel alone, launched back to back for about a second (the prefill requests only, no workspace, so
    # the call is that one kernel), with the board power read beside it: this kernel runs the board into its power
    # cap, and what a power-capped kernel reaches is set by the energy it spends, not by its schedule.
    sustained = None
    if args.sustained_launches > 0:
        n_pre = int((cu_q[1:] - cu_q[:-1] > 1).sum())
        t_pre = int(cu_q[n_pre])
        cu_pre, lens_pre, bt_pre = cu_q[:n_pre + 1].contiguous(), lens[:n_pre].contiguous(), bt[:n_pre].contiguous()
        q_pre, out_pre = q_rot[:t_pre], out[:t_pre]
        def tile_only():
            mi.ops.paged_prefill_attention(q_pre, kc, vc, cu_pre, lens_pre, bt_pre, max_kv_len=max_len, out=out_pre,
                                           k_scales=ks, v_scales=vs)
        for _ in range(5):
            tile_only()
        torch.cuda.synchronize()
        with BoardPower() as power:
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            t_a = time.perf_counter()
            e0.record()
            for _ in range(args.sustained_launches):
                tile_only()
            e1.record()
            torch.cuda.synchronize()
            t_b = time.perf_counter()
        sus_ms = e0.elapsed_time(e1) / args.sustained_launches
        sustained = {"launches": args.sustained_launches, "kernel_ms": round(sus_ms, 5),
                     "achieved": None, "board_power_w": power.mean_w(t_a + 0.6 * (t_b - t_a), t_b),
                     "power_cap_w": power.cap_w,
                     "core_clock_mhz": power.mean_clock_mhz(t_a + 0.6 * (t_b - t_a), t_b),
                     "what": "the prefill requests' tile kernel launched back to back; board power and core clock = "
                             "means of the driver's readings (hwmon power1_input, pp_dpm_sclk) over the last 40 % of "
                             "the run; the clock's ceiling is 2400 MHz"}

    lq = (cu_q[1:] - cu_q[:-1]).cpu().long()
    lk = lens.cpu().long()
    pre = lq > 1
    flops = 4 * Hq * d * int((lq[pre] * (lk - lq)[pre] + lq[pre] * (lq[pre] + 1) // 2).sum())
    kvb = 1 if args.fp8_kv else 2
    dec_bytes = mi.synthetic.decode_attention_bytes(lk[~pre].tolist(), Hq, Hkv, d, chunk, kv_bytes=kvb, fp8_scales=args.fp8_kv)
    pre_kv_bytes = int(lk[pre].sum()) * Hkv * d * 2 * kvb + int(lq[pre].sum()) * Hq * d * 4
    ms_per_step = elapsed * 1e3 / args.steps
    total_bytes = dec_bytes + pre_kv_bytes
    result = {
        "metric": "paged_decode_attention_hbm_GBps",
        "value": round(total_bytes / (ms_per_step * 1e-3) / 1e9, 1),
        "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp8-e4m3 KV, bf16 q/out, fp32 accumulate" if args.fp8_kv else "bf16 (fp32 accumulate)",
        "data": "synthetic",
        "config": {"workload": "cfg3: mixed batch, 8 x 2048-token prefill over U[0,4096] + 120 decode U[512,8192], "
                               "32/8 heads d128 chunk 256; step = fused RMSNorm+RoPE+append then paged varlen attention"
                               + (" (fp8-e4m3 KV cache, quantising append)" if args.fp8_kv else ""),
                   "new_tokens": T, "requests": int(lens.numel()), "algorithmic_bytes_per_step": total_bytes,
                   "prefill_flops_per_step": flops},
        "roofline": {"bound": "mfma", "kernel": ("paged_prefill_pp_kernel" if (args.fp8_kv or args.prefill_kernel not in (0, 3))
                                                  else "paged_prefill_woven_kernel"),
                     "achieved": round(flops / tile_ms / 1e9, 1),
                     "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(flops / tile_ms / 1e9 / MFMA_BF16_PEAK_TFLOPS, 4), "kernel_ms": round(tile_ms, 5),
                     "traffic": None if args.fp8_kv else MEASURED_HBM_TRAFFIC_BYTES["cfg3_tile"],
                     "traffic_source": None if args.fp8_kv else TRAFFIC_SOURCE["cfg3_tile"]},
        "roofline_decode_part": {"bound": "hbm", "kernel": "paged_decode_stream_kernel",
                                 "achieved": round(dec_bytes / stream_ms / 1e6, 1), "peak": HBM_PEAK_GBPS,
                                 "unit": "GB/s", "frac": round(dec_bytes / stream_ms / 1e6 / HBM_PEAK_GBPS, 4),
                                 "kernel_ms": round(stream_ms, 5),
                                 "traffic": None if args.fp8_kv else MEASURED_HBM_TRAFFIC_BYTES["cfg3_stream"],
                                 "traffic_source": None if args.fp8_kv else TRAFFIC_SOURCE["cfg3_stream"]},
    }
    if sustained is not None:
        sustained["achieved"] = round(flops / sustained["kernel_ms"] / 1e9, 1)
        sustained["frac"] = round(flops / sustained["kernel_ms"] / 1e9 / MFMA_BF16_PEAK_TFLOPS, 4)
        result["roofline"]["sustained"] = sustained
    if not args.no_cpu_baseline and not args.fp8_kv:
        result["cpu_baseline"] = cpu_baseline_mixed(q, k_new, v_new, kc, vc, cu_q, lens, bt, qw, kw, table,
                                                    n_prefill=1, n_decode=15, Hq=Hq, Hkv=Hkv, d=d, chunk=chunk,
                                                    budget_s=args.cpu_budget_s)
    return result


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU: this build's hot path is a single-GPU kernel path and --gpus "
              f"{args.gpus} is not supported (no collectives are part of it).", file=sys.stderr)
        sys.exit(2)

    import copy

    import torch

    from __graft_entry__ import load_package

    mi = load_package()
    lib = mi._lib.load()  # raises if the HIP library is missing: there is no fallback to measure
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    if args.subtiles:
        mi.ops.set_tuning("decode_tile_subtiles", args.subtiles)  # (passed with every call of the ops module)
    if args.prefill_kernel:
        mi.ops.set_tuning("prefill_two_phase", args.prefill_kernel)

    result = run_workload(args, mi, lib, torch, dev)
    # The default run carries the other single-GPU configurations beside the headline one: the mixed batch (cfg3),
    # the long-context batch (cfg4) and the fp8 cache (cfg5), each with its own roofline and a short CPU leg.
    plain = not (args.hip_graph or args.attention_only or args.separate_launches or args.fp8_kv or args.subtiles
                 or args.split_tokens or args.calibrate_copy_mib or args.prefill_kernel)
    if args.workload == "cfg2" and plain and not args.no_other_configs:
        others = {}
        # (their own step counts, stated in each entry: a step is 1.2-1.4 ms, and the first dozen launches after a
        # set-up run at a clock that has not settled, so a few more warm-up steps cost nothing and say more)
        for name, steps, warmup in (("cfg3", 50, 10), ("cfg4", 30, 5), ("cfg5", 30, 5)):
            sub = copy.copy(args)
            sub.workload, sub.steps, sub.warmup, sub.cpu_budget_s = name, steps, warmup, 3.0
            torch.cuda.empty_cache()
            r = run_workload(sub, mi, lib, torch, dev)
            others[name] = {k: r[k] for k in ("value", "unit", "steps", "warmup", "ms_per_step", "dtype", "config", "roofline",
                                              "roofline_decode_part", "separate_launches", "cpu_baseline") if k in r}
        result["other_configs"] = others
    print(json.dumps(result), flush=True)


def run_workload(args, mi, lib, torch, dev):
    """One workload -> its result line as a dictionary."""
    if args.workload == "cfg3":
        return run_mixed_batch(args, mi, lib, torch, dev)
    if args.workload == "stream_read":
        return run_stream_read(args, mi, torch, dev)
    if args.workload == "bookkeeping":
        return run_bookkeeping(args, mi, lib, torch, dev)
    if args.workload in SECONDARY_WORKLOADS:
        return run_secondary(args, mi, lib, torch, dev)
    return run_decode_config(args, mi, lib, torch, dev)


def run_decode_config(args, mi, lib, torch, dev):
    """cfg1 / cfg2 / cfg4 / cfg5 (and cfg3's decode part alone): one decode step per timed step."""
    cfg = mi.synthetic.CONFIGS[args.workload]
    case = mi.synthetic.make_decode_case(cfg, dev, on_device_rng=True)
    if cfg.fp8:
        k8 = torch.empty(case.k_cache.shape, dtype=torch.uint8, device=dev)
        v8 = torch.empty_like(k8)
        case.k_scales = torch.empty(case.k_cache.size(0), cfg.Hkv, dtype=torch.float32, device=dev)
        case.v_scales = torch.empty_like(case.k_scales)
        mi.ops.quantize_chunks_fp8(case.k_cache, k8, case.k_scales)
        mi.ops.quantize_chunks_fp8(case.v_cache, v8, case.v_scales)
        torch.cuda.synchronize()
        case.k_cache, case.v_cache = k8, v8
        torch.cuda.empty_cache()

    lens_host = case.kv_lens.cpu()
    max_len = int(lens_host.max())
    gen = torch.Generator().manual_seed(cfg.seed + 1)
    qw = (1 + 0.02 * torch.randn(cfg.d, generator=gen)).bfloat16().to(dev)
    kw = (1 + 0.02 * torch.randn(cfg.d, generator=gen)).bfloat16().to(dev)
    theta = cfg.rope_theta or 500000.0
    table = mi.synthetic.rotary_angle_table(max_len + 1, cfg.d, base=theta).to(dev)
    pos = (case.kv_lens.long() - 1).contiguous()
    q_in = case.q.clone()
    out = torch.empty_like(case.q)
    use_norm = "rms"

    # the whole step inside the streaming kernel unless asked otherwise
    one_kernel = (not args.attention_only and not args.separate_launches
                  and mi.ops.decode_step_supported(cfg.d, cfg.d, False, cfg.fp8))

    def step():
        if one_kernel:
            mi.ops.decode_step_attention(case.q, case.k_new, case.v_new, case.k_cache, case.v_cache, case.kv_lens,
                                         case.block_table, q_weight=qw, k_weight=kw, eps=1e-5, norm=use_norm,
                                         rotary_emb=table, positions=None, out=out, max_kv_len=max_len,
                                         split_tokens=args.split_tokens, k_scales=case.k_scales,
                                         v_scales=case.v_scales)  # (positions: kv_lens - 1)
            return
        if not args.attention_only:
            if cfg.fp8:
                mi.ops.norm_rope_append(case.q, case.k_new, query_out=q_in, key_out=k_rot, q_weight=qw, k_weight=kw, eps=1e-5,
                                        norm=use_norm, rotary_emb=table, q_positions=pos, k_positions=pos)
                mi.ops.kv_append_decode_fp8(k_rot, case.v_new, case.k_cache, case.v_cache, case.k_scales,
                                            case.v_scales, case.block_table, case.kv_lens)
            else:
                mi.ops.norm_rope_append(case.q, case.k_new, query_out=q_in, value=case.v_new, q_weight=qw, k_weight=kw, eps=1e-5,
                                        norm=use_norm, rotary_emb=table, q_positions=pos, k_positions=pos,
                                        k_cache=case.k_cache, v_cache=case.v_cache, block_table=case.block_table,
                                        kv_lens=case.kv_lens)
        mi.ops.paged_decode_attention(q_in, case.k_cache, case.v_cache, case.kv_lens, case.block_table, out=out,
                                      max_kv_len=max_len, split_tokens=args.split_tokens,
                                      k_scales=case.k_scales, v_scales=case.v_scales)

    if args.calibrate_copy_mib:
        src = torch.empty(args.calibrate_copy_mib << 20, dtype=torch.uint8, device=dev).random_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    k_rot = torch.empty_like(case.k_new)
    nbytes = mi.synthetic.decode_attention_bytes(lens_host.tolist(), cfg.Hq, cfg.Hkv, cfg.d, cfg.chunk,
                                       kv_bytes=1 if cfg.fp8 else 2, fp8_scales=cfg.fp8)
    buf = (ctypes.c_float * args.steps)()

    # The same step as three launches (norm / RoPE / append, then the attention-only streaming kernel, then the
    # merge), timed first (the extra leg then also brings the device to its running state before the leg that
    # counts): its streaming kernel does attention alone, so its rate is the one to hold
    # against the HBM roofline kernel for kernel; the one-kernel step trades a little of that for a launch.
    separate = None
    if one_kernel:
        def step_separate():
            if cfg.fp8:
                mi.ops.norm_rope_append(case.q, case.k_new, query_out=q_in, key_out=k_rot, q_weight=qw, k_weight=kw,
                                        eps=1e-5, norm=use_norm, rotary_emb=table, q_positions=pos, k_positions=pos)
                mi.ops.kv_append_decode_fp8(k_rot, case.v_new, case.k_cache, case.v_cache, case.k_scales,
                                            case.v_scales, case.block_table, case.kv_lens)
            else:
                mi.ops.norm_rope_append(case.q, case.k_new, query_out=q_in, value=case.v_new, q_weight=qw, k_weight=kw,
                                        eps=1e-5, norm=use_norm, rotary_emb=table, q_positions=pos, k_positions=pos,
                                        k_cache=case.k_cache, v_cache=case.v_cache, block_table=case.block_table,
                                        kv_lens=case.kv_lens)
            mi.ops.paged_decode_attention(q_in, case.k_cache, case.v_cache, case.kv_lens, case.block_table, out=out,
                                          max_kv_len=max_len, split_tokens=args.split_tokens,
                                          k_scales=case.k_scales, v_scales=case.v_scales)
        for _ in range(args.warmup):
            step_separate()
        torch.cuda.synchronize()
        lib.mi_profile_enable(1)
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step_separate()
        torch.cuda.synchronize()
        sep_ms = (time.perf_counter() - t0) * 1e3 / args.steps
        n_sep = lib.mi_profile_collect(buf, args.steps)
        lib.mi_profile_enable(0)
        sep_kernel_ms = sum(buf[i] for i in range(min(n_sep, args.steps))) / max(1, min(n_sep, args.steps))
        separate = {"ms_per_step": round(sep_ms, 5), "value": round(nbytes / (sep_ms * 1e-3) / 1e9, 1),
                    "kernel": "paged_decode_stream_kernel", "kernel_ms": round(sep_kernel_ms, 5),
                    "achieved": round(nbytes / (sep_kernel_ms * 1e-3) / 1e9, 1),
                    "frac": round(nbytes / (sep_kernel_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                    "traffic": MEASURED_HBM_TRAFFIC_BYTES.get(args.workload),
                    "traffic_source": TRAFFIC_SOURCE.get(args.workload)}
    # The GPU's clocks take a few hundred launches to settle after the set-up (allocation, input generation, the
    # host-side CPU legs of earlier workloads): steps until `settle_s` seconds have passed come before the W warm-up
    # steps and the K timed ones, so that a short run (K = 20) measures the same steady state as a long one.
    t_settle = time.perf_counter()
    n_settle = 0
    while time.perf_counter() - t_settle < args.settle_s:
        for _ in range(10):
            step()
        torch.cuda.synchronize()
        n_settle += 10
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()

    graph = None
    if args.hip_graph:
        # the step as one HIP graph (the reference replays CUDA graphs for decode steps); the
        # per-kernel events cannot be recorded inside a graph, so kernel_ms then comes from the
        # eager steps timed right after the graph loop
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            step()
        for _ in range(3):
            graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            graph.replay()
        torch.cuda.synchronize()
        graph_elapsed = time.perf_counter() - t0

    lib.mi_profile_enable(1)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    if graph is not None:
        elapsed = graph_elapsed
    n_ev = lib.mi_profile_collect(buf, args.steps)
    lib.mi_profile_enable(0)
    kernel_ms = sum(buf[i] for i in range(min(n_ev, args.steps))) / max(1, min(n_ev, args.steps))

    ms_per_step = elapsed * 1e3 / args.steps

    value = nbytes / (ms_per_step * 1e-3) / 1e9
    achieved = nbytes / (kernel_ms * 1e-3) / 1e9

    result = {
        "metric": "paged_decode_attention_hbm_GBps",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp8-e4m3 KV, bf16 q/out, fp32 accumulate" if cfg.fp8 else "bf16 (fp32 accumulate)",
        "data": "synthetic",
        "config": {
            "workload": cfg.name + (", attention call only" if args.attention_only
                                    else ", step = RMSNorm+RoPE+KV-append inside the paged decode attention kernel, then merge"
                                    if one_kernel
                                    else ", step = fused RMSNorm+RoPE+KV-append then paged decode attention")
            + (", replayed as one HIP graph" if args.hip_graph else ""),
            "batch": case.q.size(0), "q_heads": cfg.Hq, "kv_heads": cfg.Hkv, "head_dim": cfg.d,
            "chunk_tokens": cfg.chunk, "kv_tokens_total": int(lens_host.sum()), "kv_len_max": max_len,
            "algorithmic_bytes_per_step": nbytes,
            "untimed_steps_before_warmup": n_settle,
        },
        "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBPS, 2),
        "decode_steps_per_sec": round(1e3 / ms_per_step, 1),
        "roofline": {
            "bound": "hbm",
            "kernel": "decode_step_stream_kernel" if one_kernel else "paged_decode_stream_kernel",
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBPS, 4),
            "kernel_ms": round(kernel_ms, 5),
            "traffic": MEASURED_HBM_TRAFFIC_BYTES.get(args.workload + "_step" if one_kernel else args.workload),
            "traffic_source": TRAFFIC_SOURCE.get(args.workload + "_step" if one_kernel else args.workload),
        },
    }
    if separate is not None:
        result["separate_launches"] = separate
    if not args.no_cpu_baseline:
        sample = {"cfg1": 4, "cfg2": 64, "cfg3_decode": 64, "cfg4": 1, "cfg5": 16}[args.workload]
        result["cpu_baseline"] = cpu_baseline(case, cfg, sample, qw, kw, table, args.attention_only, args.cpu_budget_s)
    return result


if __name__ == "__main__":
    main()
