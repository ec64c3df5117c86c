"""GPU parity: the decode-sized projections (`mi_linear_decode`, `mi_linear_qkv_decode_step`,
`mi_attention_out_linear_proj`) against fp32 matrix products, and the attention layer from hidden states to hidden
states against the checker's chain (projection -> split -> head norm -> RoPE -> append -> attention -> projection).

Tolerance of a projection: the result is one rounding to the 16-bit type of an fp32 sum whose order differs from
the library's, so the two may land on neighbouring values of the 16-bit type: one unit in the last place
(2^-7 relative for bf16, 2^-10 for fp16).  The layer chain is held to the path's 2e-2.
"""
import ctypes

import pytest
import torch

from oracle import paged_attention as oa
from oracle import projections as opj
from oracle import rope_norm as orn

pytestmark = pytest.mark.gpu


def _ulp_close(got, ref, dtype, what):
    got, ref = got.float().cpu(), ref.float().cpu()
    assert torch.isfinite(got).all(), f"{what}: non-finite"
    ulp = 2.0 ** (-7 if dtype == torch.bfloat16 else -10)   # largest relative spacing of the 16-bit type
    err = (got - ref).abs()
    bound = 1.01 * ulp * torch.maximum(ref.abs(), got.abs()) + 1e-3   # one unit in the last place
    assert (err <= bound).all(), f"{what}: max err {err.max().item():.4e} at ref {ref.flatten()[err.argmax()].item():.4e}"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("T,N,K,bias", [
    (64, 6144, 4096, False), (64, 4096, 4096, False), (1, 6144, 4096, True), (17, 4096, 4096, True),
    (256, 6144, 4096, True), (130, 1536, 1024, False), (5, 64, 512, True), (33, 48, 96, True), (64, 16, 32, False),
    (100, 2064, 4000, True), (3, 10240, 8192, False)])
def test_linear_decode_matches_an_fp32_product(mi, dev, T, N, K, bias, dtype):
    gen = torch.Generator().manual_seed(T + N + K)
    x = (torch.randn(T, K, generator=gen) * 0.5).to(dtype).to(dev)
    w = (torch.randn(N, K, generator=gen) * 0.05).to(dtype).to(dev)
    b = (torch.randn(N, generator=gen)).to(dtype).to(dev) if bias else None
    out = mi.ops.linear_decode(x, w, b)
    torch.cuda.synchronize()
    ref = x.float() @ w.float().t()
    if bias:
        ref = ref + b.float()
    _ulp_close(out, ref.to(dtype), dtype, f"linear {T}x{N}x{K}")
    # twice the same bits (fixed summation order), and rows of x beyond T / strided inputs are respected
    out2 = mi.ops.linear_decode(x, w, b)
    assert torch.equal(out, out2)


def test_strided_inputs_and_leading_dimensions(mi, dev):
    gen = torch.Generator().manual_seed(5)
    big_x = (torch.randn(24, 1, 2 * 512, generator=gen) * 0.5).bfloat16().to(dev)
    big_w = (torch.randn(256, 3 * 512, generator=gen) * 0.05).bfloat16().to(dev)
    x, w = big_x[..., :512], big_w[:, 512:1024]
    out = torch.full((24, 1, 300), 7.0, dtype=torch.bfloat16, device=dev)
    mi.ops.linear_decode(x, w, out=out[..., :256])
    torch.cuda.synchronize()
    ref = (x.float().reshape(24, 512) @ w.float().t()).bfloat16()
    _ulp_close(out[..., :256].reshape(24, 256), ref, torch.bfloat16, "strided")
    assert (out[..., 256:] == 7.0).all(), "columns beyond N were touched"


def test_rejections(mi, dev):
    x = torch.zeros(300, 64, dtype=torch.bfloat16, device=dev)
    w = torch.zeros(32, 64, dtype=torch.bfloat16, device=dev)
    with pytest.raises(mi._lib.KernelError, match="1..256 tokens"):
        mi.ops.linear_decode(x, w)
    with pytest.raises(mi._lib.KernelError, match="multiple of 16"):
        mi.ops.linear_decode(x[:4], torch.zeros(24, 64, dtype=torch.bfloat16, device=dev))
    with pytest.raises(ValueError):
        mi.ops.linear_decode(x[:4], w.float())


def test_named_entry_points_through_the_c_abi(mi, dev):
    """mi_linear_qkv_decode_step / mi_attention_out_linear_proj with raw pointers, as a C caller would."""
    lib = mi._lib.load()
    T, hidden, Hq, Hkv, d = 8, 256, 8, 2, 64
    gen = torch.Generator().manual_seed(9)
    x = (torch.randn(T, hidden, generator=gen) * 0.5).bfloat16().to(dev)
    wqkv = (torch.randn((Hq + 2 * Hkv) * d, hidden, generator=gen) * 0.05).bfloat16().to(dev)
    bqkv = torch.randn((Hq + 2 * Hkv) * d, generator=gen).bfloat16().to(dev)
    wo = (torch.randn(hidden, Hq * d, generator=gen) * 0.05).bfloat16().to(dev)
    mixed = torch.empty(T, (Hq + 2 * Hkv) * d, dtype=torch.bfloat16, device=dev)
    n_ws = max(lib.mi_linear_decode_workspace_bytes(T, (Hq + 2 * Hkv) * d, hidden), lib.mi_linear_decode_workspace_bytes(T, hidden, Hq * d), 16)
    ws = torch.empty(n_ws, dtype=torch.uint8, device=dev)
    st = torch.cuda.current_stream().cuda_stream
    rc = lib.mi_linear_qkv_decode_step(x.data_ptr(), hidden, wqkv.data_ptr(), hidden, bqkv.data_ptr(), mixed.data_ptr(),
                                       mixed.stride(0), ws.data_ptr(), n_ws, T, hidden, Hq, Hkv, d, 0, st)
    assert rc == 0, lib.mi_last_error()
    _ulp_close(mixed, opj.linear(x.cpu(), wqkv.cpu(), bqkv.cpu())[0], torch.bfloat16, "qkv")
    attn = (torch.randn(T, Hq * d, generator=gen) * 0.5).bfloat16().to(dev)
    out = torch.empty(T, hidden, dtype=torch.bfloat16, device=dev)
    rc = lib.mi_attention_out_linear_proj(attn.data_ptr(), Hq * d, wo.data_ptr(), Hq * d, out.data_ptr(), hidden,
                                          ws.data_ptr(), n_ws, T, hidden, Hq, d, 0, st)
    assert rc == 0, lib.mi_last_error()
    torch.cuda.synchronize()
    _ulp_close(out, opj.linear(attn.cpu(), wo.cpu())[0], torch.bfloat16, "proj")
    # a workspace that is too small is refused before anything is launched
    rc = lib.mi_linear_decode(x.data_ptr(), hidden, wqkv.data_ptr(), hidden, None, mixed.data_ptr(), mixed.stride(0),
                              ws.data_ptr(), 16, 64, (Hq + 2 * Hkv) * d, hidden, 0, st)
    assert rc == -5


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
def test_attention_layer_from_hidden_states_to_hidden_states(mi, dev, dtype):
    """cfg2's layer shape on a small batch: hidden 4096 -> QKV projection -> (split, RMSNorm, RoPE, append, decode
    attention) -> output projection, against the checker's chain in fp32 / the tensors' type."""
    hidden, Hq, Hkv, d, chunk = 4096, 32, 8, 128, 256
    lens = torch.tensor([1, 255, 256, 257, 900, 3000, 17, 512, 2049, 64, 5, 1500], dtype=torch.int32)
    R = lens.numel()
    cfg = mi.synthetic.DecodeConfig("layer", R, Hq, Hkv, d, 0, 0, chunk=chunk, seed=21)
    case = mi.synthetic.make_decode_case(cfg, dev, lens=lens, dtype=dtype)
    gen = torch.Generator().manual_seed(22)
    x = torch.randn(R, 1, hidden, generator=gen).to(dtype)
    wqkv = (torch.randn((Hq + 2 * Hkv) * d, hidden, generator=gen) * hidden ** -0.5).to(dtype)
    bqkv = (torch.randn((Hq + 2 * Hkv) * d, generator=gen) * 0.1).to(dtype)
    wo = (torch.randn(hidden, Hq * d, generator=gen) * (Hq * d) ** -0.5).to(dtype)
    qw = (1 + 0.05 * torch.randn(d, generator=gen)).to(dtype)
    kw = (1 + 0.05 * torch.randn(d, generator=gen)).to(dtype)
    table = orn.rotary_table(4096, d, base=500000.0)
    pos = lens.long() - 1

    # ---- checker chain (CPU) ----
    mixed_ref, _ = opj.linear(x.squeeze(1), wqkv, bqkv)
    q_ref, k_ref, v_ref = opj.qkv_split(mixed_ref, Hq, Hkv, d)
    qn = orn.norm_rope(q_ref, pos, table, norm="rms", weight=qw, eps=1e-5)
    kn = orn.norm_rope(k_ref, pos, table, norm="rms", weight=kw, eps=1e-5)
    kc, vc = case.k_cache.cpu().clone(), case.v_cache.cpu().clone()
    rows, ids, loc = oa.decode_slots(case.block_table.cpu(), lens, chunk)
    oa.kv_append(kc, vc, kn[rows], v_ref[rows], ids, loc)
    attn_ref = oa.paged_decode_attention(qn, kc, vc, lens, case.block_table.cpu())
    out_ref, _ = opj.linear(attn_ref.reshape(R, Hq * d).to(dtype), wo)

    # ---- product (GPU): three launches + merge ----
    layer = mi.attention.PagedSelfAttentionLayer(1, hidden, Hq, Hkv, d, qk_norm="rms", eps=1e-5, add_qkv_bias=True,
                                                 dtype=dtype, device=dev)
    with torch.no_grad():
        layer.linear_qkv.weight.copy_(wqkv); layer.linear_qkv.bias.copy_(bqkv); layer.linear_proj.weight.copy_(wo)
        layer.core.q_layernorm_weight.copy_(qw); layer.core.k_layernorm_weight.copy_(kw)
    mixed, _ = layer.linear_qkv(x.to(dev))
    out_attn = mi.ops.decode_step_attention(None, None, None, case.k_cache, case.v_cache, case.kv_lens, case.block_table,
                                            mixed_qkv=mixed, num_query_heads=Hq, num_kv_heads=Hkv, q_weight=qw.to(dev),
                                            k_weight=kw.to(dev), norm="rms", eps=1e-5, rotary_emb=table.to(dev))
    out, bias = layer.linear_proj(out_attn.reshape(R, 1, Hq * d))
    torch.cuda.synchronize()
    assert bias is None
    _ulp_close(mixed.squeeze(1), mixed_ref, dtype, "mixed_qkv")
    got_k = case.k_cache.cpu().float()
    assert (got_k - kc.float()).abs().max().item() <= 4e-2, "appended keys"
    assert torch.equal(case.v_cache.cpu()[ids, loc], vc[ids, loc]) or (case.v_cache.cpu().float() - vc.float()).abs().max().item() <= 2e-2
    err = (out.float().cpu().squeeze(1) - out_ref.float()).abs()
    assert (err <= 2e-2 + 2e-2 * out_ref.float().abs()).all(), f"layer output: max err {err.max().item():.4e}"
