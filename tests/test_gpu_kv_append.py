"""GPU parity: KV-append is a bit-exact scatter (both addressing modes)."""
import pytest
import torch

from oracle import paged_attention as oa

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("Hkv,d", [(8, 128), (2, 8), (3, 5)])
def test_append_with_token_rows(mi, dev, dtype, Hkv, d):
    """Slots from the per-token rows; padded tokens all target the dummy chunk's slot 0."""
    gen = torch.Generator().manual_seed(Hkv * 100 + d)
    N, C, T, T_pad = 9, 16, 21, 32
    kc = torch.full((N, C, Hkv, d), -1, dtype=dtype)
    vc = torch.full((N, C, Hkv, d), -1, dtype=dtype)
    key = torch.randn(T_pad, 1, Hkv, d, generator=gen).to(dtype)
    val = torch.randn(T_pad, 1, Hkv, d, generator=gen).to(dtype)
    slots = torch.randperm((N - 1) * C, generator=gen)[:T]
    chunk_idx = torch.full((64,), N - 1, dtype=torch.int64)
    local = torch.zeros(64, dtype=torch.int64)
    chunk_idx[:T], local[:T] = slots // C, slots % C
    kc_d, vc_d = kc.to(dev), vc.to(dev)
    mi.ops.kv_append(key.to(dev), val.to(dev), kc_d, vc_d, chunk_idx.to(dev), local.to(dev))
    torch.cuda.synchronize()
    oa.kv_append(kc, vc, key.squeeze(1)[:T], val.squeeze(1)[:T], chunk_idx[:T], local[:T])
    # every slot outside the dummy chunk's slot 0 is bit-identical; untouched slots keep the fill
    assert torch.equal(kc_d.cpu()[: N - 1].view(torch.uint8), kc[: N - 1].view(torch.uint8))
    assert torch.equal(vc_d.cpu()[: N - 1].view(torch.uint8), vc[: N - 1].view(torch.uint8))
    assert torch.equal(kc_d.cpu()[N - 1, 1:], kc[N - 1, 1:])
    # the dummy slot holds padded-row data (duplicates race element by element, any writer may win)
    dummy = kc_d.cpu()[N - 1, 0]
    assert (dummy.unsqueeze(0) == key[T:T_pad, 0]).any(dim=0).all()


def test_append_decode_slots_on_gpu(mi, dev):
    """One new token per request; slot = (block_table[r][(len-1)//C], (len-1)%C); len 0 rows write nothing."""
    lens = torch.tensor([1, 256, 257, 700, 0, 512, 513, 3], dtype=torch.int32)
    cfg = mi.synthetic.DecodeConfig("app", lens.numel(), 32, 8, 128, 0, 0, seed=42)
    case = mi.synthetic.make_decode_case(cfg, dev, lens=lens)
    kc, vc = case.k_cache.cpu().clone(), case.v_cache.cpu().clone()
    mi.ops.kv_append_decode(case.k_new, case.v_new, case.k_cache, case.v_cache, case.block_table, case.kv_lens)
    torch.cuda.synchronize()
    rows, ids, loc = oa.decode_slots(case.block_table.cpu(), lens, cfg.chunk)
    oa.kv_append(kc, vc, case.k_new.cpu().squeeze(1)[rows], case.v_new.cpu().squeeze(1)[rows], ids, loc)
    assert torch.equal(case.k_cache.cpu().view(torch.int16), kc.view(torch.int16))
    assert torch.equal(case.v_cache.cpu().view(torch.int16), vc.view(torch.int16))


def test_append_into_layer_views_of_memory_buffer(mi, dev):
    """The cache views handed out by the context are strided slices of memory_buffer[2, L, N, C, H, d]."""
    L, N, C, H, d, T = 3, 5, 32, 4, 64, 7
    buf = torch.full((2, L, N, C, H, d), -1, dtype=torch.bfloat16, device=dev)
    gen = torch.Generator().manual_seed(0)
    key = torch.randn(T, 1, H, d, generator=gen).bfloat16().to(dev)
    val = torch.randn(T, 1, H, d, generator=gen).bfloat16().to(dev)
    slots = torch.randperm(N * C, generator=gen)[:T]
    ci, lo = (slots // C).to(dev), (slots % C).to(dev)
    mi.ops.kv_append(key, val, buf[0, 1], buf[1, 1], ci, lo)
    torch.cuda.synchronize()
    ref = torch.full((2, L, N, C, H, d), -1, dtype=torch.bfloat16)
    ref[0, 1, slots // C, slots % C] = key.cpu().squeeze(1)
    ref[1, 1, slots // C, slots % C] = val.cpu().squeeze(1)
    assert torch.equal(buf.cpu(), ref)
