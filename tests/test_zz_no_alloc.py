"""GPU parity of the entry point that allocates nothing, ``mi_paged_decode_attention_noalloc``.

It shares every kernel with ``mi_paged_decode_attention``; only the home of the partials differs (the
library's built-in device scratch instead of a caller workspace), so its output must be BIT-EQUAL to the
existing entry point's on the same inputs -- on a first call, and on a second call with a smaller batch
that finds the first call's partials still lying in the scratch.  Both entry points are called through
the raw C ABI (ctypes), the allocating one with a workspace this test owns.
"""
import ctypes

import pytest
import torch

from oracle import paged_attention as oa

pytestmark = pytest.mark.gpu

SCRATCH_BYTES = 16 * 1024 * 1024  # MI_NOALLOC_SCRATCH_BYTES of include/mi355_decode.h


def _args(case, out):
    q3, o3 = case.q.squeeze(1), out.squeeze(1)
    kc, vc = case.k_cache, case.v_cache
    R, Hq, D = q3.shape
    fp8 = kc.element_size() == 1
    head = [q3.data_ptr(), q3.stride(0), q3.stride(1), kc.data_ptr(), vc.data_ptr(), kc.stride(0), kc.stride(1),
            kc.stride(2), case.block_table.data_ptr(), case.block_table.stride(0), case.kv_lens.data_ptr(),
            o3.data_ptr(), o3.stride(0), o3.stride(1)]
    tail = [R, Hq, kc.size(2), D, kc.size(1), case.block_table.size(1) * kc.size(1), 0, float(D) ** -0.5,
            1 if fp8 else 0,
            case.k_scales.data_ptr() if fp8 else None, case.v_scales.data_ptr() if fp8 else None,
            1 if q3.dtype == torch.float16 else 0, None,   # element type, knobs (NULL = defaults)
            torch.cuda.current_stream().cuda_stream]
    return head, tail


def _with_workspace(lib, case):
    out = torch.full_like(case.q, float("nan"))
    head, tail = _args(case, out)
    need = lib.mi_decode_workspace_bytes(*tail[:6], 0, None)
    ws = torch.empty(need, dtype=torch.uint8, device=case.q.device)
    rc = lib.mi_paged_decode_attention(*head, ws.data_ptr(), need, *tail)
    assert rc == 0, lib.mi_last_error()
    torch.cuda.synchronize()
    return out


def _no_alloc(lib, case):
    out = torch.full_like(case.q, float("nan"))
    head, tail = _args(case, out)
    # the device's own free-memory figure sees every allocation of the process (the library's hipMalloc or event
    # pools included), torch's counter only its caching allocator's
    torch.cuda.synchronize()
    before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
    rc = lib.mi_paged_decode_attention_noalloc(*head, *tail)
    assert rc == 0, lib.mi_last_error()
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.cuda.mem_get_info()[0] >= free_before, "device memory was taken during the call"
    return out


def _check_vs_oracle(case, out):
    ref = oa.paged_decode_attention(case.q.cpu().squeeze(1), case.k_cache.cpu(), case.v_cache.cpu(),
                                    case.kv_lens.cpu(), case.block_table.cpu())
    got = out.float().cpu().squeeze(1)
    assert ((got - ref).abs() <= 2e-2 + 2e-2 * ref.abs()).all()


def test_two_calls_in_a_row_second_smaller(mi, dev):
    lib = mi._lib.load()
    syn = mi.synthetic
    # call 1: 24 requests, long enough to be cut over several workgroups each (split partials + merge)
    big = syn.make_decode_case(syn.DecodeConfig("na-big", 24, 32, 8, 128, 300, 6000, chunk=256, seed=41), dev)
    # call 2: 5 requests incl. a zero-length row and lengths at tile / chunk edges; it lands on the scratch
    # the first call left behind
    lens = torch.tensor([700, 0, 257, 16, 4099], dtype=torch.int32)
    small = syn.make_decode_case(syn.DecodeConfig("na-small", 5, 32, 8, 128, 0, 0, chunk=256, seed=42), dev, lens=lens)

    want_big, want_small = _with_workspace(lib, big), _with_workspace(lib, small)
    got_big = _no_alloc(lib, big)
    got_small = _no_alloc(lib, small)
    assert torch.equal(got_big.view(torch.int16), want_big.view(torch.int16)), "first call differs from the workspace entry point"
    assert torch.equal(got_small.view(torch.int16), want_small.view(torch.int16)), "second (smaller) call differs"
    assert (got_small[1] == 0).all(), "a zero-length row must be zeros"
    _check_vs_oracle(small, got_small)
    _check_vs_oracle(big, got_big)


def test_fp8_cache_and_the_python_wrapper(mi, dev):
    """The same through ``ops.paged_decode_attention_noalloc`` over an fp8-e4m3 cache (bit-equal to the op with a
    workspace)."""
    syn = mi.synthetic
    case = syn.make_decode_case(syn.DecodeConfig("na-fp8", 9, 32, 8, 128, 100, 3000, chunk=256, seed=43), dev)
    N, C, H, D = case.k_cache.shape
    kq = torch.empty(N, C, H, D, dtype=torch.uint8, device=dev)
    vq = torch.empty_like(kq)
    ks = torch.empty(N, H, dtype=torch.float32, device=dev)
    vs = torch.empty_like(ks)
    mi.ops.quantize_chunks_fp8(case.k_cache, kq, ks)
    mi.ops.quantize_chunks_fp8(case.v_cache, vq, vs)
    want = mi.ops.paged_decode_attention(case.q, kq, vq, case.kv_lens, case.block_table, k_scales=ks, v_scales=vs)
    out = torch.full_like(case.q, float("nan"))
    got = mi.ops.paged_decode_attention_noalloc(case.q, kq, vq, case.kv_lens, case.block_table, out,
                                                k_scales=ks, v_scales=vs)
    torch.cuda.synchronize()
    assert got is out and torch.equal(got.view(torch.int16), want.view(torch.int16))


def test_sizes_beyond_the_scratch_are_rejected(mi, dev):
    """A problem whose partials do not fit the built-in scratch is refused with a message, nothing is launched."""
    lib = mi._lib.load()
    R, Hq, Hkv, D = 2048, 64, 8, 128
    assert lib.mi_decode_workspace_bytes(R, Hq, Hkv, D, 256, 4096, 0, None) > SCRATCH_BYTES
    one = ctypes.c_void_p(256)
    rc = lib.mi_paged_decode_attention_noalloc(one, Hq * D, D, one, one, 256 * Hkv * D, Hkv * D, D, one, 16, one, one,
                                               Hq * D, D, R, Hq, Hkv, D, 256, 4096, 0, 0.1, 0, None, None, 0, None, None)
    assert rc == -5 and b"16 MiB" in lib.mi_last_error()


def test_refused_while_kernel_timing_is_on(mi, dev):
    """Timed launches draw event pairs from a pool that grows by creating events, so the entry point that must not
    allocate returns an error instead while timing is enabled."""
    lib = mi._lib.load()
    syn = mi.synthetic
    case = syn.make_decode_case(syn.DecodeConfig("na-prof", 4, 32, 8, 128, 100, 400, chunk=256, seed=43), dev)
    out = torch.full_like(case.q, float("nan"))
    head, tail = _args(case, out)
    assert lib.mi_profile_enable(1) == 0
    try:
        rc = lib.mi_paged_decode_attention_noalloc(*head, *tail)
        assert rc < 0 and "timing" in lib.mi_last_error().decode()
    finally:
        assert lib.mi_profile_enable(0) == 0
    torch.cuda.synchronize()
    assert torch.isnan(out.float()).all(), "nothing may have been launched"
    assert lib.mi_paged_decode_attention_noalloc(*head, *tail) == 0, lib.mi_last_error()
    torch.cuda.synchronize()
    _check_vs_oracle(case, out)
