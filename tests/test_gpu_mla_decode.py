"""GPU parity: absorbed multi-latent decode attention over the latent cache (through the C ABI),
against the fp32 checker: 2e-2 abs/rel as for the other bf16 attention paths."""
import pytest
import torch

from oracle import paged_attention as oa

pytestmark = pytest.mark.gpu

DK, DV = 576, 512


def _case(mi, dev, lens, Hq, chunk, seed, pool_extra=3):
    g = torch.Generator().manual_seed(seed)
    lens = torch.tensor(lens, dtype=torch.int32)
    bt, N = mi.synthetic.build_block_table(lens, chunk, g)
    cache = (torch.randn(N + pool_extra, chunk, DK, generator=g) * 0.5).bfloat16()
    q = torch.randn(lens.numel(), 1, Hq, DK, generator=g).bfloat16()
    return q, cache, lens, bt


def _check(mi, dev, q, cache, lens, bt, scale):
    out = mi.ops.paged_mla_decode_attention(q.to(dev), cache.to(dev), lens.to(dev), bt.to(dev), softmax_scale=scale)
    torch.cuda.synchronize()
    ref = oa.mla_decode_attention(q.squeeze(1), cache, lens, bt, scale, DV)
    got = out.float().cpu().squeeze(1)
    assert got.shape == ref.shape and torch.isfinite(got).all()
    err = (got - ref).abs()
    assert (err <= 2e-2 + 2e-2 * ref.abs()).all(), f"max err {err.max().item():.4e}"
    return out


@pytest.fixture(params=[0, -1, 2], ids=["lds_tile", "streaming", "lds_tile_eight_wavefronts"])
def kernel_choice(request, mi):
    """The decode kernels: latent tiles shared through LDS (chunk sizes that are multiples of 64, or of 32 at
    multiples of 128 heads, where the default is the four-wavefront kernel with 32 heads per wavefront and 2 asks
    for the eight-wavefront one; other sizes stream either way) and one streaming wavefront per head group."""
    mi.ops.set_tuning("mla_decode_lds", request.param)  # 0 = default (an LDS-tile kernel), -1 = never
    yield request.param
    mi.ops.set_tuning("mla_decode_lds", 0)


@pytest.mark.parametrize("Hq", [1, 8, 16, 32, 48, 128])
@pytest.mark.parametrize("chunk", [16, 64, 256])
def test_mla_decode_matches_checker(mi, dev, Hq, chunk, kernel_choice):
    if chunk == 16 and kernel_choice == -1:
        pytest.skip("chunk 16 always streams")
    lens = [0, 1, 15, 16, 17, chunk - 1, chunk, chunk + 1, 3 * chunk + 5, 700, 0, 2049]
    q, cache, lens, bt = _case(mi, dev, lens, Hq, chunk, seed=Hq + chunk)
    out = _check(mi, dev, q, cache, lens, bt, scale=(128 + 64) ** -0.5)
    assert (out.cpu()[lens == 0] == 0).all()


@pytest.mark.parametrize("Hq", [16, 64, 128])
def test_mla_decode_long_contexts_and_splits(mi, dev, Hq, kernel_choice):
    """Enough tokens that every request is cut over many workgroups and merged."""
    q, cache, lens, bt = _case(mi, dev, [20000, 4097, 12345, 1], Hq, 64, seed=9)
    _check(mi, dev, q, cache, lens, bt, scale=0.07)
    for grid in (3, 37):
        mi.ops.set_tuning("decode_grid", grid)
        try:
            _check(mi, dev, q, cache, lens, bt, scale=0.07)
        finally:
            mi.ops.set_tuning("decode_grid", 0)


@pytest.mark.parametrize("Hq", [128, 256])
@pytest.mark.parametrize("chunk", [32, 96, 256])
def test_mla_decode_128_heads_per_workgroup(mi, dev, Hq, chunk):
    """The four-wavefront kernel (multiples of 128 heads, chunk sizes that are multiples of 32): tile edges, empty
    requests, requests cut over workgroups, forced grids."""
    lens = [0, 1, 15, 16, 17, 31, 32, 33, 63, 64, 65, chunk - 1, chunk, chunk + 1, 3 * chunk + 5, 700, 0, 2049]
    q, cache, lens, bt = _case(mi, dev, lens, Hq, chunk, seed=Hq + chunk)
    out = _check(mi, dev, q, cache, lens, bt, scale=(128 + 64) ** -0.5)
    assert (out.cpu()[lens == 0] == 0).all()
    for grid in (1, 5, 64):
        with mi.ops.tuning(decode_grid=grid):
            _check(mi, dev, q, cache, lens, bt, scale=(128 + 64) ** -0.5)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("choice", [0, 2])
def test_mla_decode_128_heads_scores_that_keep_growing(mi, dev, dtype, choice):
    """Keys whose scores grow along the sequence by far more than a factor 2^30: the four-wavefront kernel leaves its
    fast loop (exponentials against the first tile's maxima) for the one that follows every maximum, in the middle
    of a segment, whole requests and cut ones alike."""
    lens = [900, 333, 64, 2500, 33]
    q, cache, lens, bt = _case(mi, dev, lens, 128, 64, seed=11)
    cache = cache.float()
    for r in range(lens.numel()):
        pos = torch.arange(int(lens[r]))
        # (only the 64 values past the value part of a row grow: the outputs keep their size and the tolerance its meaning)
        cache[bt[r, pos // 64].long(), pos % 64, DV:] *= (1.0 + 0.05 * pos)[:, None]
    q, cache = q.to(dtype), cache.to(dtype)
    for grid in (0, 7):
        with mi.ops.tuning(mla_decode_lds=choice, decode_grid=grid):
            _check(mi, dev, q, cache, lens, bt, scale=0.07)


def test_mla_decode_many_requests_fall_back_to_streaming(mi, dev):
    """More requests than the LDS-tile kernel has room for next to its tiles: the call still succeeds."""
    g = torch.Generator().manual_seed(12)
    lens = torch.randint(0, 200, (1000,), generator=g).tolist()
    q, cache, lens, bt = _case(mi, dev, lens, 16, 64, seed=13)
    _check(mi, dev, q, cache, lens, bt, scale=0.07)


def test_mla_decode_more_requests_than_one_launch_takes(mi, dev):
    """Beyond 7 680 requests (8 bytes of LDS each) the call runs in slices."""
    g = torch.Generator().manual_seed(21)
    lens = torch.randint(0, 40, (7680 + 500,), generator=g).tolist()
    q, cache, lens, bt = _case(mi, dev, lens, 8, 16, seed=22)
    _check(mi, dev, q, cache, lens, bt, scale=0.07)


@pytest.mark.parametrize("Hq", [32, 128])
def test_mla_decode_chunk_permutation_and_cache_view(mi, dev, Hq):
    """Moving the rows to other physical chunks changes nothing; a [N, C, 1, 576] cache view is accepted; so is a
    cache that is a slice of a wider buffer (a token stride beyond 576 values)."""
    q, cache, lens, bt = _case(mi, dev, [100, 333, 64], Hq, 64, seed=4)
    a = mi.ops.paged_mla_decode_attention(q.to(dev), cache.to(dev), lens.to(dev), bt.to(dev), softmax_scale=0.1)
    wide = torch.zeros(cache.size(0), cache.size(1), 640, dtype=cache.dtype)
    wide[..., :DK] = cache
    c = mi.ops.paged_mla_decode_attention(q.to(dev), wide.to(dev)[..., :DK], lens.to(dev), bt.to(dev), softmax_scale=0.1)
    assert torch.equal(a, c)
    N = cache.size(0)
    perm = torch.randperm(N, generator=torch.Generator().manual_seed(1))
    moved = torch.empty_like(cache)
    moved[perm] = cache
    bt2 = torch.where(bt >= 0, perm[bt.clamp(min=0).long()].int(), bt)
    b = mi.ops.paged_mla_decode_attention(q.to(dev), moved.unsqueeze(2).to(dev), lens.to(dev), bt2.to(dev),
                                          softmax_scale=0.1)
    torch.cuda.synchronize()
    assert torch.equal(a, b)


def test_mla_decode_argument_errors(mi, dev):
    q, cache, lens, bt = _case(mi, dev, [10, 20], 24, 16, seed=2)
    with pytest.raises(mi._lib.KernelError, match="multiple of 16"):
        mi.ops.paged_mla_decode_attention(q.to(dev), cache.to(dev), lens.to(dev), bt.to(dev), softmax_scale=0.1)
    q, cache, lens, bt = _case(mi, dev, [10, 20], 16, 16, seed=2)
    with pytest.raises(ValueError, match="576"):
        mi.ops.paged_mla_decode_attention(q.to(dev)[..., :512].contiguous(), cache.to(dev), lens.to(dev), bt.to(dev),
                                          softmax_scale=0.1)
    with pytest.raises(mi._lib.KernelError, match="softmax_scale"):
        mi.ops.paged_mla_decode_attention(q.to(dev), cache.to(dev), lens.to(dev), bt.to(dev), softmax_scale=0.0)
