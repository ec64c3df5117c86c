"""Pins for the CPU checker of the rotary table, RoPE application and head norms."""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import rope_norm as orn


def test_table_closed_form_and_layout():
    tab = orn.rotary_table(50, 8, base=10000.0)
    assert tab.shape == (50, 1, 1, 8) and tab.dtype == torch.float32
    for pos in (0, 1, 7, 49):
        for i in range(4):
            theta = pos / (10000.0 ** (2 * i / 8))
            assert abs(tab[pos, 0, 0, i].item() - theta) < 1e-4 * max(1.0, theta)
            assert tab[pos, 0, 0, i + 4].item() == tab[pos, 0, 0, i].item()  # cat(freqs, freqs)
    inter = orn.rotary_table(5, 8, interleaved=True)
    assert torch.equal(inter[3, 0, 0, 0::2], inter[3, 0, 0, 1::2])
    assert torch.equal(inter[3, 0, 0, 0::2], tab[3, 0, 0, :4])


def test_position_zero_is_identity():
    x = torch.randn(3, 2, 16).bfloat16()
    tab = orn.rotary_table(4, 16)
    y = orn.norm_rope(x, torch.zeros(3, dtype=torch.long), tab)
    assert torch.equal(x, y)


@pytest.mark.parametrize("interleaved", [False, True])
def test_rotation_equals_complex_multiplication(interleaved):
    """(x_a + i x_b) * e^{i theta} with a/b = (i, i+d/2) or (2i, 2i+1)."""
    d = 16
    x = torch.randn(5, 3, d, dtype=torch.float64)
    tab = orn.rotary_table(100, d, base=500000.0, interleaved=interleaved).double()
    pos = torch.tensor([0, 3, 17, 64, 99])
    ang = tab.reshape(100, d)[pos]
    got = orn.apply_rope(x, ang.float().double(), interleaved)
    for t in range(5):
        for h in range(3):
            for i in range(d // 2):
                a, b = (2 * i, 2 * i + 1) if interleaved else (i, i + d // 2)
                th = float(ang[t, a])
                z = complex(x[t, h, a], x[t, h, b]) * complex(math.cos(th), math.sin(th))
                assert abs(got[t, h, a].item() - z.real) < 1e-9 and abs(got[t, h, b].item() - z.imag) < 1e-9
    # norm of every rotated pair is preserved
    assert torch.allclose(got.pow(2).sum(-1), x.pow(2).sum(-1), atol=1e-9)


def test_partial_rotary_passes_tail_through():
    x = torch.randn(4, 2, 16)
    tab = orn.rotary_table(10, 8)
    y = orn.norm_rope(x, torch.tensor([1, 2, 3, 4]), tab)
    assert torch.equal(y[..., 8:], x[..., 8:]) and not torch.equal(y[..., :8], x[..., :8])


def test_bf16_chain_rounds_cos_sin_before_multiplying():
    """The reference casts cos/sin to the tensor dtype first: check one element by hand."""
    x = torch.tensor([[[1.0, 2.0, 3.0, 4.0]]]).bfloat16()
    ang = torch.tensor([[0.3, 1.1, 0.3, 1.1]])
    y = orn.apply_rope(x, ang)
    c = torch.cos(torch.tensor(0.3)).bfloat16()
    s = torch.sin(torch.tensor(0.3)).bfloat16()
    expect0 = (x[0, 0, 0] * c) + ((-x[0, 0, 2]) * s)  # bf16 ops, each rounded
    assert y[0, 0, 0].item() == expect0.item()
    exact = 1.0 * math.cos(0.3) - 3.0 * math.sin(0.3)
    assert abs(y[0, 0, 0].item() - exact) < 2e-2


def test_llama3_frequency_scaling_three_bands():
    dim, base, factor = 128, 500000.0, 8.0
    f = 1.0 / (base ** (torch.arange(0, dim, 2, dtype=torch.float64) / dim))
    got = orn.inv_freq(dim, base, rope_scaling=True, factor=factor).double()
    wavelen = 2 * math.pi / f
    seen = set()
    for i in range(dim // 2):
        w = wavelen[i].item()
        if w < 8192 / 4:
            exp, band = f[i].item(), "high"
        elif w > 8192:
            exp, band = f[i].item() / factor, "low"
        else:
            smooth = (8192 / w - 1.0) / (4.0 - 1.0)
            exp, band = (1 - smooth) * f[i].item() / factor + smooth * f[i].item(), "mid"
        seen.add(band)
        assert abs(got[i].item() - exp) <= 1e-6 * exp
    assert seen == {"high", "mid", "low"}


def test_rms_norm_equals_library_routine_and_fp64():
    x = torch.randn(64, 4, 128).bfloat16()
    w = (1 + 0.02 * torch.randn(128)).bfloat16()
    assert torch.equal(orn.rms_norm(x, w, 1e-5), F.rms_norm(x, (128,), w, 1e-5))
    xd = x.double()
    ref = xd / torch.sqrt(xd.pow(2).mean(-1, keepdim=True) + 1e-5) * w.double()
    assert (orn.rms_norm(x, w, 1e-5).double() - ref).abs().max() < 2e-2
    l2 = orn.l2_norm(x, 1e-6).double()
    assert torch.allclose(l2.pow(2).mean(-1), torch.ones(64, 4, dtype=torch.float64), atol=2e-2)


def test_split_mixed_qkv_offsets():
    """Hand-computed column offsets: Hq=4, Hkv=2, d=2 -> per group [q q k v] of width 2 each, so a
    row 0..15 splits into q = [0 1 | 2 3 | 8 9 | 10 11], k = [4 5 | 12 13], v = [6 7 | 14 15]."""
    row = torch.arange(16.0).view(1, 1, 16)
    q, k, v = orn.split_mixed_qkv(row, 4, 2)
    assert q.flatten().tolist() == [0, 1, 2, 3, 8, 9, 10, 11]
    assert k.flatten().tolist() == [4, 5, 12, 13]
    assert v.flatten().tolist() == [6, 7, 14, 15]


def test_split_mixed_qkv_scalar_loop():
    t, hq, hkv, d = 3, 6, 2, 4
    g = hq // hkv
    x = torch.randn(t, 1, (hq + 2 * hkv) * d)
    q, k, v = orn.split_mixed_qkv(x, hq, hkv)
    assert q.shape == (t, 1, hq, d) and k.shape == (t, 1, hkv, d) and v.shape == (t, 1, hkv, d)
    for ti in range(t):
        for grp in range(hkv):
            base = grp * (g + 2) * d
            for j in range(g):
                assert torch.equal(q[ti, 0, grp * g + j], x[ti, 0, base + j * d: base + (j + 1) * d])
            assert torch.equal(k[ti, 0, grp], x[ti, 0, base + g * d: base + (g + 1) * d])
            assert torch.equal(v[ti, 0, grp], x[ti, 0, base + (g + 1) * d: base + (g + 2) * d])
