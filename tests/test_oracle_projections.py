"""The projection checker (oracle/projections.py) against a library routine, closed forms and a hand-laid-out split."""
import torch

from oracle import projections as op


def test_linear_equals_the_library_routine_in_float64():
    gen = torch.Generator().manual_seed(3)
    x = torch.randn(7, 96, generator=gen).bfloat16()
    w = torch.randn(48, 96, generator=gen).bfloat16()
    b = torch.randn(48, generator=gen).bfloat16()
    want = torch.nn.functional.linear(x.double(), w.double(), b.double())
    got, rest = op.linear(x, w, b)
    assert rest is None and got.dtype == torch.bfloat16
    # one rounding to bf16 of an fp32 sum of 96 products: within half a bf16 ulp of the float64 value, plus fp32 noise
    assert ((got.double() - want).abs() <= 2.0 ** -8 * want.abs() + 1e-4).all()
    got2, rest2 = op.linear(x, w, b, skip_bias_add=True)
    assert rest2 is b
    want2 = torch.nn.functional.linear(x.double(), w.double())
    assert ((got2.double() - want2).abs() <= 2.0 ** -8 * want2.abs() + 1e-4).all()


def test_linear_closed_forms():
    x = torch.arange(12, dtype=torch.float32).reshape(3, 4).bfloat16()
    eye = torch.eye(4).bfloat16()
    assert torch.equal(op.linear(x, eye)[0], x)
    w = torch.tensor([[1.0, 2.0, 0.0, -1.0], [0.5, 0.0, 0.0, 4.0]]).bfloat16()
    b = torch.tensor([10.0, -3.0]).bfloat16()
    got = op.linear(x, w, b)[0].float()
    for t in range(3):
        for n in range(2):
            assert got[t, n].item() == sum(float(x[t, k]) * float(w[n, k]) for k in range(4)) + float(b[n])


def test_qkv_split_layout():
    # entry = 1000 * group + 100 * role (0.. G-1 query heads, G key, G + 1 value) + element
    T, Hq, Hkv, d = 2, 6, 2, 4
    G = Hq // Hkv
    row = torch.tensor([1000 * g + 100 * role + e for g in range(Hkv) for role in range(G + 2) for e in range(d)],
                       dtype=torch.float32)
    mixed = torch.stack([row, row + 0.5])
    q, k, v = op.qkv_split(mixed, Hq, Hkv, d)
    assert q.shape == (T, Hq, d) and k.shape == (T, Hkv, d) and v.shape == (T, Hkv, d)
    for g in range(Hkv):
        for u in range(G):
            assert q[0, g * G + u].tolist() == [1000 * g + 100 * u + e for e in range(d)]
        assert k[0, g].tolist() == [1000 * g + 100 * G + e for e in range(d)]
        assert v[1, g].tolist() == [1000 * g + 100 * (G + 1) + e + 0.5 for e in range(d)]
