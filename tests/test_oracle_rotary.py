"""Pins oracle/rotary.py (CPU): the rotation restated from
diffulex/layer/rotary_embedding.py:7-17,29-37 against independent evaluations, so that a wrong
sign, swapped halves or a wrong table column fails."""
import numpy as np
import pytest
import torch

from oracle import rotary

HD, MAXPOS, BASE = 128, 4096, 1.0e6


def _data(T=9, H=3, hd=HD, seed=0):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, H * hd, generator=g).to(torch.bfloat16)
    pos = torch.randint(0, MAXPOS, (T,), generator=g)
    return x, pos


def test_table_matches_closed_form_in_float64():
    tab = rotary.cos_sin_cache(HD, MAXPOS, BASE).double().numpy()
    i = np.arange(0, HD, 2, dtype=np.float64)
    ang = np.arange(MAXPOS, dtype=np.float64)[:, None] * BASE ** (-i / HD)[None, :]
    # fp32 angles: error grows with the position (4095 * 2^-24 relative to the largest angle)
    assert np.abs(tab[:, :HD // 2] - np.cos(ang)).max() < 1e-3
    assert np.abs(tab[:, HD // 2:] - np.sin(ang)).max() < 1e-3
    assert tab.shape == (MAXPOS, HD)
    assert np.all(tab[0, :HD // 2] == 1.0) and np.all(tab[0, HD // 2:] == 0.0)


def test_equals_complex_multiplication():
    """(x1 + i x2) * (cos + i sin) in float64, to bf16 rounding of the result."""
    x, pos = _data()
    tab = rotary.cos_sin_cache(HD, MAXPOS, BASE)
    y = rotary.apply_rotary(x, pos, tab, HD).double().view(x.shape[0], -1, HD)
    xd = x.double().view(x.shape[0], -1, HD)
    z = torch.complex(xd[..., :HD // 2], xd[..., HD // 2:])
    cs = tab[pos].double()
    w = torch.complex(cs[:, None, :HD // 2], cs[:, None, HD // 2:])
    want = z * w
    got = torch.complex(y[..., :HD // 2], y[..., HD // 2:])
    err = (got - want).abs()
    assert (err <= 2.0 ** -8 * want.abs().clamp_min(1e-3) * 1.5 + 1e-6).all()


def test_position_zero_is_the_identity_bit_for_bit():
    x, _ = _data()
    tab = rotary.cos_sin_cache(HD, MAXPOS, BASE)
    y = rotary.apply_rotary(x, torch.zeros(x.shape[0], dtype=torch.long), tab, HD)
    assert torch.equal(y.view(torch.int16), x.view(torch.int16))


def test_pair_norms_are_preserved():
    x, pos = _data(seed=3)
    tab = rotary.cos_sin_cache(HD, MAXPOS, BASE)
    y = rotary.apply_rotary(x, pos, tab, HD).double().view(x.shape[0], -1, HD)
    xd = x.double().view(x.shape[0], -1, HD)
    n0 = xd[..., :HD // 2] ** 2 + xd[..., HD // 2:] ** 2
    n1 = y[..., :HD // 2] ** 2 + y[..., HD // 2:] ** 2
    assert ((n1 - n0).abs() <= 0.02 * n0 + 1e-6).all()


def test_rotations_add_up():
    """Rotating by p then by q lands (to rounding) where rotating by p + q does."""
    g = torch.Generator().manual_seed(5)
    x = torch.randn(6, 2 * HD, generator=g).to(torch.bfloat16)
    p = torch.randint(0, MAXPOS // 2, (6,), generator=g)
    q = torch.randint(0, MAXPOS // 2, (6,), generator=g)
    tab = rotary.cos_sin_cache(HD, MAXPOS, BASE)
    twice = rotary.apply_rotary(rotary.apply_rotary(x, p, tab, HD), q, tab, HD).float()
    once = rotary.apply_rotary(x, p + q, tab, HD).float()
    assert (twice - once).abs().max() < 0.06


def test_scalar_loop_bit_exact():
    """Element by element with every intermediate rounded to fp32, then bf16."""
    x, pos = _data(T=3, H=2, hd=16, seed=7)
    tab = rotary.cos_sin_cache(16, 64, 10000.0)
    pos = pos % 64
    y = rotary.apply_rotary(x, pos, tab, 16)
    xf = x.float().numpy().reshape(3, 2, 16)
    want = np.zeros_like(xf)
    for t in range(3):
        for h in range(2):
            for i in range(8):
                c, s = np.float32(tab[pos[t], i]), np.float32(tab[pos[t], 8 + i])
                x1, x2 = np.float32(xf[t, h, i]), np.float32(xf[t, h, 8 + i])
                want[t, h, i] = np.float32(np.float32(x1 * c) - np.float32(x2 * s))
                want[t, h, 8 + i] = np.float32(np.float32(x2 * c) + np.float32(x1 * s))
    want = torch.from_numpy(want).to(torch.bfloat16).reshape(3, 32)
    assert torch.equal(y.view(torch.int16), want.view(torch.int16))


@pytest.mark.parametrize("hd,H", [(128, 4), (64, 5)])
def test_matches_torch_tensor_ops_bit_exact(hd, H):
    """The same formula written with torch's tensor operations (each one rounding on its own)."""
    x, pos = _data(T=33, H=H, hd=hd, seed=11)
    tab = rotary.cos_sin_cache(hd, MAXPOS, BASE)
    y = rotary.apply_rotary(x, pos, tab, hd)
    cos, sin = tab[pos].chunk(2, dim=-1)
    cos, sin = cos.unsqueeze(-2), sin.unsqueeze(-2)
    x1, x2 = torch.chunk(x.view(33, H, hd).to(torch.float32), 2, dim=-1)
    want = torch.cat((x1 * cos - x2 * sin, x2 * cos + x1 * sin), dim=-1).to(torch.bfloat16).view(33, H * hd)
    assert torch.equal(y.view(torch.int16), want.view(torch.int16))
    y3 = rotary.apply_rotary(x.view(33, H, hd), pos, tab, hd)
    assert y3.shape == (33, H, hd) and torch.equal(y3.reshape(33, -1).view(torch.int16), y.view(torch.int16))
