"""Pins oracle/fp8_e4m3.py against the library cast torch.float8_e4m3fn, exhaustively."""
import numpy as np
import torch

from oracle import fp8_e4m3


def _all_bf16_as_f32():
    bits = (np.arange(65536, dtype=np.uint32) << 16)
    return bits.view(np.float32)


def test_decode_all_codes_matches_library():
    codes = np.arange(256, dtype=np.uint8)
    want = torch.from_numpy(codes).view(torch.float8_e4m3fn).to(torch.float32).numpy()
    got = fp8_e4m3.decode_e4m3fn(codes)
    assert np.array_equal(np.isnan(want), np.isnan(got))
    ok = ~np.isnan(want)
    assert np.array_equal(want[ok].view(np.uint32), got[ok].view(np.uint32))


def test_encode_all_bf16_matches_library():
    x = _all_bf16_as_f32()
    want = torch.from_numpy(x.copy()).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    got = fp8_e4m3.encode_e4m3fn(x)
    nan = np.isnan(x)
    # NaN: any NaN code is acceptable as long as both are NaN codes
    assert np.all((got[nan] & 0x7F) == 0x7F) and np.all((want[nan] & 0x7F) == 0x7F)
    assert np.array_equal(want[~nan], got[~nan])


def test_encode_random_fp32_and_ties_match_library():
    rng = np.random.default_rng(0)
    x = np.concatenate([
        rng.standard_normal(200000).astype(np.float32) * 100,
        rng.standard_normal(200000).astype(np.float32) * 0.01,
        # exact ties between neighbouring codes, in the normal and the subnormal range
        np.array([(a + b) / 2 for a, b in zip(fp8_e4m3.decode_e4m3fn(np.arange(0, 126, dtype=np.uint8)),
                                               fp8_e4m3.decode_e4m3fn(np.arange(1, 127, dtype=np.uint8)))],
                 dtype=np.float32),
    ])
    x = np.concatenate([x, -x])
    want = torch.from_numpy(x.copy()).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(want, fp8_e4m3.encode_e4m3fn(x))


def test_quantize_per_head_is_divide_clamp_cast():
    x = _all_bf16_as_f32()
    x = x[np.isfinite(x)].reshape(-1, 1, 1)
    for scale in (1.0, 0.0123, 3.7, 2.0 ** -20, 11.0):
        s = np.array([scale], dtype=np.float32)
        got = fp8_e4m3.quantize_per_head(x, s)
        y = (torch.from_numpy(x.copy()) / torch.tensor(scale, dtype=torch.float32)).clamp(-448, 448)
        want = y.to(torch.float8_e4m3fn).view(torch.uint8).numpy()
        assert np.array_equal(got, want)
        assert not np.any((got & 0x7F) == 0x7F)  # finite input never produces the NaN code


def test_round_trip_is_identity_on_codes():
    codes = np.arange(256, dtype=np.uint8)
    vals = fp8_e4m3.decode_e4m3fn(codes)
    ok = ~np.isnan(vals)
    back = fp8_e4m3.encode_e4m3fn(vals[ok])
    assert np.array_equal(back & 0x7F, codes[ok] & 0x7F)
    nz = (codes[ok] & 0x7F) != 0
    assert np.array_equal(back[nz], codes[ok][nz])


def test_dequant_to_bf16_is_exact():
    codes = np.arange(256, dtype=np.uint8)
    vals = torch.from_numpy(fp8_e4m3.decode_e4m3fn(codes))
    ok = ~torch.isnan(vals)
    assert torch.equal(vals[ok].to(torch.bfloat16).to(torch.float32), vals[ok])
