"""The oracle's 16-bit / 8-bit float codecs against torch's own casts (library
routines), exhaustively where the domain is small."""
import ctypes

import numpy as np
import torch


def _vec(fn, xs, out_dtype):
    return np.array([fn(x) for x in xs], dtype=out_dtype)


def test_f16_decode_all_codes(oracle):
    L = oracle.lib()
    codes = np.arange(65536, dtype=np.uint16)
    want = torch.from_numpy(codes.view(np.int16)).view(torch.float16).float().numpy()
    got = _vec(lambda c: L.oracle_f16_to_f32(int(c)), codes, np.float32)
    assert np.array_equal(got.view(np.uint32)[~np.isnan(want)], want.view(np.uint32)[~np.isnan(want)])
    assert np.isnan(got[np.isnan(want)]).all()


def test_bf16_decode_all_codes(oracle):
    L = oracle.lib()
    codes = np.arange(65536, dtype=np.uint16)
    want = torch.from_numpy(codes.view(np.int16)).view(torch.bfloat16).float().numpy()
    got = _vec(lambda c: L.oracle_bf16_to_f32(int(c)), codes, np.float32)
    ok = ~np.isnan(want)
    assert np.array_equal(got.view(np.uint32)[ok], want.view(np.uint32)[ok])


def test_e5m2_decode_all_256_codes(oracle):
    """E5M2 -> fp16 is exact and equals the byte placed in the top half of a binary16."""
    L = oracle.lib()
    codes = torch.arange(256, dtype=torch.int32).to(torch.uint8)
    want = codes.view(torch.float8_e5m2).to(torch.float16)
    shifted = (codes.to(torch.int32) << 8).to(torch.int16).view(torch.float16)
    ok = ~torch.isnan(want)
    assert torch.equal(want[ok], shifted[ok])
    got = _vec(lambda c: L.oracle_e5m2_to_f32(int(c)), codes.numpy(), np.float32)
    w = want.float().numpy()
    assert np.array_equal(got[ok.numpy()], w[ok.numpy()])
    assert np.isnan(got[~ok.numpy()]).all()


def test_e4m3_decode_all_256_codes(oracle):
    """E4M3 "fn" decode against torch.float8_e4m3fn, NaN codes included."""
    L = oracle.lib()
    codes = torch.arange(256, dtype=torch.int32).to(torch.uint8)
    want = codes.view(torch.float8_e4m3fn).float().numpy()
    got = _vec(lambda c: L.oracle_e4m3_to_f32(int(c)), codes.numpy(), np.float32)
    ok = ~np.isnan(want)
    assert np.array_equal(got.view(np.uint32)[ok], want.view(np.uint32)[ok])
    assert np.isnan(got[~ok]).all() and (~ok).sum() == 2


def _encode_cases():
    rng = np.random.default_rng(0)
    xs = [rng.standard_normal(20000).astype(np.float32),
          (rng.standard_normal(20000) * 1e-6).astype(np.float32),
          (rng.standard_normal(5000) * 3e4).astype(np.float32)]
    # every fp16 value, its neighbours' midpoints (ties) and one ulp either side of them
    h = torch.arange(0, 0x7C00, dtype=torch.int32).to(torch.int16).view(torch.float16).float().numpy()
    mid = ((h[:-1].astype(np.float64) + h[1:].astype(np.float64)) / 2).astype(np.float32)
    xs += [h, mid, np.nextafter(mid, np.float32(np.inf)), np.nextafter(mid, np.float32(-np.inf))]
    xs += [np.array([0.0, -0.0, 65504.0, 65519.99, 65520.0, 65536.0, 1e10, np.inf, -np.inf,
                     2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0000001, 2.0 ** -26, 6.1e-5],
                    dtype=np.float32)]
    x = np.concatenate(xs)
    return np.concatenate([x, -x])


def test_f32_to_f16_round_to_nearest_even(oracle):
    L = oracle.lib()
    x = _encode_cases()
    want = torch.from_numpy(x).to(torch.float16).view(torch.int16).numpy().view(np.uint16)
    got = _vec(lambda v: L.oracle_f32_to_f16(ctypes.c_float(float(v))), x, np.uint16)
    assert np.array_equal(got, want)


def test_f32_to_bf16_round_to_nearest_even(oracle):
    L = oracle.lib()
    rng = np.random.default_rng(1)
    x = np.concatenate([rng.standard_normal(30000).astype(np.float32),
                        (rng.standard_normal(3000) * 1e30).astype(np.float32),
                        (rng.standard_normal(3000) * 1e-30).astype(np.float32)])
    # exact ties: bf16 value plus half an ulp
    b = torch.from_numpy(x[:3000]).to(torch.bfloat16).float().numpy()
    tie = (b.view(np.uint32) | 0x8000).view(np.float32)
    x = np.concatenate([x, tie, np.array([0.0, -0.0, np.inf, -np.inf, 3.3895e38], dtype=np.float32)])
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = _vec(lambda v: L.oracle_f32_to_bf16(ctypes.c_float(float(v))), x, np.uint16)
    assert np.array_equal(got, want)
