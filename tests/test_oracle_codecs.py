"""Pins the oracle's scalar codecs against library routines (numpy float16,
torch bfloat16 / float8) and the formats' closed forms."""
import numpy as np
import pytest
import torch


def _interesting_f32(rng, n=20000, lim=None):
    x = np.concatenate([
        rng.standard_normal(n).astype(np.float32),
        (rng.standard_normal(n) * 100).astype(np.float32),
        (rng.standard_normal(n) * 1e-3).astype(np.float32),
        (rng.standard_normal(n) * 1e-6).astype(np.float32),
        np.array([0.0, -0.0, 1.0, -1.0, 65504.0, 65519.0, 65520.0, 1e-8, 6e-8,
                  5.96e-8, 2.98e-8, 2.9802322e-8, 448.0, 449.0, 464.0, 465.0,
                  0.0009765625, 0.001953125, 0.0146484375], np.float32)])
    if lim is not None:
        x = x[np.abs(x) <= lim]
    return x


def test_f16_matches_numpy(oracle):
    rng = np.random.default_rng(1)
    x = _interesting_f32(rng)
    got = oracle.narrow(x, oracle.F16)
    want = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(got, want)
    # every f16 code widens exactly
    codes = np.arange(65536, dtype=np.uint16)
    w = oracle.widen(codes, oracle.F16)
    ref = codes.view(np.float16).astype(np.float32)
    assert np.array_equal(np.isnan(w), np.isnan(ref))
    ok = ~np.isnan(ref)
    assert np.array_equal(w[ok], ref[ok])


def test_f16_overflow_and_inf(oracle):
    x = np.array([np.inf, -np.inf, 1e6, -1e6, np.nan], np.float32)
    got = oracle.narrow(x, oracle.F16).view(np.float16)
    assert got[0] == np.inf and got[1] == -np.inf
    assert got[2] == np.inf and got[3] == -np.inf and np.isnan(got[4])


def test_bf16_matches_torch(oracle):
    rng = np.random.default_rng(2)
    x = _interesting_f32(rng)
    got = oracle.narrow(x, oracle.BF16)
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got, want)
    back = oracle.widen(got, oracle.BF16)
    assert np.array_equal(back, torch.from_numpy(x).to(torch.bfloat16).float().numpy())


def test_e4m3fn_all_codes_widen(oracle):
    codes = np.arange(256, dtype=np.uint8)
    w = oracle.widen(codes, oracle.FP8)
    ref = torch.from_numpy(codes).view(torch.float8_e4m3fn).float().numpy()
    assert np.array_equal(np.isnan(w), np.isnan(ref))
    ok = ~np.isnan(ref)
    assert np.array_equal(w[ok], ref[ok])
    # OCP format facts: max finite 448, NaN only at 0x7f / 0xff, no inf
    assert w[0x7e] == 448.0 and w[0xfe] == -448.0
    assert np.isnan(w[0x7f]) and np.isnan(w[0xff])
    assert not np.isinf(w).any()
    assert w[0x01] == 2.0 ** -9  # smallest subnormal


def test_e4m3fn_narrow_in_range_matches_torch(oracle):
    rng = np.random.default_rng(3)
    x = _interesting_f32(rng, lim=448.0)
    x = np.concatenate([x, np.linspace(-448, 448, 100001, dtype=np.float32)])
    got = oracle.narrow(x, oracle.FP8)
    want = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(got, want)


def test_e4m3fn_saturates(oracle):
    # the GPU path clamps (Pipelines.cpp:238): overflow -> +-448, not NaN
    x = np.array([449.0, 464.0, 465.0, 1e9, np.inf, -1e9, -np.inf], np.float32)
    got = oracle.widen(oracle.narrow(x, oracle.FP8), oracle.FP8)
    assert np.array_equal(got, np.array([448, 448, 448, 448, 448, -448, -448], np.float32))
    assert np.isnan(oracle.widen(oracle.narrow(np.array([np.nan], np.float32), oracle.FP8), oracle.FP8))[0]
    # the reference's host-side truncation does not saturate: overflow -> NaN
    lib = oracle.lib()
    assert lib.orc_f32_to_e4m3fn_nosat(1e9) == 0x7f
    assert lib.orc_f32_to_e4m3fn_nosat(-1e9) == 0xff
    # 464 is the rounding boundary between 448 and the (non-existent) 480
    assert lib.orc_f32_to_e4m3fn_nosat(463.9) == 0x7e


def test_e5m2_matches_torch(oracle):
    codes = np.arange(256, dtype=np.uint8)
    w = oracle.widen(codes, oracle.BF8)
    ref = torch.from_numpy(codes).view(torch.float8_e5m2).float().numpy()
    assert np.array_equal(np.isnan(w), np.isnan(ref))
    ok = ~np.isnan(ref)
    assert np.array_equal(w[ok], ref[ok])
    rng = np.random.default_rng(4)
    x = _interesting_f32(rng, lim=57344.0)
    got = oracle.narrow(x, oracle.BF8)
    want = torch.from_numpy(x).to(torch.float8_e5m2).view(torch.uint8).numpy()
    assert np.array_equal(got, want)
    sat = oracle.widen(oracle.narrow(np.array([1e9, -np.inf], np.float32), oracle.BF8), oracle.BF8)
    assert np.array_equal(sat, np.array([57344.0, -57344.0], np.float32))


def test_int_cast_round_half_even_and_saturate(oracle):
    x = np.array([0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 126.5, 127.5, 300.0, -128.5, -129.0, -1000.0],
                 np.float32)
    got = oracle.narrow(x, oracle.I8)
    assert got.tolist() == [0, 2, 2, 0, -2, -2, 126, 127, 127, -128, -128, -128]


def test_round_through(oracle):
    x = np.array([0.1, 1.0 / 3.0, 1000.123], np.float32)
    assert np.array_equal(oracle.round_through(x, oracle.F16),
                          x.astype(np.float16).astype(np.float32))
    assert np.array_equal(oracle.round_through(x, oracle.F32), x)
