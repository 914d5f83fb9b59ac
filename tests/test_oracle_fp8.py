"""Pins the fp8 / bf16 codecs of the oracle: closed forms, exhaustive tables, and
agreement between three independent statements (torch CPU casts, oracle/fp8_codec.c,
numpy closed-form decode)."""
import ctypes

import numpy as np
import pytest
import torch


def _decode_e4m3(c: int) -> float:
    s, e, m = c >> 7, (c >> 3) & 15, c & 7
    if e == 15 and m == 7:
        return float("nan")
    v = m / 8 * 2.0 ** -6 if e == 0 else (1 + m / 8) * 2.0 ** (e - 7)
    return -v if s else v


def _decode_e5m2(c: int) -> float:
    s, e, m = c >> 7, (c >> 2) & 31, c & 3
    if e == 31:
        v = float("inf") if m == 0 else float("nan")
    else:
        v = m / 4 * 2.0 ** -14 if e == 0 else (1 + m / 4) * 2.0 ** (e - 15)
    return -v if s else v


@pytest.mark.parametrize("fmt", ["e4m3", "e5m2"])
def test_decode_all_codes_three_ways(oracle_c, fmt):
    dec_c = oracle_c.ngpt_oracle_e4m3fn_to_f32 if fmt == "e4m3" else oracle_c.ngpt_oracle_e5m2_to_f32
    dec_py = _decode_e4m3 if fmt == "e4m3" else _decode_e5m2
    dt = torch.float8_e4m3fn if fmt == "e4m3" else torch.float8_e5m2
    tv = torch.arange(256, dtype=torch.int32).to(torch.uint8).view(dt).float()
    for c in range(256):
        a, b, t = dec_c(c), dec_py(c), float(tv[c])
        if np.isnan(b):
            assert np.isnan(a) and np.isnan(t)
        else:
            assert a == b == t, (c, a, b, t)
    assert dec_py(0x7e if fmt == "e4m3" else 0x7b) == (448.0 if fmt == "e4m3" else 57344.0)


@pytest.mark.parametrize("fmt", ["e4m3", "e5m2"])
def test_encode_roundtrip_monotone_and_ties(oracle_c, fmt):
    enc = oracle_c.ngpt_oracle_f32_to_e4m3fn if fmt == "e4m3" else oracle_c.ngpt_oracle_f32_to_e5m2
    dec = _decode_e4m3 if fmt == "e4m3" else _decode_e5m2
    top = 0x7e if fmt == "e4m3" else 0x7b
    # every finite code is a fixed point of encode(decode(.)), both signs
    for c in range(top + 1):
        assert enc(dec(c)) == c
        if c:
            assert enc(-dec(c)) == (c | 0x80)
    # midpoints between adjacent codes round to the even code; just off the
    # midpoint rounds to the nearer one
    for c in range(top):
        lo, hi = dec(c), dec(c + 1)
        mid = (lo + hi) / 2
        assert np.float32(mid) == mid
        even = c if c % 2 == 0 else c + 1
        assert enc(mid) == even, (c, mid)
        assert enc(float(np.nextafter(np.float32(mid), np.float32(0)))) == c
        assert enc(float(np.nextafter(np.float32(mid), np.float32(1e9)))) == c + 1
    # overflow rule: the tie above max rounds to the odd side's neighbour
    if fmt == "e4m3":
        assert enc(464.0) == 0x7e                      # tie -> even mantissa (448)
        assert enc(float(np.nextafter(np.float32(464), np.float32(1e9)))) == 0x7f   # NaN, not saturate
        assert enc(1e9) == 0x7f and enc(float("inf")) == 0x7f
        assert enc(2.0 ** -10) == 0 and enc(2.0 ** -9) == 1   # half the smallest subnormal ties to 0
    else:
        assert enc(61440.0) == 0x7c                    # tie -> inf (even)
        assert enc(float(np.nextafter(np.float32(61440), np.float32(0)))) == 0x7b
        assert enc(1e9) == 0x7c and enc(float("inf")) == 0x7c
        assert oracle_c.ngpt_oracle_f32_to_e5m2_sat(1e9) == 0x7b
        assert oracle_c.ngpt_oracle_f32_to_e5m2_sat(-1e9) == 0xfb
        assert enc(2.0 ** -17) == 0 and enc(2.0 ** -16) == 1


def test_exhaustive_bf16_tables(oracle_c, fp8_tables):
    """C encoder == committed torch tables == a fresh torch cast, on all 65536 bf16 patterns."""
    e4, e5 = fp8_tables
    bits = np.arange(65536, dtype=np.uint16)
    out = np.empty(65536, dtype=np.uint8)
    vals = torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16)
    for fmt, table, dt in ((0, e4, torch.float8_e4m3fn), (1, e5, torch.float8_e5m2)):
        oracle_c.ngpt_oracle_quant_bf16(bits.ctypes.data, out.ctypes.data, 65536, ctypes.c_float(1.0), fmt)
        fresh = vals.to(dt).view(torch.uint8).numpy()
        nan_t = np.isnan(vals.float().numpy())
        # NaN inputs: any NaN code is acceptable; compare payload-free
        assert np.array_equal(out[~nan_t], table[~nan_t])
        assert np.array_equal(fresh[~nan_t], table[~nan_t])
        if fmt == 0:
            assert np.all((out[nan_t] & 0x7f) == 0x7f) and np.all((table[nan_t] & 0x7f) == 0x7f)
        else:
            assert np.all((out[nan_t] & 0x7f) > 0x7c) and np.all((table[nan_t] & 0x7f) > 0x7c)


def test_bf16_rounding(oracle_c):
    rng = np.random.default_rng(0)
    x = rng.standard_normal(20000).astype(np.float32) * np.float32(10.0) ** rng.integers(-20, 20, 20000).astype(np.float32)
    t = torch.from_numpy(x).bfloat16().view(torch.int16).numpy().view(np.uint16)
    for xi, ti in zip(x[:5000], t[:5000]):
        assert oracle_c.ngpt_oracle_f32_to_bf16(float(xi)) == int(ti)
    # tie to even: 1 + 2^-8 is halfway between bf16(1) and the next bf16
    assert oracle_c.ngpt_oracle_f32_to_bf16(1.0 + 2.0 ** -8) == 0x3f80
    assert oracle_c.ngpt_oracle_f32_to_bf16(1.0 + 3 * 2.0 ** -8) == 0x3f82


@pytest.mark.parametrize("s", [1.0, 1 / 32, 100 / 448, 1.6 / 448, 0.75 / 448])
def test_eager_quantiser_formula(oracle, oracle_c, s):
    """oracle.quant_* (torch eager) == fp8(bf16(fp32(x)/fp32(s))) stated in C, bit for bit."""
    g = torch.Generator().manual_seed(1)
    x = (torch.randn(50000, generator=g) * 3).bfloat16()
    bits = x.view(torch.int16).numpy().view(np.uint16).copy()
    out = np.empty(bits.size, dtype=np.uint8)
    for fmt, fn in ((0, oracle.quant_e4m3), (1, oracle.quant_e5m2)):
        oracle_c.ngpt_oracle_quant_bf16(bits.ctypes.data, out.ctypes.data, bits.size,
                                        ctypes.c_float(np.float32(s)), fmt)
        ref = fn(x, s).view(torch.uint8).numpy()
        assert np.array_equal(out, ref)


def test_quantiser_bf16_intermediate_matters(oracle):
    """The bf16 rounding between the division and the fp8 cast is observable for the
    lm_head scales (a plausible mistake -- casting the fp32 quotient directly -- changes codes)."""
    g = torch.Generator().manual_seed(2)
    x = torch.randn(100000, generator=g).bfloat16()
    s = 100 / 448
    single = (x.float() / s).to(torch.float8_e4m3fn).view(torch.uint8)
    double = oracle.quant_e4m3(x, s).view(torch.uint8)
    frac = (single != double).float().mean().item()
    assert 0.005 < frac < 0.1
    # multiply-by-reciprocal differs from IEEE division for the lm_head grad scale
    gs = 0.75 / 448
    recip = (x.float() * (1.0 / gs)).bfloat16()
    assert (recip != x.div(gs)).any()


def test_e5m2_satfinite(oracle):
    v = torch.tensor([0.0, 1e-9, 57344.0, 61439.0, 61440.0, 1e9, -1e9, 3.0, -2.5])
    got = oracle.e5m2_satfinite(v).view(torch.uint8).tolist()
    assert got == [0, 0, 0x7b, 0x7b, 0x7b, 0x7b, 0xfb, 0x42, 0xc1]
