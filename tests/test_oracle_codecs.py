"""Pins the oracle's scalar codecs against library codecs (torch / numpy) and
the reference's own known-answer tests."""
import numpy as np
import torch


def _all_f32_patterns_sample(rng, n):
    """Random fp32 bit patterns (finite), plus every rounding-tie pattern family."""
    bits = rng.integers(0, 2**32, size=n, dtype=np.uint64).astype(np.uint32)
    x = bits.view(np.float32)
    return x[np.isfinite(x)]


def test_bf16_rne_matches_torch(oracle):
    rng = np.random.default_rng(1)
    x = _all_f32_patterns_sample(rng, 400000)
    # exact ties: low 16 bits == 0x8000, both parities of the kept bit
    hi = rng.integers(0, 0x7F7F, size=20000, dtype=np.uint32)
    ties = ((hi << 16) | 0x8000).view(np.float32)
    x = np.concatenate([x, ties, -ties, np.float32([0.0, -0.0, 1.0, 3.3895314e38])])
    got = oracle.f32_to_bf16(x)
    want = torch.from_numpy(x.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    np.testing.assert_array_equal(got, want)


def test_bf16_rne_arithmetic_definition(oracle):
    """serenitymojo/ops/torch_bf16.mojo:27-60: nearest multiple of 2^(e-7), ties to even k."""
    rng = np.random.default_rng(2)
    x = (rng.standard_normal(20000) * np.exp(rng.uniform(-20, 20, 20000))).astype(np.float32)
    got = oracle.bf16_to_f32(oracle.f32_to_bf16(x)).astype(np.float64)
    a = np.abs(x.astype(np.float64))
    e = np.floor(np.log2(a))
    step = 2.0 ** (e - 7)
    y = a / step
    kf = np.floor(y)
    frac = y - kf
    k = kf + ((frac > 0.5) | ((frac == 0.5) & (kf % 2 == 1)))
    want = np.sign(x) * k * step
    np.testing.assert_array_equal(got, want)


def test_f16_rne_matches_numpy(oracle):
    rng = np.random.default_rng(3)
    x = _all_f32_patterns_sample(rng, 400000)
    x = x[np.abs(x) < 65520.0]
    # all fp16 midpoints: (h + h_next)/2 is exactly representable in fp32
    h = np.arange(0, 0x7BFF, dtype=np.uint16)
    lo = h.view(np.float16).astype(np.float32)
    hi = (h + 1).astype(np.uint16).view(np.float16).astype(np.float32)
    mid = ((lo.astype(np.float64) + hi.astype(np.float64)) / 2).astype(np.float32)
    x = np.concatenate([x, mid, -mid, lo, -lo, np.float32([0.0, -0.0, 2.0**-25, 2.0**-24, 1.5 * 2.0**-25])])
    got = oracle.f32_to_f16(x)
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    np.testing.assert_array_equal(got, want)


def test_f16_overflow_saturates(oracle):
    x = np.float32([65519.9, 65520.0, 1e9, np.inf, -65520.0, -np.inf])
    got = oracle.f32_to_f16(x)
    np.testing.assert_array_equal(got, np.uint16([0x7BFF, 0x7BFF, 0x7BFF, 0x7BFF, 0xFBFF, 0xFBFF]))


def test_f16_decode_all_codes(oracle):
    L = oracle.lib()
    codes = np.arange(0, 65536, dtype=np.uint32).astype(np.uint16)
    want = codes.view(np.float16).astype(np.float32)
    got = np.float32([L.sage_oracle_f16_to_f32(int(c)) for c in codes])
    m = np.isfinite(want)
    np.testing.assert_array_equal(got[m], want[m])
    assert np.all(np.isnan(got[np.isnan(want)]))


def test_e4m3_decode_all_codes_matches_torch(oracle):
    codes = np.arange(256, dtype=np.uint8)
    got = oracle.e4m3_to_f32(codes)
    want = torch.from_numpy(codes.copy()).view(torch.float8_e4m3fn).to(torch.float32).numpy()
    m = ~np.isnan(want)                     # 0x7F / 0xFF are NaN in e4m3fn; the decoder is never fed them
    np.testing.assert_array_equal(got[m], want[m])
    assert np.signbit(got[0x80]) and got[0x80] == 0.0


def test_e4m3_encode_matches_torch(oracle):
    rng = np.random.default_rng(4)
    x = (rng.standard_normal(300000) * np.exp(rng.uniform(-12, 6.2, 300000))).astype(np.float32)
    x = x[np.abs(x) <= 448.0]
    # all midpoints between adjacent e4m3 values
    codes = np.arange(0, 0x7E, dtype=np.uint8)
    lo = oracle.e4m3_to_f32(codes)
    hi = oracle.e4m3_to_f32((codes + 1).astype(np.uint8))
    mid = ((lo.astype(np.float64) + hi.astype(np.float64)) / 2).astype(np.float32)
    x = np.concatenate([x, mid, -mid, lo, -lo])
    got = oracle.f32_to_e4m3(x)
    want = torch.from_numpy(x.copy()).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    np.testing.assert_array_equal(got, want)


def test_e4m3_reference_kats(oracle):
    """serenitymojo/ops/tests/fp8_quant_smoke.mojo:108-143: grid values round-trip
    exactly at scale 1; 460 / -470 saturate to +-448; NaN -> +-0."""
    grid = np.float32([448.0, -448.0, 1.0, -1.0, 1.5, 0.5, 0.25, 240.0,
                       0.015625, -0.015625, 0.001953125, 0.0, 2.0, -3.5, 96.0, 20.0])
    np.testing.assert_array_equal(oracle.e4m3_to_f32(oracle.f32_to_e4m3(grid)), grid)
    sat = oracle.e4m3_to_f32(oracle.f32_to_e4m3(np.float32([448.0, 460.0, -470.0, 1.0])))
    np.testing.assert_array_equal(sat, np.float32([448.0, 448.0, -448.0, 1.0]))
    assert oracle.f32_to_e4m3(np.float32([np.nan]))[0] in (0x00, 0x80)
    # 0x7F (NaN code) is never produced
    rng = np.random.default_rng(5)
    x = (rng.standard_normal(100000) * 1000).astype(np.float32)
    assert not np.any((oracle.f32_to_e4m3(x) & 0x7F) == 0x7F)
