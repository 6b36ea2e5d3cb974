"""Pins the oracle's storage codecs against the format definitions and torch."""
import numpy as np
import torch

from oracle import paged_attention_oracle as O


def test_bf16_decode_exhaustive_vs_torch():
    bits = np.arange(65536, dtype=np.uint16)
    ours = O.bf16_bits_to_f32(bits)
    ref = torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16).float().numpy()
    assert np.array_equal(ours.view(np.uint32), ref.view(np.uint32))


def test_bf16_encode_roundtrip_exhaustive():
    bits = np.arange(65536, dtype=np.uint16)
    f = O.bf16_bits_to_f32(bits)
    back = O.f32_to_bf16_bits(f)
    nan = np.isnan(f)
    assert np.array_equal(back[~nan], bits[~nan])
    assert np.all(np.isnan(O.bf16_bits_to_f32(back[nan])))


def test_bf16_encode_rne_vs_torch(rng):
    x = np.concatenate([
        rng.standard_normal(200000).astype(np.float32),
        (rng.standard_normal(50000) * 1e-30).astype(np.float32),
        (rng.standard_normal(50000) * 1e30).astype(np.float32),
        np.array([0.0, -0.0, np.inf, -np.inf, 3.3895314e38, 1.0 + 2 ** -8, 1.0 + 3 * 2 ** -8], np.float32),
    ])
    ours = O.f32_to_bf16_bits(x)
    ref = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(ours, ref)
    # ties go to even: 1 + 2^-8 is halfway between 1.0 (even) and 1 + 2^-7
    assert O.f32_to_bf16_bits(np.float32(1.0 + 2 ** -8)) == 0x3F80
    assert O.f32_to_bf16_bits(np.float32(1.0 + 3 * 2 ** -8)) == 0x3F82


def test_fp8_lut_definition_and_torch():
    lut = O.FP8_E4M3FN_LUT
    assert lut[0x7E] == 448.0 and lut[0xFE] == -448.0
    assert np.isnan(lut[0x7F]) and np.isnan(lut[0xFF])
    assert lut[0x01] == 2.0 ** -9 and lut[0x08] == 2.0 ** -6 and lut[0x38] == 1.0
    assert not np.any(np.isinf(lut))
    codes = np.arange(256, dtype=np.uint8)
    ref = torch.from_numpy(codes).view(torch.float8_e4m3fn).float().numpy()
    ok = ~np.isnan(lut)
    assert np.array_equal(lut[ok], ref[ok]) and np.all(np.isnan(ref[~ok]))


def test_fp8_encode_roundtrip_and_rne(rng):
    codes = np.arange(256, dtype=np.uint8)
    vals = O.fp8_e4m3fn_decode(codes)
    ok = ~np.isnan(vals)
    back = O.fp8_e4m3fn_encode(vals[ok])
    # -0.0 keeps its sign bit, every finite code is a fixed point
    assert np.array_equal(back, codes[ok])
    # midpoints between neighbours go to the even code; saturation at 448
    mags = O.FP8_E4M3FN_LUT[:0x7F].astype(np.float64)
    mid = ((mags[:-1] + mags[1:]) / 2).astype(np.float32)
    got = O.fp8_e4m3fn_encode(mid)
    lo = np.arange(0, 0x7E)
    want = np.where(lo % 2 == 0, lo, lo + 1).astype(np.uint8)
    assert np.array_equal(got, want)
    assert O.fp8_e4m3fn_encode(np.float32(1e9)) == 0x7E
    assert O.fp8_e4m3fn_encode(np.float32(-1e9)) == 0xFE
    x = (rng.standard_normal(300000) * rng.choice([0.01, 1.0, 100.0], 300000)).astype(np.float32)
    x = np.clip(x, -448, 448)
    ref = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(O.fp8_e4m3fn_encode(x), ref)


def test_quantize_kv_scale_rule(rng):
    pool = rng.standard_normal((5, 4, 3, 8)).astype(np.float32)
    pool[2] = 0.0
    codes, scale = O.quantize_kv_fp8(pool)
    absmax = np.abs(pool).max(axis=(1, 3))
    assert np.allclose(scale[absmax > 0], absmax[absmax > 0] / 448.0, rtol=1e-7)
    assert np.all(scale[2] == 1.0) and np.all(codes[2] == 0)
    deq = O.dequantize_kv_fp8(codes, scale)
    # e4m3 has 3 mantissa bits: relative step 2^-3, so error <= 2^-4 of magnitude
    # (plus the subnormal floor of scale * 2^-10)
    err = np.abs(deq - pool)
    assert np.all(err <= np.abs(pool) * 2.0 ** -4 + scale[:, None, :, None] * 2.0 ** -10 + 1e-12)
    # the absmax element maps to +-448 exactly
    assert np.abs(O.fp8_e4m3fn_decode(codes)).max() == 448.0
