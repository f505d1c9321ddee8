"""Pins oracle/rounding.py against library conversions and double-rounding traps."""
import numpy as np
import torch

from oracle import rounding as R


def test_bf16_matches_torch_on_fp32_inputs():
    rng = np.random.default_rng(0)
    x = np.concatenate([
        rng.standard_normal(200000).astype(np.float32),
        (rng.standard_normal(50000) * 1e-30).astype(np.float32),
        (rng.standard_normal(50000) * 1e30).astype(np.float32),
        np.array([0.0, -0.0, np.inf, -np.inf, 3.3895314e38, 3.4e38, 1e-40, -1e-40, 2.0 ** -133, 2.0 ** -134],
                 dtype=np.float32),
    ])
    got = R.f64_to_bf16(x.astype(np.float64))
    ref = torch.from_numpy(x).to(torch.bfloat16).to(torch.float32).numpy()
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))


def test_bf16_single_rounding_trap():
    # 1 + 2^-8 is the tie between 1 and 1+2^-7; + 2^-30 puts the exact value above the tie.
    # Rounding through fp32 first loses the 2^-30 and resolves the tie to even (1.0).
    x = np.float64(1.0) + 2.0 ** -8 + 2.0 ** -30
    assert R.f64_to_bf16(x) == np.float32(1.0 + 2.0 ** -7)
    via_f32 = torch.tensor(np.float32(x)).to(torch.bfloat16).item()
    assert via_f32 == 1.0


def test_fp16_single_rounding_trap_and_library():
    x = np.float64(1.0) + 2.0 ** -11 + 2.0 ** -40
    assert R.f64_to_f16(x) == np.float32(1.0 + 2.0 ** -10)
    rng = np.random.default_rng(1)
    y = rng.standard_normal(100000).astype(np.float32) * 10
    ref = torch.from_numpy(y).to(torch.float16).to(torch.float32).numpy()
    assert np.array_equal(R.f64_to_f16(y.astype(np.float64)), ref)


def test_bits16_roundtrip():
    for tag in (R.BF16, R.FP16):
        b = np.arange(0, 0x7C00 if tag == R.FP16 else 0x7F80, dtype=np.uint16)
        v = R.from_bits16(b, tag)
        assert np.array_equal(R.bits16(v, tag), b)
        assert np.all(np.diff(v) > 0)        # non-negative patterns are value-ordered


def test_e4m3_table_matches_torch():
    codes = torch.arange(256, dtype=torch.uint8)
    ref = codes.view(torch.float8_e4m3fn).to(torch.float32).numpy()
    mine = R.E4M3_VALUES
    assert np.array_equal(np.isnan(ref), np.isnan(mine))
    ok = ~np.isnan(ref)
    assert np.array_equal(ref[ok], mine[ok])


def test_e4m3_encode_matches_torch_exhaustive_fp16_range():
    # every fp16 value with |x| <= 448 (torch's cast is RNE; no saturation is involved in this range)
    h = np.arange(0x10000, dtype=np.uint32).astype(np.uint16).view(np.float16).astype(np.float32)
    h = h[np.isfinite(h) & (np.abs(h) <= 448)]
    ref = torch.from_numpy(h).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    got = R.f32_to_e4m3fn(h)
    assert np.array_equal(got, ref)


def test_e4m3_encode_random_fp32_and_ties():
    rng = np.random.default_rng(2)
    x = (rng.standard_normal(300000) * rng.choice([1e-3, 0.05, 1, 30, 200], 300000)).astype(np.float32)
    x = x[np.abs(x) <= 448]
    ref = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(R.f32_to_e4m3fn(x), ref)
    # exact ties between neighbours go to the even code
    v = R.E4M3_VALUES[:0x7E].astype(np.float64)
    mid = ((v[:-1] + v[1:]) / 2).astype(np.float32)
    got = R.f32_to_e4m3fn(mid)
    assert np.all(got % 2 == 0)
    assert np.all((got == np.arange(0x7D)) | (got == np.arange(1, 0x7E)))


def test_e4m3_saturates_and_nan():
    x = np.array([448.0, 449.0, 464.0, 1e9, np.inf, -1e9, np.nan], dtype=np.float32)
    got = R.f32_to_e4m3fn(x)
    assert list(got[:6]) == [0x7E, 0x7E, 0x7E, 0x7E, 0x7E, 0xFE]
    assert got[6] & 0x7F == 0x7F
