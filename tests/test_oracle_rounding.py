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


def test_fp32_subtraction_then_rne_equals_single_rounding():
    """Lemma the GPU smoothing step relies on: for a, b in T, RN_T(RN_f32(a - b)) == RN_T(a - b).

    Checked on random pairs with every exponent gap from 0 to 30 (where the binary32 difference stops being exact)
    and on values next to powers of two, for both 16-bit formats."""
    rng = np.random.default_rng(11)
    for tag in (R.BF16, R.FP16):
        pats = np.arange(0x0080 if tag == R.BF16 else 0x0001, 0x7F80 if tag == R.BF16 else 0x7C00, dtype=np.uint16)
        vals = R.from_bits16(pats, tag).astype(np.float64)
        vals = vals[(vals > 1e-30) & (vals < 1e30)]
        a = rng.choice(vals, 400000) * rng.choice([-1.0, 1.0], 400000)
        gaps = rng.integers(0, 31, 400000)
        b = rng.choice(vals, 400000)
        b = b * 2.0 ** (np.floor(np.log2(np.abs(a))) - gaps - np.floor(np.log2(b)))      # force the exponent gap
        b = R.round_to(b, tag).astype(np.float64) * rng.choice([-1.0, 1.0], 400000)
        keep = np.isfinite(b) & (b != 0)
        a, b = a[keep], b[keep]
        exact = R.round_to(a - b, tag)
        via32 = R.round_to((a.astype(np.float32) - b.astype(np.float32)).astype(np.float64), tag)
        assert np.array_equal(exact, via32), tag
        # neighbours of powers of two (where the spacing halves)
        p2 = 2.0 ** rng.integers(-10, 10, 100000)
        ulp = p2 * (2.0 ** -7 if tag == R.BF16 else 2.0 ** -10)
        a2 = R.round_to(p2 + rng.integers(-2, 3, 100000) * ulp / 2, tag).astype(np.float64)
        b2 = R.round_to(p2 * 2.0 ** -rng.integers(8, 26, 100000), tag).astype(np.float64)
        assert np.array_equal(R.round_to(a2 - b2, tag),
                              R.round_to((a2.astype(np.float32) - b2.astype(np.float32)).astype(np.float64), tag))


def _safe_for_two_step(r32, tag):
    """The predicate of the kernels' binary64 -> 16-bit shortcut (csrc/maskpred.hip, f64_to_elem_fast): the binary32 image
    is zero, or inside the 16-bit format's normal range and not exactly on one of its rounding ties."""
    b = np.ascontiguousarray(r32, dtype=np.float32).view(np.uint32)
    mag = b & np.uint32(0x7fffffff)
    drop = 16 if tag == R.BF16 else 13
    low, tie = np.uint32((1 << drop) - 1), np.uint32(1 << (drop - 1))
    lo = np.uint32(0x00800000 if tag == R.BF16 else 0x38800000)
    hi = np.uint32(0x7f000000 if tag == R.BF16 else 0x47000000)
    return (mag == 0) | ((mag >= lo) & (mag < hi) & ((b & low) != tie))


def test_binary64_to_16_bits_through_binary32_where_the_kernels_take_that_way():
    """Rounding a binary64 value to binary32 first changes its rounding to a 16-bit format only when the binary32 image
    lands exactly on a tie of that format: wherever the kernels' predicate holds, both ways give the same bits - also
    for a value two units in the last place away (the reciprocal-based probabilities)."""
    rng = np.random.default_rng(4)
    for tag in (R.BF16, R.FP16):
        drop = 16 if tag == R.BF16 else 13
        # random magnitudes over the whole normal range, values sitting on and next to ties, next to binade edges
        e = rng.integers(-14, 15, size=400000) if tag == R.FP16 else rng.integers(-126, 127, size=400000)
        x = np.ldexp(1.0 + rng.random(400000), e) * rng.choice([-1.0, 1.0], size=400000)
        grid = np.ldexp(1.0 + rng.integers(0, 1 << (23 - drop), size=200000) * 2.0 ** -(23 - drop),
                        rng.integers(-10, 10, size=200000))                  # values of the 16-bit format
        ulp = np.ldexp(1.0, np.floor(np.log2(grid)).astype(np.int64) - (23 - drop))
        tie = grid + 0.5 * ulp
        near = np.concatenate([tie, tie * (1 + 2.0 ** -30), tie * (1 - 2.0 ** -30), tie * (1 + 2.0 ** -52),
                               tie * (1 - 2.0 ** -52), tie + 2.0 ** -24 * grid, grid * (1 - 2.0 ** -40),
                               grid * (1 + 2.0 ** -40)])
        for vals, least in ((x, 0.95), (near, 0.25)):
            r32 = vals.astype(np.float32)
            safe = _safe_for_two_step(r32, tag)
            assert safe.mean() > least
            direct = R.bits16(R.round_to(vals, tag), tag)
            two_step = R.bits16(R.round_to(r32.astype(np.float64), tag), tag)
            assert np.array_equal(direct[safe], two_step[safe])
            # a neighbour within two units in the last place of binary64 rounds like the value itself
            for k in (-2, 2):
                nb = (vals.view(np.int64) + k).view(np.float64)
                assert np.array_equal(R.bits16(R.round_to(nb, tag), tag)[safe], two_step[safe])
        # and the predicate is not vacuous: on the ties themselves the two ways differ somewhere
        r32 = (tie * (1 + 2.0 ** -30)).astype(np.float32)
        assert (~_safe_for_two_step(r32, tag)).any()
        assert not np.array_equal(R.bits16(R.round_to(tie * (1 + 2.0 ** -30), tag), tag),
                                  R.bits16(R.round_to(r32.astype(np.float64), tag), tag))
