"""Pins of the oracle's scalar numerics against independent implementations (numpy's float16, torch's bfloat16),
closed forms, and the worked examples of the reference's precision-conversion document."""
import ctypes as C

import numpy as np
import pytest
import torch

import orc
from ascq import _abi as abi


def test_f16_to_f32_all_patterns():
    bits = np.arange(65536, dtype=np.uint16)
    got = orc.f16_bits_to_f32(bits)
    want = bits.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))
    assert np.all(np.isnan(got[nan]))


def test_f32_to_f16_roundtrip_and_random():
    bits = np.arange(65536, dtype=np.uint16)
    f = bits.view(np.float16).astype(np.float32)
    ok = ~np.isnan(f)
    assert np.array_equal(orc.f32_to_f16_bits(f)[ok], bits[ok])
    rng = np.random.default_rng(1)
    x = np.concatenate([
        rng.standard_normal(2_000_000).astype(np.float32) * np.float32(100.0),
        (rng.standard_normal(500_000) * 1e-6).astype(np.float32),           # subnormal results
        rng.integers(0, 2**32, 2_000_000, dtype=np.uint64).astype(np.uint32).view(np.float32),  # any bit pattern
    ])
    x = x[~np.isnan(x)]
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(orc.f32_to_f16_bits(x), want)


def test_f64_to_f16_ties_go_to_even():
    # the exact midpoint of two adjacent half values must round to the one with an even mantissa
    bits = np.arange(0, 0x7BFF, dtype=np.uint16)
    lo = bits.view(np.float16).astype(np.float64)
    hi = (bits + 1).astype(np.uint16).view(np.float16).astype(np.float64)
    mid = (lo + hi) / 2
    L = orc.lib()
    got = np.array([L.orc_f64_to_f16(float(v)) for v in mid[::7]], dtype=np.uint16)
    b = bits[::7]
    want = np.where(b % 2 == 0, b, b + 1).astype(np.uint16)
    assert np.array_equal(got, want)
    # doc example: 0.5 + 2^-12 -> 0.5 under RINT (precision_conversion.md:520-534)
    assert L.orc_f32_to_f16(0.5 + 2.0**-12) == np.float16(0.5).view(np.uint16)
    # overflow goes to infinity, 65520 is the first value that does
    assert L.orc_f32_to_f16(65519.0) == 0x7BFF and L.orc_f32_to_f16(65520.0) == 0x7C00


def test_f16_mul_add_against_numpy_half():
    rng = np.random.default_rng(2)
    n = 4_000_000
    a = rng.integers(0, 65536, n).astype(np.uint16)
    b = rng.integers(0, 65536, n).astype(np.uint16)
    # concentrate half of the pairs where products / sums stay finite and hit subnormals and ties
    a[: n // 2] = (rng.standard_normal(n // 2) * 8).astype(np.float16).view(np.uint16)
    b[: n // 2] = (rng.standard_normal(n // 2) * 0.01).astype(np.float16).view(np.uint16)
    af, bf = a.view(np.float16), b.view(np.float16)
    with np.errstate(all="ignore"):
        wm = (af * bf)
        wa = (af + bf)
    gm = orc.f16_mul_bits(a, b).view(np.float16)
    ga = orc.f16_add_bits(a, b).view(np.float16)
    for got, want in ((gm, wm), (ga, wa)):
        ok = ~np.isnan(want)
        assert np.array_equal(got[ok].view(np.uint16), want[ok].view(np.uint16))
        assert np.all(np.isnan(got[~ok]))


def test_bf16_against_torch():
    rng = np.random.default_rng(3)
    x = np.concatenate([
        rng.standard_normal(1_000_000).astype(np.float32),
        rng.integers(0, 2**32, 1_000_000, dtype=np.uint64).astype(np.uint32).view(np.float32),
    ])
    x = x[~np.isnan(x)]
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(orc.f32_to_bf16_bits(x), want)
    # doc example precision_conversion.md:541-553: 0.5 + 2^-9 + 2^-11 -> 0.5 + 2^-8 under RINT
    got = orc.f32_to_bf16_bits(np.array([0.5 + 2.0**-9 + 2.0**-11], dtype=np.float32))
    assert orc.bf16_bits_to_f32(got)[0] == np.float32(0.5 + 2.0**-8)


def test_int32_to_float_doc_example():
    # precision_conversion.md:427-437: 2^25 + 3 -> 2^25 + 4 under RINT; the oracle uses the C cast (RNE)
    d = abi.DequantDesc(policy=abi.PER_TENSOR, src_dtype=abi.I32, scale_dtype=abi.F32, dst_dtype=abi.F32,
                        mode=abi.DEQUANT_WITH_MULTI_ROW, scale=1.0, m=1, n=8, cal_count=8)
    src = np.full((1, 8), 2**25 + 3, dtype=np.int32)
    assert orc.dequant(d, src)[0, 0] == np.float32(2**25 + 4)


@pytest.mark.parametrize("mode,fn", [
    (abi.CAST_RINT, np.rint), (abi.CAST_NONE, np.rint), (abi.CAST_FLOOR, np.floor), (abi.CAST_CEIL, np.ceil),
    (abi.CAST_TRUNC, np.trunc), (abi.CAST_ROUND, lambda v: np.sign(v) * np.floor(np.abs(v) + 0.5)),
])
def test_round_sat8_modes(mode, fn):
    x = np.concatenate([np.arange(-140, 140, 0.25), [127.5, 127.49, -128.5, -128.51, 1e9, -1e9, np.inf, -np.inf]])
    x = x.astype(np.float32)
    want = np.clip(fn(x.astype(np.float64)), -128, 127).astype(np.int8)
    assert np.array_equal(orc.round_sat8(x, mode), want)


def test_round_sat8_doc_example():
    # precision_conversion.md:242-252: half 2^7 - 0.5 saturates to 2^7 - 1 in every mode
    for mode in (abi.CAST_RINT, abi.CAST_FLOOR, abi.CAST_CEIL, abi.CAST_ROUND, abi.CAST_TRUNC):
        assert orc.round_sat8(np.array([127.5], np.float32), mode)[0] == 127
    # ties to even under RINT
    assert list(orc.round_sat8(np.array([0.5, 1.5, 2.5, -0.5, -1.5, -2.5], np.float32))) == [0, 2, 2, 0, -2, -2]


# ------------------------------------------------------------------ 8-bit floats
def _fp8_lib():
    L = orc.lib()
    L.orc_f32_to_fp8.restype = C.c_uint8
    L.orc_f32_to_fp8.argtypes = [C.c_float, C.c_int]
    L.orc_fp8_to_f32.restype = C.c_float
    L.orc_fp8_to_f32.argtypes = [C.c_uint8, C.c_int]
    return L


@pytest.mark.parametrize("e5m2", [0, 1])
def test_fp8_codes_decode_like_torch_and_round_trip(e5m2):
    """All 256 codes: the value equals torch's float8 (the OCP formats the reference's own golden scripts take from
    ml_dtypes, examples/.../matmul_fp8/scripts/gen_data.py:142-147), and encoding a representable value gives its
    code back."""
    L = _fp8_lib()
    tdt = torch.float8_e5m2 if e5m2 else torch.float8_e4m3fn
    vals = torch.arange(256, dtype=torch.int32).to(torch.uint8).view(tdt).float().numpy()
    for code in range(256):
        mine = L.orc_fp8_to_f32(code, e5m2)
        if np.isnan(vals[code]):
            assert np.isnan(mine)
            continue
        assert mine == vals[code]
        if np.isfinite(mine):
            back = L.orc_f32_to_fp8(mine, e5m2)
            assert back == code or (mine == 0 and (back & 0x7F) == 0)


@pytest.mark.parametrize("e5m2", [0, 1])
def test_fp8_encode_matches_torch_in_range_and_saturates(e5m2):
    """Round-half-even to the nearest representable value agrees with torch's conversion for every input below the
    overflow threshold (random values, every midpoint between neighbours and its two fp32 neighbours); from the
    largest finite value up the result saturates (the reference's SatMode::SAT) where torch gives NaN / infinity."""
    L = _fp8_lib()
    tdt = torch.float8_e5m2 if e5m2 else torch.float8_e4m3fn
    top_code = 0x7B if e5m2 else 0x7E
    top = L.orc_fp8_to_f32(top_code, e5m2)
    grid = np.array([L.orc_fp8_to_f32(c, e5m2) for c in range(top_code + 1)], dtype=np.float64)
    mids = ((grid[:-1] + grid[1:]) / 2).astype(np.float32)
    rng = np.random.default_rng(8)
    rand = (np.exp(rng.uniform(np.log(1e-8), np.log(top), 20000)) * rng.choice([-1, 1], 20000)).astype(np.float32)
    xs = np.concatenate([mids, np.nextafter(mids, np.float32(0)), np.nextafter(mids, np.float32(np.inf)), -mids, rand,
                         grid.astype(np.float32), np.float32([0.0, -0.0])])
    want = torch.from_numpy(xs).to(tdt).view(torch.uint8).numpy()
    got = np.array([L.orc_f32_to_fp8(float(v), e5m2) for v in xs], dtype=np.uint8)
    assert np.array_equal(got, want)
    for v in (top, np.nextafter(np.float32(top), np.float32(np.inf)), top * 1.04, top * 2, 1e30, np.inf):
        assert L.orc_f32_to_fp8(float(v), e5m2) == top_code
        assert L.orc_f32_to_fp8(-float(v), e5m2) == 0x80 | top_code
    # NaN -> +0: the saturation-mode column of the reference's boundary table for float -> fp8_e5m2_t
    # (docs/zh/api/附录/Reg矢量计算接口边界值汇总.md); its e4m3 cell is empty and follows the same rule here
    assert L.orc_f32_to_fp8(float("nan"), e5m2) == 0



# ---------------------------------------------------------------- 4-bit floats (fp4x2_e2m1_t / fp4x2_e1m2_t)
def _fp4_lib():
    return orc.lib()


@pytest.mark.parametrize("e1m2", [0, 1])
def test_fp4_value_grid_and_the_reference_boundary_table(e1m2):
    """The value sets of the two formats (e2m1 is the OCP microscaling FP4: 0, 0.5, 1, 1.5, 2, 3, 4, 6; e1m2 with the
    same bias has 0 .. 1.75 in steps of 0.25), built here from sign / exponent / mantissa fields, and the rows
    bfloat16_t/fp4x2_* of the reference's boundary table in saturation mode: MIN / -inf -> -max, MAX / inf -> +max,
    nan -> 0.0 (docs/zh/api/附录/Reg矢量计算接口边界值汇总.md)."""
    L = _fp4_lib()
    ebits, mbits = (1, 2) if e1m2 else (2, 1)
    for code in range(16):
        e, m = (code >> mbits) & ((1 << ebits) - 1), code & ((1 << mbits) - 1)
        mag = (m / (1 << mbits)) if e == 0 else (1 + m / (1 << mbits)) * 2.0 ** (e - 1)   # bias 1, e == 0 subnormal
        want = -mag if code & 8 else mag
        got = L.orc_fp4_to_f32(code, e1m2)
        assert got == want and np.signbit(got) == bool(code & 8)
        for mode in (abi.CAST_RINT, abi.CAST_FLOOR, abi.CAST_CEIL, abi.CAST_ROUND, abi.CAST_TRUNC):
            assert L.orc_f32_to_fp4(want, e1m2, mode) == code          # representable values are fixed points
    top = 1.75 if e1m2 else 6.0
    bf16_max = float(np.float32(3.3895313892515355e38))
    for mode in (abi.CAST_RINT, abi.CAST_FLOOR, abi.CAST_CEIL, abi.CAST_ROUND, abi.CAST_TRUNC):
        for v in (bf16_max, float("inf"), top * 1.01, 8.0):
            assert L.orc_fp4_to_f32(L.orc_f32_to_fp4(v, e1m2, mode), e1m2) == top
            assert L.orc_fp4_to_f32(L.orc_f32_to_fp4(-v, e1m2, mode), e1m2) == -top
        assert L.orc_f32_to_fp4(float("nan"), e1m2, mode) == 0
        assert L.orc_f32_to_fp4(0.0, e1m2, mode) == 0


def test_fp4_rounding_modes_known_answers():
    """Midpoints and off-grid values worked by hand for each rounding mode: half-even goes to the even code (the one
    whose mantissa bit is 0), ROUND away from zero, FLOOR / CEIL are directed on the signed value, TRUNC towards 0."""
    L = _fp4_lib()
    R, F, Cc, A, T = abi.CAST_RINT, abi.CAST_FLOOR, abi.CAST_CEIL, abi.CAST_ROUND, abi.CAST_TRUNC

    def q(v, e1m2, mode):
        return L.orc_fp4_to_f32(L.orc_f32_to_fp4(v, e1m2, mode), e1m2)

    # e2m1: neighbours (0, .5) (.5, 1) (1, 1.5) (1.5, 2) (2, 3) (3, 4) (4, 6); even codes are 0, 1, 2, 4
    for v, want in [(0.25, 0.0), (0.75, 1.0), (1.25, 1.0), (1.75, 2.0), (2.5, 2.0), (3.5, 4.0), (5.0, 4.0),
                    (-0.25, -0.0), (-2.5, -2.0), (-5.0, -4.0), (0.26, 0.5), (2.49, 2.0), (2.51, 3.0), (5.01, 6.0)]:
        assert q(v, 0, R) == want, (v, want)
    for v, want in [(0.25, 0.5), (1.25, 1.5), (2.5, 3.0), (5.0, 6.0), (-0.25, -0.5), (-2.5, -3.0), (4.9, 4.0)]:
        assert q(v, 0, A) == want, (v, want)
    for v, f, c, t in [(0.3, 0.0, 0.5, 0.0), (2.2, 2.0, 3.0, 2.0), (5.9, 4.0, 6.0, 4.0), (-0.3, -0.5, -0.0, -0.0),
                       (-2.2, -3.0, -2.0, -2.0), (-5.9, -6.0, -4.0, -4.0)]:
        assert (q(v, 0, F), q(v, 0, Cc), q(v, 0, T)) == (f, c, t), v
    # e1m2: a uniform grid of 0.25; even codes are the even multiples
    for v, want in [(0.125, 0.0), (0.375, 0.5), (0.625, 0.5), (1.625, 1.5), (1.7, 1.75), (-0.875, -1.0)]:
        assert q(v, 1, R) == want, (v, want)
    for v, want in [(0.125, 0.25), (0.625, 0.75), (-0.875, -1.0), (-0.125, -0.25)]:
        assert q(v, 1, A) == want, (v, want)
    for v, f, c, t in [(0.3, 0.25, 0.5, 0.25), (-0.3, -0.5, -0.25, -0.25), (1.74, 1.5, 1.75, 1.5)]:
        assert (q(v, 1, F), q(v, 1, Cc), q(v, 1, T)) == (f, c, t), v
    # a zero result keeps the sign of the input
    assert L.orc_f32_to_fp4(-0.1, 0, R) == 8 and L.orc_f32_to_fp4(-0.0, 1, R) == 8


@pytest.mark.parametrize("e1m2", [0, 1])
def test_fp4_rint_is_monotone_and_nearest(e1m2):
    """Over a dense sweep: the result is one of the two neighbours, never farther than the other neighbour, and the
    map is monotone."""
    L = _fp4_lib()
    xs = np.linspace(-7, 7, 5601).astype(np.float32)
    out = np.array([L.orc_fp4_to_f32(L.orc_f32_to_fp4(float(v), e1m2, abi.CAST_RINT), e1m2) for v in xs])
    assert np.all(np.diff(out) >= 0)
    grid = np.array(sorted({L.orc_fp4_to_f32(c, e1m2) for c in range(16)}))
    clipped = np.clip(xs, grid[0], grid[-1])
    best = np.min(np.abs(clipped[:, None] - grid[None, :]), axis=1)
    assert np.allclose(np.abs(out - clipped), best, atol=0)
