"""Pins the CPU checker's conversions (oracle/skl_oracle.c) before anything is
compared with it: the format definitions, known answers, round-trip and
nearest-value properties, and - where it was built - the reference's own
scalar library on the reference's test inputs (test/cvt/cvt_f32_f8.c:29-35).
"""
import os

import numpy as np
import pytest

import support
from support import decode_table, oracle, ref

FMTS = ("f8e4m3", "f8e5m2")
MAXB = {"f8e4m3": 0x7E, "f8e5m2": 0x7B}


def encode(fmt, x, sat):
    fn = getattr(oracle(), f"skl_oracle_f32_to_{fmt}")
    return fn(float(np.float32(x)), int(sat))


def encode_array(fmt, x, sat, scale=1.0, lib=None, suffix="_oracle"):
    lib = lib or oracle()
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.full(x.size, 0xAA, dtype=np.uint8)
    getattr(lib, f"skl_cvt_{'sat_' if sat else ''}f32_{fmt}{suffix}")(out, x, float(scale), x.size)
    return out


@pytest.mark.parametrize("fmt", FMTS)
def test_decode_matches_format_definition(fmt):
    table = decode_table(fmt)
    fn = getattr(oracle(), f"skl_oracle_{fmt}_to_f32")
    for code in range(256):
        v = np.float32(fn(code))
        if np.isnan(table[code]):
            # the reference returns the sign-less quiet NaN (ref/cvt/cvt_ofp8.c:41-43, 83-85)
            assert v.view(np.uint32) == 0x7FC00000, hex(code)
        else:
            assert v == np.float32(table[code]) and np.signbit(v) == np.signbit(table[code]), hex(code)


def test_decode_f4_values():
    want = [0, .5, 1, 1.5, 2, 3, 4, 6]
    for nib in range(16):
        v = oracle().skl_oracle_f4e2m1_to_f32(nib)
        assert abs(v) == want[nib & 7] and bool(np.signbit(np.float32(v))) == bool(nib & 8)


@pytest.mark.parametrize("fmt", FMTS)
def test_decode_vs_reference(fmt):
    if ref() is None:
        pytest.skip("reference library not built")
    for code in range(256):
        a = np.float32(getattr(oracle(), f"skl_oracle_{fmt}_to_f32")(code))
        b = np.float32(getattr(ref(), f"skl_cvt_{fmt}_f32")(code))
        assert a.view(np.uint32) == b.view(np.uint32), hex(code)
    for nib in range(16):
        a = np.float32(oracle().skl_oracle_f4e2m1_to_f32(nib))
        b = np.float32(ref().skl_cvt_f4e2m1_f32(nib))
        assert a.view(np.uint32) == b.view(np.uint32)


def test_encode_known_answers():
    # ties to even in the normal range, underflow tie to zero, the overflow
    # threshold of E4M3 (464 is the tie between 448 and the non-existent 480)
    assert encode("f8e4m3", 1.0625, 0) == 0x38
    assert encode("f8e4m3", 1.1875, 0) == 0x3A
    assert encode("f8e4m3", 2.0 ** -10, 0) == 0x00
    assert encode("f8e4m3", 3 * 2.0 ** -10, 0) == 0x02
    assert encode("f8e4m3", 464.0, 0) == 0x7E
    assert encode("f8e4m3", 465.0, 0) == 0x7F
    assert encode("f8e4m3", 465.0, 1) == 0x7E
    assert encode("f8e4m3", -465.0, 0) == 0x7F   # sign dropped
    assert encode("f8e4m3", -465.0, 1) == 0xFE
    assert encode("f8e4m3", 448.0, 0) == 0x7E
    assert encode("f8e4m3", 2.0 ** -6, 0) == 0x08
    assert encode("f8e4m3", 2.0 ** -9, 0) == 0x01
    assert encode("f8e4m3", 0.9375 * 2.0 ** -6, 0) == 0x08  # 7.5 * 2^-9: tie, even is 8 = min normal
    assert encode("f8e5m2", 57344.0, 0) == 0x7B
    assert encode("f8e5m2", 61439.0, 0) == 0x7B
    assert encode("f8e5m2", 61440.0, 0) == 0x7C  # tie rounds to even = overflow -> inf
    assert encode("f8e5m2", 61440.0, 1) == 0x7B
    assert encode("f8e5m2", -61440.0, 0) == 0xFC
    assert encode("f8e5m2", 2.0 ** -16, 0) == 0x01
    assert encode("f8e5m2", 2.0 ** -17, 0) == 0x00
    assert encode("f8e5m2", 1.125, 0) == 0x3C  # tie 1.0 / 1.25 -> even mantissa 0
    assert encode("f8e5m2", 1.375, 0) == 0x3E  # tie 1.25 / 1.5 -> even mantissa 2


@pytest.mark.parametrize("fmt", FMTS)
def test_encode_specials(fmt):
    inf_ns = {"f8e4m3": (0x7F, 0x7F), "f8e5m2": (0x7C, 0xFC)}[fmt]
    m = MAXB[fmt]
    for sat in (0, 1):
        assert encode(fmt, np.nan, sat) == 0x7F
        assert encode(fmt, -np.nan, sat) == 0x7F
        assert encode(fmt, 0.0, sat) == 0x00
        assert encode(fmt, -0.0, sat) == 0x80
        assert encode(fmt, 1e-45, sat) == 0x00      # fp32 subnormal
        assert encode(fmt, -1e-45, sat) == 0x80
    assert (encode(fmt, np.inf, 0), encode(fmt, -np.inf, 0)) == inf_ns
    assert (encode(fmt, np.inf, 1), encode(fmt, -np.inf, 1)) == (m, 0x80 | m)
    assert (encode(fmt, 3e38, 1), encode(fmt, -3e38, 1)) == (m, 0x80 | m)
    assert (encode(fmt, 3e38, 0), encode(fmt, -3e38, 0)) == inf_ns


@pytest.mark.parametrize("fmt", FMTS)
def test_encode_decode_round_trip(fmt):
    table = decode_table(fmt)
    for code in range(256):
        v = table[code]
        if np.isnan(v):
            continue
        if np.isinf(v):
            assert encode(fmt, v, 0) == code
            continue
        for sat in (0, 1):
            assert encode(fmt, v, sat) == code, hex(code)


@pytest.mark.parametrize("fmt", FMTS)
def test_encode_is_round_to_nearest_even(fmt):
    """Independent of the reference: the byte chosen must decode to the nearest
    representable value, ties to the even code, computed in fp64 from the table."""
    table = decode_table(fmt)
    finite = np.array([c for c in range(0x80) if np.isfinite(table[c])])
    vals = table[finite]            # ascending, starts at +0
    rng = np.random.default_rng(7)
    top = vals[-1]
    x = np.concatenate([
        rng.uniform(0, top, 20000), rng.uniform(0, vals[9], 20000),
        np.exp(rng.uniform(np.log(vals[1] / 8), np.log(top), 20000)),
        (vals[:-1] + vals[1:]) / 2,          # every tie
        np.nextafter(((vals[:-1] + vals[1:]) / 2).astype(np.float32), np.float32(0)).astype(np.float64),
        np.nextafter(((vals[:-1] + vals[1:]) / 2).astype(np.float32), np.float32(1e9)).astype(np.float64),
    ]).astype(np.float32)
    x = x[x <= np.float32(top)]
    got = encode_array(fmt, x, sat=True)
    xd = x.astype(np.float64)
    idx = np.searchsorted(vals, xd)          # vals[idx-1] < x <= vals[idx]
    idx = np.clip(idx, 1, len(vals) - 1)
    lo, hi = vals[idx - 1], vals[idx]
    want = np.where(xd - lo < hi - xd, finite[idx - 1], finite[idx])
    tie = (xd - lo) == (hi - xd)
    want = np.where(tie, np.where(finite[idx - 1] % 2 == 0, finite[idx - 1], finite[idx]), want)
    want = np.where(xd == hi, finite[idx], want)
    assert np.array_equal(got, want.astype(np.uint8))
    neg = encode_array(fmt, -x, sat=True)
    assert np.array_equal(neg, want.astype(np.uint8) | 0x80)


@pytest.mark.parametrize("fmt", FMTS)
def test_encode_monotonic(fmt):
    x = np.sort(np.random.default_rng(3).uniform(-600, 600, 50000).astype(np.float32))
    table = decode_table(fmt)
    y = table[encode_array(fmt, x, sat=True)]
    assert np.all(np.diff(y) >= 0)


def _structured_f32_patterns():
    hi = np.arange(1 << 16, dtype=np.uint32) << 16
    lows = np.array([0x0000, 0x0001, 0x7FFF, 0x8000, 0x8001, 0xFFFF, 0x1000, 0xF000], dtype=np.uint32)
    pats = (hi[:, None] | lows[None, :]).ravel()
    rnd = np.random.default_rng(11).integers(0, 1 << 32, size=1 << 21, dtype=np.uint64).astype(np.uint32)
    return np.concatenate([pats, rnd]).view(np.float32)


@pytest.mark.parametrize("sat", (False, True))
@pytest.mark.parametrize("fmt", FMTS)
def test_encode_vs_reference_bit_patterns(fmt, sat):
    """All 2^16 upper halves x 8 lower halves plus 2M random patterns."""
    if ref() is None:
        pytest.skip("reference library not built")
    x = _structured_f32_patterns()
    a = encode_array(fmt, x, sat)
    b = encode_array(fmt, x, sat, lib=ref(), suffix="_ref")
    assert np.array_equal(a, b)


@pytest.mark.slow
@pytest.mark.parametrize("fmt", FMTS)
def test_encode_vs_reference_exhaustive(fmt):
    if ref() is None or os.environ.get("SKL_EXHAUSTIVE") != "1":
        pytest.skip("set SKL_EXHAUSTIVE=1 (and build the reference library) for the 2^32 sweep")
    for chunk in range(256):
        x = (np.arange(1 << 24, dtype=np.uint32) | np.uint32(chunk << 24)).view(np.float32)
        for sat in (False, True):
            assert np.array_equal(encode_array(fmt, x, sat), encode_array(fmt, x, sat, lib=ref(), suffix="_ref"))


def reference_cvt_input(n, seed):
    """test/cvt/cvt_f32_f8.h:55-57 + cvt_f32_f8.c:29-35: uniform [-512, 512] with
    the first three elements forced to NaN, +inf, -inf."""
    x = np.random.default_rng(seed).uniform(-512, 512, n).astype(np.float32)
    x[:3] = [np.nan, np.inf, -np.inf]
    return x


@pytest.mark.parametrize("row", support.table_rows("test/cvt/cvt_f32_f8_zvfofp8min.c"),
                         ids=lambda r: f"L{r['line']}")
def test_cvt_f32_reference_table(row):
    if ref() is None:
        pytest.skip("reference library not built")
    fmt = "f8e4m3" if row["kind"].endswith("E4M3") else "f8e5m2"
    x = reference_cvt_input(row["len"], row["line"])
    a = encode_array(fmt, x, row["saturation"], row["scale"])
    b = encode_array(fmt, x, row["saturation"], row["scale"], lib=ref(), suffix="_ref")
    assert np.array_equal(a, b)


@pytest.mark.parametrize("scale", (1.0, 1.5, 2.0 ** 100, 2.0 ** -100, 3.0e38))
@pytest.mark.parametrize("fmt", FMTS)
def test_cvt_scaled_vs_reference(fmt, scale):
    """The scale multiply is one fp32 operation: subnormal inputs times a large
    scale, and products that overflow to infinity, must agree."""
    if ref() is None:
        pytest.skip("reference library not built")
    rng = np.random.default_rng(5)
    x = np.concatenate([
        rng.uniform(-512, 512, 4096).astype(np.float32),
        rng.integers(0, 1 << 23, 2048, dtype=np.uint32).view(np.float32),                    # subnormals
        (rng.integers(0, 1 << 23, 2048, dtype=np.uint32) | np.uint32(0x80000000)).view(np.float32),
        np.float32([np.nan, np.inf, -np.inf, 0.0, -0.0]),
    ])
    for sat in (False, True):
        a = encode_array(fmt, x, sat, scale)
        b = encode_array(fmt, x, sat, scale, lib=ref(), suffix="_ref")
        assert np.array_equal(a, b)


@pytest.mark.parametrize("scale", (1.0, 1.5, 0.001, 1e30))
@pytest.mark.parametrize("sat", (False, True))
@pytest.mark.parametrize("fmt", FMTS)
def test_cvt_bf16_all_patterns(fmt, sat, scale):
    src = np.arange(1 << 16, dtype=np.uint16)
    name = f"skl_cvt_{'sat_' if sat else ''}bf16_{fmt}"
    a = np.zeros(src.size, np.uint8)
    getattr(oracle(), name + "_oracle")(a, src, scale, src.size)
    # same thing through the f32 routine on the widened values
    widened = support.bf16_bits_to_f32(src)
    assert np.array_equal(a, encode_array(fmt, widened, sat, scale))
    if ref() is not None:
        b = np.zeros(src.size, np.uint8)
        getattr(ref(), name + "_ref")(b, src, scale, src.size)
        assert np.array_equal(a, b)


@pytest.mark.parametrize("fmt", FMTS)
def test_cvt_f8_to_bf16(fmt):
    src = np.arange(256, dtype=np.uint8)   # test/cvt/cvt_f8_bf16.h:50-52: sequential bytes
    a = np.zeros(256, np.uint16)
    getattr(oracle(), f"skl_cvt_{fmt}_bf16_oracle")(a, src, 256)
    table = decode_table(fmt)
    for code in range(256):
        if np.isnan(table[code]):
            assert a[code] == 0x7FC0
        else:
            assert support.bf16_bits_to_f32(a[code:code + 1])[0] == np.float32(table[code])
    if ref() is not None:
        b = np.zeros(256, np.uint16)
        getattr(ref(), f"skl_cvt_{fmt}_bf16_ref")(b, src, 256)
        assert np.array_equal(a, b)


@pytest.mark.parametrize("n", (0, 1, 2, 7, 511, 512))
def test_cvt_f4_to_f8(n):
    src = np.arange(256, dtype=np.uint8)   # test/cvt/cvt_f4_f8.h:45-47
    a = np.full(n + 4, 0xAA, np.uint8)
    oracle().skl_cvt_f4e2m1_f8e4m3_oracle(a, src, n)
    e4 = decode_table("f8e4m3")
    want = [0, .5, 1, 1.5, 2, 3, 4, 6]
    for i in range(n):
        nib = (src[i // 2] >> 4) if i % 2 else (src[i // 2] & 0xF)
        v = e4[a[i]]
        assert abs(v) == want[nib & 7] and bool(a[i] & 0x80) == bool(nib & 8)
    assert np.all(a[n:] == 0xAA)
    if ref() is not None:
        b = np.full(n + 4, 0xAA, np.uint8)
        ref().skl_cvt_f4e2m1_f8e4m3_ref(b, src, n)
        assert np.array_equal(a, b)
