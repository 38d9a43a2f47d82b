"""Pins the CPU checker's GEMMs: integer results against numpy's exact integer
matmul, blocked == strided, the K-packed form, exactly-summable fp inputs that
fix the result under any summation order, the fp64 bound, and bit-equality
with the reference's own library on the reference's test tables.
"""
import numpy as np
import pytest

import support
from support import (GemmCase, colmajor_a_case, dot4_case, oracle, panel_case, ref, rowmajor_case,
                     run_oracle_gemm)


def ref_gemm(case, a, b, c):
    out = c.copy()
    getattr(ref(), case.stem() + "_ref")(*case.rcprc_args(a, b, out))
    return out


def int_expect(case, a, b, c):
    A, B, C, oc = case.dense(a, b, c)
    acc = (A.astype(np.int64) @ B.astype(np.int64))
    val = (case.beta * C.astype(np.int64) + case.alpha * acc)
    out = c.copy()
    if oc.size:
        out[oc.ravel()] = (val & 0xFFFFFFFF).astype(np.uint32).view(np.int32).ravel()
    return out


def rvv_cases(path, ta):
    out = []
    for r in support.table_rows(path, ("TEST", "BENCH")):
        out.append(rowmajor_case(ta, r["m1"], r["n1"], r["k1"], r.get("alpha", 0), r.get("beta", 0),
                                 r.get("rsa1"), r.get("rsb1"), r.get("rsc1")))
    return out


def xsfmm_c_cases(path, ta, max_k=64):
    out = []
    for r in support.table_rows(path, ("TEST", "BENCH")):
        k = min(r["k1"], max_k) if r["kind"] == "BENCH" else r["k1"]
        out.append(colmajor_a_case(ta, r["m1"], r["n1"], k, r.get("alpha", 0), r.get("beta", 0),
                                   r.get("csa1"), r.get("rsb1"), r.get("rsc1")))
    return out


def panel_cases(path, ta, stride=1, max_k=64):
    rows = support.table_rows(path, ("TEST", "BENCH"))
    out = []
    for r in rows[::stride]:
        k = min(r["k1"], max_k) if r["kind"] == "BENCH" else r["k1"]
        out.append(panel_case(ta, r["m1"], r["n1"], k, r.get("alpha", 0), r.get("beta", 0),
                              r.get("csa1", 0), r.get("rsa1", 0), r.get("rsb1", 0), r.get("csb1", 0),
                              r.get("rsc0", 0), r.get("csc0", 0), r.get("rsc1", 0), r.get("csc1", 0)))
    return out


def dot4_cases():
    out = []
    for r in support.table_rows("test/gemm/xsfvqdotq/skl_gemm_i8rcp1x4_i8p4x1c_i32_xsfvqdotq.c", ("TEST", "BENCH")):
        out.append(dot4_case(r["m1"], r["n1"], r["k1"], r.get("alpha", 0), r.get("beta", 0), r.get("rsa1", 0),
                             r.get("csa1", 0), r.get("rsb1", 0), r.get("rsc1", 0)))
    return out


INT_CASES = (rvv_cases("test/gemm/rvv/skl_gemm_i8_i8_i32_zve32x_x390.c", "i8") +
             xsfmm_c_cases("test/gemm/xsfmm/skl_gemm_i8c_i8_i32_xsfmm32a8i.c", "i8") +
             panel_cases("test/gemm/xsfmm/skl_gemm_i8rcptex1c_i8rcp1xte_i32rcptexterc_xsfmm32a8i.c", "i8", stride=9) +
             dot4_cases())


def test_int8_against_exact_integer_matmul():
    for idx, case in enumerate(INT_CASES):
        a, b, c = case.make_inputs(100 + idx)
        got = run_oracle_gemm(case, a, b, c)
        assert np.array_equal(got, int_expect(case, a, b, c)), vars(case)
        if ref() is not None:
            assert np.array_equal(got, ref_gemm(case, a, b, c)), vars(case)


def test_int8_config1_shape():
    # benchmark configuration 1: 512^3 row-major, alpha = 1, beta = 0, C = 0
    case = rowmajor_case("i8", 512, 512, 512, 1, 0)
    a, b, c = case.make_inputs(0x5EED0000)
    c[:] = 0
    got = run_oracle_gemm(case, a, b, c)
    want = (a.reshape(512, 512).astype(np.int32) @ b.reshape(512, 512).astype(np.int32))
    assert np.array_equal(got.reshape(512, 512), want)


def test_int32_wraparound_in_epilogue():
    case = rowmajor_case("i8", 3, 5, 8, alpha=0x7FFFFFF, beta=-0x12345678)
    a, b, c = case.make_inputs(9)
    c[:] = np.random.default_rng(2).integers(-2 ** 31, 2 ** 31, size=c.size)
    assert np.array_equal(run_oracle_gemm(case, a, b, c), int_expect(case, a, b, c))


def test_blocked_equals_strided():
    # packed API with 1x1x1 blocks is the strided API (src/gemm/packed-gemm.md:77)
    rng = np.random.default_rng(4)
    m, n, k = 9, 11, 13
    for ta in ("i8", "bf16", "f16", "f8e4m3", "f8e5m2"):
        case = GemmCase(ta, None, 2, 3, m0=1, n0=1, k0=1, m1=m, n1=n, k1=k, rsa0=0, csa0=0, rsa1=k + 2, csa1=1,
                        rsb0=0, csb0=0, rsb1=1, csb1=k + 1, rsc0=0, csc0=0, rsc1=2, csc1=2 * m + 3)
        a, b, c = case.make_inputs(int(rng.integers(1 << 30)))
        blocked = run_oracle_gemm(case, a, b, c)
        strided = c.copy()
        rc_name = case.stem().replace("rcprc", "rc") + "_oracle"
        getattr(oracle(), rc_name)(m, n, k, case.alpha, a, case.rsa1, case.csa1, b, case.rsb1, case.csb1,
                                   case.beta, strided, case.rsc1, case.csc1)
        assert np.array_equal(blocked.view(np.uint32), strided.view(np.uint32)), ta


FP_SUITES = {
    "bf16": ("test/gemm/rvv/skl_gemm_bf16_bf16_f32_zvfbfwma_x390.c", "test/gemm/xsfmm/skl_gemm_bf16c_bf16_f32_xsfmm32a16f.c",
             "test/gemm/xsfmm/skl_gemm_bf16rcptex1c_bf16rcp1xte_f32rcptexterc_xsfmm32a16f.c"),
    "f16": ("test/gemm/rvv/skl_gemm_f16_f16_f32_zvfh_x390.c", "test/gemm/xsfmm/skl_gemm_f16c_f16_f32_xsfmm32a16f.c",
            "test/gemm/xsfmm/skl_gemm_f16rcptex1c_f16rcp1xte_f32rcptexterc_xsfmm32a16f.c"),
    "f8e4m3": (None, "test/gemm/xsfmm/skl_gemm_f8e4m3c_f8e4m3_f32_xsfmm32a8f.c",
               "test/gemm/xsfmm/skl_gemm_f8e4m3rcptex1c_f8e4m3rcp1xte_f32rcptexterc_xsfmm32a8f.c"),
    "f8e5m2": (None, "test/gemm/xsfmm/skl_gemm_f8e5m2c_f8e5m2_f32_xsfmm32a8f.c",
               "test/gemm/xsfmm/skl_gemm_f8e5m2rcptex1c_f8e5m2rcp1xte_f32rcptexterc_xsfmm32a8f.c"),
    "f32": ("test/gemm/rvv/skl_gemm_f32_f32_f32_zve32f_x390.c", "test/gemm/xsfmm/skl_gemm_f32c_f32_f32_xsfmm32a32f.c",
            "test/gemm/xsfmm/skl_gemm_f32rcptex1c_f32rcp1xte_f32rcptexterc_xsfmm32a32f.c"),
    "f64": ("test/gemm/rvv/skl_gemm_f64_f64_f64_zve64d_x390.c", None, None),
    "f16h": ("test/gemm/rvv/skl_gemm_f16_f16_f16_zvfh_x390.c", None, None),  # f16 accumulator and C
}


def fp_cases(ta, panel_stride=17):
    rvv, xc, xp = FP_SUITES[ta]
    cases = []
    if rvv:
        cases += rvv_cases(rvv, ta)
    if xc:
        cases += xsfmm_c_cases(xc, ta)
    if xp:
        cases += panel_cases(xp, ta, stride=panel_stride)
    return cases


@pytest.mark.parametrize("ta", list(FP_SUITES))
def test_fp_within_reference_bound_and_equal_to_reference(ta):
    for idx, case in enumerate(fp_cases(ta)):
        a, b, c = case.make_inputs(500 + idx)
        got = run_oracle_gemm(case, a, b, c)
        # (the 1e-3 Frobenius target is stated for fp32 accumulation; a half accumulator has the bound only)
        support.assert_fp_gemm_close(case, a, b, c, got, frob_tol=None if ta == "f16h" else 1e-3)
        if ref() is not None:
            want = ref_gemm(case, a, b, c)
            assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), vars(case)


@pytest.mark.parametrize("ta", list(FP_SUITES))
def test_fp_exactly_summable_inputs(ta):
    """Small integers / powers of two: every partial sum is exact in fp32, so the
    result is fixed by the mathematics whatever the summation order."""
    rng = np.random.default_rng(21)
    m, n, k = 17, 19, 40
    vals = np.array([-2.0, -1.0, -0.5, 0.0, 0.5, 1.0, 2.0, 4.0])
    if ta == "f16h":  # partial sums must be exact in half precision too
        vals = np.array([-1.0, -0.5, 0.0, 0.5, 1.0, 2.0])
    A = rng.choice(vals, size=(m, k))
    B = rng.choice(vals, size=(k, n))
    C = rng.integers(-8, 9, size=(m, n)).astype(np.float64)

    def enc(x):
        x32 = x.astype(np.float32)
        if ta == "bf16":
            return support.f32_to_bf16_bits(x32)
        if ta in ("f16", "f16h"):
            return x32.astype(np.float16).view(np.uint16)
        if ta in ("f32", "f64"):
            return x.astype(support.ETYPES[ta].dtype)
        out = np.zeros(x32.size, np.uint8)
        getattr(oracle(), f"skl_cvt_f32_{ta}_oracle")(out, x32.ravel(), 1.0, x32.size)
        return out.reshape(x.shape)

    case = rowmajor_case(ta, m, n, k, alpha=2.0, beta=-3.0)
    a, b, c = enc(A).ravel(), enc(B).ravel(), C.astype(case.cdtype).ravel()
    got = run_oracle_gemm(case, a, b, c).reshape(m, n)
    assert np.array_equal(got, (2.0 * (A @ B) - 3.0 * C).astype(case.cdtype))


def test_mixed_fp8_equals_decode_then_f32_gemm():
    m, n, k = 13, 21, 37
    rng = np.random.default_rng(8)
    a = rng.integers(8, 127, size=m * k, dtype=np.uint8)
    b = rng.integers(4, 124, size=k * n, dtype=np.uint8)
    c0 = rng.uniform(-1, 1, m * n).astype(np.float32)
    got = c0.copy()
    oracle().skl_gemm_f8e4m3rc_f8e5m2rc_f32rc_oracle(m, n, k, 1.5, a, k, 1, b, n, 1, 0.5, got, n, 1)
    af = support.decode_table("f8e4m3")[a].astype(np.float32)
    bf = support.decode_table("f8e5m2")[b].astype(np.float32)
    want = c0.copy()
    oracle().skl_gemm_f32rc_f32rc_f32rc_oracle(m, n, k, 1.5, af, k, 1, bf, n, 1, 0.5, want, n, 1)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    if ref() is not None:
        want2 = c0.copy()
        ref().skl_gemm_f32rc_f32rc_f32rc_ref(m, n, k, 1.5, af, k, 1, bf, n, 1, 0.5, want2, n, 1)
        assert np.array_equal(got.view(np.uint32), want2.view(np.uint32))


def test_f64_helper_matches_numpy_and_reference():
    m, n, k = 7, 9, 33
    rng = np.random.default_rng(12)
    A, B, C = rng.normal(size=(m, k)), rng.normal(size=(k, n)), rng.normal(size=(m, n))
    got = C.copy().ravel()
    oracle().skl_gemm_f64rc_f64rc_f64rc_oracle(m, n, k, 1.25, A.ravel(), k, 1, B.ravel(), n, 1, -0.5, got, n, 1)
    assert np.allclose(got.reshape(m, n), 1.25 * A @ B - 0.5 * C, rtol=1e-13, atol=1e-13)
    if ref() is not None:
        want = C.copy().ravel()
        ref().skl_gemm_f64rc_f64rc_f64rc_ref(m, n, k, 1.25, A.ravel(), k, 1, B.ravel(), n, 1, -0.5, want, n, 1)
        assert np.array_equal(got, want)


def test_f32_to_f16_rounding_matches_numpy():
    """The half rounding the f16 -> f16 GEMM restatement is built on, against numpy's float16
    conversion (round to nearest even, subnormals, overflow to infinity): random patterns plus every
    pattern around the zero / subnormal, subnormal / normal and overflow thresholds."""
    import ctypes
    f = oracle().cdll.skl_oracle_f32_to_f16
    f.argtypes, f.restype = [ctypes.c_float], ctypes.c_uint16
    rng = np.random.default_rng(5)
    bits = np.concatenate([rng.integers(0, 1 << 32, 60000, dtype=np.uint64).astype(np.uint32),
                           np.arange(0x33000000 - 64, 0x33000000 + 64, dtype=np.uint32),
                           np.arange(0x38800000 - 9000, 0x38800000 + 9000, dtype=np.uint32),
                           np.arange(0x477FE000 - 9000, 0x477FE000 + 9000, dtype=np.uint32),
                           np.arange(0x3F800000, 0x3F800000 + 20000, dtype=np.uint32)])
    bits = np.concatenate([bits, bits | np.uint32(0x80000000)])
    x = bits.view(np.float32)
    x = x[~np.isnan(x)]
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    got = np.fromiter((f(float(v)) for v in x), dtype=np.uint16, count=x.size)
    assert np.array_equal(got, want)


FUSED_TYPES = ("i8", "bf16", "f16", "f8e4m3", "f8e5m2")


FP8_COPY_FORMATS = {1: "skl_cvt_f32_f8e4m3_oracle", 2: "skl_cvt_sat_f32_f8e4m3_oracle",
                    3: "skl_cvt_f32_f8e5m2_oracle", 4: "skl_cvt_sat_f32_f8e5m2_oracle"}   # q_format -> the conversion it fuses


def requantised(v, scale, zero, fmt=0):
    """clamp(rne((float)v * s) + zero, -128, 127) of include/skl-gfx950.h, in numpy and by another route than the
    checker's C: the product of two fp32 values is exact in fp64, so rounding it to fp32 once is the one fp32
    multiplication; np.rint rounds ties to even; a NaN counts as 0, values beyond int32 as its ends.
    With an fp8 `fmt` the bytes are the checker's fp32 -> fp8 conversion (pinned to the reference's vectors in
    test_oracle_cvt.py) of that same product (its own factor 1 changes nothing)."""
    with np.errstate(invalid="ignore", over="ignore"):
        prod = (np.asarray(v).astype(np.float32).astype(np.float64) * np.asarray(scale, np.float32).astype(np.float64)
                ).astype(np.float32)
        if fmt:
            flat = np.ascontiguousarray(prod).ravel()
            out = np.empty(flat.size, np.uint8)
            getattr(oracle(), FP8_COPY_FORMATS[fmt])(out, flat, 1.0, flat.size)
            return out.view(np.int8).reshape(prod.shape)
        r = np.rint(prod.astype(np.float64))
    r = np.where(np.isnan(r), 0.0, np.clip(r, -2147483648.0, 2147483647.0))
    return np.clip(r.astype(np.int64) + int(zero), -128, 127).astype(np.int8)


def fused_expectation(case, plain, bias, max_in, activation=0, requant=None):
    """C and *max after the fused steps, from the plain GEMM's result: the bias of the logical column
    added in C's arithmetic (one fp32 addition / int32 wrap), the activation, the maximum over what was
    written. With `requant` = dict(q=<int8 buffer before the call>, rsq, csq, scale=<1 or n floats>,
    per_column, zero, only, format) a third value follows: the int8 buffer afterwards (and C stays `plain`'s
    memory where `only` says it is not written)."""
    oc = support.blocked_offsets(case.m1, case.n1, case.m0, case.n0, case.rsc0, case.csc0, case.rsc1, case.csc1)
    want = plain.copy()
    if bias is not None:
        with np.errstate(over="ignore"):
            want[oc] = (plain[oc] + bias[None, :]).astype(plain.dtype)
    if activation == 1:
        v = want[oc]
        want[oc] = np.where(v > 0, v, 0).astype(plain.dtype)
    elif activation in (2, 3):
        want[oc] = support.activation_reference(want[oc], activation)
    top = None
    if max_in is not None:
        written = want[oc]
        with np.errstate(invalid="ignore"):
            best = written[written > max_in[0]]
        top = np.array([best.max() if best.size else max_in[0]], dtype=plain.dtype)
    if requant is None:
        return want, top
    m, n = oc.shape
    q = requant["q"].copy()
    scale = requant["scale"][None, :] if requant.get("per_column") else requant["scale"][0]
    oq = np.arange(m)[:, None] * requant["rsq"] + np.arange(n)[None, :] * requant["csq"]
    values = want[oc]
    if requant.get("only") and case.beta == 0 and not case.is_int:
        values = np.where(values == 0, np.float32(0.0), values)   # C is not read then: an exact zero is +0 (include/skl-gfx950.h)
    q[oq] = requantised(values, scale, requant.get("zero", 0), requant.get("format", 0))
    return want, top, q


@pytest.mark.parametrize("ta", FUSED_TYPES)
def test_fused_steps_follow_the_plain_gemm(ta):
    """Bias and maximum (src/gemm/fused-kernel-API.md:159-207) behind the alpha/beta step, checked
    against the plain restatement plus numpy: strided and blocked forms, each step alone and both."""
    rng = np.random.default_rng(31)
    cases = (rowmajor_case(ta, 9, 14, 21, alpha=2, beta=3),
             GemmCase(ta, None, 1, 0, m0=3, n0=4, k0=5, m1=5, n1=3, k1=4, rsa0=5, csa0=1, rsa1=100, csa1=15,
                      rsb0=4, csb0=1, rsb1=20, csb1=90, rsc0=1, csc0=3, rsc1=12, csc1=64))
    for case in cases:
        a, b, c = case.make_inputs(int(rng.integers(1 << 30)))
        n = case.n0 * case.n1
        plain = run_oracle_gemm(case, a, b, c)
        if case.is_int:
            bias = rng.integers(-1 << 20, 1 << 20, n).astype(np.int32)
            low = np.array([-(1 << 31)], np.int32)
        else:
            bias = rng.uniform(-4, 4, n).astype(np.float32)
            low = np.array([-np.inf], np.float32)
        blocked = not (case.m0 == case.n0 == case.k0 == 1)
        name = "skl_gemm_fused_" + (case.stem() if blocked else case.stem().replace("rcprc", "rc"))[len("skl_gemm_"):] + "_oracle"
        args = case.rcprc_args if blocked else (lambda a_, b_, c_: (case.m1, case.n1, case.k1, case.alpha, a_, case.rsa1,
                                                                  case.csa1, b_, case.rsb1, case.csb1, case.beta,
                                                                  c_, case.rsc1, case.csc1))
        for use_bias, use_max in ((True, True), (True, False), (False, True), (False, False)):
            for start in (low, None if not use_max else np.array([1 << 30 if case.is_int else 1e30], low.dtype)):
                if start is None:
                    continue
                got, mx = c.copy(), start.copy()
                getattr(oracle(), name)(*args(a, b, got), bias if use_bias else None, mx if use_max else None)
                want, top = fused_expectation(case, plain, bias if use_bias else None, start if use_max else None)
                assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), (ta, blocked, use_bias, use_max)
                if use_max:
                    assert mx[0] == top[0], (ta, blocked, use_bias)
                else:
                    assert mx[0] == start[0]


def test_ofp4_gemm_is_the_conversion_followed_by_the_fp8_gemm():
    """The checker's GEMM over OFP4 weights (oracle/skl_oracle.c: the reference's conversion, ref/cvt/cvt_ofp4.c:59-68,
    then its fp8 GEMM) against the same GEMM on a B converted by the format's value table in numpy: bit for bit, odd
    and even column distances, ragged everything; and against the exact product where every sum is exact."""
    import ofp4_support as f4
    o = oracle()
    # the table itself: the checker's conversion of all 16 codes, and their values
    got = np.zeros(16, np.uint8)
    o.skl_cvt_f4e2m1_f8e4m3_oracle(got, f4.pack_nibbles(np.arange(16)), 16)
    assert np.array_equal(got, f4.E2M1_AS_E4M3)
    assert np.array_equal(support.decode_table("f8e4m3")[f4.E2M1_AS_E4M3], f4.E2M1_VALUES)
    for i, (m, n, k, ldb, alpha, beta) in enumerate(((3, 5, 7, 7, 1.0, 0.0), (4, 6, 33, 40, 1.5, -0.5), (1, 9, 64, 65, 2.0, 1.0),
                                                     (17, 3, 100, 101, 1.0, 0.0), (2, 2, 0, 4, 3.0, 2.0))):
        case, a, b4, b8, c = f4.make_problem(50 + i, m, n, k, ldb, alpha, beta, rsa=k + 3, rsc=n + 2)
        got = c.copy()
        o.skl_gemm_f8e4m3rc_f4e2m1c_f32rc_oracle(m, n, k, alpha, a, case.rsa1, 1, b4, ldb, beta, got, case.rsc1, 1)
        want = run_oracle_gemm(case, a, b8, c)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (m, n, k, ldb)
        if k:
            support.assert_fp_gemm_close(case, a, b8, c, got)
    # exact sums: A in {1, 2, 4}, K = 64: every partial sum is a small multiple of 0.5
    m, n, k = 5, 11, 64
    rng = np.random.default_rng(3)
    a = rng.choice(np.array([0x38, 0x40, 0x48], np.uint8), m * k)
    codes = rng.integers(0, 16, n * k, dtype=np.uint8)
    got = np.zeros(m * n, np.float32)
    o.skl_gemm_f8e4m3rc_f4e2m1c_f32rc_oracle(m, n, k, 1.0, a, k, 1, f4.pack_nibbles(codes), k, 0.0, got, n, 1)
    A = support.decode_table("f8e4m3")[a].reshape(m, k)
    B = f4.E2M1_VALUES[codes].reshape(n, k).T
    assert np.array_equal(got.reshape(m, n).astype(np.float64), A @ B)


def test_mx_scaled_ofp4_gemm_definition():
    """The checker's GEMM over MXFP4 weights (oracle/skl_oracle.c): with every scale 2^0, or none, it is the
    unscaled routine bit for bit (which is pinned against the reference's conversion + fp8 GEMM above); raising
    every scale by one doubles every sum exactly; the result lies inside the reference's fp32-accumulation bound around
    the exact product of the decoded, scaled operands; exact where the sums are."""
    import ofp4_support as f4
    o = oracle()
    for i, (m, n, k, ldb) in enumerate(((3, 5, 70, 71), (4, 6, 64, 64), (2, 9, 200, 224), (1, 3, 31, 40))):
        case, a, b4, b8, scales, lds, c = f4.make_mx_problem(90 + i, m, n, k, ldb, 1.5, -0.5, rsa=k + 3, rsc=n + 2)
        plain, unit, none = c.copy(), c.copy(), c.copy()
        o.skl_gemm_f8e4m3rc_f4e2m1c_f32rc_oracle(m, n, k, 1.5, a, case.rsa1, 1, b4, ldb, -0.5, plain, case.rsc1, 1)
        o.skl_gemm_f8e4m3rc_mxf4e2m1c_f32rc_oracle(m, n, k, 1.5, a, case.rsa1, 1, b4, ldb, np.full_like(scales, 127), lds, -0.5, unit, case.rsc1, 1)
        o.skl_gemm_f8e4m3rc_mxf4e2m1c_f32rc_oracle(m, n, k, 1.5, a, case.rsa1, 1, b4, ldb, None, 0, -0.5, none, case.rsc1, 1)
        assert np.array_equal(plain.view(np.uint32), unit.view(np.uint32)) and np.array_equal(plain.view(np.uint32), none.view(np.uint32))
        got, twice = np.zeros_like(c), np.zeros_like(c)
        o.skl_gemm_f8e4m3rc_mxf4e2m1c_f32rc_oracle(m, n, k, 1.0, a, case.rsa1, 1, b4, ldb, scales, lds, 0.0, got, case.rsc1, 1)
        o.skl_gemm_f8e4m3rc_mxf4e2m1c_f32rc_oracle(m, n, k, 1.0, a, case.rsa1, 1, b4, ldb, scales + 1, lds, 0.0, twice, case.rsc1, 1)
        assert np.array_equal(twice, 2 * got)
        scaled = c.copy()
        o.skl_gemm_f8e4m3rc_mxf4e2m1c_f32rc_oracle(m, n, k, 1.5, a, case.rsa1, 1, b4, ldb, scales, lds, -0.5, scaled, case.rsc1, 1)
        exact, bound, oc = f4.mx_bound(case, a, b8, scales, lds, c, m, n, k, ldb)
        assert np.all(np.abs(scaled[oc] - exact) <= bound + np.abs(exact) * 2.0 ** -22)
    # exact sums: A in {1, 2, 4}, scales 2^-2 .. 2^2, K = 64
    m, n, k = 5, 11, 64
    rng = np.random.default_rng(4)
    a = rng.choice(np.array([0x38, 0x40, 0x48], np.uint8), m * k)
    codes = rng.integers(0, 16, n * k, dtype=np.uint8)
    scales = rng.integers(125, 130, size=n * 2, dtype=np.uint8)
    got = np.zeros(m * n, np.float32)
    o.skl_gemm_f8e4m3rc_mxf4e2m1c_f32rc_oracle(m, n, k, 1.0, a, k, 1, f4.pack_nibbles(codes), k, scales, 2, 0.0, got, n, 1)
    A = support.decode_table("f8e4m3")[a].reshape(m, k)
    S = np.ldexp(1.0, scales.reshape(n, 2).astype(np.int64) - 127).repeat(32, axis=1)
    B = (f4.E2M1_VALUES[codes].reshape(n, k) * S).T
    assert np.array_equal(got.reshape(m, n).astype(np.float64), A @ B)


def test_silu_and_gelu_restate_the_reference():
    """The checker's SiLU and GELU (oracle/skl_oracle.c) against the reference's own routines compiled from
    ref/sigmoid/sigmoid_f32.c and ref/gelu/gelu_f32.c - bit for bit over the ranges of the reference's tests and the
    special values - and, independently, against the closed forms in fp64 (scipy) and the identity f(x) - f(-x) = x."""
    from scipy import special
    rng = np.random.default_rng(12)
    x = np.concatenate([rng.uniform(-110, 18, 100000), rng.uniform(-3, 3, 50000), rng.uniform(-15, 6, 50000)]).astype(np.float32)
    x = np.concatenate([x, np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1e-40, -1e-40, -103.5, -88.7, 88.8, 3e38], np.float32)])
    ref = support.ref()
    for act, name in ((2, "skl_silu_f32_ref"), (3, "skl_gelu_f32_ref")):
        got = support.activation_reference(x, act)
        if ref is not None and hasattr(ref, name):
            want = np.zeros_like(x)
            getattr(ref, name)(want, x, x.size)
            same = (got.view(np.uint32) == want.view(np.uint32)) | (np.isnan(got) & np.isnan(want))  # a NaN's sign is the compiler's
            assert same.all(), name
        xd = x[:-11].astype(np.float64)
        with np.errstate(over="ignore"):
            closed = xd / (1 + np.exp(-xd)) if act == 2 else 0.5 * xd * special.erfc(-xd / np.sqrt(2))
        assert support.ulp_error_f32(got[:-11], closed.astype(np.float32)).max() <= 1.0, name
        pos = np.abs(x[:1000])
        diff = support.activation_reference(pos, act).astype(np.float64) - support.activation_reference(-pos, act).astype(np.float64)
        assert np.allclose(diff, pos, rtol=1e-6, atol=1e-30), name
    assert support.activation_reference(np.array([0.0, -0.0], np.float32), 2).tolist() == [0.0, -0.0]
    assert support.activation_reference(np.array([0.0], np.float32), 3)[0] == 0.0


def test_requantisation_rule_on_worked_values():
    """The checker's requantisation and activation (oracle/skl_oracle.c, skl_oracle_act_requant_*) against values
    worked by hand from the rule in include/skl-gfx950.h - ties go to the even integer, the zero point is added
    after rounding, both ends saturate, an int32 is rounded to fp32 before it is scaled, a NaN counts as 0 - and
    against the numpy formulation above on random values, per-call and per-column scales, strided Q."""
    o = oracle()
    half = np.array([0.5], np.float32)

    def run(values, scale, zero=0, act=0, per_column=0, suffix="f32"):
        c = np.array(values, np.float32 if suffix == "f32" else np.int32).reshape(1, -1)
        q = np.full(c.size, 99, np.int8)
        getattr(o, "skl_oracle_act_requant_" + suffix)(1, c.size, c, c.size, 1, act, q, c.size, 1,
                                                       np.asarray(scale, np.float32), per_column, zero)
        return c[0], q

    # x * 0.5 = 0.5, 1.5, 2.5, 3.5, -0.5, -1.5, -2.5: ties to even
    assert list(run([1, 3, 5, 7, -1, -3, -5], half)[1]) == [0, 2, 2, 4, 0, -2, -2]
    assert list(run([1, 3, 5, 7, -1, -3, -5], half, suffix="i32")[1]) == [0, 2, 2, 4, 0, -2, -2]
    # the zero point is added after rounding, and the sum saturates: 2.5 -> 2 (+3 = 5); 300 -> 127; -300 -> -128
    assert list(run([5, 600, -600, 250], half, zero=3)[1]) == [5, 127, -128, 127]
    assert list(run([250, 252, -260], half, zero=-3)[1]) == [122, 123, -128]
    # NaN -> 0 (+ zero); infinities and values beyond int32 end at the ends of int8 whatever the zero point
    assert list(run([np.nan, np.inf, -np.inf, 3e38, -3e38, 4e9, -4e9], [1.0], zero=-128)[1]) == [-128, 127, -128, 127, -128, 127, -128]
    assert list(run([np.nan, -4e9], [1.0], zero=127)[1]) == [127, -128]
    # int32 -> fp32 rounds to nearest even before the product: 2^24 + 1 -> 2^24, 2^24 + 3 -> 2^24 + 4;
    # times 2^-20: 16 and 16.000004 -> 16
    assert list(run([(1 << 24) + 1, (1 << 24) + 3, 100 << 20, -(101 << 20)], [2.0 ** -20], suffix="i32")[1]) == [16, 16, 100, -101]
    # relu before the requantisation, and written back to C; a NaN becomes 0
    c, q = run([-4.0, 6.0, np.nan, -0.0], [1.0], act=1)
    assert list(q) == [0, 6, 0, 0] and list(c[:2]) == [0.0, 6.0] and c[2] == 0.0 and c[3] == 0.0
    c, q = run([-7, 9], [1.0], act=1, suffix="i32")
    assert list(c) == [0, 9] and list(q) == [0, 9]
    # per-column scales
    assert list(run([10, 10, 10], [1.0, 0.25, 3.0], per_column=1)[1]) == [10, 2, 30]

    rng = np.random.default_rng(77)
    for suffix, dt in (("i32", np.int32), ("f32", np.float32)):
        for per_column in (0, 1):
            m, n, rsc, rsq, csq = 13, 29, 31, 3, 47
            if dt is np.int32:
                c = rng.integers(-1 << 31, 1 << 31, m * rsc, dtype=np.int64).astype(np.int32)
                scale = (rng.uniform(0.5, 2.0, n) * 2.0 ** rng.integers(-30, -20, n)).astype(np.float32)
            else:
                c = (rng.standard_normal(m * rsc) * 300).astype(np.float32)
                scale = rng.uniform(0.01, 2.0, n).astype(np.float32)
            c[::17] = (c[::17] // 2) * 2  # some exact ties with a scale of 0.5
            if not per_column:
                scale = scale[:1]
            for act in (0, 1):
                for zero in (0, -128, 127, 5):
                    got_c, q = c.copy(), np.full(m * rsq + n * csq, 77, np.int8)
                    getattr(o, "skl_oracle_act_requant_" + suffix)(m, n, got_c, rsc, 1, act, q, rsq, csq, scale,
                                                                   per_column, zero)
                    oc = np.arange(m)[:, None] * rsc + np.arange(n)[None, :]
                    want_c = c.copy()
                    if act:
                        want_c[oc] = np.where(c[oc] > 0, c[oc], 0)
                    assert np.array_equal(got_c, want_c)
                    want_q = np.full(m * rsq + n * csq, 77, np.int8)
                    oq = np.arange(m)[:, None] * rsq + np.arange(n)[None, :] * csq
                    want_q[oq] = requantised(want_c[oc], scale[None, :] if per_column else scale[0], zero)
                    assert np.array_equal(q, want_q), (suffix, per_column, act, zero)


def test_fp8_copy_rule_on_worked_values():
    """The fp8 forms of the 8-bit copy (q_format of include/skl-gfx950.h) as this file's tests expect them: worked
    codes for both formats - exact values, the tie at the largest value (E4M3: 464 stays 448, its last bit is even;
    E5M2: 61440 goes up and overflows), what lies beyond with and without saturation (E4M3's NaN carries no sign,
    ref/cvt/cvt_ofp8.c:97-107), the smallest subnormal - and the product taken once in fp32 before the conversion
    equal to the conversion given the scale itself."""
    def codes(values, scale, fmt):
        return list(requantised(np.array(values, np.float32), np.float32(scale), 0, fmt).view(np.uint8))

    assert codes([1.0, 448.0, 464.0, 465.0, -500.0, 2.0 ** -9, -0.0], 1.0, 1) == [0x38, 0x7E, 0x7E, 0x7F, 0x7F, 0x01, 0x80]
    assert codes([1.0, 448.0, 464.0, 465.0, -500.0, 2.0 ** -9, -0.0], 1.0, 2) == [0x38, 0x7E, 0x7E, 0x7E, 0xFE, 0x01, 0x80]
    assert codes([1.0, 57344.0, 61439.0, 61440.0, -70000.0, 2.0 ** -16], 1.0, 3) == [0x3C, 0x7B, 0x7B, 0x7C, 0xFC, 0x01]
    assert codes([1.0, 57344.0, 61439.0, 61440.0, -70000.0, 2.0 ** -16], 1.0, 4) == [0x3C, 0x7B, 0x7B, 0x7B, 0xFB, 0x01]
    assert codes([2.0, 928.0, 930.0], 0.5, 1) == [0x38, 0x7E, 0x7F]   # the scale is applied first
    rng = np.random.default_rng(8)
    v = (rng.standard_normal(20000) * np.exp2(rng.integers(-20, 18, 20000))).astype(np.float32)
    for fmt, name in FP8_COPY_FORMATS.items():
        for scale in (0.37, 3.0, 2.0 ** -7):
            direct = np.empty(v.size, np.uint8)
            getattr(oracle(), name)(direct, v, scale, v.size)
            assert np.array_equal(direct.view(np.int8), requantised(v, np.float32(scale), 0, fmt)), (fmt, scale)


def block4x8x4_case(m1, n1, k1, rsa1=None, rsb1=None, rsc1=None, accum=False):
    """The 4 x 8 by 8 x 4 block product of src/gemm/packed-gemm.md:270-298 as a blocked GEMM: "block dimensions
    m0 = 4, n0 = 4, k0 = 8; intra-block row strides rsa0 = 8, rsb0 = 4, rsc0 = 4; all intra-block column strides
    equal to 1", block-row-major with csa1 = 32, csb1 = 32, csc1 = 16."""
    return support.GemmCase("i8", None, 1, 1 if accum else 0, m0=4, n0=4, k0=8, m1=m1, n1=n1, k1=k1,
                            rsa0=8, csa0=1, rsa1=rsa1 if rsa1 is not None else 32 * k1, csa1=32,
                            rsb0=4, csb0=1, rsb1=rsb1 if rsb1 is not None else 32 * n1, csb1=32,
                            rsc0=4, csc0=1, rsc1=rsc1 if rsc1 is not None else 16 * n1, csc1=16)


def test_block4x8x4_layout_against_numpy_blocks():
    """Pins the checker on that layout without its own index arithmetic: the buffers reshaped into
    [block row][block column][row][column] arrays, the product formed block by block with numpy in 64 bits."""
    m1, n1, k1 = 5, 3, 4
    for accum in (False, True):
        case = block4x8x4_case(m1, n1, k1, accum=accum)
        a, b, c = case.make_inputs(77 + accum)
        got = support.run_oracle_gemm(case, a, b, c)
        A = a.astype(np.int64).reshape(m1, k1, 4, 8)
        B = b.astype(np.int64).reshape(k1, n1, 8, 4)
        want = np.einsum("ipak,pjkb->ijab", A, B) + (c.astype(np.int64).reshape(m1, n1, 4, 4) if accum else 0)
        assert np.array_equal(got.reshape(m1, n1, 4, 4), want.astype(np.int32))
