"""GPU parity of the GEMM entry points with the CPU checker.

Every row of the reference's gemm suites (tests/golden/ref_tables.json) is run
through the entry point the reference's suite calls, with inputs drawn as the
reference's harnesses draw them (int8 in [-128,127]; bf16/f16 in [-1,1]; fp8
bytes 8..126 / 4..123). Integer results must equal the checker bit for bit over
the whole C buffer (stride gaps included: the clobber check); floating-point
results must satisfy the reference's elementwise bound
2*((1+2^-24)^(K+2)-1)*(|alpha||A||B| + |beta||C|) and a relative Frobenius
error <= 1e-3 against the fp64 result. For fp8 operands the elementwise bound
is widened by 2^-10 * |alpha||A||B| (support.FP8_MFMA_REL): the fp8 matrix-core
instructions add the products of one instruction with about 12 bits below the
largest term, which the reference's fp32-accumulation bound does not allow for
at small K; the Frobenius bound is not relaxed."""
import numpy as np
import pytest

import skl_amd
import support
from gpu_support import MODES, run_fused_gemm, run_gemm
from support import colmajor_a_case, rowmajor_case, run_oracle_gemm
from test_oracle_gemm import FP_SUITES, dot4_cases, fused_expectation, panel_cases, rvv_cases, xsfmm_c_cases

pytestmark = pytest.mark.gpu


def check(gpu, kind, case, seed, mode):
    a, b, c = case.make_inputs(seed)
    got = run_gemm(gpu, kind, case, a, b, c, mode)
    if case.is_int or case.ta == "f16h":  # the half-accumulating GEMM is defined operation by operation
        want = run_oracle_gemm(case, a, b, c)
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), (kind, vars(case))
        if case.ta == "f16h":
            # Bit-identity holds against the reference as compiled for x86 (product in float, one rounding to half per
            # step); hardware with half arithmetic rounds the product too. What every evaluation must meet is the
            # reference test's own bound (P = 11, test/gemm/gemm_f16rcprc_f16rcprc_f16rcprc.c:157): applied as well.
            support.assert_fp_gemm_close(case, a, b, c, got, frob_tol=None)
    else:
        fp8 = case.ta.startswith("f8")
        support.assert_fp_gemm_close(case, a, b, c, got, extra_rel=support.FP8_MFMA_REL if fp8 else 0.0)


@pytest.mark.parametrize("mode", MODES)
def test_int8_rowmajor_table(gpu, mode):
    for path in ("test/gemm/rvv/skl_gemm_i8_i8_i32_zve32x.c", "test/gemm/rvv/skl_gemm_i8_i8_i32_zve32x_x390.c"):
        for i, case in enumerate(rvv_cases(path, "i8")):
            check(gpu, "rowmajor", case, 1000 + i, mode)


@pytest.mark.parametrize("mode", MODES)
def test_int8_colmajor_a_table(gpu, mode):
    for i, case in enumerate(xsfmm_c_cases("test/gemm/xsfmm/skl_gemm_i8c_i8_i32_xsfmm32a8i.c", "i8", max_k=8192)):
        check(gpu, "colmajor_a", case, 2000 + i, mode)


@pytest.mark.parametrize("mode", MODES)
def test_int8_panel_table(gpu, mode):
    path = "test/gemm/xsfmm/skl_gemm_i8rcptex1c_i8rcp1xte_i32rcptexterc_xsfmm32a8i.c"
    stride = 1 if mode == "device" else 5
    for i, case in enumerate(panel_cases(path, "i8", stride=stride, max_k=8192)):
        check(gpu, "panel", case, 3000 + i, mode)


@pytest.mark.parametrize("mode", MODES)
def test_int8_dot4_table(gpu, mode):
    for i, case in enumerate(dot4_cases()):
        check(gpu, "dot4", case, 4000 + i, mode)


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("ta", list(FP_SUITES))
def test_fp_tables(gpu, ta, mode):
    rvv, xc, xp = FP_SUITES[ta]
    seed = 5000
    if rvv:
        for path in (rvv, rvv.replace("_x390", "")):
            for case in rvv_cases(path, ta):
                seed += 1
                check(gpu, "rowmajor", case, seed, mode)
    for case in (xsfmm_c_cases(xc, ta, max_k=8192) if xc else ()):
        seed += 1
        check(gpu, "colmajor_a", case, seed, mode)
    stride = 1 if mode == "device" else 7
    for case in (panel_cases(xp, ta, stride=stride, max_k=8192) if xp else ()):
        seed += 1
        check(gpu, "panel", case, seed, mode)


@pytest.mark.parametrize("kind", ("rc", "rcprc"))
def test_general_strides(gpu, kind):
    """Column-major B and C, gapped strides, blocked layouts with k0 > 1: the
    layouts only the full-stride forms can express."""
    rng = np.random.default_rng(77)
    for ta in ("i8", "bf16", "f16", "f8e4m3", "f8e5m2", "f32", "f64", "f16h"):
        m, n, k = 37, 29, 53
        if kind == "rc":
            case = support.GemmCase(ta, None, 2, 3, m0=1, n0=1, k0=1, m1=m, n1=n, k1=k, rsa0=0, csa0=0,
                                    rsa1=k + 3, csa1=1, rsb0=0, csb0=0, rsb1=1, csb1=k + 5, rsc0=0, csc0=0,
                                    rsc1=2, csc1=2 * m + 1)
        else:
            case = support.GemmCase(ta, None, 2, 3, m0=3, n0=4, k0=5, m1=5, n1=3, k1=4, rsa0=5, csa0=1,
                                    rsa1=100, csa1=15, rsb0=4, csb0=1, rsb1=20, csb1=90, rsc0=1, csc0=3,
                                    rsc1=12, csc1=64)
        check(gpu, kind, case, int(rng.integers(1 << 30)), "device")
        check(gpu, kind, case, int(rng.integers(1 << 30)), "host")


@pytest.mark.parametrize("ta", ("i8", "bf16", "f8e4m3"))
def test_ragged_mid_size_bounds_checked_tiles(gpu, ta):
    """1000 x 1100 x 333 with gapped leading dimensions: 72 tiles of 128 x 128, none of them whole in
    every dimension (the small shapes of the tables run on 64 x 64 tiles, the aligned large ones on the
    streaming kernel)."""
    m, n, k = 1000, 1100, 336 if ta != "i8" else 333
    for a_kc in (True, False):
        case = (rowmajor_case(ta, m, n, k, 2, 1, rsa=k + 16 - k % 16 + 16, rsb=1104 + 16, rsc=1101) if a_kc else
                colmajor_a_case(ta, m, n, k, 2, 1, csa=1008, rsb=1104, rsc=1100))
        a, b, c = case.make_inputs(77 + a_kc)
        got = run_gemm(gpu, "rc", case, a, b, c, "device")
        A, B, C, oc = case.dense(a, b, c)
        exact = case.alpha * (A @ B) + case.beta * C
        if case.is_int:
            assert np.array_equal(got, run_oracle_gemm(case, a, b, c))
        else:
            rel = np.linalg.norm(got[oc] - exact) / np.linalg.norm(exact)
            assert rel <= 1e-3, rel
            support.assert_fp_gemm_close(case, a, b, c, got, extra_rel=support.FP8_MFMA_REL if ta.startswith("f8") else 0.0)


def test_f32_f64_bit_identical_to_the_checker(gpu):
    """The f32 and f64 contractions evaluate the reference's loop with a separately rounded multiply and add: for
    finite data the result equals the checker's (and the compiled reference's) bit for bit, stride gaps
    included. (A row-major case on the register-tiled kernel, a blocking only the any-stride kernel takes.)"""
    rng = np.random.default_rng(91)
    for ta in ("f32", "f64"):
        for case in (rowmajor_case(ta, 33, 47, 129, alpha=1.5, beta=-0.25, rsa=131, rsb=50, rsc=49),
                     support.GemmCase(ta, None, 2, 3, m0=3, n0=4, k0=5, m1=5, n1=3, k1=4, rsa0=5, csa0=1, rsa1=100,
                                      csa1=15, rsb0=4, csb0=1, rsb1=20, csb1=90, rsc0=1, csc0=3, rsc1=12, csc1=64)):
            a, b, c = case.make_inputs(int(rng.integers(1 << 30)))
            want = run_oracle_gemm(case, a, b, c)
            for mode in MODES:
                got = run_gemm(gpu, "rcprc", case, a, b, c, mode)
                assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), (ta, mode)


BETA_ZERO_SHAPES = (
    # ta, m, n, k, what serves it
    ("bf16", 130, 200, 64, "64 x 64 bounds-checked tiles"),
    ("f8e4m3", 256, 256, 128, "bounds-checked tiles"),
    ("f16", 512, 2048 + 128, 256, "streaming kernel"),
    ("bf16", 128, 256, 4096, "bounds-checked tiles with K shared between workgroups"),
    ("bf16", 256, 8192, 4096, "streaming kernel with K shared between two workgroups (too long for the checker)"),
    ("f32", 33, 47, 17, "any-stride kernel"),
    ("f32", 256, 192, 64, "register-tiled kernel"),
    ("f64", 20, 31, 9, "any-stride kernel"),
    ("f16h", 21, 30, 19, "any-stride kernel"),
    ("bf16", 1, 4096, 512, "M = 1, one workgroup per strip"),
    ("bf16", 1, 4096, 2048, "M = 1, four workgroups per strip"),
    ("f8e4m3", 1, 2048, 4096, "M = 1, fp8"),
    ("f16", 2, 1024, 2048, "two rows, fp32 multiply-adds"),
    ("f8e4m3", 4, 2048, 2048, "four rows on the matrix cores (second pass adds the planes)"),
)


def _spoil(c, m, n, rows):
    """Inf and NaN planted in rows `rows` of a row-major m x n C."""
    spoiled = c.copy()
    if len(rows):
        view = spoiled.reshape(m, n)
        view[rows[::3], ::5] = np.nan
        view[rows[1::3], 1::7] = np.inf
        view[rows[2::3], 2::11] = -np.inf
    return spoiled


@pytest.mark.parametrize("ta,m,n,k,what", BETA_ZERO_SHAPES)
def test_beta_zero_as_the_reference_evaluates_it(gpu, ta, m, n, k, what):
    """skl_hip_set_beta_zero_mode(SKL_HIP_BETA_ZERO_AS_REFERENCE): beta == 0 still evaluates beta*C + alpha*acc
    (ref/gemm/gemm_bf16rc_bf16rc_f32rc.c:21). An Inf or NaN in C gives NaN exactly where the checker gives NaN, every
    other element has the bits of the same call on a clean C (which the table tests check against the bound), and
    where alpha*acc is an exact zero - rows of A are zeroed to make such elements, C holds both signs - the sign of
    the result is the checker's."""
    gpu.skl_hip_set_beta_zero_mode(1)
    try:
        assert gpu.skl_hip_get_beta_zero_mode() == 1
        _beta_zero_as_reference(gpu, ta, m, n, k)
    finally:
        gpu.skl_hip_set_beta_zero_mode(0)


def _beta_zero_as_reference(gpu, ta, m, n, k):
    rng = np.random.default_rng(77)
    for alpha, beta in ((-1.5, 0.0), (2.0, -0.0)):
        case = rowmajor_case(ta, m, n, k, alpha, beta)
        a, b, c = case.make_inputs(int(rng.integers(1 << 30)))
        zero_rows = sorted(set((0, m // 2, m - 1))) if m > 2 else []
        for i in zero_rows:
            a[i * k:(i + 1) * k] = 0
        live = np.ones(m, dtype=bool)
        live[zero_rows] = False
        spoiled = _spoil(c, m, n, np.flatnonzero(live))
        nan_want = ~np.isfinite(spoiled.astype(np.float64))  # 0 * Inf and 0 * NaN are NaN, and NaN + x is NaN
        assert nan_want.sum() > 0
        checker = m * n * k <= 1 << 30  # the checker's scalar loop takes seconds beyond that
        if checker:
            want = run_oracle_gemm(case, a, b, c)
            assert np.array_equal(np.isnan(run_oracle_gemm(case, a, b, spoiled).astype(np.float64)), nan_want)
        for mode in MODES:
            got = run_gemm(gpu, "rc", case, a, b, c, mode)
            again = run_gemm(gpu, "rc", case, a, b, spoiled, mode)
            for i in zero_rows if checker else ():
                row = slice(i * n, (i + 1) * n)
                assert np.array_equal(got[row].view(np.uint8), want[row].view(np.uint8)), (ta, mode, alpha, i)
            nan_got = np.isnan(again.astype(np.float64))
            assert np.array_equal(nan_got, nan_want), (ta, mode, alpha, int(nan_got.sum()), int(nan_want.sum()))
            assert np.array_equal(got[~nan_want].view(np.uint8), again[~nan_want].view(np.uint8)), (ta, mode, alpha)
            if ta in ("f32", "f64", "f16h"):
                assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), (ta, mode, alpha)
                assert np.array_equal(again[~nan_want].view(np.uint8), want[~nan_want].view(np.uint8)), (ta, mode, alpha)


@pytest.mark.parametrize("ta,m,n,k,what", BETA_ZERO_SHAPES)
def test_beta_zero_initialises_c(gpu, ta, m, n, k, what):
    """The default: beta == 0 is the initialising call (src/gemm/README.md:43). The old C contributes nothing but the
    sign of an exact zero, so an Inf or NaN in C is overwritten exactly as a finite value is - also in the rows whose
    products are exact zeros, where the old sign is all that is read - and every result has the bits of the
    reference-evaluation mode's result on a clean C. (f64: C is always read.)"""
    if ta == "f64":
        pytest.skip("f64 GEMMs always read C")
    rng = np.random.default_rng(78)
    case = rowmajor_case(ta, m, n, k, -1.5, 0.0)
    a, b, c = case.make_inputs(int(rng.integers(1 << 30)))
    zero_rows = sorted(set((0, m // 2, m - 1))) if m > 2 else []
    for i in zero_rows:
        a[i * k:(i + 1) * k] = 0
    live = np.ones(m, dtype=bool)
    live[zero_rows] = False
    spoiled = _spoil(c, m, n, np.flatnonzero(live))
    for i in zero_rows:  # the zero rows too: NaN and Inf that keep the sign of the value they replace
        row = spoiled.reshape(m, n)[i]
        row[::2] = np.copysign(np.nan, row[::2])
        row[1::4] = np.copysign(np.inf, row[1::4])
    assert gpu.skl_hip_get_beta_zero_mode() == 0
    for mode in MODES:
        gpu.skl_hip_set_beta_zero_mode(1)
        try:
            reference_mode = run_gemm(gpu, "rc", case, a, b, c, mode)
        finally:
            gpu.skl_hip_set_beta_zero_mode(0)
        got = run_gemm(gpu, "rc", case, a, b, c, mode)
        again = run_gemm(gpu, "rc", case, a, b, spoiled, mode)
        assert np.all(np.isfinite(again.astype(np.float64))), (ta, mode)
        assert np.array_equal(got.view(np.uint8), again.view(np.uint8)), (ta, mode)
        assert np.array_equal(got.view(np.uint8), reference_mode.view(np.uint8)), (ta, mode)


SCANNED_C_SHAPES = (
    # ta, layout of C, m, n, k, what serves it
    ("f8e4m3", "row", 4096, 4096, 4096, "256 x 256 tiles, exactly the slices of K it takes to look through a wave's block (64)"),
    ("f8e4m3", "row", 4096, 4096, 4096 + 128, "256 x 256 tiles, two slices more"),
    ("f8e4m3", "row", 4096, 4096, 8192, "256 x 256 tiles, twice the slices: the last rows are requested again"),
    ("bf16", "row", 1024, 3072, 1024, "256 x 128 tiles, exactly the slices it takes (32)"),
    ("f8e4m3", "row", 1024, 16640, 4096, "260 tiles: 256-column tiles and, for the last 256 columns, 128-column ones (two launches)"),
    ("bf16", "row", 1024, 3072, 2048 + 64, "256 x 128 tiles"),
    ("f16", "column", 4096, 4096, 4096, "column-major C"),
    ("bf16", "panel", 4096, 4096, 4096, "C in 64 x 64 panels, 256 x 256 tiles"),
    ("bf16", "panel", 1024, 3072, 1024 + 64, "C in 64 x 64 panels, 256 x 128 tiles"),
)


@pytest.mark.parametrize("ta,layout,m,n,k,what", SCANNED_C_SHAPES)
def test_beta_zero_as_the_reference_scans_c_under_the_product(gpu, ta, layout, m, n, k, what):
    """The streaming kernel with a long K looks through the old C while it multiplies (four rows of every wave's block
    per two slices of K) instead of reading all of it in the epilogue. Single NaNs and infinities planted in a few blocks - first
    and last row of a block, first and last column, neighbouring blocks, the matrix's corners - become NaN exactly
    there (ref/gemm/gemm_bf16rc_bf16rc_f32rc.c:21: 0 * c), every other element has the bits of the same call on a
    clean C and of the initialising mode's call, and rows of exact zeros (a zeroed row of A) take their sign from the
    old C in blocks with and without a planted value."""
    rng = np.random.default_rng(79)
    if layout == "panel":
        case = support.panel_case(ta, m // support.TE, n // support.TE, k, -1.5, 0.0)
        kind = "rcprc"
    else:
        case = rowmajor_case(ta, m, n, k, -1.5, 0.0)
        if layout == "column":
            case.rsc1, case.csc1 = 1, m
        kind = "rc"
    a, b, c = case.make_inputs(int(rng.integers(1 << 30)))
    if layout != "panel":  # row 5 and the last row of A: exact zeros in those rows of C
        for i in (5, m - 1):
            a[i * k:(i + 1) * k] = 0
    c[::3] = -c[::3]
    oc = support.blocked_offsets(case.m1, case.n1, case.m0, case.n0, case.rsc0, case.csc0, case.rsc1, case.csc1)
    spots = [(0, 0), (127, 63), (128, 64), (255, 255), (256 + 63, 191), (256 + 64, 192), (m - 1, n - 1), (m - 1, 0),
             (0, n - 1), (m // 2 + 31, n // 2 + 33), (m - 129, n - 65), (700, 1500)]
    spoiled = c.copy()
    for idx, (i, j) in enumerate(spots):
        spoiled[oc[i, j]] = (np.nan, np.inf, -np.inf)[idx % 3]
    nan_want = np.zeros(c.size, dtype=bool)
    nan_want[[oc[i, j] for i, j in spots]] = True
    initialised = run_gemm(gpu, kind, case, a, b, c, "device")
    assert np.all(np.isfinite(initialised))
    gpu.skl_hip_set_beta_zero_mode(1)
    try:
        clean = run_gemm(gpu, kind, case, a, b, c, "device")
        again = run_gemm(gpu, kind, case, a, b, spoiled, "device")
    finally:
        gpu.skl_hip_set_beta_zero_mode(0)
    assert np.array_equal(clean.view(np.uint8), initialised.view(np.uint8)), (ta, layout)
    assert np.array_equal(np.isnan(again), nan_want), (ta, layout, int(np.isnan(again).sum()))
    assert np.array_equal(again[~nan_want].view(np.uint8), clean[~nan_want].view(np.uint8)), (ta, layout)
    if layout != "panel":  # the zero rows hold zeros of both signs, following the old C
        zeros = clean[oc[5, :]]
        assert np.all(zeros == 0) and np.signbit(zeros).any() and not np.signbit(zeros).all()


@pytest.mark.parametrize("ta,tb", (("f8e4m3", "f8e4m3"), ("f8e5m2", "f8e5m2"), ("f8e4m3", "f8e5m2")))
@pytest.mark.parametrize("a_rowmajor", (True, False))
def test_fp8_short_k_is_multiplied_exactly(gpu, ta, tb, a_rowmajor):
    """Up to K = 2304 the fp8 kinds run with the bytes widened to f16 and exact products. One-hot rows of A (1.0 at
    position p_i): row i of C is row p_i of B as the format defines it, every finite code, subnormal ones included,
    whichever lane, k-step half and instruction of the pair its k falls into. Then random operands: the
    reference's elementwise bound with nothing added, at a K where the fp8 instructions would exceed it."""
    m, n, k = 96, 256, 160
    one = 0x38 if ta == "f8e4m3" else 0x3C
    table = support.decode_table(tb)
    finite_codes = np.flatnonzero(np.isfinite(table)).astype(np.uint8)  # 0 * Inf would spoil whole columns
    b = finite_codes[(np.arange(k * n) * 7 + np.arange(k * n) // n) % finite_codes.size].astype(np.uint8)
    assert set(b.tolist()) == set(finite_codes.tolist())
    a = np.zeros(m * k, np.uint8)
    pos = [(i * 37 + 5) % k for i in range(m)]
    for i in range(m):
        a[(i * k + pos[i]) if a_rowmajor else (pos[i] * m + i)] = one
    case = (rowmajor_case if a_rowmajor else colmajor_a_case)(ta, m, n, k, 1.0, 0.0, tb=tb)
    got = run_gemm(gpu, "rc", case, a, b, np.zeros(m * n, np.float32), "device").reshape(m, n)
    for i in range(m):
        assert np.array_equal(got[i].astype(np.float64), table[b[pos[i] * n:(pos[i] + 1) * n]]), (ta, tb, i)
    for (mm, nn, kk) in ((200, 300, 64), (384, 512, 2304)):
        case = (rowmajor_case if a_rowmajor else colmajor_a_case)(ta, mm, nn, kk, 1.5, -0.5, tb=tb)
        a, b, c = case.make_inputs(mm + kk)
        support.assert_fp_gemm_close(case, a, b, c, run_gemm(gpu, "rc", case, a, b, c, "device"))


FUSED_SHAPES = (
    # m, n, k, what serves it
    (130, 200, 64, "64 x 64 bounds-checked tiles"),
    (300, 1100, 96, "128 x 128 bounds-checked tiles"),
    (2048, 2048, 128, "streaming kernel, 256 x 128 tiles"),
    (2048, 9216, 128, "streaming kernel, 256 x 256 tiles and a last round of 256 x 128"),
    (1, 4096, 512, "M = 1: the fused call must not take the GEMV path"),
)


@pytest.mark.parametrize("m,n,k,what", FUSED_SHAPES)
@pytest.mark.parametrize("ta", ("i8", "bf16", "f8e4m3"))
def test_fused_epilogue(gpu, ta, m, n, k, what):
    """Bias and running maximum behind the alpha/beta step (include/skl-gfx950.h, fused section). int8:
    C and *max equal the checker's GEMM followed by the two steps, bit for bit. Floating point: the fused call's C equals
    the plain call's C plus the bias in one fp32 addition, bit for bit (same kernel, same summation), and
    *max is the largest value written."""
    rng = np.random.default_rng(m * 7 + n)
    case = rowmajor_case(ta, m, n, k, alpha=1, beta=1 if m != 2048 else 0)
    a, b, c = case.make_inputs(int(rng.integers(1 << 30)))
    if case.is_int:
        bias = rng.integers(-1 << 20, 1 << 20, n).astype(np.int32)
        start = np.array([-(1 << 31)], np.int32)
    else:
        bias = rng.uniform(-4, 4, n).astype(np.float32)
        start = np.array([-np.inf], np.float32)
    checker_plain = run_oracle_gemm(case, a, b, c) if case.is_int else None
    for mode in MODES:
        if m == 1 and not case.is_int:
            plain = None  # the plain M = 1 call sums with floating-point atomics: no bit-level anchor
        else:
            plain = run_gemm(gpu, "rc", case, a, b, c, mode)
        for use_bias, use_max in ((True, True), (False, True), (True, False)):
            got, top = run_fused_gemm(gpu, "rc", case, a, b, c, bias if use_bias else None,
                                      start if use_max else None, mode)
            if case.is_int:
                want_c, want_top = fused_expectation(case, checker_plain, bias if use_bias else None,
                                                     start if use_max else None)
                assert np.array_equal(got, want_c), (what, mode, use_bias, use_max)
                if use_max:
                    assert top[0] == want_top[0], (what, mode)
            elif plain is not None:
                want_c, want_top = fused_expectation(case, plain, bias if use_bias else None,
                                                     start if use_max else None)
                assert np.array_equal(got.view(np.uint8), want_c.view(np.uint8)), (what, mode, use_bias, use_max)
                if use_max:
                    assert top[0] == want_top[0], (what, mode)
            else:
                if not use_bias:
                    support.assert_fp_gemm_close(case, a, b, c, got,
                                                 extra_rel=support.FP8_MFMA_REL if ta.startswith("f8") else 0.0)
                else:  # the same kernel with and without the bias: one rounded addition apart
                    unbiased, _ = run_fused_gemm(gpu, "rc", case, a, b, c, None, start, mode)
                    assert np.array_equal(got, (unbiased + bias).astype(np.float32)), (what, mode)
                if use_max:
                    assert top[0] == got.max(), (what, mode)
    # a maximum already above every element stays
    high = np.array([1 << 30], np.int32) if case.is_int else np.array([1e30], np.float32)
    _, top = run_fused_gemm(gpu, "rc", case, a, b, c, None, high, "device")
    assert top[0] == high[0]


EXTRA_STEP_SHAPES = (
    # m, n, k, beta, what serves it
    (130, 200, 64, 1, "64 x 64 bounds-checked tiles"),
    (300, 1100, 96, 0, "128 x 128 bounds-checked tiles"),
    (512, 768, 256, 1, "whole tiles, too few for the streaming kernel"),
    (2048, 2048, 128, 1, "streaming kernel, 256 x 128 tiles (int8 with a row-major copy; everything else: bounds-checked kernels)"),
    (2048, 9216, 128, 0, "streaming kernel, 256 x 256 tiles and a second launch of 256 x 128 on the last columns (int8)"),
    (2048, 2048, 2560, 1, "streaming kernel, K beyond the exact fp8 kernels' range (int8 and fp8 kinds with a row-major copy)"),
    (1000, 1100, 520, 0, "ragged and large enough for padded copies: must stay on the bounds-checked kernels"),
    (16, 4096, 4096, 1, "a decode batch"),
    (40, 300, 8192, 1, "K shared between workgroups: the steps ride on the pass that adds the shares"),
    (1, 4096, 512, 0, "M = 1"),
)


@pytest.mark.parametrize("m,n,k,beta,what", EXTRA_STEP_SHAPES)
@pytest.mark.parametrize("ta", ("i8", "bf16", "f8e4m3"))
def test_fused_activation_and_requantised_copy(gpu, ta, m, n, k, beta, what):
    """Activation and the requantised int8 copy (include/skl-gfx950.h, fused section), which follow the bias and
    precede the maximum. The fused call without them is the anchor for C (bit for bit: same kernel family, same
    summation - the plain steps are checked against the checker elsewhere); C, Q and *max must then be exactly what
    the rules make of that C: relu in C's type, Q = clamp(rne((float)v * s_j) + zero). Row-major and transposed Q,
    one scale and one per column, both kinds of memory, and q_only, which must leave C alone."""
    rng = np.random.default_rng(m * 11 + n + k)
    case = rowmajor_case(ta, m, n, k, alpha=1, beta=beta)
    a, b, c = case.make_inputs(int(rng.integers(1 << 30)))
    if case.is_int:
        bias = rng.integers(-1 << 12, 1 << 12, n).astype(np.int32)
        start = np.array([-(1 << 31)], np.int32)
    else:
        bias = rng.uniform(-4, 4, n).astype(np.float32)
        start = np.array([-np.inf], np.float32)
    spread = float(np.abs(run_fused_gemm(gpu, "rc", case, a, b, c, None, None, "device")[0].astype(np.float64)).max())
    scales = (rng.uniform(0.5, 2.0, n) * 100.0 / max(spread, 1e-3)).astype(np.float32)  # some values saturate
    layouts = ((n + 4, 1), (1, m + 5))  # (rsq, csq); row-major rows on 4-byte boundaries: the streaming kernel writes them as dwords (int8)
    for mode in MODES:
        anchor, _ = run_fused_gemm(gpu, "rc", case, a, b, c, bias, None, mode)
        for act, per_column, (rsq, csq), zero, only in ((1, True, layouts[0], 3, False), (0, False, layouts[1], -7, False),
                                                        (1, False, layouts[0], 0, True)):
            q0 = np.full((m - 1) * rsq + (n - 1) * csq + 1, 0x55, np.int8)
            rq = dict(q=q0, rsq=rsq, csq=csq, scale=scales if per_column else scales[:1], per_column=per_column,
                      zero=zero, only=only)
            got, top, q = run_fused_gemm(gpu, "rc", case, a, b, c, bias, start, mode, activation=act, requant=rq)
            want_c, want_top, want_q = fused_expectation(case, anchor, None, start, activation=act, requant=rq)
            tag = (ta, what, mode, act, per_column, rsq, only)
            assert np.array_equal(q, want_q), tag
            if only:
                assert np.array_equal(got.view(np.uint8), c.view(np.uint8)), tag
            else:
                assert np.array_equal(got.view(np.uint8), want_c.view(np.uint8)), tag
            assert top[0] == want_top[0], tag
            assert len(np.unique(want_q)) > 20, "a degenerate scale would test nothing"
        # the activation alone
        got, top = run_fused_gemm(gpu, "rc", case, a, b, c, bias, start, mode, activation=1)
        want_c, want_top = fused_expectation(case, anchor, None, start, activation=1)
        assert np.array_equal(got.view(np.uint8), want_c.view(np.uint8)) and top[0] == want_top[0], (ta, what, mode)


@pytest.mark.parametrize("m,n,k,beta,what", EXTRA_STEP_SHAPES)
@pytest.mark.parametrize("ta", ("i8", "bf16", "f8e4m3", "f8e5m2"))
def test_fused_fp8_copy(gpu, ta, m, n, k, beta, what):
    """The 8-bit copy as OCP fp8 (q_format): each byte must be what the reference's fp32 -> fp8 conversion
    (skl_cvt_[sat_]f32_f8e4m3 / _f8e5m2, ref/cvt/cvt_ofp8.c:174-198, through the checker) makes of the value written to
    C times the column's scale, on every kernel family; the scales put a good part of the values beyond the format's
    largest, so the saturating and the non-saturating rule differ, and (one scale per column) others among its subnormals."""
    rng = np.random.default_rng(m * 13 + n + k)
    case = rowmajor_case(ta, m, n, k, alpha=1, beta=beta)
    a, b, c = case.make_inputs(int(rng.integers(1 << 30)))
    bias = rng.integers(-1 << 12, 1 << 12, n).astype(np.int32) if case.is_int else rng.uniform(-4, 4, n).astype(np.float32)
    for mode in MODES:
        anchor, _ = run_fused_gemm(gpu, "rc", case, a, b, c, bias, None, mode)
        spread = float(np.abs(anchor.astype(np.float64)).max())
        for fmt, (rsq, csq), per_column, act, only in ((1, (n + 4, 1), True, 0, False), (2, (1, m + 3), False, 1, False),
                                                       (3, (n, 1), False, 0, True), (4, (n + 1, 1), True, 1, False)):
            largest = 448.0 if fmt <= 2 else 57344.0
            base = largest * 1.25 / max(spread, 1e-3)   # the widest values land a quarter beyond the format's largest
            scales = (base * np.exp2(rng.integers(-24, 4, n))).astype(np.float32) if per_column else np.array([base], np.float32)
            q0 = np.full((m - 1) * rsq + (n - 1) * csq + 1, 0x55, np.int8)
            rq = dict(q=q0, rsq=rsq, csq=csq, scale=scales, per_column=per_column, only=only, format=fmt)
            got, _, q = run_fused_gemm(gpu, "rc", case, a, b, c, bias, None, mode, activation=act, requant=rq)
            want_c, _, want_q = fused_expectation(case, anchor, None, None, activation=act, requant=rq)
            tag = (ta, what, mode, fmt, per_column, rsq, only)
            assert np.array_equal(q, want_q), tag
            assert np.array_equal(got.view(np.uint8), (c if only else want_c).view(np.uint8)), tag
            oq = np.arange(m)[:, None] * rsq + np.arange(n)[None, :] * csq
            codes = want_q[oq].view(np.uint8) & 0x7F
            beyond = {1: 0x7F, 2: 0x7E, 3: 0x7C, 4: 0x7B}[fmt]   # what a value past the largest becomes
            assert np.count_nonzero(codes == beyond) > 0 and len(np.unique(codes)) > (40 if per_column else 2), tag


@pytest.mark.parametrize("ta,m,n,k,what", (
    ("bf16", 300, 1100, 96, "bounds-checked tiles"),
    ("f8e4m3", 2048, 2048, 2560, "streaming kernel"),
    ("f16", 2048, 2048, 128, "streaming kernel, 16-bit operands"),
    ("f8e5m2", 40, 300, 8192, "K shared between workgroups"),
    ("bf16", 16, 4096, 4096, "a decode batch"),
    ("f16", 1, 2048, 512, "M = 1"),
))
def test_q_only_with_beta_zero_leaves_c_untouched(gpu, ta, m, n, k, what):
    """A floating-point call that writes only the 8-bit copy, with beta == 0, neither writes nor reads C
    (include/skl-gfx950.h): rows of A that are all zero make exact zeros, whose sign an old C would decide - C holds
    -1 everywhere and alpha is negative, so alpha * acc is -0 there and a kernel that looked at C would add the -0 that
    0 * -1 is and write the fp8 code of -0 (0x80), as the call that also writes C does; an old C of +0 gives +0
    (0x00). Everything else equals the call that also writes C, and C comes back bit for bit."""
    rng = np.random.default_rng(m + n)
    case = rowmajor_case(ta, m, n, k, alpha=-1.0, beta=0.0)
    a, b, _ = case.make_inputs(int(rng.integers(1 << 30)))
    zero_rows = sorted({0, m - 1, m // 2})
    a.reshape(m, k)[zero_rows] = 0
    c = np.full(m * n, -1.0, np.float32)
    scale = np.array([0.125], np.float32)
    for mode in MODES:
        rq = dict(q=np.full(m * n, 0x55, np.int8), rsq=n, csq=1, scale=scale, format=2)
        _, _, q_with_c = run_fused_gemm(gpu, "rc", case, a, b, c, None, None, mode, requant=rq)
        got, _, q = run_fused_gemm(gpu, "rc", case, a, b, c, None, None, mode, requant=dict(rq, only=True))
        assert np.array_equal(got.view(np.uint32), c.view(np.uint32)), (ta, what, mode)
        q, q_with_c = q.reshape(m, n).view(np.uint8), q_with_c.reshape(m, n).view(np.uint8)
        assert np.all(q_with_c[zero_rows] == 0x80) and np.all(q[zero_rows] == 0x00), (ta, what, mode)
        rest = np.setdiff1d(np.arange(m), zero_rows)
        assert np.array_equal(q[rest], q_with_c[rest]), (ta, what, mode)


@pytest.mark.parametrize("ta,m,n,k,what", (
    ("f8e4m3", 2048, 2048, 2560, "streaming kernel: four values per lane packed into a dword"),
    ("bf16", 2048, 2048, 128, "streaming kernel, 16-bit operands"),
    ("f16", 2048, 9216, 64, "streaming kernel, 256 x 256 tiles and a second launch"),
    ("bf16", 512, 1024, 64, "bounds-checked tiles: byte by byte"),
))
def test_fp8_copy_of_any_fp32_value(gpu, ta, m, n, k, what):
    """The epilogues' fp32 -> fp8 conversion over fp32 values of every kind: with alpha = 0 and beta = 1 the value
    written is C itself, so C can hold any bit pattern - every exponent with a spread of significands around the
    rounding ties, both signs, zeros, subnormals, infinities, NaNs, the neighbourhood of each format's largest value,
    and random patterns. Each byte of the copy must be the checker's conversion of what was written to C."""
    from test_oracle_gemm import requantised
    rng = np.random.default_rng(k)
    case = rowmajor_case(ta, m, n, k, alpha=0.0, beta=1.0)
    a, b, _ = case.make_inputs(3)
    sig = np.array([0, 1, 0x7FFFFF, 0x400000, 0x400001, 0x3FFFFF, 0x100000, 0x080000, 0x0FFFFF, 0x200000, 0x600000, 0x700000,
                    0x500000, 0x300000, 0x0FFFFE, 0x100001, 0x680000, 0x680001, 0x67FFFF], np.uint32)
    special = (np.arange(256, dtype=np.uint32)[:, None, None] << 23 | np.array([0, 1], np.uint32)[None, :, None] << 31 | sig[None, None, :]).ravel()
    near_max = np.concatenate([np.float32(x).view(np.uint32) + np.arange(-64, 65, dtype=np.int64).astype(np.uint32)
                               for x in (448.0, 464.0, 480.0, 57344.0, 61440.0, 65536.0, 2.0 ** -6, 2.0 ** -9, 2.0 ** -10, 2.0 ** -14,
                                         2.0 ** -16, 2.0 ** -17)])
    near_max = np.concatenate([near_max, near_max | np.uint32(0x80000000)])
    for fmt in (1, 2, 3, 4):
        bits = rng.integers(0, 1 << 32, m * n, dtype=np.uint64).astype(np.uint32)
        bits[:special.size] = special
        bits[special.size:special.size + near_max.size] = near_max
        c = bits.view(np.float32)
        rq = dict(q=np.zeros(m * n, np.int8), rsq=n, csq=1, scale=np.array([1.0], np.float32), format=fmt)
        got, _, q = run_fused_gemm(gpu, "rc", case, a, b, c, None, None, "device", requant=rq)
        assert np.array_equal(q, requantised(got, np.float32(1.0), 0, fmt)), (ta, what, fmt)
        same = ~np.isnan(c)
        assert np.array_equal(got[same], c[same] + np.float32(0.0)), (ta, what, fmt)   # the values did arrive in the epilogue


@pytest.mark.parametrize("act", (2, 3))
def test_silu_and_gelu_values(gpu, act):
    """The activation alone: with alpha = 0 and beta = 1 the value it is applied to is C itself, so any fp32 value
    can be put through it - the ranges of the reference's own tests (test/sigmoid/sigmoid_f32_zve32f.c: [-110, 18];
    test/gelu/skl_gelu_f32_zve32f.c: [-14.356, 5.348]) densely, the far tails, zeros, infinities, NaN. The result must
    be the reference routine's value (skl_silu_f32_ref / skl_gelu_f32_ref through the checker) within the error the
    reference allows its own vector kernels, range by range; measured: well inside."""
    rng = np.random.default_rng(act)
    m, n, k = 256, 1024, 8
    lo, hi = ((-110.0, 18.0), (-14.356, 5.348))[act - 2]
    c = np.concatenate([rng.uniform(lo, hi, m * n - 70000), rng.uniform(-3, 3, 40000), rng.uniform(-1e-3, 1e-3, 29980),
                        np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1e-40, -1e-40, -88.7, -103.9, -109.9, 88.8, 3e38, -3e38,
                                  -17.0, -17.000002, -80.0, -80.00001, 1.0, -1.0, -2.0])]).astype(np.float32)
    case = rowmajor_case("bf16", m, n, k, alpha=0.0, beta=1.0)
    a, b, _ = case.make_inputs(1)
    for mode in MODES:
        got, _ = run_fused_gemm(gpu, "rc", case, a, b, c, None, None, mode, activation=act)
        want = support.activation_reference(c, act)
        err = support.ulp_error_f32(got, want)
        finite = np.isfinite(want)
        assert np.all(err[finite] <= support.activation_ulp_bound(c, act)[finite]), (act, mode, float(err[finite].max()))
        assert np.array_equal(np.isnan(got), np.isnan(want)) and np.array_equal(got[np.isinf(want)], want[np.isinf(want)])
        inside = finite & (c >= (-80 if act == 2 else -1)) & (np.abs(want) > 1e-30)
        assert err[inside].max() <= 4.0, (act, mode, float(err[inside].max()))   # where nothing underflows: a few ulp


@pytest.mark.parametrize("ta,m,n,k,what", (
    ("bf16", 300, 1100, 96, "bounds-checked tiles"),
    ("f16", 2048, 2048, 128, "whole tiles: still the bounds-checked kernels, which carry the steps"),
    ("f8e4m3", 40, 300, 8192, "K shared between workgroups: the pass that adds the shares"),
    ("bf16", 16, 4096, 4096, "a decode batch: the pass that adds the planes"),
    ("f8e5m2", 1, 2048, 512, "M = 1"),
))
def test_fused_silu_and_gelu(gpu, ta, m, n, k, what):
    """SiLU and GELU behind alpha / beta and the bias on every kernel family: C must be the reference routine's value
    of the fused call's own pre-activation C (the same call without an activation gives it bit for bit) within the
    reference's bounds; the maximum is the largest value written, and the requantised copy is the rule applied to the
    value written."""
    from test_oracle_gemm import requantised
    rng = np.random.default_rng(m + n + k)
    case = rowmajor_case(ta, m, n, k, alpha=0.25, beta=1.0)
    a, b, c = case.make_inputs(int(rng.integers(1 << 30)))
    bias = rng.uniform(-2, 2, n).astype(np.float32)
    start = np.array([-np.inf], np.float32)
    scale = np.array([16.0], np.float32)
    for mode in MODES:
        anchor, _ = run_fused_gemm(gpu, "rc", case, a, b, c, bias, None, mode)
        for act in (2, 3):
            rq = dict(q=np.zeros(m * n, np.int8), rsq=n, csq=1, scale=scale, zero=-3)
            got, top, q = run_fused_gemm(gpu, "rc", case, a, b, c, bias, start, mode, activation=act, requant=rq)
            want = support.activation_reference(anchor, act)
            err = support.ulp_error_f32(got, want)
            assert np.all(err <= support.activation_ulp_bound(anchor, act)), (ta, what, mode, act, float(err.max()))
            assert top[0] == got.max(), (ta, what, mode, act)
            assert np.array_equal(q, requantised(got, scale[0], -3)), (ta, what, mode, act)
    # integers have no such activation
    icase = rowmajor_case("i8", 8, 8, 8, alpha=1, beta=0)
    ia, ib, ic = icase.make_inputs(1)
    run_fused_gemm_expecting_refusal(gpu, icase, ia, ib, ic, activation=2)


def test_fused_extra_steps_blocked_form_any_strides_and_refusals(gpu):
    """The rcprc form addresses Q by the logical row and column; odd blocks and strides take the any-stride
    kernel. Descriptors the header rules out are refused before anything runs."""
    rng = np.random.default_rng(15)
    for ta in ("i8", "f16"):
        case = support.GemmCase(ta, None, 2, 3, m0=3, n0=4, k0=5, m1=5, n1=3, k1=4, rsa0=5, csa0=1, rsa1=100, csa1=15,
                                rsb0=4, csb0=1, rsb1=20, csb1=90, rsc0=1, csc0=3, rsc1=12, csc1=64)
        a, b, c = case.make_inputs(int(rng.integers(1 << 30)))
        m, n = case.m0 * case.m1, case.n0 * case.n1
        bias = (rng.integers(-99, 99, n).astype(np.int32) if case.is_int else rng.uniform(-4, 4, n).astype(np.float32))
        start = np.array([-(1 << 31)], np.int32) if case.is_int else np.array([-np.inf], np.float32)
        scales = rng.uniform(0.01, 0.05, n).astype(np.float32) * (1.0 if case.is_int else 20.0)
        for mode in MODES:
            anchor, _ = run_fused_gemm(gpu, "rcprc", case, a, b, c, bias, None, mode)
            rq = dict(q=np.full(m * 40, 9, np.int8), rsq=40, csq=2, scale=scales, per_column=True, zero=-1)
            got, top, q = run_fused_gemm(gpu, "rcprc", case, a, b, c, bias, start, mode, activation=1, requant=rq)
            want_c, want_top, want_q = fused_expectation(case, anchor, None, start, activation=1, requant=rq)
            assert np.array_equal(got.view(np.uint8), want_c.view(np.uint8)), (ta, mode)
            assert np.array_equal(q, want_q) and top[0] == want_top[0], (ta, mode)
    # the 4 x 8 by 8 x 4 block format: through copies of A and B, C where it lies (accumulating) or through a
    # row-major scratch matrix (beta == 0)
    from test_oracle_gemm import block4x8x4_case
    for accum in (True, False):
        case = block4x8x4_case(32, 40, 16, accum=accum)
        a, b, c = case.make_inputs(77)
        m, n = 128, 160
        bias = rng.integers(-999, 999, n).astype(np.int32)
        start = np.array([-(1 << 31)], np.int32)
        plain = run_oracle_gemm(case, a, b, c)
        rq = dict(q=np.full(m * n, 9, np.int8), rsq=n, csq=1, scale=np.array([1 / 64.0], np.float32), zero=4)
        got, top, q = run_fused_gemm(gpu, "rcprc", case, a, b, c, bias, start, "device", activation=1, requant=rq)
        want_c, want_top, want_q = fused_expectation(case, plain, bias, start, activation=1, requant=rq)
        assert np.array_equal(got, want_c) and np.array_equal(q, want_q) and top[0] == want_top[0], accum
        rq["only"] = True
        got, top, q = run_fused_gemm(gpu, "rcprc", case, a, b, c, bias, start, "device", activation=1, requant=rq)
        assert np.array_equal(got, c) and np.array_equal(q, want_q) and top[0] == want_top[0], accum
    case = rowmajor_case("i8", 8, 8, 8, alpha=1, beta=0)
    a, b, c = case.make_inputs(1)
    q0, one = np.zeros(64, np.int8), np.ones(1, np.float32)
    for bad in (dict(q=q0, rsq=8, csq=1, scale=None), dict(q=q0, rsq=8, csq=1, scale=one, zero=128),
                dict(q=q0, rsq=8, csq=1, scale=one, zero=-129), dict(q=q0, rsq=8, csq=1, scale=one, format=5),
                dict(q=q0, rsq=8, csq=1, scale=one, format=-1)):
        run_fused_gemm_expecting_refusal(gpu, case, a, b, c, requant=bad)
    run_fused_gemm_expecting_refusal(gpu, case, a, b, c, activation=2)
    # a Q in memory of the other kind than C
    dq = skl_amd.DeviceBuffer.from_array(q0)
    try:
        run_fused_gemm_expecting_refusal(gpu, case, a, b, c, requant=dict(q=dq, rsq=8, csq=1, scale=one))
    finally:
        dq.free()


@pytest.mark.parametrize("m", (1, 16, 50))
def test_fused_steps_on_k_packed_weights(gpu, m):
    """A fused decode call on the K-packed B of the dot-product GEMM (src/gemm/packed-gemm.md:178-219), through the
    blocked fused entry point with k0 = 4: the streaming kernels leave the plain product in scratch memory and a
    second pass applies alpha / beta and the steps. C, the requantised copy and the maximum against the checker's
    product plus the rules; padded strides, alpha / beta with wrap-around, both pointer modes, q_only."""
    from test_oracle_gemm import fused_expectation
    rng = np.random.default_rng(40 + m)
    n, k1 = 4100, 132
    for alpha, beta, only in ((1, 0, True), (0x01010101, -77, False)):
        case = support.dot4_case(m, n, k1, alpha=alpha, beta=beta, rsa1=4 * k1 + 16, rsb1=4 * n + 32, rsc1=n + 5)
        a, b, c = case.make_inputs(int(rng.integers(1 << 30)))
        c[:] = rng.integers(-2 ** 31, 2 ** 31, size=c.size)
        plain = run_oracle_gemm(case, a, b, c)
        bias = rng.integers(-1 << 12, 1 << 12, n).astype(np.int32)
        start = np.array([-(1 << 31)], np.int32)
        spread = float(np.abs(plain.astype(np.float64)).max())
        scales = (rng.uniform(0.5, 2.0, n) * 100.0 / spread).astype(np.float32)
        for mode in MODES:
            rq = dict(q=np.full(m * (n + 4), 0x55, np.int8), rsq=n + 4, csq=1, scale=scales, per_column=True, zero=3, only=only)
            got, top, q = run_fused_gemm(gpu, "rcprc", case, a, b, c, bias, start, mode, activation=1, requant=rq)
            want_c, want_top, want_q = fused_expectation(case, plain, bias, start, activation=1, requant=rq)
            assert np.array_equal(q, want_q) and top[0] == want_top[0], (m, alpha, beta, mode)
            assert np.array_equal(got, c if only else want_c), (m, alpha, beta, mode)


def run_fused_gemm_expecting_refusal(gpu, case, a, b, c, activation=0, requant=None):
    before = c.copy()
    rq = requant or {}
    gpu.skl_gemm_fused_i8rc_i8rc_i32rc_gfx950(
        case.m1, case.n1, case.k1, 1, a, case.rsa1, 1, b, case.rsb1, 1, 0, c, case.rsc1, 1,
        skl_amd.Epilogue(None, None, activation=activation, q=rq.get("q"), rsq=rq.get("rsq", 0), csq=rq.get("csq", 0),
                         q_scale=rq.get("scale"), q_zero=rq.get("zero", 0), q_format=rq.get("format", 0)))
    assert gpu.skl_hip_last_error() != 0, (activation, requant)  # reading clears it
    assert np.array_equal(c, before)


def test_fused_epilogue_blocked_form_and_null_descriptor(gpu):
    """The rcprc form indexes the bias by the logical column (block * n0 + column in the block); a call
    without descriptor operands is the plain GEMM. Odd blocks and strides: the any-stride kernel."""
    rng = np.random.default_rng(5)
    for ta in ("i8", "f16"):
        case = support.GemmCase(ta, None, 2, 3, m0=3, n0=4, k0=5, m1=5, n1=3, k1=4, rsa0=5, csa0=1, rsa1=100, csa1=15,
                                rsb0=4, csb0=1, rsb1=20, csb1=90, rsc0=1, csc0=3, rsc1=12, csc1=64)
        a, b, c = case.make_inputs(int(rng.integers(1 << 30)))
        n = case.n0 * case.n1
        plain = run_gemm(gpu, "rcprc", case, a, b, c, "device")
        bias = (rng.integers(-99, 99, n).astype(np.int32) if case.is_int else rng.uniform(-4, 4, n).astype(np.float32))
        start = np.array([-(1 << 31)], np.int32) if case.is_int else np.array([-np.inf], np.float32)
        for mode in MODES:
            got, top = run_fused_gemm(gpu, "rcprc", case, a, b, c, bias, start, mode)
            want_c, want_top = fused_expectation(case, plain, bias, start)
            assert np.array_equal(got.view(np.uint8), want_c.view(np.uint8)), (ta, mode)
            assert top[0] == want_top[0]
            got, _ = run_fused_gemm(gpu, "rcprc", case, a, b, c, None, None, mode)
            assert np.array_equal(got.view(np.uint8), plain.view(np.uint8)), (ta, mode)


@pytest.mark.parametrize("ta", ("i8", "bf16", "f16", "f8e4m3"))
@pytest.mark.parametrize("m,n,k", ((9, 1000, 4096), (16, 11008, 4096), (40, 300, 8192), (130, 520, 5000)))
def test_few_tiles_long_k_shares_k_between_workgroups(gpu, ta, m, n, k):
    """A problem with few output tiles and a long K is shared out along K: raw sums per share, then one
    pass that adds the shares in order and applies alpha / beta (and the fused steps). int8 must stay
    bit-exact, floating point inside the reference's bound; two runs give the same bits."""
    if ta != "i8":
        k -= k % 8  # 16-byte aligned rows for the 16-bit kinds
    case = rowmajor_case(ta, m, n, k, alpha=2, beta=3)
    a, b, c = case.make_inputs(m * 1000 + n)
    for mode in MODES:
        got = run_gemm(gpu, "rc", case, a, b, c, mode)
        if case.is_int:
            assert np.array_equal(got, run_oracle_gemm(case, a, b, c)), (m, n, k, mode)
        else:
            support.assert_fp_gemm_close(case, a, b, c, got, extra_rel=support.FP8_MFMA_REL if ta.startswith("f8") else 0.0)
            assert np.array_equal(got.view(np.uint8), run_gemm(gpu, "rc", case, a, b, c, mode).view(np.uint8))
    # fused steps ride on the second pass
    bias = (np.arange(n) % 7 - 3).astype(np.int32 if case.is_int else np.float32)
    start = np.array([-(1 << 31)], np.int32) if case.is_int else np.array([-np.inf], np.float32)
    plain = run_gemm(gpu, "rc", case, a, b, c, "device")
    got, top = run_fused_gemm(gpu, "rc", case, a, b, c, bias, start, "device")
    want_c, want_top = fused_expectation(case, plain, bias, start)
    assert np.array_equal(got.view(np.uint8), want_c.view(np.uint8))
    assert top[0] == want_top[0]


def test_stream_slots_run_out_and_come_back(gpu):
    """A device keeps scratch memory for 32 streams. A call on a further stream still gives the right result - on a
    kernel that needs no scratch - and records the advisory SKL_HIP_ERR_STREAM_SLOTS; once a stream has been
    released (skl_hip_release_stream), the same call runs without a word."""
    import ctypes as ct
    from skl_amd import DeviceBuffer

    hip = ct.CDLL("libamdhip64.so.7")
    hip.hipStreamCreate.restype = hip.hipStreamDestroy.restype = ct.c_int
    case = rowmajor_case("i8", 1, 2048, 4096, alpha=1, beta=0)   # a GEMV: its workgroups meet in the stream's scratch
    a, b, c = case.make_inputs(4242)
    want = run_oracle_gemm(case, a, b, c)
    da, db, dc = DeviceBuffer.from_array(a), DeviceBuffer.from_array(b), DeviceBuffer.from_array(c)
    streams, codes = [], []
    gpu.skl_hip_set_pointer_mode(1)

    def call_on(stream):
        gpu.skl_hip_set_stream(stream.value)
        gpu.skl_hip_memcpy_h2d(dc, c, c.nbytes)
        gpu.skl_gemm_i8_i8_i32_gfx950(1, 2048, 4096, 1, da, case.rsa1, db, case.rsb1, 0, dc, case.rsc1)
        assert gpu.skl_hip_synchronize() == 0
        code = gpu.skl_hip_last_error()
        assert np.array_equal(dc.download(c.dtype, c.size), want), (len(streams), code)
        return code

    try:
        for _ in range(34):   # other tests of this process may hold a few slots already
            stream = ct.c_void_p()
            assert hip.hipStreamCreate(ct.byref(stream)) == 0
            streams.append(stream)
            codes.append(call_on(stream))
            if codes[-1] != 0:
                break
        assert codes[-1] == -5 and all(code == 0 for code in codes[:-1]), codes
        assert call_on(streams[-1]) == -5           # and again: nothing was claimed meanwhile
        assert gpu.skl_hip_release_stream(streams[0].value) == 0
        assert call_on(streams[-1]) == 0            # the freed slot is this stream's now
    finally:
        gpu.skl_hip_set_stream(None)
        gpu.skl_hip_set_pointer_mode(0)
        for stream in streams:
            gpu.skl_hip_release_stream(stream.value)
            hip.hipStreamDestroy(stream)
        for d in (da, db, dc):
            d.free()
        gpu.skl_hip_last_error()


def test_mixed_e4m3_e5m2(gpu):
    for (m, n, k) in ((13, 21, 37), (128, 192, 256)):
        case = rowmajor_case("f8e4m3", m, n, k, 1.0, 0.0, tb="f8e5m2")
        check(gpu, "rc", case, 6000 + m, "device")
        case = colmajor_a_case("f8e4m3", m, n, k, 1.5, 0.5, tb="f8e5m2")
        check(gpu, "rc", case, 6100 + m, "host")


def test_config1_int8_512_cubed_bit_exact(gpu):
    """benchmark configuration 1: 512^3, row-major, C = 0, alpha = 1, beta = 0."""
    case = rowmajor_case("i8", 512, 512, 512, 1, 0)
    a, b, c = case.make_inputs(0x5EED0010)
    c[:] = 0
    for mode in MODES:
        got = run_gemm(gpu, "rowmajor", case, a, b, c, mode)
        assert np.array_equal(got, run_oracle_gemm(case, a, b, c))


def test_k_zero_scales_c_without_reading_operands(gpu):
    """k == 0: C = beta * C and A, B are never dereferenced
    (test/gemm/rvv/skl_gemm_i8_i8_i32_zve32x_x390.c:59,68-69)."""
    c = np.arange(33 * 33, dtype=np.int32)
    out = c.copy()
    gpu.skl_gemm_i8_i8_i32_gfx950(33, 33, 0, 1, None, 0, None, 33, 3, out, 33)
    skl_amd.check_error()
    assert np.array_equal(out, 3 * c)
    cf = np.linspace(-1, 1, 16 * 16).astype(np.float32)
    outf = cf.copy()
    gpu.skl_gemm_bf16_bf16_f32_gfx950(16, 16, 0, 1.0, None, 0, None, 16, 0.5, outf, 16)
    skl_amd.check_error()
    assert np.array_equal(outf, np.float32(0.5) * cf)


def test_zero_m_or_n_touches_nothing(gpu):
    c = np.full(64, 7, np.int32)
    a = np.ones(64, np.int8)
    gpu.skl_gemm_i8_i8_i32_gfx950(0, 8, 8, 1, a, 8, a, 8, 0, c, 8)
    gpu.skl_gemm_i8_i8_i32_gfx950(8, 0, 8, 1, a, 8, a, 8, 0, c, 8)
    skl_amd.check_error()
    assert np.all(c == 7)


def _dense_case(ta, m, n, k, a_kc, b_kc, alpha, beta, tb=None):
    """A (m x k) row-major if a_kc else column-major; B (k x n) column-major if b_kc else row-major."""
    return support.GemmCase(ta, tb, alpha, beta, m0=1, n0=1, k0=1, m1=m, n1=n, k1=k, rsa0=0, csa0=0,
                            rsa1=k if a_kc else 1, csa1=1 if a_kc else m, rsb0=0, csb0=0,
                            rsb1=1 if b_kc else n, csb1=k if b_kc else 1, rsc0=0, csc0=0, rsc1=n, csc1=1)


@pytest.mark.parametrize("m,n", ((4096, 4096), (2048, 1664), (2048, 8704)))
@pytest.mark.parametrize("a_kc,b_kc", ((True, False), (False, False), (True, True), (False, True)))
@pytest.mark.parametrize("ta", ("i8", "bf16", "f16", "f8e4m3", "f8e5m2", "mixed"))
def test_whole_tile_streaming_kernel(gpu, ta, a_kc, b_kc, m, n):
    """4096 x 4096 outputs (256 tiles of 256 x 256), 2048 x 1664 outputs (104
    tiles of 256 x 128) and 2048 x 8704 outputs (272 tiles: one full round of
    256 x 256 tiles and a short last round that runs as 256 x 128 tiles): the
    tile shapes of the streaming matrix-core kernel, for every operand orientation. Too large for the scalar checker: the
    expected result is numpy's fp64 product, which is exact for the integer case
    (|sum| < 2^53) and the fp64-accumulated reference for the others."""
    k = 384 if ta == "i8" else 256
    tb = None
    if ta == "mixed":
        ta, tb = "f8e4m3", "f8e5m2"
    alpha, beta = (3, -2) if ta == "i8" else (1.5, 0.5)
    case = _dense_case(ta, m, n, k, a_kc, b_kc, alpha, beta, tb)
    rng = np.random.default_rng((sum(map(ord, ta + str(tb))) * 4 + a_kc * 2 + b_kc + n) % (1 << 31))
    a, b, c = case.make_inputs(int(rng.integers(1 << 30)))
    if ta.startswith("f8"):   # N(0,1)-like spread instead of log-uniform bytes: the config-4 distribution
        a = rng.integers(0x28, 0x48, size=a.size, dtype=np.uint8) | (rng.integers(0, 2, size=a.size, dtype=np.uint8) << 7)
        b = rng.integers(0x28, 0x48, size=b.size, dtype=np.uint8) | (rng.integers(0, 2, size=b.size, dtype=np.uint8) << 7)
    got = run_gemm(gpu, "rc", case, a, b, c, "device")
    A, B, C, oc = case.dense(a, b, c)
    exact = alpha * (A @ B) + beta * C
    if case.is_int:
        want = (exact.astype(np.int64) & 0xFFFFFFFF).astype(np.uint32).view(np.int32)
        assert np.array_equal(got[oc], want)
    else:
        rel = np.linalg.norm(got[oc] - exact) / np.linalg.norm(exact)
        assert rel <= 1e-3, rel
        gamma = 2.0 * ((1.0 + 2.0 ** -24) ** (k + 2) - 1.0)
        extra = support.FP8_MFMA_REL if ta.startswith("f8") else 0.0
        bound = (gamma + extra) * abs(alpha) * (np.abs(A) @ np.abs(B)) + gamma * abs(beta) * np.abs(C)
        err = np.abs(got[oc] - exact)
        assert np.all(err <= bound + np.abs(exact) * 2.0 ** -22), float((err / (bound + 1e-30)).max())


@pytest.mark.parametrize("ta,tb", (("i8", "i8"), ("bf16", "bf16"), ("f16", "f16"), ("f8e4m3", "f8e5m2")))
def test_leading_dimensions_off_the_16_byte_rule(gpu, ta, tb):
    """Operands whose leading dimension is not a multiple of 16 bytes, or that have no unit stride at all, are
    copied into aligned scratch memory and multiplied by the matrix-core kernels instead of the any-stride one:
    A alone, B alone, both; row- and column-major. Same bar as everywhere: int8 bit-exact over the whole C buffer,
    floating point inside the reference's bound."""
    from support import GemmCase
    m, n, k = 300, 260, 777
    layouts = {  # (rsa, csa), (rsb, csb)
        "A odd lda": ((k + 1, 1), (n + 12, 1)),
        "B odd ldb": ((k + 7, 1), (n + 1, 1)),
        "both odd": ((k, 1), (n + 3, 1)),
        "column-major, odd": ((1, m + 1), (1, k + 5)),
        "no unit stride": ((2 * k, 2), (3 * n, 3)),
    }
    for name, ((rsa, csa), (rsb, csb)) in layouts.items():
        alpha, beta = (2, -1) if ta == "i8" else (1.5, -0.5)
        case = GemmCase(ta, tb, alpha, beta, m0=1, n0=1, k0=1, m1=m, n1=n, k1=k, rsa0=0, csa0=0, rsa1=rsa, csa1=csa,
                        rsb0=0, csb0=0, rsb1=rsb, csb1=csb, rsc0=0, csc0=0, rsc1=n + 2, csc1=1)
        check(gpu, "rc", case, 7000 + len(name), "device")


def test_host_threads_share_one_device(gpu):
    """The entry points are re-entrant like the reference's: host threads may call them at the same time on one
    device (here all on the default stream). Problems whose kernels hand data to each other through the library's
    per-device scratch memory - K shared between workgroups, operands copied into aligned memory, few columns - must
    not pick up each other's data. int8, so every result is compared bit for bit."""
    import threading
    from support import GemmCase

    def rc(m, n, k, rsa, csa, rsb, csb):
        return GemmCase("i8", None, 3, -2, m0=1, n0=1, k0=1, m1=m, n1=n, k1=k, rsa0=0, csa0=0, rsa1=rsa, csa1=csa,
                        rsb0=0, csb0=0, rsb1=rsb, csb1=csb, rsc0=0, csc0=0, rsc1=n, csc1=1)

    cases = [rc(16, 2048, 4096, 4096, 1, 2048, 1),      # few tiles, long K: partial sums in the workspace
             rc(300, 260, 777, 778, 1, 261, 1),         # odd leading dimensions: both operands copied
             rc(1037, 2, 1040, 1040, 1, 2, 1),          # matrix times two vectors, row-major B: B copied
             rc(24, 1024, 8192, 8192, 1, 1024, 1)]
    jobs = []
    for i, case in enumerate(cases):
        a, b, c = case.make_inputs(9100 + i)
        jobs.append((case, a, b, c, run_oracle_gemm(case, a, b, c)))
    failures = []

    def worker(t):
        try:
            for it in range(6):
                case, a, b, c, want = jobs[(t + it) % len(jobs)]
                got = run_gemm(gpu, "rc", case, a, b, c, "device")
                if not np.array_equal(got, want):
                    failures.append((t, it, (t + it) % len(jobs)))
        except Exception as e:  # noqa: BLE001 - reported by the assertion below
            failures.append((t, repr(e)))

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(4)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not failures, failures


def test_host_threads_on_streams_of_their_own(gpu):
    """Scratch memory (sums shared by the workgroups of a GEMV, partial sums of a shared K, operand copies) belongs
    to the launching stream, so host threads with a stream each may have their kernels run at the same time. Every
    thread enqueues its whole list of problems back to back, so that launches of different streams overlap on the
    device, and compares bit for bit (int8)."""
    import ctypes as ct
    import threading
    from skl_amd import DeviceBuffer
    from support import GemmCase

    hip = ct.CDLL("libamdhip64.so.7")
    hip.hipStreamCreate.restype = hip.hipStreamDestroy.restype = ct.c_int

    def rc(m, n, k, rsa, csa, rsb, csb):
        return GemmCase("i8", None, 1, 0, m0=1, n0=1, k0=1, m1=m, n1=n, k1=k, rsa0=0, csa0=0, rsa1=rsa, csa1=csa,
                        rsb0=0, csb0=0, rsb1=rsb, csb1=csb, rsc0=0, csc0=0, rsc1=n, csc1=1)

    cases = [rc(1, 4096, 8192, 8192, 1, 4096, 1),       # GEMV: workgroups meet in the zeroed scratch
             rc(4, 2048, 4096, 4096, 1, 2048, 1),       # a batch of four rows on the same scratch
             rc(16, 2048, 4096, 4096, 1, 2048, 1),      # few tiles, long K: partial sums in the workspace
             rc(300, 260, 777, 778, 1, 261, 1),         # odd leading dimensions: both operands copied
             rc(1037, 2, 1040, 1040, 1, 2, 1)]          # matrix times two vectors, row-major B: B copied
    jobs = []
    for i, case in enumerate(cases):
        a, b, c = case.make_inputs(9200 + i)
        jobs.append((case, a, b, c, run_oracle_gemm(case, a, b, c)))
    failures = []

    def worker(t):
        stream = ct.c_void_p()
        bufs = []
        try:
            assert hip.hipStreamCreate(ct.byref(stream)) == 0
            gpu.skl_hip_set_stream(stream.value)
            gpu.skl_hip_set_pointer_mode(1)
            for case, a, b, c, _ in jobs:
                bufs.append((DeviceBuffer.from_array(a), DeviceBuffer.from_array(b), DeviceBuffer.from_array(c)))
            for it in range(8):
                for rep in range(3):
                    for j in range(len(jobs)):
                        idx = (j + t) % len(jobs)
                        case = jobs[idx][0]
                        da, db, dc = bufs[idx]
                        gpu.skl_gemm_i8rc_i8rc_i32rc_gfx950(case.m1, case.n1, case.k1, 1, da, case.rsa1, case.csa1, db,
                                                           case.rsb1, case.csb1, 0, dc, case.rsc1, case.csc1)
                assert gpu.skl_hip_synchronize() == 0
                skl_amd.check_error()
                for idx, (case, a, b, c, want) in enumerate(jobs):
                    if not np.array_equal(bufs[idx][2].download(c.dtype, c.size), want):
                        failures.append((t, it, idx))
        except Exception as e:  # noqa: BLE001 - reported by the assertion below
            failures.append((t, repr(e)))
        finally:
            gpu.skl_hip_synchronize()
            gpu.skl_hip_set_stream(None)
            gpu.skl_hip_set_pointer_mode(0)
            for trio in bufs:
                for d in trio:
                    d.free()
            if stream:
                gpu.skl_hip_release_stream(stream.value)
                hip.hipStreamDestroy(stream)

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(4)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not failures, failures


@pytest.mark.parametrize("mode", MODES)
def test_block4x8x4_entry_point(gpu, mode):
    """`skl_gemm_a1b01_i8p4x8_i8p8x4_i32p4x4` (documented by the reference without an implementation): small
    problems on the any-stride kernel, larger ones through aligned copies on the matrix cores; block rows with
    gaps between them; C = A*B and C += A*B; empty dimensions. Whole C buffer compared bit for bit."""
    from test_oracle_gemm import block4x8x4_case
    shapes = [(1, 1, 1, 0), (3, 2, 5, 7), (0, 2, 2, 0), (2, 0, 2, 0), (2, 2, 0, 0), (64, 96, 40, 0), (33, 50, 129, 48),
              (256, 8, 64, 16),
              # whole 256-row tiles: the streaming kernel, which writes the 4 x 4 blocks of C 16 bytes per lane (256 x 128
              # and 256 x 256 tiles); with a gap that keeps block rows on 16-byte boundaries and one that does not
              (512, 384, 32, 0), (512, 384, 16, 16), (512, 384, 16, 2), (1024, 832, 16, 0)]
    for i, (m1, n1, k1, gap) in enumerate(shapes):
        for accum in (False, True):
            case = block4x8x4_case(m1, n1, k1, 32 * k1 + gap, 32 * n1 + gap, 16 * n1 + gap, accum)
            a, b, c = case.make_inputs(8100 + i)
            want = run_oracle_gemm(case, a, b, c)
            if mode == "host":
                got = c.copy()
                gpu.skl_gemm_a1b01_i8p4x8_i8p8x4_i32p4x4_gfx950(m1, n1, k1, a, case.rsa1, b, case.rsb1, got, case.rsc1, accum)
                skl_amd.check_error()
            else:
                bufs = [skl_amd.DeviceBuffer.from_array(x) for x in (a, b, c)]
                gpu.skl_gemm_a1b01_i8p4x8_i8p8x4_i32p4x4_gfx950(m1, n1, k1, bufs[0], case.rsa1, bufs[1], case.rsb1, bufs[2],
                                                                case.rsc1, accum)
                assert gpu.skl_hip_synchronize() == 0
                skl_amd.check_error()
                got = bufs[2].download(c.dtype, c.size)
                for d in bufs:
                    d.free()
            assert np.array_equal(got, want), (m1, n1, k1, gap, accum)


@pytest.mark.parametrize("ta,tb", (("i8", "i8"), ("bf16", "bf16"), ("f16", "f16"), ("f8e4m3", "f8e4m3"), ("f8e5m2", "f8e5m2")))
def test_blockings_no_kernel_reads_in_place(gpu, ta, tb):
    """Blocks of other sizes than 1, 64 or the whole matrix (3 x 5 x 7, 32 x 32 x 16 column-major blocks with
    gaps, the 4 x 8 x 4 format): operands copied, C unpacked, multiplied and packed back. beta != 0 and beta == 0;
    gaps in C must come back untouched."""
    from support import GemmCase
    blockings = [
        dict(m0=3, n0=5, k0=7, m1=40, n1=30, k1=20, rsa0=7, csa0=1, rsa1=7 * 3 * 20 + 4, csa1=21, rsb0=5, csb0=1,
             rsb1=5 * 7 * 30 + 1, csb1=35, rsc0=5, csc0=1, rsc1=15 * 30 + 3, csc1=15),
        dict(m0=32, n0=32, k0=16, m1=5, n1=6, k1=9, rsa0=1, csa0=32, rsa1=512, csa1=5 * 512, rsb0=1, csb0=16,
             rsb1=512, csb1=9 * 512 + 16, rsc0=1, csc0=33, rsc1=33 * 32, csc1=5 * 33 * 32),
    ]
    for i, blk in enumerate(blockings):
        for alpha, beta in (((2, -1) if ta == "i8" else (1.5, -0.5)), ((1, 0) if ta == "i8" else (1.0, 0.0))):
            case = GemmCase(ta, tb, alpha, beta, **blk)
            check(gpu, "rcprc", case, 8200 + i, "device")


@pytest.mark.parametrize("ta", ("f32", "f64", "f16h"))
def test_register_tiled_kernel_bit_identical(gpu, ta):
    """f32, f64 and f16 -> f16 on the register-tiled kernel: the same bits as the checker over the whole C buffer.
    Both tile sizes (64 x 64; 128 x 128 from 512 tiles on), every pairing of row- and column-major operands, 64-row
    panels, ragged edges in M, N and K, K shorter than one slab, beta == 0 and != 0."""
    from support import GemmCase
    te = support.TE

    def rc(m, n, k, a_rows, b_rows, alpha, beta):
        rsa, csa = (k + 3, 1) if a_rows else (1, m + 1)
        rsb, csb = (n + 2, 1) if b_rows else (1, k + 5)
        return GemmCase(ta, None, alpha, beta, m0=1, n0=1, k0=1, m1=m, n1=n, k1=k, rsa0=0, csa0=0, rsa1=rsa, csa1=csa,
                        rsb0=0, csb0=0, rsb1=rsb, csb1=csb, rsc0=0, csc0=0, rsc1=n + 1, csc1=1)

    cases = []
    for a_rows in (True, False):
        for b_rows in (True, False):
            cases.append(rc(130, 203, 77, a_rows, b_rows, 1.5, -0.5))
            cases.append(rc(64, 64, 5, a_rows, b_rows, 1.0, 0.0))
    cases.append(rc(2890, 2950, 24, True, True, 0.5, 2.0))     # 128 x 128 tiles, ragged
    cases.append(rc(2944, 2944, 9, False, True, 1.0, 0.0))
    # 64-row panels of A and B, 64 x 64 blocks of C (the panel entry points' layout)
    m1, n1, k = 3, 5, 50
    cases.append(GemmCase(ta, None, 2.0, 1.0, m0=te, n0=te, k0=1, m1=m1, n1=n1, k1=k, rsa0=1, csa0=0, rsa1=k * te, csa1=te,
                          rsb0=0, csb0=1, rsb1=te, csb1=k * te, rsc0=te, csc0=1, rsc1=n1 * te * te, csc1=te * te))
    for i, case in enumerate(cases):
        a, b, c = case.make_inputs(9300 + i)
        want = run_oracle_gemm(case, a, b, c)
        got = run_gemm(gpu, "rcprc", case, a, b, c, "device")
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), (ta, i, vars(case))


@pytest.mark.parametrize("ta,tb", (("i8", "i8"), ("bf16", "bf16"), ("f16", "f16"), ("f8e4m3", "f8e4m3"), ("f8e4m3", "f8e5m2")))
def test_ragged_problems_on_padded_copies(gpu, ta, tb):
    """Ragged M, N and K (and odd leading dimensions) on a problem large enough to fill the chip: A and B are copied
    into tile-padded scratch memory and the streaming kernel runs with an epilogue that stops at C's true edges.
    256 x 128 and 256 x 256 tiles, row- and column-major operands, beta == 0 and != 0, C with padded rows (the
    clobber check), fused bias and maximum. int8 bit-exact, floating point inside the reference's bound."""
    from support import GemmCase
    fp8 = ta.startswith("f8")
    shapes = [(1500, 2100, 500 if ta == "i8" or fp8 else 250, True, True),      # 6 x 17 tiles of 256 x 128
              (3300, 4000, 250 if ta == "i8" or fp8 else 125, False, False),    # 13 x 16 tiles of 256 x 256
              (1537, 2049, 1000, True, False)]
    for i, (m, n, k, a_rows, b_rows) in enumerate(shapes):
        rsa, csa = (k + 1, 1) if a_rows else (1, m + 3)
        rsb, csb = (n + 5, 1) if b_rows else (1, k + 7)
        alpha, beta = ((2, -1) if ta == "i8" else (1.5, -0.5)) if i != 1 else ((1, 0) if ta == "i8" else (1.0, 0.0))
        case = GemmCase(ta, tb, alpha, beta, m0=1, n0=1, k0=1, m1=m, n1=n, k1=k, rsa0=0, csa0=0, rsa1=rsa, csa1=csa,
                        rsb0=0, csb0=0, rsb1=rsb, csb1=csb, rsc0=0, csc0=0, rsc1=n + 3, csc1=1)
        a, b, c = case.make_inputs(9500 + i)
        got = run_gemm(gpu, "rc", case, a, b, c, "device")
        if case.is_int:
            want = run_oracle_gemm(case, a, b, c)
            assert np.array_equal(got, want), (m, n, k)
        else:
            support.assert_fp_gemm_close(case, a, b, c, got, extra_rel=support.FP8_MFMA_REL if fp8 else 0.0)
        if i == 0 and ta == tb:
            rng = np.random.default_rng(i)
            bias = (rng.integers(-99, 99, n).astype(np.int32) if case.is_int else rng.uniform(-4, 4, n).astype(np.float32))
            start = np.array([-(1 << 31)], np.int32) if case.is_int else np.array([-np.inf], np.float32)
            fused, top = run_fused_gemm(gpu, "rc", case, a, b, c, bias, start, "device")
            want_c, want_top = fused_expectation(case, got, bias, start)
            assert np.array_equal(fused.view(np.uint8), want_c.view(np.uint8)), (ta, m, n, k)
            assert top[0] == want_top[0]


@pytest.mark.parametrize("ta", ("i8", "bf16", "f8e4m3"))
def test_streaming_kernel_shares_k_when_tiles_fill_half_the_chip(gpu, ta):
    """96 to 128 tiles of 256 x 128: two workgroups per tile take half of K each, a second pass adds the planes and
    applies alpha / beta and the fused steps. Whole tiles in place and a ragged problem on padded copies. int8
    bit-exact; floating point inside the bound and the same bits on two runs."""
    from support import GemmCase
    k = 8192 if ta != "bf16" else 4096  # 8 KiB of K per row: the shortest K that is shared
    for i, (m, n, kk, ld_extra) in enumerate(((1536, 2048, k, 0), (1500, 2040, k - 40, 1), (256, 11008, k, 0))):  # 96, 96, 86 tiles
        case = GemmCase(ta, None, 2 if ta == "i8" else 1.5, -1 if ta == "i8" else -0.5, m0=1, n0=1, k0=1, m1=m, n1=n, k1=kk,
                        rsa0=0, csa0=0, rsa1=kk + ld_extra, csa1=1, rsb0=0, csb0=0, rsb1=n + ld_extra, csb1=1,
                        rsc0=0, csc0=0, rsc1=n + 2, csc1=1)
        a, b, c = case.make_inputs(9700 + i)
        got = run_gemm(gpu, "rc", case, a, b, c, "device")
        if case.is_int:
            # 25 G multiply-adds are minutes of the scalar checker; every partial sum here is below 2^53, so the
            # fp64 matrix product of the widened operands is the exact integer result
            A, B, C, oc = case.dense(a, b, c)
            want = c.copy()
            want[oc] = (case.alpha * (A @ B) + case.beta * C).astype(np.int64).astype(np.int32)
            assert np.array_equal(got, want), (m, n, kk)
        else:
            support.assert_fp_gemm_close(case, a, b, c, got, extra_rel=support.FP8_MFMA_REL if ta.startswith("f8") else 0.0)
            assert np.array_equal(got.view(np.uint8), run_gemm(gpu, "rc", case, a, b, c, "device").view(np.uint8))
        rng = np.random.default_rng(i)
        bias = (rng.integers(-99, 99, n).astype(np.int32) if case.is_int else rng.uniform(-4, 4, n).astype(np.float32))
        start = np.array([-(1 << 31)], np.int32) if case.is_int else np.array([-np.inf], np.float32)
        fused, top = run_fused_gemm(gpu, "rc", case, a, b, c, bias, start, "device")
        want_c, want_top = fused_expectation(case, got, bias, start)
        assert np.array_equal(fused.view(np.uint8), want_c.view(np.uint8)), (ta, m, n, kk)
        assert top[0] == want_top[0]
