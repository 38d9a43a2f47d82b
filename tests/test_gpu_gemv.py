"""GPU parity of the M == 1 streaming path with the CPU checker (bit-exact:
integer sums are order-independent), at the benchmark configuration 2 shape and around
the kernel's tiling edges, including back-to-back calls that share the
library's zero-initialised reduction scratch."""
import numpy as np
import pytest

import skl_amd
import support
from gpu_support import run_gemm
from support import GemmCase, colmajor_a_case, rowmajor_case, run_oracle_gemm

pytestmark = pytest.mark.gpu


def test_config2_decode_shape_bit_exact(gpu):
    """1 x 4096 times 4096 x 11008, int8 -> int32, beta = 0."""
    case = rowmajor_case("i8", 1, 11008, 4096, 1, 0)
    a, b, c = case.make_inputs(0x5EED0020)
    want = run_oracle_gemm(case, a, b, c)
    for mode in ("device", "host"):
        got = run_gemm(gpu, "rowmajor", case, a, b, c, mode)
        assert np.array_equal(got, want)
    # independent of the checker: exact integer matmul in numpy
    ref = a.astype(np.int64)[None, :] @ b.reshape(4096, 11008).astype(np.int64)
    assert np.array_equal(want, ref.ravel().astype(np.int32))


def test_back_to_back_calls_reuse_scratch(gpu):
    """Three calls in a row, shrinking shapes, accumulating into the same y: the
    scratch accumulators and tickets must be back at zero after every call."""
    rng = np.random.default_rng(3)
    y = rng.integers(-1000, 1000, size=11008).astype(np.int32)
    dy = skl_amd.DeviceBuffer.from_array(y)
    want = y.copy()
    for (n, k, alpha, beta) in ((11008, 4096, 1, 1), (4096, 1000, -3, 2), (1024, 128, 7, -1), (16, 4, 1, 0)):
        case = rowmajor_case("i8", 1, n, k, alpha, beta)
        a, b, _ = case.make_inputs(n + k)
        da, db = skl_amd.DeviceBuffer.from_array(a), skl_amd.DeviceBuffer.from_array(b)
        gpu.skl_gemm_i8_i8_i32_gfx950(1, n, k, alpha, da, k, db, n, beta, dy, n)
        gpu.skl_hip_synchronize()
        skl_amd.check_error()
        want = run_oracle_gemm(case, a, b, want)
        assert np.array_equal(dy.download(np.int32), want), (n, k)
        da.free(), db.free()


@pytest.mark.parametrize("n,k", ((16, 1), (1024, 127), (1040, 129), (2048, 4), (33 * 16, 1000), (11008, 4095)))
def test_tiling_edges(gpu, n, k):
    case = rowmajor_case("i8", 1, n, k, alpha=0x01010101, beta=-77, rsb=n + 32, rsc=n)
    a, b, c = case.make_inputs(n * 7 + k)
    c[:] = np.random.default_rng(k).integers(-2 ** 31, 2 ** 31, size=c.size)
    assert np.array_equal(run_gemm(gpu, "rowmajor", case, a, b, c, "device"), run_oracle_gemm(case, a, b, c))


def test_strided_x_and_y(gpu):
    """x read with a stride (column-major A with m = 1) and y written with a
    stride (column-major-like C): gaps in y must be preserved."""
    n, k = 2048, 300
    case = GemmCase("i8", None, 2, 3, m0=1, n0=1, k0=1, m1=1, n1=n, k1=k, rsa0=0, csa0=0, rsa1=1, csa1=5,
                    rsb0=0, csb0=0, rsb1=n, csb1=1, rsc0=0, csc0=0, rsc1=1, csc1=3)
    a, b, c = case.make_inputs(99)
    assert np.array_equal(run_gemm(gpu, "rc", case, a, b, c, "device"), run_oracle_gemm(case, a, b, c))


def test_panel_packed_weights(gpu):
    """B in 1 x TE row panels (B_p[j/64][k][j%64]) with one block row of A."""
    te = support.TE
    k, n1 = 200, 5
    case = GemmCase("i8", None, 1, 0, m0=1, n0=te, k0=1, m1=1, n1=n1, k1=k, rsa0=0, csa0=0, rsa1=k, csa1=1,
                    rsb0=0, csb0=1, rsb1=te, csb1=k * te, rsc0=0, csc0=1, rsc1=n1 * te, csc1=te)
    a, b, c = case.make_inputs(5)
    assert np.array_equal(run_gemm(gpu, "rcprc", case, a, b, c, "device"), run_oracle_gemm(case, a, b, c))


def test_m1_shapes_outside_the_streaming_kernel(gpu):
    """N not a multiple of 16 or a misaligned row stride: served by another
    kernel, same answer (test/gemm/rvv/skl_gemm_i8_i8_i32_zve32x_x390.c:64)."""
    for (n, k, rsb) in ((33, 31, 33), (255, 12, 255), (256, 31, 257)):
        case = rowmajor_case("i8", 1, n, k, 1, 1, rsb=rsb)
        a, b, c = case.make_inputs(n + k)
        assert np.array_equal(run_gemm(gpu, "rowmajor", case, a, b, c, "device"), run_oracle_gemm(case, a, b, c))


@pytest.mark.parametrize("ta", ("bf16", "f16"))
@pytest.mark.parametrize("n,k", ((256, 12), (256, 31), (1024, 1000), (11008, 4096)))
def test_16bit_decode_shapes(gpu, ta, n, k):
    """bf16 / f16 weights, fp32 accumulation: the M = 1 rows of the reference's suites
    (test/gemm/rvv/skl_gemm_f16_f16_f32_zvfh_x390.c:66-72) and the decode shape. The
    order of the sum over k differs from the reference's k-ascending loop - compared through the reference's
    elementwise bound - but it is a fixed order: every run gives the same bits."""
    case = rowmajor_case(ta, 1, n, k, 1.5, -0.5)
    a, b, c = case.make_inputs(n + k)
    runs = []
    for _ in range(3):   # more than once: the tickets must come back clean, and the sums in the same order
        got = run_gemm(gpu, "rowmajor", case, a, b, c, "device")
        support.assert_fp_gemm_close(case, a, b, c, got)
        runs.append(got)
    assert all(np.array_equal(r.view(np.uint8), runs[0].view(np.uint8)) for r in runs[1:])


@pytest.mark.parametrize("n,k1", ((64, 1), (128, 4), (192, 3), (256, 17), (11008, 1024)))
def test_k_packed_int8_decode(gpu, n, k1):
    """The dot4 layout with M = 1 (src/gemm/gemm_i8rcp1x4_i8p4x1c_i32_xsfvqdotq.c:645-660
    dispatches this case to its own GEMV kernels): A 1 x 4 K-blocks, B 4 x 1 K-blocks."""
    case = support.dot4_case(1, n, k1, alpha=-3, beta=5)
    a, b, c = case.make_inputs(n * 3 + k1)
    for mode in ("device", "host"):
        assert np.array_equal(run_gemm(gpu, "dot4", case, a, b, c, mode), run_oracle_gemm(case, a, b, c))


@pytest.mark.parametrize("m", (2, 3, 7, 16, 17, 33, 48, 100, 112, 128, 129, 200, 257))
def test_k_packed_int8_decode_batches(gpu, m):
    """The dot4 layout with 2 or more rows of A (src/gemm/gemm_i8rcp1x4_i8p4x1c_i32_xsfvqdotq.c:645-660 has its own
    kernels for these): the K-packed B is read in place by the decode-batch kernels - four loads give a lane 16 k of
    four columns, no transposes; B stays in registers for up to eight groups of 16 rows (ragged last group: 17, 33,
    100), more rows go through in chunks of 128 (a last chunk of one row through the one-row kernel: 129, 257).
    K <= 4096: one workgroup per 64 columns takes all of K and writes C once; beyond (one shape here) workgroups
    share a column tile and meet in C. Problems with few column tiles (the reference's own benchmark shape, 126 x 128
    with k1 = 64, test/gemm/xsfvqdotq/skl_gemm_i8rcp1x4_i8p4x1c_i32_xsfvqdotq.c:56) run a workgroup per tile and group of
    16 rows. The config-2 weights prepacked, N and K off the kernel's 1024 x 64
    blocks, padded strides of A, B and C, alpha / beta with wrap-around, both pointer modes; whole-buffer compare."""
    rng = np.random.default_rng(600 + m)
    shapes = [(11008, 1024, 0, 0, 0), (4100, 132, 16, 32, 5), (2052, 516, 48, 16, 0),
              (128, 64, 0, 0, 0), (132, 68, 16, 16, 3)]  # few column tiles: a workgroup per tile and group of 16 rows
    if m in (7, 100):
        shapes.append((1028, 1284, 16, 0, 3))  # K = 5136 > 4096: the sums of a column tile meet in C, not in LDS
    for (n, k1, pad_a, pad_b, pad_c) in shapes:
        for alpha, beta in ((1, 0), (0x01010101, -77), (-3, 1)):
            case = support.dot4_case(m, n, k1, alpha=alpha, beta=beta, rsa1=4 * k1 + pad_a, rsb1=4 * n + pad_b,
                                     rsc1=n + pad_c)
            a, b, c = case.make_inputs(int(rng.integers(1 << 30)))
            c[:] = rng.integers(-2 ** 31, 2 ** 31, size=c.size)
            want = run_oracle_gemm(case, a, b, c)
            for mode in ("device", "host"):
                assert np.array_equal(run_gemm(gpu, "dot4", case, a, b, c, mode), want), (m, n, k1, alpha, beta, mode)


@pytest.mark.parametrize("m", (300, 600, 1100))
def test_k_packed_int8_many_rows(gpu, m):
    """The dot4 layout with more rows of A than the decode-batch kernels take in two passes over B: the K-packed B is
    copied into rows contiguous in K - as 32-bit groups that is a transpose - and the tile kernels run on the copy
    (A, K-contiguous already, is copied alongside; C is updated where it lies). Padded strides of A, B and C, alpha /
    beta with wrap-around, both pointer modes; whole-buffer compare."""
    rng = np.random.default_rng(900 + m)
    for (n, k1, pad_a, pad_b, pad_c) in ((4100, 132, 16, 32, 5), (2052, 516, 48, 16, 0), (1024, 256, 0, 0, 0)):
        for alpha, beta in ((1, 0), (0x01010101, -77)):
            case = support.dot4_case(m, n, k1, alpha=alpha, beta=beta, rsa1=4 * k1 + pad_a, rsb1=4 * n + pad_b,
                                     rsc1=n + pad_c)
            a, b, c = case.make_inputs(int(rng.integers(1 << 30)))
            c[:] = rng.integers(-2 ** 31, 2 ** 31, size=c.size)
            want = run_oracle_gemm(case, a, b, c)
            for mode in ("device", "host"):
                assert np.array_equal(run_gemm(gpu, "dot4", case, a, b, c, mode), want), (m, n, k1, alpha, beta, mode)


def _exact_int8_gemv(x, w, k, n):
    """x (k) times row-major w (k x n) in exact integer arithmetic, through fp64 BLAS in slices of K."""
    acc = np.zeros(n, np.float64)
    for k0 in range(0, k, 2048):
        k1 = min(k, k0 + 2048)
        acc += x[k0:k1].astype(np.float64) @ w[k0 * n:k1 * n].reshape(k1 - k0, n).astype(np.float64)
    return acc.astype(np.int64).astype(np.int32)


def test_long_streams_take_sixteen_loads_per_lane(gpu):
    """A stream of more than two rounds of workgroups (here 138 MB of int8 / fp8 weights, 143 MB of bf16, 134 MB in
    the K-packed layout) runs with sixteen loads per lane and groups of 1024 rows: ragged K against those groups,
    int8 bit for bit, floating point inside the reference's bound."""
    rng = np.random.default_rng(88)
    n, k = 8192, 16900
    x, w = rng.integers(-128, 128, k, dtype=np.int8), rng.integers(-128, 128, k * n, dtype=np.int8)
    case = rowmajor_case("i8", 1, n, k, -3, 5)
    c = rng.integers(-2 ** 31, 2 ** 31, size=n).astype(np.int32)
    want = (5 * c.astype(np.int64) - 3 * _exact_int8_gemv(x, w, k, n).astype(np.int64)).astype(np.int32)
    assert np.array_equal(run_gemm(gpu, "rowmajor", case, x, w, c, "device"), want)
    k1 = 4100  # K-packed: B(4P + p, j) at P * 4n + 4j + p
    case = support.dot4_case(1, n, k1, alpha=1, beta=0)
    a, b, c = case.make_inputs(3)
    assert np.array_equal(run_gemm(gpu, "dot4", case, a, b, c, "device"), run_oracle_gemm(case, a, b, c))
    for ta, kk in (("bf16", 8712), ("f8e4m3", 16900)):
        case = rowmajor_case(ta, 1, n, kk, 1.5, -0.5)
        a, b, c = case.make_inputs(kk)
        support.assert_fp_gemm_close(case, a, b, c, run_gemm(gpu, "rc", case, a, b, c, "device"))


@pytest.mark.parametrize("m", (2, 3, 4, 5, 6, 7, 8))
def test_small_batch_rows_bit_exact(gpu, m):
    """2 to 8 rows of A against a row-major int8 B (the streaming kernel that shares the byte transposes
    between the rows): the config-2 shape, ragged K, tiling edges, padded row strides of A, B and C,
    alpha / beta with wrap-around, and back-to-back calls on the shared reduction scratch."""
    rng = np.random.default_rng(40 + m)
    shapes = ((11008, 4096, 0, 0, 0), (1040, 129, 0, 32, 16), (16, 4, 4, 0, 0), (2048, 1000, 24, 16, 48),
              (33 * 16, 515, 0, 0, 0))
    for (n, k, pad_a, pad_b, pad_c) in shapes:
        for alpha, beta in ((1, 0), (0x01010101, -77)):
            case = rowmajor_case("i8", m, n, k, alpha, beta, rsa=k + pad_a if (k + pad_a) % 4 == 0 else None,
                                 rsb=n + pad_b, rsc=n + pad_c)
            a, b, c = case.make_inputs(int(rng.integers(1 << 30)))
            c[:] = rng.integers(-2 ** 31, 2 ** 31, size=c.size)
            want = run_oracle_gemm(case, a, b, c)
            for mode in ("device", "host"):
                assert np.array_equal(run_gemm(gpu, "rowmajor", case, a, b, c, mode), want), (m, n, k, mode)


@pytest.mark.parametrize("m", (4, 5, 8, 9, 13, 16, 17, 25, 32, 33, 64, 128))
def test_decode_batch_on_the_matrix_cores_bit_exact(gpu, m):
    """4 to 32 rows of A against a row-major int8 B of at least 1 MiB (the stream over B whose multiply-adds run
    on the matrix cores and whose workgroups add into C with atomics; beyond 16 rows in two groups of 16 with B held
    in registers, ragged second group: 17, 25), and row counts beyond, which the tile kernels take: the config-2 weights, K and N off the kernel's 512 x 256 blocks, a K
    of a single block, padded row strides of A, B and C (whole-buffer compare: the padding must survive), beta 0 / 1 /
    other with wrap-around, a C full of extreme values, both pointer modes."""
    rng = np.random.default_rng(400 + m)
    shapes = ((11008, 4096, 0, 0, 0), (4112, 528, 16, 32, 16), (16 * 4099, 16, 0, 0, 3), (2064, 1008, 48, 16, 48),
              (256, 4096, 0, 0, 0))
    if m > 16:  # the checker's time grows with m: the config-2 width at a quarter of its K, and no 65 584-column case
        shapes = ((11008, 1040, 0, 0, 0),) + shapes[1:2] + shapes[3:]
    for (n, k, pad_a, pad_b, pad_c) in shapes:
        for alpha, beta in ((1, 0), (0x01010101, -77), (-3, 1)):
            case = rowmajor_case("i8", m, n, k, alpha, beta, rsa=k + pad_a, rsb=n + pad_b, rsc=n + pad_c)
            a, b, c = case.make_inputs(int(rng.integers(1 << 30)))
            c[:] = rng.integers(-2 ** 31, 2 ** 31, size=c.size)
            want = run_oracle_gemm(case, a, b, c)
            for mode in ("device", "host"):
                assert np.array_equal(run_gemm(gpu, "rowmajor", case, a, b, c, mode), want), (m, n, k, alpha, beta, mode)


def test_decode_batch_on_the_matrix_cores_panels_and_strided_c(gpu):
    """The same kernel with a column-major C through the full-stride entry point, and with B in panels of 64
    columns (the 1 x TE panel format) through the blocked one."""
    rng = np.random.default_rng(77)
    m, n, k = 12, 2560, 1024
    case = GemmCase("i8", None, 3, -5, m0=1, n0=1, k0=1, m1=m, n1=n, k1=k, rsa0=0, csa0=0, rsa1=k, csa1=1,
                    rsb0=0, csb0=0, rsb1=n, csb1=1, rsc0=0, csc0=0, rsc1=1, csc1=m + 3)
    a, b, c = case.make_inputs(6)
    c[:] = rng.integers(-2 ** 31, 2 ** 31, size=c.size)
    assert np.array_equal(run_gemm(gpu, "rc", case, a, b, c, "device"), run_oracle_gemm(case, a, b, c))
    # B in panels of 64 columns with 16 rows of A: blocked description, m0 = 16 rows in one block
    n1 = 40
    case = GemmCase("i8", None, 1, 0, m0=16, n0=64, k0=1, m1=1, n1=n1, k1=k, rsa0=k, csa0=0, rsa1=16 * k, csa1=1,
                    rsb0=0, csb0=1, rsb1=64, csb1=k * 64, rsc0=64 * n1, csc0=1, rsc1=16 * 64 * n1, csc1=64)
    a, b, c = case.make_inputs(7)
    assert np.array_equal(run_gemm(gpu, "rcprc", case, a, b, c, "device"), run_oracle_gemm(case, a, b, c))


@pytest.mark.parametrize("ta,tb", (("f8e4m3", "f8e4m3"), ("f8e5m2", "f8e5m2"), ("f8e4m3", "f8e5m2")))
@pytest.mark.parametrize("m", (2, 7, 16))
def test_decode_batch_on_the_matrix_cores_fp8(gpu, ta, tb, m):
    """The fp8 kinds of the same kernel (raw sums in planes, a second pass adds them in order): the reference's
    bound widened by the accuracy of the fp8 matrix-core instructions, shapes off the kernel's blocks, padded
    strides, the same bits on a second run, and the fused steps (bias, maximum) applied to the same sums."""
    from gpu_support import run_fused_gemm
    from test_oracle_gemm import fused_expectation
    for (n, k, pad) in ((11008, 4096, 0), (4112, 528, 16), (2064, 1008, 48)):
        case = rowmajor_case(ta, m, n, k, 1.5, -0.5, tb=tb, rsa=k + pad, rsb=n + pad, rsc=n + pad)
        a, b, c = case.make_inputs(m * 100 + n + k)
        # two or three rows against less than 12 MiB of B run on the kernel with fp32 multiply-adds (a fixed order
        # too, but not the sums of the fused call)
        here = m >= 4 or n * k >= (12 << 20)
        for mode in ("device", "host"):
            got = run_gemm(gpu, "rc", case, a, b, c, mode)
            support.assert_fp_gemm_close(case, a, b, c, got, extra_rel=support.FP8_MFMA_REL)
            assert np.array_equal(got.view(np.uint8), run_gemm(gpu, "rc", case, a, b, c, mode).view(np.uint8))
        if ta != tb or not here:
            continue  # the mixed pair has no fused entry point
        bias = (np.arange(n) % 7 - 3).astype(np.float32)
        start = np.array([-np.inf], np.float32)
        plain = run_gemm(gpu, "rc", case, a, b, c, "device")
        got, top = run_fused_gemm(gpu, "rc", case, a, b, c, bias, start, "device")
        want_c, want_top = fused_expectation(case, plain, bias, start)
        assert np.array_equal(got.view(np.uint8), want_c.view(np.uint8))
        assert top[0] == want_top[0]


@pytest.mark.parametrize("ta", ("bf16", "f16"))
@pytest.mark.parametrize("m", (2, 7, 16))
def test_decode_batch_on_the_matrix_cores_16bit(gpu, ta, m):
    """bf16 / f16 on the same kernel (8 x 8 halfword transposes, v_mfma_f32_16x16x32): products are exact in fp32
    and the sums are fp32, so the reference's own bound holds; shapes off the kernel's 512 x 128 blocks, padded
    strides, the same bits on a second run and with the fused steps."""
    from gpu_support import run_fused_gemm
    from test_oracle_gemm import fused_expectation
    for (n, k, pad) in ((11008, 4096, 0), (4104, 520, 8), (2056, 1000, 24)):
        case = rowmajor_case(ta, m, n, k, 1.5, -0.5, rsa=k + pad, rsb=n + pad, rsc=n + pad)
        a, b, c = case.make_inputs(m * 100 + n + k)
        # two or three rows against less than 12 MiB of B run on the kernel with fp32 multiply-adds (a fixed order
        # too, but not the sums of the fused call)
        here = m >= 4 or 2 * n * k >= (12 << 20)
        for mode in ("device", "host"):
            got = run_gemm(gpu, "rc", case, a, b, c, mode)
            support.assert_fp_gemm_close(case, a, b, c, got)
            assert np.array_equal(got.view(np.uint8), run_gemm(gpu, "rc", case, a, b, c, mode).view(np.uint8))
        if not here:
            continue
        bias = (np.arange(n) % 7 - 3).astype(np.float32)
        start = np.array([-np.inf], np.float32)
        plain = run_gemm(gpu, "rc", case, a, b, c, "device")
        got, top = run_fused_gemm(gpu, "rc", case, a, b, c, bias, start, "device")
        want_c, want_top = fused_expectation(case, plain, bias, start)
        assert np.array_equal(got.view(np.uint8), want_c.view(np.uint8))
        assert top[0] == want_top[0]


def test_decode_batch_on_the_matrix_cores_16bit_one_hot(gpu):
    """Rows of A with a single 1.0 each: row i of C is row p_i of B widened to fp32, exactly and in the right
    columns, for positions in every lane group and every halfword of a lane's eight."""
    m, n, k = 16, 4096, 256
    rng = np.random.default_rng(5)
    for ta in ("bf16", "f16"):
        b = support.ETYPES[ta].gen(rng, k * n)
        wide = support.ETYPES[ta].widen(b).reshape(k, n)
        one = 0x3F80 if ta == "bf16" else 0x3C00
        for base in (0, 3, 32 + 8, 128 + 48 - 15):
            a = np.zeros(m * k, np.uint16)
            for i in range(m):
                a[i * k + base + i] = one
            case = rowmajor_case(ta, m, n, k, 1.0, 0.0)
            got = run_gemm(gpu, "rc", case, a, b, np.zeros(m * n, np.float32), "device").reshape(m, n)
            for i in range(m):
                assert np.array_equal(got[i].astype(np.float64), wide[base + i]), (ta, base, i)


def test_decode_batch_on_the_matrix_cores_decodes_fp8_exactly(gpu):
    """A = rows of one-hot vectors (1.0 at position p of row i), alpha = 1, beta = 0: row i of C is row p_i of B
    decoded to fp32 - every finite code of both formats must come out as the format defines it, in its column,
    whichever lane group and half of the instruction its k falls into."""
    m, n, k = 16, 4096, 256
    for ta, tb in (("f8e4m3", "f8e4m3"), ("f8e5m2", "f8e5m2"), ("f8e4m3", "f8e5m2")):
        one = 0x38 if ta == "f8e4m3" else 0x3C
        table = support.decode_table(tb)
        finite_codes = np.flatnonzero(np.isfinite(table)).astype(np.uint8)  # 0 * Inf would spoil whole columns
        b = finite_codes[(np.arange(k * n) * 7 + np.arange(k * n) // n) % finite_codes.size].astype(np.uint8)
        for base in (0, 5, 64 + 8, 128 + 48 - 15):
            a = np.zeros(m * k, np.uint8)
            for i in range(m):
                a[i * k + base + i] = one
            case = rowmajor_case(ta, m, n, k, 1.0, 0.0, tb=tb)
            got = run_gemm(gpu, "rc", case, a, b, np.zeros(m * n, np.float32), "device").reshape(m, n)
            for i in range(m):
                p = base + i
                assert np.array_equal(got[i].astype(np.float64), table[b[p * n:(p + 1) * n]]), (ta, tb, base, i)


def test_small_batch_unaligned_rows_fall_back(gpu):
    """Rows of A that are not 4-byte aligned (odd row stride) are served by the tile kernels: same result."""
    case = rowmajor_case("i8", 4, 1024, 131, 3, 2, rsa=133)
    a, b, c = case.make_inputs(77)
    assert np.array_equal(run_gemm(gpu, "rowmajor", case, a, b, c, "device"), run_oracle_gemm(case, a, b, c))


FP8_PAIRS = (("f8e4m3", "f8e4m3"), ("f8e5m2", "f8e5m2"), ("f8e4m3", "f8e5m2"))


@pytest.mark.parametrize("ta,tb", FP8_PAIRS)
def test_fp8_rows_of_b_are_decoded_exactly(gpu, ta, tb):
    """x = one-hot (1.0 at position p), alpha = 1, beta = 0: y is row p of B decoded to fp32. Every code
    of the format (NaN codes aside) must come out as the format defines it, in the right column."""
    n, k = 256, 24
    one = 0x38 if ta == "f8e4m3" else 0x3C
    table = support.decode_table(tb)
    finite_codes = np.flatnonzero(np.isfinite(table)).astype(np.uint8)  # 0 * Inf would spoil whole columns
    b = np.zeros(k * n, np.uint8)
    for p in range(k):
        b[p * n:(p + 1) * n] = finite_codes[(np.arange(n) * (2 * p + 1) + 5 * p) % finite_codes.size]
    assert set(b.tolist()) == set(finite_codes.tolist())
    for p in (0, 7, 8, 23):
        x = np.zeros(k, np.uint8)
        x[p] = one
        case = rowmajor_case(ta, 1, n, k, 1.0, 0.0, tb=tb)
        got = run_gemm(gpu, "rc", case, x, b, np.zeros(n, np.float32), "device")
        assert np.array_equal(got.astype(np.float64), table[b[p * n:(p + 1) * n]]), (ta, tb, p)


@pytest.mark.parametrize("ta,tb", FP8_PAIRS)
@pytest.mark.parametrize("n,k", ((11008, 4096), (1040, 129), (16, 5), (2048, 1000)))
def test_fp8_streaming_path_within_reference_bound(gpu, ta, tb, n, k):
    """fp8 x and weights on the streaming kernel: fp32 accumulation (no matrix-core instruction), so the
    reference's own elementwise bound holds without the fp8-MFMA allowance."""
    case = rowmajor_case(ta, 1, n, k, 1.5, -0.5, tb=tb, rsb=n + 48)
    a, b, c = case.make_inputs(n + 3 * k)
    for mode in ("device", "host"):
        got = run_gemm(gpu, "rc", case, a, b, c, mode)
        support.assert_fp_gemm_close(case, a, b, c, got)


@pytest.mark.parametrize("ta,tb", (("bf16", "bf16"), ("f16", "f16")) + FP8_PAIRS)
@pytest.mark.parametrize("m", (2, 3))
def test_small_batch_rows_floating_point(gpu, ta, tb, m):
    """2 or 3 rows of A for bf16 / f16 / fp8: with less than 1 MiB of B (or K off the 16-byte rule) on the
    streaming kernel with fp32 multiply-adds - the reference's elementwise bound, no matrix-core allowance -,
    larger ones on the kernel that multiplies on the matrix cores (fp8: with the allowance of those instructions).
    Strides with padding, both pointer modes, and a second call right behind the first on the shared scratch."""
    for (n, k) in ((11008, 4096), (1040, 136), (16, 8), (2048, 1000)):
        case = rowmajor_case(ta, m, n, k, 1.5, -0.5, tb=tb, rsa=k + 8, rsb=n + 48, rsc=n + 3)
        a, b, c = case.make_inputs(m * 100 + n + k)
        on_matrix_cores = ta.startswith("f8") and n * k >= (1 << 20) and k % 16 == 0
        extra = support.FP8_MFMA_REL if on_matrix_cores else 0.0
        for mode in ("device", "host"):
            got = run_gemm(gpu, "rc", case, a, b, c, mode)
            support.assert_fp_gemm_close(case, a, b, c, got, extra_rel=extra)
            again = run_gemm(gpu, "rc", case, a, b, c, mode)
            support.assert_fp_gemm_close(case, a, b, c, again, extra_rel=extra)


def _kc_case(ta, tb, m, n, k, alpha, beta, pad=0):
    """Row-major A (m x k), B with K contiguous (column j at j * (k + pad)), row-major C."""
    return GemmCase(ta, tb, alpha, beta, m0=1, n0=1, k0=1, m1=m, n1=n, k1=k, rsa0=0, csa0=0, rsa1=k + pad, csa1=1,
                    rsb0=0, csb0=0, rsb1=1, csb1=k + pad, rsc0=0, csc0=0, rsc1=n + 5, csc1=1)


@pytest.mark.parametrize("m", (1, 2, 3, 4))
def test_k_contiguous_b_int8_bit_exact(gpu, m):
    """B stored column by column (a linear layer's [out][in] weight): one dot product over contiguous memory per
    output, no sums between workgroups. Config-2 sizes, K tails of every residue of 16 bytes per KiB, few columns."""
    rng = np.random.default_rng(60 + m)
    for (n, k, pad) in ((11008, 4096, 0), (1037, 4096 + 16, 16), (5, 16, 0), (70, 1008, 32), (513, 5040, 0)):
        for alpha, beta in ((1, 0), (-3, 2)):
            case = _kc_case("i8", None, m, n, k, alpha, beta, pad)
            a, b, c = case.make_inputs(int(rng.integers(1 << 30)))
            want = run_oracle_gemm(case, a, b, c)
            for mode in ("device", "host"):
                assert np.array_equal(run_gemm(gpu, "rc", case, a, b, c, mode), want), (m, n, k, mode)


@pytest.mark.parametrize("m", (5, 16, 17, 40, 90, 96, 100, 128))
def test_k_contiguous_b_decode_batches_int8_bit_exact(gpu, m):
    """5 to 96 rows of A against a B stored column by column, K <= 4096 (ref/gemm/gemm_i8rc_i8rc_i32rc.c:9-24 with
    rsb = 1): one workgroup per 64 columns takes 4096 k on the matrix cores, row groups of 16 (ragged last groups:
    5, 17, 40, 90), C written once per 4096 k; 100 and 128 rows: the tile kernels. The config-2 width, N off the
    64-column workgroups, K off the waves' 512 and the chunks of 256, padded strides, alpha / beta with wrap-around on
    a C of extreme values, both pointer modes; a K beyond 4096 against a narrow B (the tile kernels) and against a
    wide one (two launches, the second of 16 k)."""
    rng = np.random.default_rng(160 + m)
    for (n, k, pad) in ((11008, 1024 if m > 16 else 4096, 0), (1037, 4080, 16), (300, 3504, 32), (4100, 272, 0), (260, 4112, 0),
                        (8200, 4112, 0)):
        for alpha, beta in ((1, 0), (0x01010101, -77), (-3, 1)):
            case = _kc_case("i8", None, m, n, k, alpha, beta, pad)
            a, b, c = case.make_inputs(int(rng.integers(1 << 30)))
            c[:] = rng.integers(-2 ** 31, 2 ** 31, size=c.size)
            want = run_oracle_gemm(case, a, b, c)
            for mode in ("device", "host"):
                assert np.array_equal(run_gemm(gpu, "rc", case, a, b, c, mode), want), (m, n, k, alpha, beta, mode)


@pytest.mark.parametrize("ta,tb", FP8_PAIRS)
@pytest.mark.parametrize("m", (5, 16, 33, 96))
def test_k_contiguous_b_decode_batches_fp8(gpu, ta, tb, m):
    """The fp8 kinds of the same kernel (operands widened to f16 in registers: exact products, fp32 sums in a fixed
    order): inside the reference's bound without any allowance, and the same bits on every run."""
    for (n, k, pad) in ((11008, 1024 if m > 16 else 4096, 0), (1037, 2064, 16), (300, 3504, 32), (8200, 4128, 0)):
        case = _kc_case(ta, tb, m, n, k, 1.5, -0.5, pad)
        a, b, c = case.make_inputs(m * 37 + n + k)
        for mode in ("device", "host"):
            got = run_gemm(gpu, "rc", case, a, b, c, mode)
            support.assert_fp_gemm_close(case, a, b, c, got)
            assert np.array_equal(got.view(np.uint8), run_gemm(gpu, "rc", case, a, b, c, mode).view(np.uint8))


@pytest.mark.parametrize("ta,tb", (("bf16", "bf16"), ("f16", "f16")) + FP8_PAIRS)
@pytest.mark.parametrize("m", (1, 4))
def test_k_contiguous_b_floating_point(gpu, ta, tb, m):
    """Same layout for bf16 / f16 / fp8: fp32 accumulation in a fixed order - inside the reference's bound,
    and the same bits on every run."""
    for (n, k, pad) in ((11008, 4096, 0), (1037, 1040, 16), (5, 16, 0)):
        case = _kc_case(ta, tb, m, n, k, 1.5, -0.5, pad)
        a, b, c = case.make_inputs(m * 31 + n + k)
        for mode in ("device", "host"):
            got = run_gemm(gpu, "rc", case, a, b, c, mode)
            support.assert_fp_gemm_close(case, a, b, c, got)
            assert np.array_equal(got.view(np.uint8), run_gemm(gpu, "rc", case, a, b, c, mode).view(np.uint8))


@pytest.mark.parametrize("ta", ("i8", "bf16", "f8e4m3"))
@pytest.mark.parametrize("m", (1, 3, 4, 7, 40))
def test_k_contiguous_b_with_fused_steps(gpu, ta, m):
    """A decode step on a linear layer's [out][in] weight with the fused steps of include/skl-gfx950.h: the kernel's
    last stage applies bias, ReLU, the 8-bit copy (int8 behind int32, saturating E4M3 behind fp32) and the maximum
    (1 to 4 rows: the dot-product kernel; 7 and 40 rows: the matrix-core kernel for int8 and fp8, bf16 on the tile kernels).
    int8 against the checker's product plus the rules; floating point against the plain call of the same kernel
    (same sums, bit for bit) plus the rules. Row tails, padded strides, both pointer modes, q_only."""
    from gpu_support import run_fused_gemm
    from test_oracle_gemm import fused_expectation
    rng = np.random.default_rng(70 + m)
    for (n, k, pad) in ((11008, 4096, 0), (1037, 1040, 16), (70, 1008, 32), (8200, 4128, 16)):
        for beta, only in ((0, True), (1, False)):
            case = _kc_case(ta, None, m, n, k, 2 if ta == "i8" else 0.5, beta, pad)
            a, b, c = case.make_inputs(int(rng.integers(1 << 30)))
            if case.is_int:
                plain = run_oracle_gemm(case, a, b, c)
                bias = rng.integers(-1 << 12, 1 << 12, n).astype(np.int32)
                start = np.array([-(1 << 31)], np.int32)
            else:
                plain = run_gemm(gpu, "rc", case, a, b, c, "device")
                bias = rng.uniform(-4, 4, n).astype(np.float32)
                start = np.array([-np.inf], np.float32)
            rows = np.arange(m)[:, None] * case.rsc1 + np.arange(n)[None, :]
            spread = float(np.abs(plain[rows].astype(np.float64)).max())
            scales = (rng.uniform(0.5, 2.0, n) * 100.0 / max(spread, 1e-3)).astype(np.float32)
            rq = dict(q=np.full(m * (n + 3), 0x55, np.int8), rsq=n + 3, csq=1, scale=scales, per_column=True, zero=-5, only=only,
                      format=0 if case.is_int else 2)
            for mode in ("device", "host"):
                got, top, q = run_fused_gemm(gpu, "rc", case, a, b, c, bias, start, mode, activation=1, requant=rq)
                want_c, want_top, want_q = fused_expectation(case, plain, bias, start, activation=1, requant=rq)
                assert np.array_equal(q, want_q) and top[0] == want_top[0], (ta, m, n, k, beta, mode)
                assert np.array_equal(got.view(np.uint8), (c if only else want_c).view(np.uint8)), (ta, m, n, k, beta, mode)


def _few_columns_case(ta, tb, m, n, k, alpha, beta, a_rows_contiguous, b_cols_contiguous, pad=0):
    """A tall problem with 1..8 columns: A row-major (lda = k + pad) or column-major (lda = m + pad); B column by
    column (a vector with unit stride when n == 1) or row-major; C row-major with a padded row."""
    rsa, csa = (k + pad, 1) if a_rows_contiguous else (1, m + pad)
    rsb, csb = (1, k + pad) if b_cols_contiguous else (n, 1)
    return GemmCase(ta, tb, alpha, beta, m0=1, n0=1, k0=1, m1=m, n1=n, k1=k, rsa0=0, csa0=0, rsa1=rsa, csa1=csa,
                    rsb0=0, csb0=0, rsb1=rsb, csb1=csb, rsc0=0, csc0=0, rsc1=n + 3, csc1=1)


@pytest.mark.parametrize("n", (1, 2, 3, 4, 8))
def test_few_columns_int8_bit_exact(gpu, n):
    """Matrix times vector (and up to 8 vectors): served by the streaming kernels with the roles of A and B
    exchanged. Every pairing of operand layouts, sizes on and off the kernels' alignment rules (those fall back
    to the tile kernels) - all bit-exact."""
    rng = np.random.default_rng(90 + n)
    for (m, k, pad) in ((11008, 4096, 0), (1037, 1040, 16), (5, 16, 0), (513, 1000, 0), (4096, 4096, 64)):
        for a_rows in (True, False):
            for b_cols in (True, False):
                for alpha, beta in ((1, 0), (-3, 2)):
                    case = _few_columns_case("i8", None, m, n, k, alpha, beta, a_rows, b_cols, pad)
                    a, b, c = case.make_inputs(int(rng.integers(1 << 30)))
                    want = run_oracle_gemm(case, a, b, c)
                    got = run_gemm(gpu, "rc", case, a, b, c, "device")
                    assert np.array_equal(got, want), (m, n, k, a_rows, b_cols, alpha, beta)


@pytest.mark.parametrize("ta,tb", (("bf16", "bf16"), ("f16", "f16")) + FP8_PAIRS)
@pytest.mark.parametrize("n", (1, 3))
def test_few_columns_floating_point(gpu, ta, tb, n):
    """The E4M3 x E5M2 pair has no exchanged form on the streaming kernels (they decode the vector as E4M3) and
    runs on the matrix-core kernels, whose fp8 summation term is allowed for."""
    extra = support.FP8_MFMA_REL if ta != tb else 0.0
    for (m, k, pad) in ((11008, 4096, 0), (1037, 1040, 16), (5, 16, 0)):
        for a_rows in (True, False):
            case = _few_columns_case(ta, tb, m, n, k, 1.5, -0.5, a_rows, True, pad)
            a, b, c = case.make_inputs(n * 17 + m + k)
            for mode in ("device", "host"):
                got = run_gemm(gpu, "rc", case, a, b, c, mode)
                support.assert_fp_gemm_close(case, a, b, c, got, extra_rel=extra)


@pytest.mark.parametrize("ta", ("i8", "bf16", "f8e4m3"))
def test_few_rows_of_a_in_a_layout_no_kernel_reads(gpu, ta):
    """A with 2..40 rows stored column by column (rows 2..40 elements apart: below the kernels' 16-byte rule): A is
    copied into scratch memory with K contiguous and the problem leaves the any-stride kernel. int8 bit-exact."""
    for (m, n, k) in ((2, 11008, 4096), (3, 1040, 1000), (7, 4096, 512), (40, 2048, 777)):
        case = GemmCase(ta, None, 2 if ta == "i8" else 1.5, 1 if ta == "i8" else -0.5, m0=1, n0=1, k0=1, m1=m, n1=n,
                        k1=k, rsa0=0, csa0=0, rsa1=1, csa1=m, rsb0=0, csb0=0, rsb1=n, csb1=1, rsc0=0, csc0=0,
                        rsc1=n, csc1=1)
        a, b, c = case.make_inputs(m + n + k)
        got = run_gemm(gpu, "rc", case, a, b, c, "device")
        if ta == "i8":
            assert np.array_equal(got, run_oracle_gemm(case, a, b, c)), (m, n, k)
        else:
            support.assert_fp_gemm_close(case, a, b, c, got, extra_rel=support.FP8_MFMA_REL if ta.startswith("f8") else 0.0)
