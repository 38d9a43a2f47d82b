"""GPU parity of the GEMM over OFP4 (E2M1) weights, skl_gemm_f8e4m3rc_f4e2m1c_f32rc_gfx950: the reference has no
such routine - its users convert the weights (skl_cvt_f4e2m1_f8e4m3, ref/cvt/cvt_ofp4.c:59-68) and call the fp8 GEMM
(ref/gemm/gemm_f8e4m3rc_f8e4m3rc_f32rc.h:48). The result must lie inside that GEMM's own bound
(test/gemm/gemm_f8rcprc_f8rcprc_f32rcprc.c:132-204, no allowance on top) around the exact product of the decoded
operands, on the kernel that streams the 4-bit weights (1 to 16 rows: matrix-core FP4 format for long K, f16
instructions on widened operands up to K = 2304) and on the route through a converted copy."""
import numpy as np
import pytest

import ofp4_support as f4
import skl_amd
import support
from gpu_support import MODES, _finish
from skl_amd import DeviceBuffer

pytestmark = pytest.mark.gpu


def run(lib, case, a, b4, c, mode, m, n, k, ldb, scales=None, lds=0):
    def call(a_, b_, c_, s_):
        if scales is None:
            lib.skl_gemm_f8e4m3rc_f4e2m1c_f32rc_gfx950(m, n, k, case.alpha, a_, case.rsa1, case.csa1, b_, ldb, case.beta, c_, case.rsc1, case.csc1)
        else:
            lib.skl_gemm_f8e4m3rc_mxf4e2m1c_f32rc_gfx950(m, n, k, case.alpha, a_, case.rsa1, case.csa1, b_, ldb, s_, lds, case.beta, c_,
                                                         case.rsc1, case.csc1)
    if mode == "host":
        out = c.copy()
        call(a, b4, out, scales)
        skl_amd.check_error()
        return out
    bufs = [DeviceBuffer.from_array(x) if x is not None else None for x in (a, b4, c, scales)]
    call(bufs[0], bufs[1], bufs[2], bufs[3])
    _finish(lib)
    out = bufs[2].download(c.dtype, c.size)
    for d in bufs:
        if d is not None:
            d.free()
    return out


SHAPES = (
    # m, n, k, ldb, rsa, what
    (1, 11008, 4096, 4096, None, "decode, FP4 operand format of the matrix cores"),
    (16, 1000, 4352, 4384, 4368, "16 rows, n off the 16-column groups, K off the chunk of 1024"),
    (16, 8200, 2592, 2624, 2608, "workgroups of 64 columns (n >= 8192, 3 rows or more): n off them, K off the chunk"),
    (3, 8256, 2304, 2304, None, "workgroups of 64 columns, multiplied exactly"),
    (3, 500, 2304, 2304, None, "longest K multiplied exactly (operands widened to f16)"),
    (7, 48, 2336, 2336, None, "shortest K on the FP4 format"),
    (5, 48, 32, 32, None, "one piece of K"),
    (1, 17, 64, 96, None, "a last group of one column"),
    (17, 300, 512, 512, None, "more than 16 rows, little of B: through the converted copy"),
    (17, 4100, 512, 544, 528, "17 rows (two row groups, the second of one row), multiplied exactly, n off the 32-column workgroups"),
    (100, 1040, 4096, 4096, None, "100 rows in seven row groups, the longest K held in registers"),
    (128, 520, 2336, 2368, 2352, "eight full row groups on the FP4 format"),
    (40, 300, 4128, 4128, None, "K beyond what the registers hold: two passes, the second of one piece of K"),
    (100, 520, 11008, 11040, 11024, "K of a down projection: three passes"),
    (300, 260, 1000, 1000, None, "a GEMM: through the converted copy"),
    (4, 64, 100, 101, None, "K off 32 and an odd column distance (columns start inside a byte): converted copy"),
    (2, 40, 64, 64, 67, "rows of A off 16 bytes: converted copy"),
)


@pytest.mark.parametrize("m,n,k,ldb,rsa,what", SHAPES)
def test_ofp4_weights(gpu, m, n, k, ldb, rsa, what):
    for i, (alpha, beta) in enumerate(((1.0, 0.0), (1.5, -0.5))):
        case, a, b4, b8, c = f4.make_problem(700 + m + n + i, m, n, k, ldb, alpha, beta, rsa=rsa, rsc=n + 3)
        for mode in MODES:
            got = run(gpu, case, a, b4, c, mode, m, n, k, ldb)
            support.assert_fp_gemm_close(case, a, b8, c, got)
            assert np.array_equal(got.view(np.uint32), run(gpu, case, a, b4, c, mode, m, n, k, ldb).view(np.uint32)), what


@pytest.mark.parametrize("m,n,k,ldb,rsa,what", SHAPES)
def test_mx_scaled_ofp4_weights(gpu, m, n, k, ldb, rsa, what):
    """The same shapes with one E8M0 scale per 32 k of a column (OCP microscaling): inside the reference's
    fp32-accumulation bound around the exact product of the decoded, scaled operands - the decode kernel hands the
    scales to the matrix cores (or folds them into the bf16 widening up to K = 2304), the other shapes run the bf16
    GEMM on exactly converted copies - and the same bits on a second run."""
    for i, (alpha, beta) in enumerate(((1.0, 0.0), (1.5, -0.5))):
        case, a, b4, b8, scales, lds, c = f4.make_mx_problem(800 + m + n + i, m, n, k, ldb, alpha, beta, rsa=rsa, rsc=n + 3)
        exact, bound, oc = f4.mx_bound(case, a, b8, scales, lds, c, m, n, k, ldb)
        for mode in MODES:
            got = run(gpu, case, a, b4, c, mode, m, n, k, ldb, scales, lds)
            err = np.abs(got[oc] - exact)
            assert np.all(err <= bound + np.abs(exact) * 2.0 ** -22 + 1e-30), (what, mode, float((err / (bound + 1e-30)).max()))
            mask = np.ones(c.size, bool)
            mask[oc.ravel()] = False
            assert np.array_equal(got[mask], c[mask]), "elements outside the addressed C were modified"
            again = run(gpu, case, a, b4, c, mode, m, n, k, ldb, scales, lds)
            assert np.array_equal(got.view(np.uint32), again.view(np.uint32)), what


@pytest.mark.parametrize("n", (48, 8208))
@pytest.mark.parametrize("k", (2304, 2560))
def test_scales_reach_their_blocks(gpu, k, n):
    """A row of A that is 1.0 at one k reads B(k, :) times its block's scale back exactly: every block of 32 k gets the
    scale stored for it, in both kernel variants and both workgroup widths (16 and, from n = 8192, 64 columns)."""
    lds = k // 32 + 1
    rng = np.random.default_rng(k + 1)
    codes = rng.integers(1, 8, size=n * k, dtype=np.uint8)        # positive, non-zero values
    scales = rng.integers(117, 138, size=n * lds, dtype=np.uint8)
    b4 = f4.pack_nibbles(codes)
    values = f4.E2M1_VALUES[codes].reshape(n, k) * np.ldexp(1.0, scales.reshape(n, lds)[:, :k // 32].astype(np.int64) - 127).repeat(32, axis=1)
    for p0 in range(0, k, 16 * 32):
        pos = np.minimum(p0 + np.arange(16) * 32 + (np.arange(16) * 7) % 32, k - 1)   # one k in each of 16 blocks
        a = np.zeros(16 * k, np.uint8)
        a[np.arange(16) * k + pos] = 0x38
        case = f4.f8_case(16, n, k, k, 1.0, 0.0)
        got = run(gpu, case, a, b4, np.zeros(16 * n, np.float32), "device", 16, n, k, k, scales, lds).reshape(16, n)
        assert np.array_equal(got.astype(np.float64), values[:, pos].T), (k, p0)


@pytest.mark.parametrize("n", (64, 8256))
@pytest.mark.parametrize("k", (2304, 2560))
def test_every_position_and_code_is_read_back(gpu, k, n):
    """A row of A that is 1.0 at one k and zero elsewhere reads B(k, :) back exactly: every position of a 256-k chunk
    (16 rows per call), every E2M1 code, both kernel variants (k = 2304: f16 instructions, 2560: FP4 format). This
    is what fixes which nibble is which k and that A's and B's lanes hold the same k. Both workgroup widths."""
    rng = np.random.default_rng(k)
    codes = rng.integers(0, 16, size=n * k, dtype=np.uint8)
    codes[:16 * k:k + 1] = np.arange(16)          # and every code at least once on a diagonal
    b4 = f4.pack_nibbles(codes)
    table = f4.E2M1_VALUES[codes].reshape(n, k)
    for base in (0, k - 256):
        for p0 in range(0, 256, 16):
            a = np.zeros(16 * k, np.uint8)
            pos = base + p0 + np.arange(16)
            a[np.arange(16) * k + pos] = 0x38      # 1.0
            case = f4.f8_case(16, n, k, k, 1.0, 0.0)
            got = run(gpu, case, a, b4, np.full(16 * n, np.nan, np.float32), "device", 16, n, k, k).reshape(16, n)
            assert np.array_equal(got.astype(np.float64), table[:, pos].T), (k, base, p0)


def test_ofp4_edges(gpu):
    """K = 0 scales C; empty problems touch nothing; a NaN in C is overwritten by beta == 0 (the library's default)
    and kept by the reference's evaluation of 0 * C when that is asked for; mixed pointers are refused."""
    case, a, b4, b8, c = f4.make_problem(9, 4, 32, 64, 64, 2.0, 3.0)
    got = run(gpu, case, a, b4, c, "device", 4, 32, 0, 64)
    assert np.array_equal(got, (np.float32(3.0) * c).astype(np.float32))
    assert np.array_equal(run(gpu, case, a, b4, c, "device", 0, 32, 64, 64), c)
    spoiled = c.copy()
    spoiled[5] = np.nan
    case0 = f4.f8_case(4, 32, 64, 64, 1.0, 0.0)
    got = run(gpu, case0, a, b4, spoiled, "device", 4, 32, 64, 64)
    support.assert_fp_gemm_close(case0, a, b8, c, got)
    gpu.skl_hip_set_beta_zero_mode(1)
    try:
        got = run(gpu, case0, a, b4, spoiled, "device", 4, 32, 64, 64)
        assert np.isnan(got[5]) and not np.isnan(np.delete(got, 5)).any()
    finally:
        gpu.skl_hip_set_beta_zero_mode(0)
    d = DeviceBuffer.from_array(a)
    gpu.skl_gemm_f8e4m3rc_f4e2m1c_f32rc_gfx950(4, 32, 64, 1.0, d, 64, 1, b4, 64, 0.0, c.copy(), 32, 1)
    assert gpu.skl_hip_last_error() == -1
    d.free()


def test_converted_copy_without_a_scratch_slot(gpu):
    """A stream beyond the 32 that hold scratch blocks on a device: a 4-bit-weight GEMM that needs a converted copy of
    its operands (more than 16 rows) still writes the right C - through a buffer of its own - and leaves only the
    advisory SKL_HIP_ERR_STREAM_SLOTS behind, with and without block scales."""
    import ctypes as ct

    hip = ct.CDLL("libamdhip64.so.7")
    hip.hipStreamCreate.restype = hip.hipStreamDestroy.restype = ct.c_int
    m, n, k = 40, 96, 512
    case, a, b4, b8, c = f4.make_problem(4711, m, n, k, k, 1.25, 0.5, rsc=n + 1)
    rng = np.random.default_rng(5)
    scales = rng.integers(120, 135, size=n * (k // 32), dtype=np.uint8)
    streams = []
    gpu.skl_hip_last_error()
    try:
        # claim slots with an int8 GEMV (its workgroups meet in the stream's scratch) until one is refused
        x, w, y = DeviceBuffer.from_array(np.ones(4096, np.int8)), DeviceBuffer.from_array(np.ones(4096 * 2048, np.int8)), DeviceBuffer(4 * 2048)
        gpu.skl_hip_set_pointer_mode(1)
        for _ in range(34):
            stream = ct.c_void_p()
            assert hip.hipStreamCreate(ct.byref(stream)) == 0
            streams.append(stream)
            gpu.skl_hip_set_stream(stream.value)
            gpu.skl_gemm_i8_i8_i32_gfx950(1, 2048, 4096, 1, x, 4096, w, 2048, 0, y, 2048)
            assert gpu.skl_hip_synchronize() == 0
            if gpu.skl_hip_last_error() == -5:
                break
        else:
            pytest.fail("no stream was refused a slot")
        gpu.skl_hip_set_pointer_mode(0)
        for sc in (None, scales):   # the stream set above is the one without a slot
            bufs = [DeviceBuffer.from_array(v) if v is not None else None for v in (a, b4, c, sc)]
            if sc is None:
                gpu.skl_gemm_f8e4m3rc_f4e2m1c_f32rc_gfx950(m, n, k, case.alpha, bufs[0], case.rsa1, case.csa1, bufs[1], k, case.beta, bufs[2],
                                                           case.rsc1, case.csc1)
            else:
                gpu.skl_gemm_f8e4m3rc_mxf4e2m1c_f32rc_gfx950(m, n, k, case.alpha, bufs[0], case.rsa1, case.csa1, bufs[1], k, bufs[3], k // 32,
                                                             case.beta, bufs[2], case.rsc1, case.csc1)
            assert gpu.skl_hip_synchronize() == 0
            assert gpu.skl_hip_last_error() in (0, -5)
            got = bufs[2].download(c.dtype, c.size)
            if sc is None:
                support.assert_fp_gemm_close(case, a, b8, c, got)
            else:
                gpu.skl_hip_set_stream(None)
                want = run(gpu, case, a, b4, c, "device", m, n, k, k, scales=sc, lds=k // 32)   # the same call on a stream with scratch
                gpu.skl_hip_set_stream(streams[-1].value)
                assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
            for d in bufs:
                if d is not None:
                    d.free()
        for d in (x, w, y):
            d.free()
    finally:
        gpu.skl_hip_set_stream(None)
        gpu.skl_hip_set_pointer_mode(0)
        for stream in streams:
            gpu.skl_hip_release_stream(stream.value)
            hip.hipStreamDestroy(stream)
        gpu.skl_hip_last_error()
