"""Randomised differential test of the GEMM dispatch at mid and large sizes: problems of random kind, shape (1 to
4500 rows and columns, K up to 9000), layout, leading-dimension padding, base misalignment and alpha / beta through
the full-stride entry points, where the streaming kernels, the padded and realigned copies, the decode-batch kernels
and the shared-K variants take over from one another. The check is independent of the CPU checker: numpy's fp64
matrix product, which is exact for int8 operands (sums below 2^53), so int8 results are compared bit for bit over
the whole C buffer (int32 wrap-around of alpha / beta included) and floating point against the reference's bound."""
import numpy as np
import pytest

import skl_amd
import support
from skl_amd import DeviceBuffer
from support import GemmCase

pytestmark = pytest.mark.gpu

KINDS = (("i8", "i8"), ("i8", "i8"), ("bf16", "bf16"), ("f16", "f16"), ("f8e4m3", "f8e4m3"), ("f8e5m2", "f8e5m2"),
         ("f8e4m3", "f8e5m2"))


def _extent(rng):
    pick = rng.integers(6)
    if pick == 0:
        return int(rng.integers(1, 9))
    if pick == 1:
        return int(rng.integers(9, 130))
    if pick == 2:
        return int(rng.integers(130, 700))
    if pick == 3:
        return 64 * int(rng.integers(1, 70))
    if pick == 4:
        return 256 * int(rng.integers(1, 18))
    return int(rng.integers(700, 4500))


def _depth(rng):
    pick = rng.integers(5)
    if pick == 0:
        return int(rng.integers(1, 200))
    if pick == 1:
        return 128 * int(rng.integers(1, 65))
    if pick == 2:
        return 16 * int(rng.integers(1, 300))
    if pick == 3:
        return int(rng.integers(200, 9000))
    return 1024 * int(rng.integers(1, 9))


def _random_case(rng):
    ta, tb = KINDS[int(rng.integers(len(KINDS)))]
    while True:
        m, n, k = _extent(rng), _extent(rng), _depth(rng)
        if m * n * k <= 1.2e10 and m * n <= 1.2e7:
            break
    align = int(rng.choice([1, 3, 8, 16, 64]))

    def ld(extent):
        return extent + align * int(rng.integers(0, 3)) if rng.integers(2) else extent

    a_row_major, b_row_major, c_row_major = bool(rng.integers(2)), bool(rng.integers(2)), bool(rng.integers(4))
    rsa, csa = (ld(k), 1) if a_row_major else (1, ld(m))
    rsb, csb = (ld(n), 1) if b_row_major else (1, ld(k))
    rsc, csc = (ld(n), 1) if c_row_major else (1, ld(m))
    if ta == "i8":
        alpha, beta = int(rng.choice([1, 1, -3, 0x01010101])), int(rng.choice([0, 0, 1, -77]))
    else:
        alpha, beta = float(rng.choice([1.0, 1.0, -0.5, 2.0])), float(rng.choice([0.0, 0.0, 1.0, -1.5]))
    return GemmCase(ta, tb, alpha, beta, m0=1, n0=1, k0=1, m1=m, n1=n, k1=k, rsa0=0, csa0=0, rsa1=rsa, csa1=csa,
                    rsb0=0, csb0=0, rsb1=rsb, csb1=csb, rsc0=0, csc0=0, rsc1=rsc, csc1=csc)


@pytest.mark.parametrize("chunk", range(6))
def test_random_mid_size_problems_match_numpy(gpu, chunk):
    rng = np.random.default_rng(50000 + 1000 * chunk)
    for _ in range(20):
        case = _random_case(rng)
        a, b, c = case.make_inputs(int(rng.integers(1 << 30)))
        if case.is_int:
            c[:] = rng.integers(-2 ** 31, 2 ** 31, size=c.size)
        # operands a few elements into their buffers now and then: bases off the 16-byte rule
        off_a, off_b = (int(rng.choice([0, 0, 0, 1, 2, 4, 8])) * x.dtype.itemsize if rng.integers(3) == 0 else 0
                        for x in (a, b))
        what = (case.ta, case.tb, case.m1, case.n1, case.k1, case.rsa1, case.csa1, case.rsb1, case.csb1, case.rsc1,
                case.csc1, case.alpha, case.beta, off_a, off_b)
        da, db, dc = DeviceBuffer(a.nbytes + 64), DeviceBuffer(b.nbytes + 64), DeviceBuffer.from_array(c)
        try:
            assert gpu.skl_hip_memcpy_h2d(da.offset(off_a), a, a.nbytes) == 0
            assert gpu.skl_hip_memcpy_h2d(db.offset(off_b), b, b.nbytes) == 0
            name = f"skl_gemm_{case.atag}rc_{case.btag}rc_{case.ctag}rc_gfx950"
            getattr(gpu, name)(case.m1, case.n1, case.k1, case.alpha, da.offset(off_a), case.rsa1, case.csa1,
                               db.offset(off_b), case.rsb1, case.csb1, case.beta, dc, case.rsc1, case.csc1)
            assert gpu.skl_hip_synchronize() == 0
            skl_amd.check_error()
            got = dc.download(c.dtype, c.size)
        finally:
            for d in (da, db, dc):
                d.free()
        if case.is_int:
            A, B, C, oc = case.dense(a, b, c)
            acc = (A @ B).astype(np.int64)
            want = c.copy()
            want[oc] = ((case.beta * C.astype(np.int64) + case.alpha * acc) & 0xFFFFFFFF).astype(np.uint32) \
                .view(np.int32).reshape(oc.shape)
            assert np.array_equal(got, want), what
        else:
            try:
                support.assert_fp_gemm_close(case, a, b, c, got,
                                             extra_rel=support.FP8_MFMA_REL if case.ta.startswith("f8") else 0.0)
            except AssertionError as e:
                raise AssertionError(f"{what}: {e}") from None
