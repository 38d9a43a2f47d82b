"""Randomised differential test of the GEMM dispatch: small problems of random kind, shape, layout, padding,
base misalignment and alpha / beta are run through the full-stride entry points and compared with the CPU
checker (int8: bit for bit over the whole C buffer; floating point: the reference's bound). Every specialised
kernel (streaming GEMV and its multi-row and K-contiguous variants, tile kernels with and without shared K, the
any-stride kernel) has eligibility rules; this test walks their borders."""
import numpy as np
import pytest

import support
from gpu_support import run_gemm
from support import GemmCase, run_oracle_gemm

pytestmark = pytest.mark.gpu

KINDS = (("i8", "i8"), ("bf16", "bf16"), ("f16", "f16"), ("f8e4m3", "f8e4m3"), ("f8e5m2", "f8e5m2"),
         ("f8e4m3", "f8e5m2"), ("f32", "f32"))


def _random_case(rng):
    ta, tb = KINDS[int(rng.integers(len(KINDS)))]
    m = int(rng.choice([1, 1, 2, 3, 4, 5, 8, 9, int(rng.integers(1, 70))]))
    n = int(rng.choice([int(rng.integers(1, 40)), 16 * int(rng.integers(1, 20)), 64 * int(rng.integers(1, 6))]))
    k = int(rng.choice([int(rng.integers(1, 50)), 16 * int(rng.integers(1, 40)), 128 * int(rng.integers(1, 40))]))
    align = int(rng.choice([1, 1, 8, 16]))  # padding granularity in elements: 1 makes odd strides likely

    def ld(extent):
        return extent + align * int(rng.integers(0, 3))

    a_row_major, b_row_major, c_row_major = bool(rng.integers(2)), bool(rng.integers(2)), bool(rng.integers(4))
    rsa, csa = (ld(k), 1) if a_row_major else (1, ld(m))
    rsb, csb = (ld(n), 1) if b_row_major else (1, ld(k))
    rsc, csc = (ld(n), 1) if c_row_major else (1, ld(m))
    if ta == "i8":
        alpha, beta = int(rng.choice([1, -3, 0x01010101])), int(rng.choice([0, 1, -77]))
    else:
        alpha, beta = float(rng.choice([1.0, -0.5, 2.0])), float(rng.choice([0.0, 1.0, -1.5]))
    return GemmCase(ta, tb, alpha, beta, m0=1, n0=1, k0=1, m1=m, n1=n, k1=k, rsa0=0, csa0=0, rsa1=rsa, csa1=csa,
                    rsb0=0, csb0=0, rsb1=rsb, csb1=csb, rsc0=0, csc0=0, rsc1=rsc, csc1=csc)


@pytest.mark.parametrize("chunk", range(20))
def test_random_problems_match_the_checker(gpu, chunk):
    rng = np.random.default_rng(9000 + chunk)
    for _ in range(60):
        case = _random_case(rng)
        a, b, c = case.make_inputs(int(rng.integers(1 << 30)))
        if case.is_int:
            c[:] = rng.integers(-2 ** 31, 2 ** 31, size=c.size)
        mode = "device" if rng.integers(4) else "host"
        got = run_gemm(gpu, "rc", case, a, b, c, mode)
        what = (case.ta, case.tb, case.m1, case.n1, case.k1, case.rsa1, case.csa1, case.rsb1, case.csb1, case.rsc1,
                case.csc1, case.alpha, case.beta, mode)
        if case.is_int:
            assert np.array_equal(got, run_oracle_gemm(case, a, b, c)), what
        elif case.ta == "f32":
            assert np.array_equal(got.view(np.uint8), run_oracle_gemm(case, a, b, c).view(np.uint8)), what
        else:
            try:
                support.assert_fp_gemm_close(case, a, b, c, got,
                                             extra_rel=support.FP8_MFMA_REL if case.ta.startswith("f8") else 0.0)
            except AssertionError as e:
                raise AssertionError(f"{what}: {e}") from None
