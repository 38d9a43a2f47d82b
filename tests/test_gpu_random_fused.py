"""Randomised differential test of the fused int8 calls (include/skl-gfx950.h, fused section): decode shapes and
small tiles with random layouts of B (row-major, K contiguous, K-packed), strides, alpha / beta and a random
descriptor - bias, maximum, ReLU, the 8-bit copy in either orientation, with one scale or one per column, as int8
or in one of the four fp8 forms, written next to C or alone - against the checker's product plus the rules, bit for
bit over the whole C and copy buffers. The fused calls are served by several routes (steps in the last stage of
the one-row and K-contiguous kernels, the product into scratch memory followed by a pass that applies the steps,
the tile kernels' epilogues, the pass that adds the shares of K); this test walks their borders."""
import numpy as np
import pytest

import support
from gpu_support import run_fused_gemm
from support import GemmCase, run_oracle_gemm
from test_oracle_gemm import fused_expectation

pytestmark = pytest.mark.gpu


def _random_case(rng):
    layout = int(rng.integers(3))  # 0 row-major B, 1 B with K contiguous, 2 K-packed B (groups of four k)
    m = int(rng.choice([1, 1, 1, 2, 3, 4, 5, 8, 16, 17, 40]))
    n = int(rng.choice([48, 208, 1024, 2064, 16 * int(rng.integers(1, 60)), int(rng.integers(1, 90))]))
    k = int(rng.choice([64, 528, 1040, 2048, 16 * int(rng.integers(1, 80))]))
    pad = int(rng.choice([0, 0, 16, 32]))
    alpha, beta = int(rng.choice([1, -3, 0x01010101])), int(rng.choice([0, 0, 1, -77]))
    if layout == 2:
        n = max(4, n // 4 * 4)
        return "rcprc", support.dot4_case(m, n, k // 4, alpha=alpha, beta=beta, rsa1=k + pad, rsb1=4 * n + pad, rsc1=n + int(rng.integers(0, 6)))
    rsb, csb = (n + pad, 1) if layout == 0 else (1, k + pad)
    return "rc", GemmCase("i8", None, alpha, beta, m0=1, n0=1, k0=1, m1=m, n1=n, k1=k, rsa0=0, csa0=0, rsa1=k + pad, csa1=1,
                          rsb0=0, csb0=0, rsb1=rsb, csb1=csb, rsc0=0, csc0=0, rsc1=n + int(rng.integers(0, 6)), csc1=1)


@pytest.mark.parametrize("chunk", range(10))
def test_random_fused_int8_calls_match_the_checker(gpu, chunk):
    rng = np.random.default_rng(7100 + chunk)
    for _ in range(40):
        kind, case = _random_case(rng)
        m, n = case.m0 * case.m1, case.n0 * case.n1
        a, b, c = case.make_inputs(int(rng.integers(1 << 30)))
        c[:] = rng.integers(-2 ** 31, 2 ** 31, size=c.size)
        plain = run_oracle_gemm(case, a, b, c)
        bias = rng.integers(-1 << 12, 1 << 12, n).astype(np.int32) if rng.integers(2) else None
        start = np.array([int(rng.integers(-1 << 20, 1 << 20))], np.int32) if rng.integers(2) else None
        act = int(rng.integers(2))
        rq = None
        if rng.integers(4):
            rsq, csq = (n + int(rng.choice([0, 3, 4])), 1) if rng.integers(3) else (1, m + int(rng.integers(0, 3)))
            per_column = bool(rng.integers(2))
            fmt = int(rng.choice([0, 0, 1, 2, 3, 4]))
            rows = support.blocked_offsets(case.m1, case.n1, case.m0, case.n0, case.rsc0, case.csc0, case.rsc1, case.csc1)
            spread = max(float(np.abs(plain[rows].astype(np.float64)).max()), 1.0)
            top = {0: 100.0, 1: 500.0, 2: 500.0, 3: 60000.0, 4: 60000.0}[fmt]
            scales = (rng.uniform(0.25, 2.0, n if per_column else 1) * top / spread).astype(np.float32)
            rq = dict(q=np.full((m - 1) * rsq + (n - 1) * csq + 1, 0x55, np.int8), rsq=rsq, csq=csq, scale=scales,
                      per_column=per_column, zero=int(rng.integers(-128, 128)), only=bool(rng.integers(2)), format=fmt)
        if bias is None and start is None and act == 0 and rq is None:
            bias = rng.integers(-9, 9, n).astype(np.int32)
        mode = "device" if rng.integers(4) else "host"
        what = (kind, m, n, case.k0 * case.k1, case.rsb1, case.csb1, case.alpha, case.beta, bias is not None, start is not None, act,
                None if rq is None else {key: rq[key] for key in ("rsq", "csq", "per_column", "zero", "only", "format")}, mode)
        out = run_fused_gemm(gpu, kind, case, a, b, c, bias, start, mode, activation=act, requant=rq)
        want = fused_expectation(case, plain, bias, start, activation=act, requant=rq)
        only = rq is not None and rq["only"]
        assert np.array_equal(out[0], c if only else want[0]), what
        if start is not None:
            assert out[1][0] == want[1][0], what
        if rq is not None:
            assert np.array_equal(out[2], want[2]), what
