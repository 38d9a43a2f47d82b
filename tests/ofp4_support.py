"""Helpers of the OFP4-weight GEMM tests: the packing of ref/cvt/cvt_ofp4.c:59-68 (value 2i in the low nibble of
byte i) and the E2M1 value table from the format's definition (1 sign, 2 exponent bits with bias 1, 1 mantissa bit:
0, 0.5, 1, 1.5, 2, 3, 4, 6 and their negatives; no infinities, no NaN)."""
import numpy as np

import support

E2M1_VALUES = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0])
# the E4M3 byte of each E2M1 value (exact): sign, exponent + 6 (E4M3's bias 7 against E2M1's 1), mantissa bit on top
E2M1_AS_E4M3 = np.array([0x00, 0x30, 0x38, 0x3C, 0x40, 0x44, 0x48, 0x4C, 0x80, 0xB0, 0xB8, 0xBC, 0xC0, 0xC4, 0xC8, 0xCC], np.uint8)


def pack_nibbles(values):
    """A flat array of 4-bit codes as bytes, value 2i in the low nibble of byte i."""
    v = np.asarray(values, np.uint8)
    if v.size % 2:
        v = np.concatenate([v, np.zeros(1, np.uint8)])
    return (v[0::2] | (v[1::2] << 4)).astype(np.uint8)


def f8_case(m, n, k, ldb, alpha, beta, rsa=None, csa=1, rsc=None, csc=1):
    """The fp8 problem that defines the result: B converted to E4M3, stored column by column (rsb = 1, csb = ldb)."""
    return support.GemmCase("f8e4m3", None, alpha, beta, m0=1, n0=1, k0=1, m1=m, n1=n, k1=k, rsa0=0, csa0=0,
                            rsa1=rsa if rsa is not None else k, csa1=csa, rsb0=0, csb0=0, rsb1=1, csb1=ldb,
                            rsc0=0, csc0=0, rsc1=rsc if rsc is not None else n, csc1=csc)


def make_problem(seed, m, n, k, ldb, alpha=1.0, beta=0.0, **strides):
    """(case, a, packed b, b as E4M3 bytes, c): random E4M3 A in the reference's test range, every E2M1 code in B."""
    rng = np.random.default_rng(seed)
    case = f8_case(m, n, k, ldb, alpha, beta, **strides)
    na, nb, nc = case.spans()
    a = support.ETYPES["f8e4m3"].gen(rng, max(na, 1))
    codes = rng.integers(0, 16, size=max(nb, 1), dtype=np.uint8)
    c = rng.uniform(-1.0, 1.0, size=max(nc, 1)).astype(np.float32)
    return case, a, pack_nibbles(codes), E2M1_AS_E4M3[codes], c


def make_mx_problem(seed, m, n, k, ldb, alpha=1.0, beta=0.0, **strides):
    """make_problem plus block scales: (case, a, packed b, B as fp64 values (k x n), scales, lds, c). Scales within
    2^-6 .. 2^6 so that nothing leaves fp32's comfortable range."""
    case, a, b4, b8, c = make_problem(seed, m, n, k, ldb, alpha, beta, **strides)
    rng = np.random.default_rng(seed + 1)
    blocks = (k + 31) // 32
    lds = blocks + int(rng.integers(0, 3))
    scales = rng.integers(121, 134, size=max(n * lds, 1), dtype=np.uint8)
    return case, a, b4, b8, scales, lds, c


def mx_bound(case, a, b8, scales, lds, c, m, n, k, ldb):
    """(exact fp64 result, elementwise bound of the reference's fp8 GEMM test) with B's values times their scales."""
    A = support.decode_table("f8e4m3")[a[(np.arange(m)[:, None] * case.rsa1 + np.arange(k)[None, :] * case.csa1)]] if k else np.zeros((m, 0))
    Bv = support.decode_table("f8e4m3")[b8[(np.arange(n)[None, :] * ldb + np.arange(k)[:, None])]] if k else np.zeros((0, n))
    S = np.ldexp(1.0, scales[(np.arange(n)[None, :] * lds + (np.arange(k) // 32)[:, None])].astype(np.int64) - 127) if k else np.zeros((0, n))
    B = Bv * S
    oc = np.arange(m)[:, None] * case.rsc1 + np.arange(n)[None, :] * case.csc1
    C = c[oc].astype(np.float64)
    gamma = 2.0 * np.expm1((k + 2) * np.log1p(2.0 ** -24))
    bound = gamma * (abs(case.alpha) * (np.abs(A) @ np.abs(B)) + abs(case.beta) * np.abs(C))
    return case.alpha * (A @ B) + case.beta * C, bound, oc
