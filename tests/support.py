"""Shared helpers of the test-suite: libraries, the reference's test tables,
seeded input generators, stride bookkeeping and comparators.

The comparison rules are the reference's own (test/gemm/gemm_i8rcprc_i8rcprc_i32rcprc.c:89-147,
test/gemm/gemm_bf16rcprc_bf16rcprc_f32rcprc.c:131-168, test/pack/pack_e8rc_e8rcprc.c:61-88):
integer GEMM, pack and cvt are compared exactly over the WHOLE buffer (so stride
gaps double as a clobber check); floating-point GEMM elementwise against
``2*((1+2^-24)^(K+2)-1) * (|alpha| |A||B| + |beta| |C|)`` with the products
evaluated in fp64.
"""
import json
import os

import numpy as np

from oracle import loader as oracle_loader

HERE = os.path.dirname(os.path.abspath(__file__))
TE = 64

_oracle = None
_ref = None
_tables = None


def oracle():
    global _oracle
    if _oracle is None:
        _oracle = oracle_loader.load_oracle()
    return _oracle


def ref():
    """The reference's scalar library built from its sources, or None."""
    global _ref
    if _ref is None and oracle_loader.ref_available():
        _ref = oracle_loader.load_ref()
    return _ref


def ref_tables():
    global _tables
    if _tables is None:
        with open(os.path.join(HERE, "golden", "ref_tables.json")) as fh:
            _tables = json.load(fh)
    return _tables


def table_rows(rel_path, kinds=("TEST",)):
    return [r for r in ref_tables()[rel_path] if any(r["kind"].startswith(k) for k in kinds)]


# --------------------------------------------------------------------------
# element types
# --------------------------------------------------------------------------

def f32_to_bf16_bits(x):
    """Round-to-nearest-even fp32 -> bf16 bit patterns (finite inputs)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    u = u + 0x7FFF + ((u >> 16) & 1)
    return (u >> 16).astype(np.uint16)


def bf16_bits_to_f32(b):
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def f16_bits_to_f32(b):
    return np.ascontiguousarray(b, dtype=np.uint16).view(np.float16).astype(np.float32)


def decode_table(fmt):
    """256-entry fp32 table of an OFP8 format from its definition
    (value = (-1)^s 2^(e-bias) (1 + m/2^M), subnormals 2^(1-bias) m/2^M; E4M3 has
    no infinities and one NaN code per sign, E5M2 is IEEE-like)."""
    mant, bias = (3, 7) if fmt == "f8e4m3" else (2, 15)
    out = np.zeros(256, dtype=np.float64)
    for code in range(256):
        s = -1.0 if code & 0x80 else 1.0
        e = (code & 0x7F) >> mant
        m = code & ((1 << mant) - 1)
        if fmt == "f8e4m3" and (code & 0x7F) == 0x7F:
            v = np.nan
        elif fmt == "f8e5m2" and e == 31:
            v = s * np.inf if m == 0 else np.nan
        elif e == 0:
            v = s * m * 2.0 ** (1 - bias - mant)
        else:
            v = s * (1 + m / 2.0 ** mant) * 2.0 ** (e - bias)
        out[code] = v
    return out


class EType:
    """One GEMM operand type: storage dtype, generator, widening to fp64."""

    def __init__(self, name, dtype, gen, widen):
        self.name, self.dtype, self.gen, self.widen = name, np.dtype(dtype), gen, widen


def _gen_i8(rng, n):
    return rng.integers(-128, 128, size=n, dtype=np.int8)


def _gen_bf16(rng, n):
    return f32_to_bf16_bits(rng.uniform(-1.0, 1.0, size=n).astype(np.float32))


def _gen_f16(rng, n):
    return rng.uniform(-1.0, 1.0, size=n).astype(np.float16).view(np.uint16)


def _gen_e4m3(rng, n):  # test/gemm/gemm_f8rcprc_f8rcprc_f32rcprc.h:72-78: bytes 8..126
    return rng.integers(8, 127, size=n, dtype=np.uint8)


def _gen_e5m2(rng, n):  # test/gemm/gemm_f8rcprc_f8rcprc_f32rcprc.h:80-86: bytes 4..123
    return rng.integers(4, 124, size=n, dtype=np.uint8)


def _gen_f32(rng, n):  # test/gemm/gemm_f32rcprc_f32rcprc_f32rcprc.h:64-66: uniform in [-1, 1]
    return rng.uniform(-1.0, 1.0, size=n).astype(np.float32)


def _gen_f64(rng, n):
    return rng.uniform(-1.0, 1.0, size=n)


ETYPES = {
    "f32": EType("f32", np.float32, _gen_f32, lambda a: a.astype(np.float64)),
    "f64": EType("f64", np.float64, _gen_f64, lambda a: a.astype(np.float64)),
    "i8": EType("i8", np.int8, _gen_i8, lambda a: a.astype(np.float64)),
    "bf16": EType("bf16", np.uint16, _gen_bf16, lambda a: bf16_bits_to_f32(a).astype(np.float64)),
    "f16": EType("f16", np.uint16, _gen_f16, lambda a: f16_bits_to_f32(a).astype(np.float64)),
    # f16 operands with an f16 accumulator and an f16 C (the f16 -> f16 GEMMs)
    "f16h": EType("f16h", np.uint16, _gen_f16, lambda a: f16_bits_to_f32(a).astype(np.float64)),
    "f8e4m3": EType("f8e4m3", np.uint8, _gen_e4m3, lambda a: decode_table("f8e4m3")[a]),
    "f8e5m2": EType("f8e5m2", np.uint8, _gen_e5m2, lambda a: decode_table("f8e5m2")[a]),
}


# --------------------------------------------------------------------------
# blocked-matrix bookkeeping
# --------------------------------------------------------------------------

def span(dims, strides):
    if any(d == 0 for d in dims):
        return 0
    return sum((d - 1) * s for d, s in zip(dims, strides)) + 1


def blocked_offsets(b1r, b1c, b0r, b0c, rs0, cs0, rs1, cs1):
    """Offsets of every element of a blocked matrix as a (b1r*b0r, b1c*b0c) array."""
    r = np.arange(b1r * b0r)
    c = np.arange(b1c * b0c)
    row = (r // b0r) * rs1 + (r % b0r) * rs0
    col = (c // b0c) * cs1 + (c % b0c) * cs0
    return row[:, None] + col[None, :]


class GemmCase:
    """One GEMM problem in the reference's blocked description."""

    FIELDS = ("m0", "n0", "k0", "m1", "n1", "k1", "rsa0", "csa0", "rsa1", "csa1", "rsb0", "csb0",
              "rsb1", "csb1", "rsc0", "csc0", "rsc1", "csc1")

    def __init__(self, ta, tb=None, alpha=1, beta=0, **kw):
        self.ta, self.tb = ta, tb or ta
        self.alpha, self.beta = alpha, beta
        for f in self.FIELDS:
            setattr(self, f, int(kw[f]))

    @property
    def is_int(self):
        return self.ta == "i8"

    @property
    def cdtype(self):
        return {"i8": np.int32, "f64": np.float64, "f16h": np.float16}.get(self.ta, np.float32)

    @property
    def ctag(self):
        """C's element type as the function names spell it."""
        return {"i8": "i32", "f64": "f64", "f16h": "f16"}.get(self.ta, "f32")

    @property
    def atag(self):
        """A's element type as the function names spell it."""
        return "f16" if self.ta == "f16h" else self.ta

    @property
    def btag(self):
        return "f16" if self.tb == "f16h" else self.tb

    @property
    def unit_roundoff_bits(self):
        """P of the reference's bound: accumulator precision (test/gemm/gemm_f64rcprc_f64rcprc_f64rcprc.c:190,
        test/gemm/gemm_f16rcprc_f16rcprc_f16rcprc.c:157)."""
        return {"f64": 53, "f16h": 11}.get(self.ta, 24)

    def spans(self):
        a = span((self.m1, self.k1, self.m0, self.k0), (self.rsa1, self.csa1, self.rsa0, self.csa0))
        b = span((self.k1, self.n1, self.k0, self.n0), (self.rsb1, self.csb1, self.rsb0, self.csb0))
        c = span((self.m1, self.n1, self.m0, self.n0), (self.rsc1, self.csc1, self.rsc0, self.csc0))
        return a, b, c

    def make_inputs(self, seed):
        rng = np.random.default_rng(seed)
        na, nb, nc = self.spans()
        a = ETYPES[self.ta].gen(rng, max(na, 1))
        b = ETYPES[self.tb].gen(rng, max(nb, 1))
        if self.is_int:
            c = rng.integers(-128, 128, size=max(nc, 1)).astype(np.int32)
        else:
            c = rng.uniform(-1.0, 1.0, size=max(nc, 1)).astype(self.cdtype)
        return a, b, c

    def rcprc_args(self, a, b, c):
        """Argument tuple of the blocked C entry points."""
        return (self.m0, self.n0, self.k0, self.m1, self.n1, self.k1, self.alpha, a, self.rsa0,
                self.csa0, self.rsa1, self.csa1, b, self.rsb0, self.csb0, self.rsb1, self.csb1,
                self.beta, c, self.rsc0, self.csc0, self.rsc1, self.csc1)

    def stem(self):
        return f"skl_gemm_{self.atag}rcprc_{self.btag}rcprc_{self.ctag}rcprc"

    def dense(self, a, b, c):
        """Logical (M x K), (K x N), (M x N) views gathered from the buffers, widened to fp64."""
        oa = blocked_offsets(self.m1, self.k1, self.m0, self.k0, self.rsa0, self.csa0, self.rsa1, self.csa1)
        ob = blocked_offsets(self.k1, self.n1, self.k0, self.n0, self.rsb0, self.csb0, self.rsb1, self.csb1)
        oc = blocked_offsets(self.m1, self.n1, self.m0, self.n0, self.rsc0, self.csc0, self.rsc1, self.csc1)
        A = ETYPES[self.ta].widen(a[oa]) if oa.size else np.zeros(oa.shape)
        B = ETYPES[self.tb].widen(b[ob]) if ob.size else np.zeros(ob.shape)
        C = c[oc].astype(np.float64) if oc.size else np.zeros(oc.shape)
        return A, B, C, oc

    def fp_bound(self, a, b, c_before):
        """Elementwise tolerance of the reference's fp GEMM tests
        (test/gemm/gemm_bf16rcprc_bf16rcprc_f32rcprc.c:131-168)."""
        A, B, C, oc = self.dense(a, b, c_before)
        K = self.k0 * self.k1
        gamma = 2.0 * np.expm1((K + 2) * np.log1p(2.0 ** -self.unit_roundoff_bits))
        bound = gamma * (abs(self.alpha) * (np.abs(A) @ np.abs(B)) + abs(self.beta) * np.abs(C))
        exact = self.alpha * (A @ B) + self.beta * C
        return exact, bound, oc


def rowmajor_case(ta, m, n, k, alpha=1, beta=0, rsa=None, rsb=None, rsc=None, tb=None):
    return GemmCase(ta, tb, alpha, beta, m0=1, n0=1, k0=1, m1=m, n1=n, k1=k, rsa0=0, csa0=0,
                    rsa1=rsa or k, csa1=1, rsb0=0, csb0=0, rsb1=rsb or n, csb1=1, rsc0=0, csc0=0,
                    rsc1=rsc or n, csc1=1)


def colmajor_a_case(ta, m, n, k, alpha=1, beta=0, csa=None, rsb=None, rsc=None, tb=None):
    return GemmCase(ta, tb, alpha, beta, m0=1, n0=1, k0=1, m1=m, n1=n, k1=k, rsa0=0, csa0=0, rsa1=1,
                    csa1=csa or m, rsb0=0, csb0=0, rsb1=rsb or n, csb1=1, rsc0=0, csc0=0,
                    rsc1=rsc or n, csc1=1)


def panel_case(ta, m1, n1, k, alpha=1, beta=0, csa1=0, rsa1=0, rsb1=0, csb1=0, rsc0=0, csc0=0,
               rsc1=0, csc1=0):
    """Defaults of the reference's packed suites
    (test/gemm/xsfmm/skl_gemm_i8rcptex1c_i8rcp1xte_i32rcptexterc_xsfmm32a8i.c:258-282)."""
    csa1 = csa1 or TE
    rsa1 = rsa1 or k * csa1
    rsb1 = rsb1 or TE
    csb1 = csb1 or k * rsb1
    csc0 = csc0 or 1
    rsc0 = rsc0 or TE * csc0
    csc1 = csc1 or (TE - 1) * rsc0 + (TE - 1) * csc0 + 1
    rsc1 = rsc1 or n1 * csc1
    return GemmCase(ta, None, alpha, beta, m0=TE, n0=TE, k0=1, m1=m1, n1=n1, k1=k, rsa0=1, csa0=TE,
                    rsa1=rsa1, csa1=csa1, rsb0=TE, csb0=1, rsb1=rsb1, csb1=csb1, rsc0=rsc0, csc0=csc0,
                    rsc1=rsc1, csc1=csc1)


def dot4_case(m, n, k1, alpha=1, beta=0, rsa1=0, csa1=0, rsb1=0, rsc1=0):
    """Defaults of test/gemm/xsfvqdotq/skl_gemm_i8rcp1x4_i8p4x1c_i32_xsfvqdotq.c:143-165."""
    csa1 = csa1 or 4
    rsa1 = rsa1 or k1 * csa1
    rsb1 = rsb1 or n * 4
    rsc1 = rsc1 or n
    return GemmCase("i8", None, alpha, beta, m0=1, n0=1, k0=4, m1=m, n1=n, k1=k1, rsa0=4, csa0=1,
                    rsa1=rsa1, csa1=csa1, rsb0=1, csb0=4, rsb1=rsb1, csb1=4, rsc0=1, csc0=1,
                    rsc1=rsc1, csc1=1)


# --------------------------------------------------------------------------
# checks
# --------------------------------------------------------------------------

def run_oracle_gemm(case, a, b, c):
    out = c.copy()
    fn = getattr(oracle(), case_oracle_name(case))
    fn(*case_args(case, a, b, out))
    return out


def case_oracle_name(case):
    if case.ta != case.tb:
        return "skl_gemm_f8e4m3rc_f8e5m2rc_f32rc_oracle"
    return case.stem() + "_oracle"


def case_args(case, a, b, c):
    if case.ta != case.tb:  # only the strided form exists for mixed formats
        assert case.m0 == case.n0 == case.k0 == 1
        return (case.m1, case.n1, case.k1, case.alpha, a, case.rsa1, case.csa1, b, case.rsb1, case.csb1,
                case.beta, c, case.rsc1, case.csc1)
    return case.rcprc_args(a, b, c)


#: Allowance on top of the reference's elementwise bound for fp8 operands: none. Up to K = 2304 the fp8 kinds are
#: multiplied exactly (bytes widened to f16, f16 matrix-core instructions, fp32 sums - the arithmetic the bound
#: assumes); beyond that the fp8 instructions are used, whose error (products of one instruction aligned to a
#: common exponent, about 12 bits kept below the largest: <= 2^-11.9 * sum|a||b|) is inside the bound
#: 2((1 + 2^-24)^(K+2) - 1) * sum|a||b| from K = 2193 on.
FP8_MFMA_REL = 0.0


def assert_fp_gemm_close(case, a, b, c_before, c_after, frob_tol=1e-3, extra_rel=0.0):
    """Reference's elementwise bound (+ `extra_rel` * |alpha| |A||B|) and relative
    Frobenius error vs the fp64 result; every element outside the addressed set
    unchanged. Returns the worst error / reference-bound ratio."""
    exact, bound, oc = case.fp_bound(a, b, c_before)
    ref_bound = bound
    if extra_rel:
        A, B, _, _ = case.dense(a, b, c_before)
        bound = bound + extra_rel * abs(case.alpha) * (np.abs(A) @ np.abs(B))
    got = c_after[oc].astype(np.float64) if oc.size else exact
    err = np.abs(got - exact)
    # a few ulps of slack on top of the bound for the final rounding of tiny results
    slack = np.abs(exact) * 2.0 ** -(case.unit_roundoff_bits - 2) + 1e-30
    bad = err > bound + slack
    assert not bad.any(), (f"{int(bad.sum())} elements exceed the reference bound; worst ratio "
                           f"{float((err / (bound + slack)).max()):.3g}")
    denom = np.linalg.norm(exact)
    if denom > 0 and frob_tol is not None:
        rel = np.linalg.norm(got - exact) / denom
        assert rel <= frob_tol, f"relative Frobenius error {rel:.3e} > {frob_tol}"
    mask = np.ones(c_after.shape, dtype=bool)
    if oc.size:
        mask[oc.ravel()] = False
    assert np.array_equal(c_after[mask].view(np.uint8), c_before[mask].view(np.uint8)), \
        "elements outside the addressed C were modified"
    return float((err / (ref_bound + slack)).max()) if err.size else 0.0


def ulp_error_f32(x, r):
    """skl_abs_error_ulp_f32 of the reference's test driver (test/skl-test-driver.h:565-592): the distance between
    x and the reference value r in units of ulp(r), denormal results counted in units of 2^-149."""
    x, r = np.asarray(x, np.float32), np.asarray(r, np.float32)
    with np.errstate(invalid="ignore", over="ignore"):
        d = np.abs(x.astype(np.float64) - r.astype(np.float64))
        _, e = np.frexp(r.astype(np.float64))
        e = np.where((e < -125) | (r == 0), -125 - 24, e - 24)
        err = np.ldexp(d, -e)
    same = (x == r) | (np.isnan(x) & np.isnan(r))
    bad = np.isinf(r) | np.isnan(x) | np.isnan(r)
    return np.where(same, 0.0, np.where(bad, np.inf, err))


def activation_reference(values, activation):
    """skl_silu_f32_ref (2) / skl_gelu_f32_ref (3) through the checker's restatement, for a float32 array."""
    v = np.ascontiguousarray(values, np.float32).copy().reshape(-1)
    oracle().skl_oracle_act_requant_f32(1, v.size, v, v.size, 1, activation, None, 0, 0, None, 0, 0)
    return v.reshape(np.shape(values))


#: what the reference's own vector kernels are held to (test/sigmoid/sigmoid_f32_zve32f.c: 52 ulp on [-110, 18];
#: test/gelu/skl_gelu_f32_zve32f.c, the tightest variant: 4 ulp for x >= 0, 5 in [-1, 0), 62 in [-2, -1), 1.7e7 below)
def activation_ulp_bound(x, activation):
    x = np.asarray(x, np.float64)
    if activation == 2:
        return np.full(x.shape, 52.0)
    return np.where(x >= 0, 4.0, np.where(x >= -1, 5.0, np.where(x >= -2, 62.0, 1.7e7)))
