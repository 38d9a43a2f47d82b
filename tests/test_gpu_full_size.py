"""The benchmark's full-size configurations, checked through properties that do not
need the scalar checker to run at that size:

* integer GEMM: Freivalds' identity  (A B) v = A (B v)  and  u^T (A B) = (u^T A) B  with
  random +-1 vectors, exact in int64, plus a sample of full rows recomputed exactly;
* fp GEMM: the same identities in fp64 with the reference's error bound summed
  along the contraction, plus sampled rows against the fp64 product;
* the fp8 operands are produced by the library's own saturating cvt from N(0,1)
  fp32 data (config 4) and checked against the CPU checker on a sample.
"""
import numpy as np
import pytest

import skl_amd
import support
from skl_amd import DeviceBuffer
from support import oracle

pytestmark = pytest.mark.gpu


def _sample_rows(rng, m, count=48):
    return np.sort(rng.choice(m, size=count, replace=False))


def test_int8_gemm_8192_cubed(gpu):
    """Target shape: int8 8192^3, alpha = 1, beta = 0, row-major."""
    n = 8192
    rng = np.random.default_rng(0x5EED0060)
    a = rng.integers(-128, 128, size=(n, n), dtype=np.int8)
    b = rng.integers(-128, 128, size=(n, n), dtype=np.int8)
    da, db, dc = DeviceBuffer.from_array(a), DeviceBuffer.from_array(b), DeviceBuffer(4 * n * n)
    gpu.skl_hip_memset(dc, 0xAA, 4 * n * n)   # poison: beta = 0 must overwrite every element
    gpu.skl_gemm_i8_i8_i32_gfx950(n, n, n, 1, da, n, db, n, 0, dc, n)
    gpu.skl_hip_synchronize()
    skl_amd.check_error()
    c = dc.download(np.int32).reshape(n, n).astype(np.int64)
    v = rng.choice(np.array([-1, 1], dtype=np.int64), size=n)
    u = rng.choice(np.array([-1, 1], dtype=np.int64), size=n)
    a64, b64 = a.astype(np.int64), b.astype(np.int64)
    assert np.array_equal(c @ v, a64 @ (b64 @ v))
    assert np.array_equal(u @ c, (u @ a64) @ b64)
    rows = _sample_rows(rng, n)
    want = (a[rows].astype(np.float64) @ b.astype(np.float64)).astype(np.int64)   # |sum| < 2^53: exact
    assert np.array_equal(c[rows], want)
    for d in (da, db, dc):
        d.free()


@pytest.mark.parametrize("fmt_b", ("f8e4m3", "f8e5m2"))
def test_fp8_gemm_8192_cubed(gpu, fmt_b):
    """Config 4: fp32 ~ N(0,1) -> E4M3 (A, stored column-major) and E4M3 / E5M2 (B) through
    the saturating cvt with scale 1, then the 8192^3 GEMM with alpha = 1, beta = 0."""
    n = 8192
    rng = np.random.default_rng(0x5EED0040)
    xa = rng.normal(size=n * n).astype(np.float32)
    xb = rng.normal(size=n * n).astype(np.float32)
    dxa, dxb = DeviceBuffer.from_array(xa), DeviceBuffer.from_array(xb)
    da, db, dc = DeviceBuffer(n * n), DeviceBuffer(n * n), DeviceBuffer(4 * n * n)
    gpu.skl_cvt_sat_f32_f8e4m3_gfx950(da, dxa, 1.0, n * n)
    getattr(gpu, f"skl_cvt_sat_f32_{fmt_b}_gfx950")(db, dxb, 1.0, n * n)
    gpu.skl_hip_memset(dc, 0, 4 * n * n)
    if fmt_b == "f8e4m3":
        gpu.skl_gemm_f8e4m3c_f8e4m3_f32_gfx950(n, n, n, 1.0, da, n, db, n, 0.0, dc, n)
    else:
        gpu.skl_gemm_f8e4m3rc_f8e5m2rc_f32rc_gfx950(n, n, n, 1.0, da, 1, n, db, n, 1, 0.0, dc, n, 1)
    gpu.skl_hip_synchronize()
    skl_amd.check_error()
    a8, b8 = da.download(np.uint8), db.download(np.uint8)
    # cvt bit-exact on a 1M-element sample of each operand
    idx = slice(123456, 123456 + (1 << 20))
    wa = np.zeros(1 << 20, np.uint8)
    oracle().skl_cvt_sat_f32_f8e4m3_oracle(wa, xa[idx], 1.0, 1 << 20)
    assert np.array_equal(a8[idx], wa)
    wb = np.zeros(1 << 20, np.uint8)
    getattr(oracle(), f"skl_cvt_sat_f32_{fmt_b}_oracle")(wb, xb[idx], 1.0, 1 << 20)
    assert np.array_equal(b8[idx], wb)
    At = support.decode_table("f8e4m3")[a8].reshape(n, n)        # A^T: k x m (column-major A)
    B = support.decode_table(fmt_b)[b8].reshape(n, n)
    c = dc.download(np.float32).reshape(n, n).astype(np.float64)
    v = rng.choice(np.array([-1.0, 1.0]), size=n)
    exact_v = At.T @ (B @ v)
    bound_v = np.abs(At).T @ (np.abs(B) @ np.ones(n))             # sum over j of (|A||B|)_ij
    gamma = 2.0 * ((1.0 + 2.0 ** -24) ** (n + 2) - 1.0) + support.FP8_MFMA_REL
    assert np.all(np.abs(c @ v - exact_v) <= gamma * bound_v)
    rows = _sample_rows(rng, n, 32)
    exact = At[:, rows].T @ B
    got = c[rows]
    rel = np.linalg.norm(got - exact) / np.linalg.norm(exact)
    assert rel <= 1e-3, rel
    bound = gamma * (np.abs(At[:, rows]).T @ np.abs(B))
    assert np.all(np.abs(got - exact) <= bound)
    for d in (dxa, dxb, da, db, dc):
        d.free()


def test_bf16_gemm_config3(gpu):
    """Config 3: bf16 2048 x 4096 x 4096, A ~ N(0,1), B ~ N(0, 0.02^2), alpha = 1, beta = 1, C ~ N(0,1)."""
    m, n, k = 2048, 4096, 4096
    rng = np.random.default_rng(0x5EED0030)
    a = support.f32_to_bf16_bits(rng.normal(size=m * k).astype(np.float32))
    b = support.f32_to_bf16_bits((rng.normal(size=k * n) * 0.02).astype(np.float32))
    c0 = rng.normal(size=m * n).astype(np.float32)
    da, db, dc = DeviceBuffer.from_array(a), DeviceBuffer.from_array(b), DeviceBuffer.from_array(c0)
    gpu.skl_gemm_bf16_bf16_f32_gfx950(m, n, k, 1.0, da, k, db, n, 1.0, dc, n)
    gpu.skl_hip_synchronize()
    skl_amd.check_error()
    got = dc.download(np.float32).reshape(m, n).astype(np.float64)
    A = support.bf16_bits_to_f32(a).reshape(m, k).astype(np.float64)
    B = support.bf16_bits_to_f32(b).reshape(k, n).astype(np.float64)
    C0 = c0.reshape(m, n).astype(np.float64)
    exact = A @ B + C0
    rel = np.linalg.norm(got - exact) / np.linalg.norm(exact)
    assert rel <= 1e-3, rel
    gamma = 2.0 * ((1.0 + 2.0 ** -24) ** (k + 2) - 1.0)
    bound = gamma * (np.abs(A) @ np.abs(B) + np.abs(C0))
    assert np.all(np.abs(got - exact) <= bound + np.abs(exact) * 2.0 ** -22)
    for d in (da, db, dc):
        d.free()


def test_f16_pipeline_config5(gpu):
    """Config 5: pack A and B into TE = 64 panels, panel GEMM into TE x TE blocks of C,
    unpack C; pack/unpack checked by the closed-form index map, the product by sampled
    rows and Freivalds in fp64."""
    te, m, k, n = 64, 4096, 4096, 14336
    rng = np.random.default_rng(0x5EED0050)
    a = rng.uniform(-1, 1, m * k).astype(np.float16)
    b = rng.uniform(-1, 1, k * n).astype(np.float16)
    da, db = DeviceBuffer.from_array(a.view(np.uint16)), DeviceBuffer.from_array(b.view(np.uint16))
    dap, dbp = DeviceBuffer(2 * m * k), DeviceBuffer(2 * k * n)
    dcp, dc = DeviceBuffer(4 * m * n), DeviceBuffer(4 * m * n)
    gpu.skl_hip_memset(dcp, 0, 4 * m * n)
    m1, n1 = m // te, n // te
    gpu.skl_pack_e16_e16rcptex1c_gfx950(m, k, da, k, dap, k * te, te, 0)
    gpu.skl_pack_e16rc_e16rcprc_gfx950(k, n, db, n, 1, 1, te, dbp, te, 1, te, k * te, 0)
    gpu.skl_gemm_f16rcptex1c_f16rcp1xte_f32rcptexterc_gfx950(m1, n1, k, 1.0, dap, k * te, te, dbp, te, k * te, 0.0, dcp,
                                                             te, 1, n1 * te * te, te * te)
    gpu.skl_unpack_e32rcprc_e32rc_gfx950(te, te, dcp, te, 1, n1 * te * te, te * te, m, n, dc, n, 1)
    gpu.skl_hip_synchronize()
    skl_amd.check_error()
    ap = dap.download(np.uint16).reshape(m1, k, te)
    assert np.array_equal(ap, a.view(np.uint16).reshape(m1, te, k).transpose(0, 2, 1))
    bp = dbp.download(np.uint16).reshape(n1, k, te)
    assert np.array_equal(bp, b.view(np.uint16).reshape(k, n1, te).transpose(1, 0, 2))
    cp = dcp.download(np.float32)
    c = dc.download(np.float32).reshape(m, n)
    assert np.array_equal(c, cp.reshape(m1, n1, te, te).transpose(0, 2, 1, 3).reshape(m, n))   # unpack is bit-exact
    A, B = a.reshape(m, k).astype(np.float64), b.reshape(k, n).astype(np.float64)
    rows = _sample_rows(rng, m, 32)
    exact = A[rows] @ B
    got = c[rows].astype(np.float64)
    rel = np.linalg.norm(got - exact) / np.linalg.norm(exact)
    assert rel <= 1e-3, rel
    gamma = 2.0 * ((1.0 + 2.0 ** -24) ** (k + 2) - 1.0)
    assert np.all(np.abs(got - exact) <= gamma * (np.abs(A[rows]) @ np.abs(B)) + np.abs(exact) * 2.0 ** -22)
    v = rng.choice(np.array([-1.0, 1.0]), size=n)
    assert np.all(np.abs(c.astype(np.float64) @ v - A @ (B @ v)) <= gamma * (np.abs(A) @ (np.abs(B) @ np.ones(n))))
    for d in (da, db, dap, dbp, dcp, dc):
        d.free()
