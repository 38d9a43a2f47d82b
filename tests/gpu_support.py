"""Helpers of the GPU parity tests: every call goes through the C-ABI of
libskl_gfx950.so, either with ordinary host arrays (the library stages them) or
with device buffers (asynchronous launch, explicit synchronise + download)."""
import numpy as np

import skl_amd
from skl_amd import DeviceBuffer

MODES = ("host", "device")


def _finish(lib):
    rc = lib.skl_hip_synchronize()
    skl_amd.check_error()
    assert rc == 0


def gemm_entry_args(kind, case, a, b, c):
    """(function name, argument tuple) of the entry point `kind` for a case that
    fits it; mirrors the execute() callbacks of the reference's suites."""
    t = case.atag
    cty = case.ctag
    if kind == "rcprc":
        return case.stem() + "_gfx950", case.rcprc_args(a, b, c)
    if kind == "rc":
        tb = case.btag
        return (f"skl_gemm_{t}rc_{tb}rc_{cty}rc_gfx950",
                (case.m1, case.n1, case.k1, case.alpha, a, case.rsa1, case.csa1, b, case.rsb1, case.csb1,
                 case.beta, c, case.rsc1, case.csc1))
    if kind == "rowmajor":   # test/gemm/rvv/skl_gemm_i8_i8_i32_zve32x_x390.c:106-113
        return (f"skl_gemm_{t}_{t}_{cty}_gfx950",
                (case.m1, case.n1, case.k1, case.alpha, a, case.rsa1, b, case.rsb1, case.beta, c, case.rsc1))
    if kind == "colmajor_a":  # test/gemm/xsfmm/skl_gemm_i8c_i8_i32_xsfmm32a8i.c:118-120
        return (f"skl_gemm_{t}c_{t}_{cty}_gfx950",
                (case.m1, case.n1, case.k1, case.alpha, a, case.csa1, b, case.rsb1, case.beta, c, case.rsc1))
    if kind == "panel":
        return (f"skl_gemm_{t}rcptex1c_{t}rcp1xte_{cty}rcptexterc_gfx950",
                (case.m1, case.n1, case.k1, case.alpha, a, case.rsa1, case.csa1, b, case.rsb1, case.csb1,
                 case.beta, c, case.rsc0, case.csc0, case.rsc1, case.csc1))
    if kind == "dot4":
        return ("skl_gemm_i8rcp1x4_i8p4x1c_i32_gfx950",
                (case.m1, case.n1, case.k1, case.alpha, a, case.rsa1, case.csa1, b, case.rsb1, case.beta, c,
                 case.rsc1))
    raise ValueError(kind)


def run_gemm(lib, kind, case, a, b, c, mode):
    """Runs one GEMM through the library; returns C's whole buffer afterwards."""
    if mode == "host":
        out = c.copy()
        name, args = gemm_entry_args(kind, case, a, b, out)
        getattr(lib, name)(*args)
        skl_amd.check_error()
        return out
    da, db, dc = DeviceBuffer.from_array(a), DeviceBuffer.from_array(b), DeviceBuffer.from_array(c)
    name, args = gemm_entry_args(kind, case, da, db, dc)
    getattr(lib, name)(*args)
    _finish(lib)
    out = dc.download(c.dtype, c.size)
    for d in (da, db, dc):
        d.free()
    return out


def run_fused_gemm(lib, kind, case, a, b, c, bias, mx, mode, activation=0, requant=None):
    """Runs `skl_gemm_fused_*` (kind "rc" or "rcprc"); returns (C's whole buffer, *max) afterwards.
    `bias` / `mx` are arrays of C's type (n values / one value) or None. `requant` = dict(q=<int8 buffer>,
    rsq, csq, scale=<float32 array>, per_column, zero, only, format) asks for the requantised copy, whose buffer
    afterwards is returned as a third value."""
    rq = requant or {}

    def call(a_, b_, c_, bias_, mx_, q_, scale_):
        name, args = gemm_entry_args(kind, case, a_, b_, c_)
        fused = name.replace("skl_gemm_", "skl_gemm_fused_")
        getattr(lib, fused)(*args, skl_amd.Epilogue(bias_, mx_, activation=activation, q=q_, rsq=rq.get("rsq", 0),
                                                    csq=rq.get("csq", 0), q_scale=scale_,
                                                    q_scale_per_column=rq.get("per_column", False),
                                                    q_zero=rq.get("zero", 0), q_only=rq.get("only", False),
                                                    q_format=rq.get("format", 0)))

    q, scale = rq.get("q"), rq.get("scale")
    if mode == "host":
        out, mo, qo = c.copy(), None if mx is None else mx.copy(), None if q is None else q.copy()
        call(a, b, out, bias, mo, qo, scale)
        skl_amd.check_error()
        return (out, mo) if requant is None else (out, mo, qo)
    bufs = [DeviceBuffer.from_array(x) if x is not None else None for x in (a, b, c, bias, mx, q, scale)]
    call(*bufs)
    _finish(lib)
    out = bufs[2].download(c.dtype, c.size)
    mo = None if mx is None else bufs[4].download(mx.dtype, mx.size)
    qo = None if q is None else bufs[5].download(q.dtype, q.size)
    for d in bufs:
        if d is not None:
            d.free()
    return (out, mo) if requant is None else (out, mo, qo)


def run_inout(lib, name, build_args, src, dst, mode):
    """Runs an entry point with one input and one in/out buffer. `build_args(src, dst)`
    returns the C argument tuple."""
    if mode == "host":
        out = dst.copy()
        getattr(lib, name)(*build_args(src, out))
        skl_amd.check_error()
        return out
    ds, dd = DeviceBuffer.from_array(src), DeviceBuffer.from_array(dst)
    getattr(lib, name)(*build_args(ds, dd))
    _finish(lib)
    out = dd.download(dst.dtype, dst.size)
    ds.free()
    dd.free()
    return out
