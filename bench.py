#!/usr/bin/env python3
"""Benchmark of the GEMM / GEMV / pack / cvt hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-extra] [--full] [--no-cpu] [--out FILE]
    python bench.py --vendor-only      (the vendor BLAS through torch on three of the products, for comparison)

Prints ONE compact JSON line (a few KB) and writes the full record of everything it measured to the file that
`--out` names; `--full` also runs the workloads that are not benchmark configurations. The headline (`value`) is the int8 GEMV decode shape
(1x4096 times 4096x11008, benchmark configuration 2) in GB/s of algorithmic bytes with
all operands resident in HBM. A "step" is `config.calls_per_step` GEMV calls back to back,
each on the next of eight weight matrices (their total size exceeds the 256 MiB last-level
cache, so the stream comes from HBM): one 10 us call per step would time the synchronisation
around the step, not the kernel. `value` comes from the wall clock around the K steps,
`roofline.achieved` from HIP events on the library's stream around the same calls.
`roofline.configs` is the table of the other benchmark configurations (TOPS / TFLOP/s or GB/s and
fraction of the roofline, each timed the same way), `roofline.measured_peak` what a plain read of
the same buffers reaches on this device, `roofline.measured_peaks` all ceilings measured in the run (plain read;
matrix cores alone on register operands). `cpu_baseline` is the reference's scalar routine (or, where that
library was not built, the CPU checker) timed on this host for the same shape.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

import skl_amd  # noqa: E402
from skl_amd import DeviceBuffer  # noqa: E402

HBM_PEAK_GBS = 8000.0
MFMA_PEAK_TOPS = {"i8": 5000.0, "f8": 5000.0, "bf16": 2500.0, "f16": 2500.0, "f32": 157.3, "f64": 78.6}
METRIC = "GEMM TOPS (int8/fp8/bf16) + GEMV HBM GB/s on 1 MI355X, % of roofline"
MFMA_WARM_MS = 60.0  # matrix-core workloads warm up at least this long before they are timed (see Timer.run)
LLC_BYTES = 256 << 20  # buffers of HBM-bound workloads are rotated so that a step streams more than this


class Timer:
    """Times `steps` steps of `calls` calls of fn(i) each after `warmup` untimed steps: wall clock around a
    synchronised region, and HIP events on the library's stream inside it."""

    def __init__(self, lib):
        self.lib = lib
        self.e0, self.e1 = lib.skl_hip_event_create(), lib.skl_hip_event_create()

    def run(self, fn, steps, warmup, calls=1, min_warm_ms=0.0):
        lib = self.lib
        for i in range(warmup * calls):
            fn(i)
        lib.skl_hip_synchronize()
        # Matrix-core kernels: the device raises its clock over the first tens of milliseconds of such a load (fp8
        # 8192^3: 467 us per call at first, 406 us from about the 100th call on), so these workloads keep warming up
        # until `min_warm_ms` of work have passed and the figure is the sustained one.
        t_warm, i = time.perf_counter(), 0
        while (time.perf_counter() - t_warm) * 1e3 < min_warm_ms:
            for _ in range(max(1, calls)):
                fn(i)
                i += 1
            lib.skl_hip_synchronize()
        t0 = time.perf_counter()
        lib.skl_hip_event_record(self.e0)
        for i in range(steps * calls):
            fn(i)
        lib.skl_hip_event_record(self.e1)
        ev_ms = lib.skl_hip_event_elapsed_ms(self.e0, self.e1)
        lib.skl_hip_synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3
        skl_amd.check_error()
        return wall_ms / steps, ev_ms / (steps * calls)


def rand_i8(rng, n):
    return rng.integers(-128, 128, size=n, dtype=np.int8)


def bf16_bits(x):
    u = x.astype(np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


# ----------------------------------------------------------------------------
# workloads: each returns (callable(i), per-step algorithmic bytes, per-step ops, bound, dtype key)
# ----------------------------------------------------------------------------

def wl_gemv(lib, rng):
    k, n, nbuf = 4096, 11008, 8
    w = [DeviceBuffer.from_array(rand_i8(rng, k * n)) for _ in range(nbuf)]
    x = DeviceBuffer.from_array(rand_i8(rng, k))
    y = DeviceBuffer(4 * n)

    def step(i):
        lib.skl_gemm_i8_i8_i32_gfx950(1, n, k, 1, x, k, w[i % nbuf], n, 0, y, n)

    return dict(fn=step, bytes=k * n + k + 4 * n, ops=2 * k * n, bound="hbm", dtype="i8", keep=(w, x, y), nbuf=nbuf,
                name="int8 GEMV 1x4096x11008 (row-major W, beta=0)", kernel="gemv_kernel<int8 row-major>")


def wl_gemv_large(lib, rng):
    """The same kernel on a stream long enough that launch and tail no longer show: 235 MB of weights."""
    k, n, nbuf = 8192, 28672, 2
    w = [DeviceBuffer.from_array(rand_i8(rng, k * n)) for _ in range(nbuf)]
    x = DeviceBuffer.from_array(rand_i8(rng, k))
    y = DeviceBuffer(4 * n)

    def step(i):
        lib.skl_gemm_i8_i8_i32_gfx950(1, n, k, 1, x, k, w[i % nbuf], n, 0, y, n)

    return dict(fn=step, bytes=k * n + k + 4 * n, ops=2 * k * n, bound="hbm", dtype="i8", keep=(w, x, y),
                name="int8 GEMV 1x8192x28672 (row-major W, beta=0)", kernel="gemv_kernel<int8 row-major>")


def wl_gemv_kc(lib, rng):
    """The config-2 product with the weights stored column by column (B with K contiguous: a linear layer's
    [out][in] weight): one dot product over contiguous memory per output, no sums between workgroups."""
    k, n, nbuf = 4096, 11008, 8
    w = [DeviceBuffer.from_array(rand_i8(rng, k * n)) for _ in range(nbuf)]
    x = DeviceBuffer.from_array(rand_i8(rng, k))
    y = DeviceBuffer(4 * n)

    def step(i):
        lib.skl_gemm_i8rc_i8rc_i32rc_gfx950(1, n, k, 1, x, k, 1, w[i % nbuf], 1, k, 0, y, n, 1)

    return dict(fn=step, bytes=k * n + k + 4 * n, ops=2 * k * n, bound="hbm", dtype="i8", keep=(w, x, y),
                name="int8 GEMV 1x4096x11008, W with K contiguous ([n][k]), beta=0", kernel="gemv_kc_kernel<int8>")


def _wl_batch_kc(m, kind="i8", k=4096, n=11008):
    """A decode batch against weights stored column by column (B with K contiguous, [out][in])."""
    def build(lib, rng):
        nbuf = 8
        if kind == "i8":
            w = [DeviceBuffer.from_array(rand_i8(rng, k * n)) for _ in range(nbuf)]
            x = DeviceBuffer.from_array(rand_i8(rng, m * k))
        else:
            w = [DeviceBuffer.from_array(rng.integers(0, 0x78, size=k * n, dtype=np.uint8)) for _ in range(nbuf)]
            x = DeviceBuffer.from_array(rng.integers(0, 0x78, size=m * k, dtype=np.uint8))
        y = DeviceBuffer(4 * m * n)

        def step(i):
            if kind == "i8":
                lib.skl_gemm_i8rc_i8rc_i32rc_gfx950(m, n, k, 1, x, k, 1, w[i % nbuf], 1, k, 0, y, n, 1)
            else:
                lib.skl_gemm_f8e4m3rc_f8e4m3rc_f32rc_gfx950(m, n, k, 1.0, x, k, 1, w[i % nbuf], 1, k, 0.0, y, n, 1)

        return dict(fn=step, bytes=k * n + m * k + 4 * m * n, ops=2 * m * k * n, bound="hbm", dtype=kind, keep=(w, x, y),
                    name=f"{'int8' if kind == 'i8' else 'E4M3'} GEMM {m}x{k}x{n}, W with K contiguous ([n][k]), beta=0",
                    kernel="gemv_kc_kernel (up to 4 rows), gemv_kc_rows_kernel (up to 128)")
    return build


def wl_gemv_kc_fused(lib, rng):
    """A quantised linear layer at decode time on its [out][in] weight: int8 in, bias, ReLU, int8 out, C not written."""
    import skl_amd
    k, n, nbuf = 4096, 11008, 8
    w = [DeviceBuffer.from_array(rand_i8(rng, k * n)) for _ in range(nbuf)]
    x = DeviceBuffer.from_array(rand_i8(rng, k))
    y = DeviceBuffer(16)  # not written
    q = DeviceBuffer(n)
    bias = DeviceBuffer.from_array(rng.integers(-1000, 1000, n).astype(np.int32))
    scales = DeviceBuffer.from_array((rng.uniform(0.5, 2.0, n) / (74.0 * 74.0 * 64.0 * 0.4)).astype(np.float32))
    ep = skl_amd.Epilogue(bias, None, activation=skl_amd.Epilogue.ACT_RELU, q=q, rsq=n, csq=1, q_scale=scales,
                          q_scale_per_column=True, q_zero=-128, q_only=True)

    def step(i):
        lib.skl_gemm_fused_i8rc_i8rc_i32rc_gfx950(1, n, k, 1, x, k, 1, w[i % nbuf], 1, k, 0, y, n, 1, ep)

    return dict(fn=step, bytes=k * n + k + n + 8 * n, ops=2 * k * n, bound="hbm", dtype="i8", keep=(w, x, y, q, bias, scales),
                name="int8 1x4096x11008, W with K contiguous ([n][k]), with bias, ReLU and int8 output only (decode)",
                kernel="gemv_kc_kernel<int8, FUSED>")


def wl_gemv_kc_bf16(lib, rng):
    k, n, nbuf = 4096, 11008, 4
    w = [DeviceBuffer.from_array(bf16_bits(rng.normal(size=k * n) * 0.02)) for _ in range(nbuf)]
    x = DeviceBuffer.from_array(bf16_bits(rng.normal(size=k)))
    y = DeviceBuffer(4 * n)
    lib.skl_hip_memset(y, 0, 4 * n)

    def step(i):
        lib.skl_gemm_bf16rc_bf16rc_f32rc_gfx950(1, n, k, 1.0, x, k, 1, w[i % nbuf], 1, k, 0.0, y, n, 1)

    return dict(fn=step, bytes=2 * k * n + 2 * k + 4 * n, ops=2 * k * n, bound="hbm", dtype="bf16", keep=(w, x, y),
                name="bf16 GEMV 1x4096x11008, W with K contiguous ([n][k]), beta=0", kernel="gemv_kc_kernel<bf16>")


def _wl_small_batch(m):
    def build(lib, rng):
        k, n, nbuf = 4096, 11008, 8
        w = [DeviceBuffer.from_array(rand_i8(rng, k * n)) for _ in range(nbuf)]
        x = DeviceBuffer.from_array(rand_i8(rng, m * k))
        y = DeviceBuffer(4 * m * n)

        def step(i):
            lib.skl_gemm_i8_i8_i32_gfx950(m, n, k, 1, x, k, w[i % nbuf], n, 0, y, n)

        kernel = ("gemv_rows_kernel" if m <= 3 else "gemv_mfma_scale_c_kernel + gemv_mfma_rows_kernel" if m <= 16 else
                  "gemv_mfma_scale_c_kernel + gemv_rowgroups_kernel")
        return dict(fn=step, bytes=k * n + m * k + 4 * m * n, ops=2 * m * k * n, bound="hbm", dtype="i8", keep=(w, x, y),
                    name=f"int8 GEMM {m}x4096x11008 (decode with a batch of {m}: still a stream over W)", kernel=kernel)
    return build


def _wl_decode_fused(m):
    """A quantised layer at decode time: int8 in, bias, ReLU, int8 out (per-column scales), C not written."""
    def build(lib, rng):
        import skl_amd
        k, n, nbuf = 4096, 11008, 8
        w = [DeviceBuffer.from_array(rand_i8(rng, k * n)) for _ in range(nbuf)]
        x = DeviceBuffer.from_array(rand_i8(rng, m * k))
        y = DeviceBuffer(16)  # not written
        q = DeviceBuffer(m * n)
        bias = DeviceBuffer.from_array(rng.integers(-1000, 1000, n).astype(np.int32))
        scales = DeviceBuffer.from_array((rng.uniform(0.5, 2.0, n) / (74.0 * 74.0 * 64.0 * 0.4)).astype(np.float32))
        ep = skl_amd.Epilogue(bias, None, activation=skl_amd.Epilogue.ACT_RELU, q=q, rsq=n, csq=1, q_scale=scales,
                              q_scale_per_column=True, q_zero=-128, q_only=True)

        def step(i):
            lib.skl_gemm_fused_i8rc_i8rc_i32rc_gfx950(m, n, k, 1, x, k, 1, w[i % nbuf], n, 1, 0, y, n, 1, ep)

        return dict(fn=step, bytes=k * n + m * k + m * n + 8 * n, ops=2 * m * k * n, bound="hbm", dtype="i8",
                    keep=(w, x, y, q, bias, scales),
                    name=f"int8 {m}x4096x11008 with bias, ReLU and requantised int8 output only (decode, batch of {m})",
                    kernel="streaming kernel into a plane + gemm_split_reduce_kernel")
    return build


def wl_gemv_f8_fused(lib, rng):
    """An fp8 layer at decode time: E4M3 in, bias, saturating E4M3 out (per-column scales), C neither written nor read."""
    import skl_amd
    k, n, nbuf = 4096, 11008, 8
    w = [_fp8_operand(lib, rng, k * n, "f8e4m3") for _ in range(nbuf)]
    x = _fp8_operand(lib, rng, k, "f8e4m3")
    y = DeviceBuffer(4 * n)
    q = DeviceBuffer(n)
    bias = DeviceBuffer.from_array(rng.uniform(-1, 1, n).astype(np.float32))
    scales = DeviceBuffer.from_array(rng.uniform(0.5, 2.0, n).astype(np.float32) / 64.0)
    ep = skl_amd.Epilogue(bias, None, q=q, rsq=n, csq=1, q_scale=scales, q_scale_per_column=True, q_only=True,
                          q_format=skl_amd.Epilogue.Q_F8E4M3_SAT)

    def step(i):
        lib.skl_gemm_fused_f8e4m3rc_f8e4m3rc_f32rc_gfx950(1, n, k, 1.0, x, k, 1, w[i % nbuf], n, 1, 0.0, y, n, 1, ep)

    return dict(fn=step, bytes=k * n + k + n + 8 * n, ops=2 * k * n, bound="hbm", dtype="f8", keep=(w, x, y, q, bias, scales),
                name="fp8 E4M3 1x4096x11008 with bias and saturating E4M3 output only (decode)",
                kernel="gemv_mfma_rows_kernel<fp8> + gemv_mfma_add_planes_kernel")


def wl_small_batch_bf16(lib, rng):
    """Decode with a batch of 8 against bf16 weights (90 MB): the stream over W with the matrix cores multiplying."""
    m, k, n, nbuf = 8, 4096, 11008, 4
    w = [DeviceBuffer.from_array(bf16_bits(rng.normal(size=k * n) * 0.02)) for _ in range(nbuf)]
    x = DeviceBuffer.from_array(bf16_bits(rng.normal(size=m * k)))
    y = DeviceBuffer(4 * m * n)

    def step(i):
        lib.skl_gemm_bf16_bf16_f32_gfx950(m, n, k, 1.0, x, k, w[i % nbuf], n, 0.0, y, n)

    return dict(fn=step, bytes=2 * k * n + 2 * m * k + 4 * m * n, ops=2 * m * k * n, bound="hbm", dtype="bf16",
                keep=(w, x, y), name="bf16 GEMM 8x4096x11008 (decode with a batch of 8)",
                kernel="gemv_mfma_rows_kernel<bf16> + gemv_mfma_add_planes_kernel")


def wl_small_batch_f8(lib, rng):
    """Decode with a batch of 16 against fp8 weights: the stream over W with the matrix cores multiplying."""
    m, k, n, nbuf = 16, 4096, 11008, 8
    w = [DeviceBuffer.from_array(rng.integers(8, 127, size=k * n, dtype=np.uint8)) for _ in range(nbuf)]
    x = DeviceBuffer.from_array(rng.integers(8, 127, size=m * k, dtype=np.uint8))
    y = DeviceBuffer(4 * m * n)

    def step(i):
        lib.skl_gemm_f8e4m3rc_f8e4m3rc_f32rc_gfx950(m, n, k, 1.0, x, k, 1, w[i % nbuf], n, 1, 0.0, y, n, 1)

    return dict(fn=step, bytes=k * n + m * k + 4 * m * n, ops=2 * m * k * n, bound="hbm", dtype="f8e4m3", keep=(w, x, y),
                name="fp8 E4M3 GEMM 16x4096x11008 (decode with a batch of 16)",
                kernel="gemv_mfma_rows_kernel<fp8 E4M3> + gemv_mfma_add_planes_kernel")


def _wl_ofp4(m, mx=False):
    """Decode against OFP4 (E2M1) weights stored column by column: the weights cross HBM at half a byte per element
    (with `mx`: plus one E8M0 scale per 32 k, the OCP MXFP4 format). 16 buffers rotated (22.5 MB each) so that the
    stream exceeds the last-level cache."""
    def build(lib, rng):
        k, n, nbuf = 4096, 11008, 16
        w = [DeviceBuffer.from_array(rng.integers(0, 256, size=k * n // 2, dtype=np.uint8)) for _ in range(nbuf)]
        sc = [DeviceBuffer.from_array(rng.integers(120, 135, size=n * k // 32, dtype=np.uint8)) for _ in range(nbuf)] if mx else None
        x = DeviceBuffer.from_array(rng.integers(8, 127, size=m * k, dtype=np.uint8))
        y = DeviceBuffer(4 * m * n)

        def step(i):
            if mx:
                lib.skl_gemm_f8e4m3rc_mxf4e2m1c_f32rc_gfx950(m, n, k, 1.0, x, k, 1, w[i % nbuf], k, sc[i % nbuf], k // 32, 0.0, y, n, 1)
            else:
                lib.skl_gemm_f8e4m3rc_f4e2m1c_f32rc_gfx950(m, n, k, 1.0, x, k, 1, w[i % nbuf], k, 0.0, y, n, 1)

        return dict(fn=step, bytes=k * n // 2 + (k * n // 32 if mx else 0) + m * k + 4 * m * n, ops=2 * m * k * n, bound="hbm",
                    dtype="f4e2m1", keep=(w, sc or [], x, y),
                    name=f"E4M3 x {'MXFP4' if mx else 'OFP4'} GEMM {m}x4096x11008 (4-bit weights, columns contiguous in K, beta=0)",
                    kernel="gemv_f4_kernel" if m <= 16 else "gemv_f4_rows_kernel, or a converted copy + the fp8 / bf16 GEMM")
    return build


def wl_gemv_p4x1c(lib, rng):
    """Config 2 with W prepacked in the K-packed dot4 layout (B(4P+p, j) at P*rsb1 + 4j + p): same bytes."""
    k, n, nbuf = 4096, 11008, 8
    w = [DeviceBuffer.from_array(rand_i8(rng, k * n)) for _ in range(nbuf)]
    x = DeviceBuffer.from_array(rand_i8(rng, k))
    y = DeviceBuffer(4 * n)

    def step(i):
        lib.skl_gemm_i8rcp1x4_i8p4x1c_i32_gfx950(1, n, k // 4, 1, x, k, 4, w[i % nbuf], 4 * n, 0, y, n)

    return dict(fn=step, bytes=k * n + k + 4 * n, ops=2 * k * n, bound="hbm", dtype="i8", keep=(w, x, y),
                name="int8 GEMV 1x4096x11008 (W in the p4x1c K-packed layout, beta=0)", kernel="gemv_kernel<int8 K-packed>")


def _wl_small_batch_p4x1c(m):
    """Decode with a batch of m rows against the same prepacked weights: the K-packed B read in place, no transposes."""
    def build(lib, rng):
        k, n, nbuf = 4096, 11008, 8
        w = [DeviceBuffer.from_array(rand_i8(rng, k * n)) for _ in range(nbuf)]
        x = DeviceBuffer.from_array(rand_i8(rng, m * k))
        y = DeviceBuffer(4 * m * n)

        def step(i):
            lib.skl_gemm_i8rcp1x4_i8p4x1c_i32_gfx950(m, n, k // 4, 1, x, k, 4, w[i % nbuf], 4 * n, 0, y, n)

        kernel = "gemv_k4_wholek_kernel" if m <= 128 else "a copy of W with K contiguous + the tile kernels"
        return dict(fn=step, bytes=k * n + m * k + 4 * m * n, ops=2 * m * k * n, bound="hbm", dtype="i8", keep=(w, x, y),
                    name=f"int8 GEMM {m}x4096x11008 (W in the p4x1c K-packed layout, decode with a batch of {m})",
                    kernel=kernel)
    return build


def wl_gemv_bf16(lib, rng):
    k, n, nbuf = 4096, 11008, 4
    w = [DeviceBuffer.from_array(bf16_bits(rng.normal(size=k * n) * 0.02)) for _ in range(nbuf)]
    x = DeviceBuffer.from_array(bf16_bits(rng.normal(size=k)))
    y = DeviceBuffer(4 * n)
    lib.skl_hip_memset(y, 0, 4 * n)

    def step(i):
        lib.skl_gemm_bf16_bf16_f32_gfx950(1, n, k, 1.0, x, k, w[i % nbuf], n, 0.0, y, n)

    return dict(fn=step, bytes=2 * k * n + 2 * k + 8 * n, ops=2 * k * n, bound="hbm", dtype="bf16", keep=(w, x, y),
                name="bf16 GEMV 1x4096x11008 (row-major W, beta=0)", kernel="gemv_kernel<bf16>")


def wl_gemv_f8(lib, rng):
    k, n, nbuf = 4096, 11008, 8
    w = [DeviceBuffer.from_array(rng.integers(8, 127, size=k * n, dtype=np.uint8)) for _ in range(nbuf)]
    x = DeviceBuffer.from_array(rng.integers(8, 127, size=k, dtype=np.uint8))
    y = DeviceBuffer(4 * n)
    lib.skl_hip_memset(y, 0, 4 * n)

    def step(i):
        lib.skl_gemm_f8e4m3rc_f8e4m3rc_f32rc_gfx950(1, n, k, 1.0, x, k, 1, w[i % nbuf], n, 1, 0.0, y, n, 1)

    return dict(fn=step, bytes=k * n + k + 4 * n, ops=2 * k * n, bound="hbm", dtype="f8e4m3", keep=(w, x, y),
                name="fp8 E4M3 GEMV 1x4096x11008 (row-major W, beta=0)", kernel="gemv_kernel<fp8 E4M3>")


def _dense(lib, rng, name, fn_name, m, n, k, abytes, gen_a, gen_b, alpha, beta, ctype, dkey, col_major_a=False):
    a = DeviceBuffer.from_array(gen_a(m * k))
    b = DeviceBuffer.from_array(gen_b(k * n))
    c = DeviceBuffer.from_array(np.zeros(m * n, ctype) if beta == 0 else rng.normal(size=m * n).astype(ctype))
    f = getattr(lib, fn_name)
    lda = m if col_major_a else k

    def step(i):
        f(m, n, k, alpha, a, lda, b, n, beta, c, n)

    return dict(fn=step, bytes=abytes * (m * k + k * n) + 4 * m * n * (2 if beta != 0 else 1), ops=2 * m * n * k,
                bound="mfma", dtype=dkey, keep=(a, b, c), name=name, kernel="gemm_mfma_ring_kernel")


def wl_gemm_i8_8192(lib, rng):
    return _dense(lib, rng, "int8 GEMM 8192^3 (row-major, alpha=1, beta=0)", "skl_gemm_i8_i8_i32_gfx950", 8192, 8192,
                  8192, 1, lambda n: rand_i8(rng, n), lambda n: rand_i8(rng, n), 1, 0, np.int32, "i8")


def wl_gemm_f8_8192_f8_out(lib, rng):
    """An fp8 layer feeding the next: E4M3 in, bias, E4M3 out (saturating, per-column scales), the fp32 C never written."""
    import skl_amd
    m = n = k = 8192
    a, b = _fp8_operand(lib, rng, m * k, "f8e4m3"), _fp8_operand(lib, rng, k * n, "f8e4m3")
    c = DeviceBuffer(4 * m * n)  # neither written nor, with beta == 0, read
    q = DeviceBuffer(m * n)
    bias = DeviceBuffer.from_array(rng.uniform(-1, 1, n).astype(np.float32))
    scales = DeviceBuffer.from_array(rng.uniform(0.5, 2.0, n).astype(np.float32) / 64.0)
    ep = skl_amd.Epilogue(bias, None, q=q, rsq=n, csq=1, q_scale=scales, q_scale_per_column=True, q_only=True,
                          q_format=skl_amd.Epilogue.Q_F8E4M3_SAT)

    def step(i):
        lib.skl_gemm_fused_f8e4m3rc_f8e4m3rc_f32rc_gfx950(m, n, k, 1.0, a, k, 1, b, n, 1, 0.0, c, n, 1, ep)

    return dict(fn=step, bytes=m * k + k * n + m * n, ops=2 * m * n * k, bound="mfma", dtype="f8", keep=(a, b, c, q, bias, scales),
                name="fp8 E4M3 GEMM 8192^3 with bias and saturating E4M3 output only (q_only)",
                kernel="gemm_mfma_ring_kernel<E4M3, EXTRA>")


def wl_gemm_i8_blocks_4x8x4(accum):
    """The 4 x 8 by 8 x 4 block format (A in 4 x 8 blocks, B in 8 x 4, C in 4 x 4), 8192^3."""
    def make(lib, rng):
        m = n = k = 8192
        a, b = DeviceBuffer.from_array(rand_i8(rng, m * k)), DeviceBuffer.from_array(rand_i8(rng, k * n))
        c = DeviceBuffer.from_array(np.zeros(m * n, np.int32))

        def step(i):
            lib.skl_gemm_a1b01_i8p4x8_i8p8x4_i32p4x4_gfx950(m // 4, n // 4, k // 8, a, 4 * k, b, 8 * n, c, 4 * n, accum)

        return dict(fn=step, bytes=m * k + k * n + 4 * m * n * (2 if accum else 1), ops=2 * m * n * k, bound="mfma", dtype="i8",
                    keep=(a, b, c), name="int8 GEMM 8192^3 in 4x8 / 8x4 / 4x4 blocks" + (", accumulating" if accum else ""),
                    kernel="copies + gemm_mfma_ring_kernel")
    return make


def wl_gemm_i8_8192_requantised(lib, rng):
    """A quantised layer: int8 in, ReLU, int8 out (per-column scales), the int32 C never written (q_only)."""
    import skl_amd
    m = n = k = 8192
    a, b = DeviceBuffer.from_array(rand_i8(rng, m * k)), DeviceBuffer.from_array(rand_i8(rng, k * n))
    c = DeviceBuffer(16)  # not written
    q = DeviceBuffer(m * n)
    bias = DeviceBuffer.from_array(rng.integers(-1000, 1000, n).astype(np.int32))
    scales = DeviceBuffer.from_array((rng.uniform(0.5, 2.0, n) / (74.0 * 74.0 * 90.0 * 0.4)).astype(np.float32))
    ep = skl_amd.Epilogue(bias, None, activation=skl_amd.Epilogue.ACT_RELU, q=q, rsq=n, csq=1, q_scale=scales,
                          q_scale_per_column=True, q_zero=-128, q_only=True)

    def step(i):
        lib.skl_gemm_fused_i8rc_i8rc_i32rc_gfx950(m, n, k, 1, a, k, 1, b, n, 1, 0, c, n, 1, ep)

    return dict(fn=step, bytes=m * k + k * n + m * n, ops=2 * m * n * k, bound="mfma", dtype="i8", keep=(a, b, c, q, bias, scales),
                name="int8 GEMM 8192^3 with bias, ReLU and requantised int8 output only (q_only)",
                kernel="gemm_mfma_ring_kernel<int8, EXTRA>")


def wl_gemm_i8_4000(lib, rng):
    """Ragged M, N, K: A and B are copied into tile-padded scratch memory, the streaming kernel runs on the copies."""
    d = _dense(lib, rng, "int8 GEMM 4000^3 (row-major, alpha=1, beta=0; ragged: runs on tile-padded copies)",
               "skl_gemm_i8_i8_i32_gfx950", 4000, 4000, 4000, 1, lambda n: rand_i8(rng, n), lambda n: rand_i8(rng, n), 1, 0,
               np.int32, "i8")
    d["kernel"] = "realign_rows_kernel + realign_transpose_kernel + gemm_mfma_ring_kernel<EDGE>"
    return d


def _wl_reference_bench(kind, m, n, k, beta):
    """The shapes the reference's own benchmark rows use (column-major A through the `c` entry points):
    test/gemm/xsfmm/skl_gemm_i8c_i8_i32_xsfmm32a8i.c:55-56 (128 x 128 x 8192, beta 0 and 1) and
    test/gemm/xsfmm/skl_gemm_bf16c_bf16_f32_xsfmm32a16f.c:55-56 (128 x 128 x 4096). Launch-bound at GPU scale:
    a single 128 x 128 tile of C - timed as what a caller of those rows would see."""
    def build(lib, rng):
        if kind == "i8":
            a, b = DeviceBuffer.from_array(rand_i8(rng, m * k)), DeviceBuffer.from_array(rand_i8(rng, k * n))
            c = DeviceBuffer.from_array(np.zeros(m * n, np.int32))

            def step(i):
                lib.skl_gemm_i8c_i8_i32_gfx950(m, n, k, 1, a, m, b, n, beta, c, n)
            es = 1
        else:
            a = DeviceBuffer.from_array(bf16_bits(rng.normal(size=m * k)))
            b = DeviceBuffer.from_array(bf16_bits(rng.normal(size=k * n) * 0.02))
            c = DeviceBuffer.from_array(np.zeros(m * n, np.float32))

            def step(i):
                lib.skl_gemm_bf16c_bf16_f32_gfx950(m, n, k, 1.0, a, m, b, n, float(beta), c, n)
            es = 2
        return dict(fn=step, bytes=es * (m * k + k * n) + 4 * m * n * (2 if beta else 1), ops=2 * m * n * k, bound="mfma",
                    dtype=kind, keep=(a, b, c), name=f"{kind} GEMM {m}x{n}x{k}, column-major A, beta={beta} (the reference's own benchmark row)",
                    kernel="gemm_mfma_kernel (K shared between workgroups) + gemm_split_reduce_kernel")
    return build


def wl_reference_bench_dot4(lib, rng):
    """test/gemm/xsfvqdotq/skl_gemm_i8rcp1x4_i8p4x1c_i32_xsfvqdotq.c:56: 126 x 128 with k1 = 64 groups of four k."""
    m, n, k1 = 126, 128, 64
    a = DeviceBuffer.from_array(rand_i8(rng, m * 4 * k1))
    b = DeviceBuffer.from_array(rand_i8(rng, k1 * 4 * n))
    c = DeviceBuffer.from_array(np.zeros(m * n, np.int32))

    def step(i):
        lib.skl_gemm_i8rcp1x4_i8p4x1c_i32_gfx950(m, n, k1, 1, a, 4 * k1, 4, b, 4 * n, 0, c, n)

    return dict(fn=step, bytes=m * 4 * k1 + 4 * k1 * n + 4 * m * n, ops=2 * m * n * 4 * k1, bound="mfma", dtype="i8", keep=(a, b, c),
                name="int8 dot4 GEMM 126x128, k1=64 (K-packed B; the reference's own benchmark row)", kernel="gemv_k4_wholek_kernel<1> on a grid of column tiles x groups of 16 rows")


def wl_gemm_i8_512(lib, rng):
    return _dense(lib, rng, "int8 GEMM 512^3 (row-major, alpha=1, beta=0)", "skl_gemm_i8_i8_i32_gfx950", 512, 512, 512,
                  1, lambda n: rand_i8(rng, n), lambda n: rand_i8(rng, n), 1, 0, np.int32, "i8")


def _fp8_operand(lib, rng, n, fmt):
    """fp32 ~ N(0,1) converted on the GPU with the saturating cvt (scale 1)."""
    src = DeviceBuffer.from_array(rng.normal(size=n).astype(np.float32))
    dst = DeviceBuffer(n)
    getattr(lib, f"skl_cvt_sat_f32_{fmt}_gfx950")(dst, src, 1.0, n)
    lib.skl_hip_synchronize()
    src.free()
    return dst


def wl_gemm_f8_8192(lib, rng, fmt_b="f8e4m3"):
    m = n = k = 8192
    a = _fp8_operand(lib, rng, m * k, "f8e4m3")   # stored column-major (k x m row-major = A^T)
    b = _fp8_operand(lib, rng, k * n, fmt_b)
    c = DeviceBuffer.from_array(np.zeros(m * n, np.float32))
    if fmt_b == "f8e4m3":
        def step(i):
            lib.skl_gemm_f8e4m3c_f8e4m3_f32_gfx950(m, n, k, 1.0, a, m, b, n, 0.0, c, n)
        name = "fp8 E4M3xE4M3 GEMM 8192^3 (column-major A, alpha=1, beta=0)"
    else:
        def step(i):
            lib.skl_gemm_f8e4m3rc_f8e5m2rc_f32rc_gfx950(m, n, k, 1.0, a, 1, m, b, n, 1, 0.0, c, n, 1)
        name = "fp8 E4M3xE5M2 GEMM 8192^3 (column-major A, alpha=1, beta=0)"
    return dict(fn=step, bytes=m * k + k * n + 8 * m * n, ops=2 * m * n * k, bound="mfma", dtype="f8", keep=(a, b, c),
                name=name, kernel="gemm_mfma_ring_kernel")


def wl_gemm_f8_layout(a_rows_contig, b_cols_contig):
    """The same fp8 product through the full-stride (rc) entry point with other operand layouts: the A and B
    buffers are random fp8 data either way, only the strides the call passes differ."""
    def build(lib, rng):
        m = n = k = 8192
        a = _fp8_operand(lib, rng, m * k, "f8e4m3")
        b = _fp8_operand(lib, rng, k * n, "f8e4m3")
        c = DeviceBuffer.from_array(np.zeros(m * n, np.float32))
        rsa, csa = (k, 1) if a_rows_contig else (1, m)
        rsb, csb = (1, k) if b_cols_contig else (n, 1)

        def step(i):
            lib.skl_gemm_f8e4m3rc_f8e4m3rc_f32rc_gfx950(m, n, k, 1.0, a, rsa, csa, b, rsb, csb, 0.0, c, n, 1)

        name = (f"fp8 E4M3xE4M3 GEMM 8192^3 ({'row' if a_rows_contig else 'column'}-major A, "
                f"{'column' if b_cols_contig else 'row'}-major B, alpha=1, beta=0)")
        return dict(fn=step, bytes=m * k + k * n + 8 * m * n, ops=2 * m * n * k, bound="mfma", dtype="f8",
                    keep=(a, b, c), name=name, kernel="gemm_mfma_ring_kernel")
    return build


def wl_gemm_bf16(lib, rng):
    m, n, k = 2048, 4096, 4096
    return _dense(lib, rng, "bf16 GEMM 2048x4096x4096 (row-major, alpha=1, beta=1)", "skl_gemm_bf16_bf16_f32_gfx950",
                  m, n, k, 2, lambda c: bf16_bits(rng.normal(size=c)), lambda c: bf16_bits(rng.normal(size=c) * 0.02),
                  1.0, 1.0, np.float32, "bf16")


def wl_gemm_f32(lib, rng):
    """f32 and f64 results are defined operation by operation (a rounded multiply, then a rounded add, k ascending),
    so they run on the vector ALUs, not the matrix cores; the published fp32 / fp64 peaks are the denominators."""
    m = n = k = 4096
    d = _dense(lib, rng, "f32 GEMM 4096^3 (row-major, alpha=1, beta=0; bit-identical to the reference)",
               "skl_gemm_f32_f32_f32_gfx950", m, n, k, 4, lambda c: rng.normal(size=c).astype(np.float32),
               lambda c: rng.normal(size=c).astype(np.float32), 1.0, 0.0, np.float32, "f32")
    d["kernel"] = "gemm_tiled_kernel"
    return d


def wl_gemm_f64(lib, rng):
    m = n = k = 4096
    d = _dense(lib, rng, "f64 GEMM 4096^3 (row-major, alpha=1, beta=0; bit-identical to the reference)",
               "skl_gemm_f64_f64_f64_gfx950", m, n, k, 8, lambda c: rng.normal(size=c), lambda c: rng.normal(size=c),
               1.0, 0.0, np.float64, "f64")
    d["kernel"] = "gemm_tiled_kernel"
    return d


def wl_f16_pipeline(lib, rng):
    """benchmark configuration 5: pack A, pack B, panel GEMM, unpack C - one step is the whole pipeline."""
    te, m, k, n = 64, 4096, 4096, 14336
    a = DeviceBuffer.from_array(rng.uniform(-1, 1, m * k).astype(np.float16).view(np.uint16))
    b = DeviceBuffer.from_array(rng.uniform(-1, 1, k * n).astype(np.float16).view(np.uint16))
    ap, bp = DeviceBuffer(2 * m * k), DeviceBuffer(2 * k * n)
    cp, c = DeviceBuffer(4 * m * n), DeviceBuffer(4 * m * n)
    lib.skl_hip_memset(cp, 0, 4 * m * n)
    m1, n1 = m // te, n // te

    def step(i):
        lib.skl_pack_e16_e16rcptex1c_gfx950(m, k, a, k, ap, k * te, te, 0)
        lib.skl_pack_e16rc_e16rcprc_gfx950(k, n, b, n, 1, 1, te, bp, te, 1, te, k * te, 0)
        lib.skl_gemm_f16rcptex1c_f16rcp1xte_f32rcptexterc_gfx950(m1, n1, k, 1.0, ap, k * te, te, bp, te, k * te, 0.0, cp,
                                                                  te, 1, n1 * te * te, te * te)
        lib.skl_unpack_e32rcprc_e32rc_gfx950(te, te, cp, te, 1, n1 * te * te, te * te, m, n, c, n, 1)

    moved = 2 * (2 * m * k) + 2 * (2 * k * n) + 2 * (4 * m * n)
    return dict(fn=step, bytes=moved, ops=2 * m * n * k, bound="mfma", dtype="f16", keep=(a, b, ap, bp, cp, c),
                name="f16 pack->GEMM->unpack 4096x4096x14336 (TE=64 panels)", kernel="gemm_mfma_ring_kernel")


def _beta_zero_as_reference(builder):
    """The same workload with beta == 0 evaluated as the reference's loops do (0 * c + alpha * acc: a NaN or an
    infinity in the old C stays a NaN, ref/gemm/gemm_bf16rc_bf16rc_f32rc.c:21) instead of the default, which
    initialises C. The switch is per thread and set around every call."""
    def build(lib, rng):
        wl = builder(lib, rng)
        inner = wl["fn"]

        def step(i):
            lib.skl_hip_set_beta_zero_mode(1)
            inner(i)
            lib.skl_hip_set_beta_zero_mode(0)

        wl["fn"] = step
        wl["name"] += ", beta == 0 as the reference evaluates it"
        return wl
    return build


def wl_cvt(lib, rng):
    n = 8192 * 8192
    src = DeviceBuffer.from_array(rng.normal(size=n).astype(np.float32))
    dst = DeviceBuffer(n)

    def step(i):
        lib.skl_cvt_sat_f32_f8e4m3_gfx950(dst, src, 1.0, n)

    return dict(fn=step, bytes=5 * n, ops=n, bound="hbm", dtype="f32", keep=(src, dst),
                name="cvt sat f32->E4M3, 8192^2 elements", kernel="cvt_f32_f8_kernel")


def wl_pack_a(lib, rng):
    te, m, k, nbuf = 64, 4096, 4096, 5   # 5 x (32 + 32 MiB): more than the last-level cache between two uses
    a = [DeviceBuffer.from_array(rng.integers(0, 1 << 16, m * k, dtype=np.uint16)) for _ in range(nbuf)]
    ap = [DeviceBuffer(2 * m * k) for _ in range(nbuf)]

    def step(i):
        lib.skl_pack_e16_e16rcptex1c_gfx950(m, k, a[i % nbuf], k, ap[i % nbuf], k * te, te, 0)

    return dict(fn=step, bytes=4 * m * k, ops=m * k, bound="hbm", dtype="u16", keep=(a, ap),
                name="pack e16 4096x4096 -> TEx1 column panels (5 buffer pairs rotated)",
                kernel="pack_vec_kernel (transposing)")


def wl_pack_b(lib, rng):
    """Configuration 5's B: row-major 4096 x 14336 f16 into 1 x TE row panels (a copy-like pack, 112 + 112 MiB)."""
    te, k, n, nbuf = 64, 4096, 14336, 2
    b = [DeviceBuffer.from_array(rng.integers(0, 1 << 16, k * n, dtype=np.uint16)) for _ in range(nbuf)]
    bp = [DeviceBuffer(2 * k * n) for _ in range(nbuf)]

    def step(i):
        lib.skl_pack_e16rc_e16rcprc_gfx950(k, n, b[i % nbuf], n, 1, 1, te, bp[i % nbuf], te, 1, te, k * te, 0)

    return dict(fn=step, bytes=4 * k * n, ops=k * n, bound="hbm", dtype="u16", keep=(b, bp),
                name="pack e16 4096x14336 -> 1xTE row panels (2 buffer pairs rotated)", kernel="pack_vec_kernel (copy-like)")


def wl_unpack_c(lib, rng):
    """Configuration 5's C: TE x TE blocks of f32 back to row-major 4096 x 14336 (224 + 224 MiB)."""
    te, m, n = 64, 4096, 14336
    n1 = n // te
    cp = DeviceBuffer.from_array(rng.integers(0, 1 << 32, m * n, dtype=np.uint32))
    c = DeviceBuffer(4 * m * n)

    def step(i):
        lib.skl_unpack_e32rcprc_e32rc_gfx950(te, te, cp, te, 1, n1 * te * te, te * te, m, n, c, n, 1)

    return dict(fn=step, bytes=8 * m * n, ops=m * n, bound="hbm", dtype="u32", keep=(cp, c),
                name="unpack e32 TExTE blocks -> row-major 4096x14336", kernel="pack_vec_kernel (copy-like)")


def wl_copy(lib, rng):
    """Plain copy through the pack kernel (one block = the whole matrix): the
    known-size stream the HBM traffic counters are calibrated against."""
    m = n = 4096
    nbuf = 3   # 3 x (64 + 64 MiB)
    src = [DeviceBuffer.from_array(rng.integers(0, 1 << 32, m * n, dtype=np.uint32)) for _ in range(nbuf)]
    dst = [DeviceBuffer(4 * m * n) for _ in range(nbuf)]

    def step(i):
        lib.skl_pack_e32rc_e32rcprc_gfx950(m, n, src[i % nbuf], n, 1, m, n, dst[i % nbuf], n, 1, 0, 0, 0)

    return dict(fn=step, bytes=8 * m * n, ops=m * n, bound="hbm", dtype="u32", keep=(src, dst),
                name="copy 4096x4096 u32 (64 MiB read + 64 MiB write, 3 buffer pairs rotated)", kernel="pack_vec_kernel (copy)")


def wl_peak_hbm_read(lib, rng):
    """The ceiling of the headline: a plain read (128-bit non-temporal loads, nothing else) of the same eight
    45 MB buffers the GEMV streams, one launch per buffer."""
    k, n, nbuf = 4096, 11008, 8
    w = [DeviceBuffer.from_array(rand_i8(rng, k * n)) for _ in range(nbuf)]

    def step(i):
        lib.skl_hip_probe_hbm_read(w[i % nbuf], k * n)

    return dict(fn=step, bytes=k * n, ops=0, bound="hbm", dtype="u8", keep=(w,),
                name="plain read of 45 MB (8 buffers rotated): what a streaming kernel can reach on that many bytes",
                kernel="probe_read_kernel")


def _wl_peak_mfma(kind, dkey, random_operands):
    def build(lib, rng):
        iters = 20000
        ops = lib.skl_hip_probe_mfma(kind, random_operands, 16)  # also loads the kernel
        lib.skl_hip_synchronize()
        ops = ops / 16 * iters

        def step(i):
            lib.skl_hip_probe_mfma(kind, random_operands, iters)

        what = "pseudo-random" if random_operands else "all-equal"
        return dict(fn=step, bytes=0, ops=ops, bound="mfma", dtype=dkey, keep=(),
                    name=f"matrix cores alone, {dkey} 32x32 instructions on register operands ({what} values)",
                    kernel="probe_mfma_kernel")
    return build


# key: (builder, default steps, default warm-up steps, calls per step)
WORKLOADS = {
    "gemv_i8": (wl_gemv, 20, 5, 128),
    "peak_hbm_read": (wl_peak_hbm_read, 20, 5, 128),
    "gemv_i8_p4x1c": (wl_gemv_p4x1c, 10, 2, 128),
    "gemv_bf16": (wl_gemv_bf16, 10, 2, 64),
    "gemv_f8e4m3": (wl_gemv_f8, 10, 2, 128),
    "gemv_f8e4m3_f4_1x4096x11008": (_wl_ofp4(1), 10, 2, 128),
    "gemm_f8e4m3_f4_16x4096x11008": (_wl_ofp4(16), 10, 2, 128),
    "gemm_f8e4m3_f4_32x4096x11008": (_wl_ofp4(32), 10, 2, 64),
    "gemm_f8e4m3_f4_64x4096x11008": (_wl_ofp4(64), 10, 2, 32),
    "gemm_f8e4m3_f4_128x4096x11008": (_wl_ofp4(128), 10, 2, 32),
    "gemv_f8e4m3_mxf4_1x4096x11008": (_wl_ofp4(1, mx=True), 10, 2, 128),
    "gemm_f8e4m3_mxf4_16x4096x11008": (_wl_ofp4(16, mx=True), 10, 2, 128),
    "gemv_i8_1x8192x28672": (wl_gemv_large, 10, 2, 32),
    "gemv_i8_kcontig": (wl_gemv_kc, 10, 2, 128),
    "gemv_i8_kcontig_fused": (wl_gemv_kc_fused, 10, 2, 128),
    "gemv_bf16_kcontig": (wl_gemv_kc_bf16, 10, 2, 64),
    "gemm_i8_kcontig_4x4096x11008": (_wl_batch_kc(4), 10, 2, 64),
    "gemm_i8_kcontig_16x4096x11008": (_wl_batch_kc(16), 10, 2, 64),
    "gemm_i8_kcontig_64x4096x11008": (_wl_batch_kc(64), 10, 2, 32),
    "gemm_f8e4m3_kcontig_16x4096x11008": (_wl_batch_kc(16, "f8"), 10, 2, 64),
    "gemm_i8_kcontig_16x11008x4096": (_wl_batch_kc(16, "i8", 11008, 4096), 10, 2, 64),
    "gemm_i8_4x4096x11008": (_wl_small_batch(4), 10, 2, 64),
    "gemm_i8_8x4096x11008": (_wl_small_batch(8), 10, 2, 64),
    "gemm_i8_16x4096x11008": (_wl_small_batch(16), 10, 2, 64),
    "gemv_i8_fused_1x4096x11008": (_wl_decode_fused(1), 10, 2, 64),
    "gemv_f8e4m3_fused_1x4096x11008": (wl_gemv_f8_fused, 10, 2, 64),
    "gemm_i8_fused_16x4096x11008": (_wl_decode_fused(16), 10, 2, 64),
    "gemm_i8_32x4096x11008": (_wl_small_batch(32), 10, 2, 64),
    "gemm_i8_64x4096x11008": (_wl_small_batch(64), 10, 2, 32),
    "gemm_i8_128x4096x11008": (_wl_small_batch(128), 10, 2, 32),
    "gemm_i8_p4x1c_16x4096x11008": (_wl_small_batch_p4x1c(16), 10, 2, 64),
    "gemm_i8_p4x1c_32x4096x11008": (_wl_small_batch_p4x1c(32), 10, 2, 32),
    "gemm_i8_p4x1c_112x4096x11008": (_wl_small_batch_p4x1c(112), 10, 2, 32),
    "gemm_i8_p4x1c_512x4096x11008": (_wl_small_batch_p4x1c(512), 5, 1, 8),
    "gemm_f8e4m3_16x4096x11008": (wl_small_batch_f8, 10, 2, 64),
    "gemm_bf16_8x4096x11008": (wl_small_batch_bf16, 10, 2, 32),
    "peak_mfma_i8_random": (_wl_peak_mfma(0, "i8", 1), 3, 1, 1),
    "peak_mfma_i8_constant": (_wl_peak_mfma(0, "i8", 0), 3, 1, 1),
    "peak_mfma_f8_random": (_wl_peak_mfma(2, "f8", 1), 3, 1, 1),
    "peak_mfma_f8_constant": (_wl_peak_mfma(2, "f8", 0), 3, 1, 1),
    "peak_mfma_bf16_random": (_wl_peak_mfma(1, "bf16", 1), 3, 1, 1),
    "peak_mfma_bf16_constant": (_wl_peak_mfma(1, "bf16", 0), 3, 1, 1),
    "gemm_i8_8192": (wl_gemm_i8_8192, 20, 2, 1),
    "gemm_i8_8192_requantised": (wl_gemm_i8_8192_requantised, 20, 2, 1),
    "gemm_f8e4m3_8192_f8_out": (wl_gemm_f8_8192_f8_out, 20, 2, 1),
    "gemm_i8_8192_blocks_4x8x4": (wl_gemm_i8_blocks_4x8x4(False), 20, 2, 1),
    "gemm_i8_8192_blocks_4x8x4_accum": (wl_gemm_i8_blocks_4x8x4(True), 20, 2, 1),
    "gemm_f8e4m3_8192": (wl_gemm_f8_8192, 20, 2, 1),
    "gemm_f8e4m3_f8e5m2_8192": (lambda lib, rng: wl_gemm_f8_8192(lib, rng, "f8e5m2"), 20, 2, 1),
    "gemm_f8e4m3_8192_rowmajor_a": (wl_gemm_f8_layout(True, False), 20, 2, 1),
    "gemm_f8e4m3_8192_kcontig": (wl_gemm_f8_layout(True, True), 20, 2, 1),
    "gemm_f8e4m3_8192_kcontig_beta0_as_reference": (_beta_zero_as_reference(wl_gemm_f8_layout(True, True)), 20, 2, 1),
    "gemm_f8e4m3_8192_beta0_as_reference": (_beta_zero_as_reference(wl_gemm_f8_8192), 20, 2, 1),
    "pipeline_f16_4096x4096x14336_beta0_as_reference": (_beta_zero_as_reference(wl_f16_pipeline), 10, 2, 1),
    "gemm_i8_4000": (wl_gemm_i8_4000, 10, 2, 2),
    "gemm_bf16_2048x4096x4096": (wl_gemm_bf16, 20, 2, 4),
    "gemm_f32_4096": (wl_gemm_f32, 5, 1, 1),
    "gemm_f64_4096": (wl_gemm_f64, 5, 1, 1),
    "pipeline_f16_4096x4096x14336": (wl_f16_pipeline, 10, 2, 1),
    "gemm_i8_512": (wl_gemm_i8_512, 10, 2, 64),
    "ref_bench_i8c_128x128x8192_beta0": (_wl_reference_bench("i8", 128, 128, 8192, 0), 10, 2, 64),
    "ref_bench_i8c_128x128x8192_beta1": (_wl_reference_bench("i8", 128, 128, 8192, 1), 10, 2, 64),
    "ref_bench_bf16c_128x128x4096_beta0": (_wl_reference_bench("bf16", 128, 128, 4096, 0), 10, 2, 64),
    "ref_bench_dot4_126x128x256": (wl_reference_bench_dot4, 10, 2, 64),
    "cvt_f32_f8e4m3_8192sq": (wl_cvt, 10, 2, 2),
    "pack_e16_4096sq": (wl_pack_a, 10, 2, 10),
    "pack_e16_4096x14336_row_panels": (wl_pack_b, 10, 2, 2),
    "unpack_e32_4096x14336": (wl_unpack_c, 10, 2, 2),
    "copy_u32_4096sq": (wl_copy, 10, 2, 6),
}
HEADLINE = "gemv_i8"

# The benchmark configurations as rows of `roofline.configs`: label -> workload key.
CONFIG_TABLE = {
    "C1 int8 512^3": "gemm_i8_512",
    "C2 int8 GEMV 1x4096x11008": "gemv_i8",
    "C3 bf16 2048x4096x4096 beta=1": "gemm_bf16_2048x4096x4096",
    "C4 fp8 E4M3xE4M3 8192^3": "gemm_f8e4m3_8192",
    "C4 fp8 E4M3xE5M2 8192^3": "gemm_f8e4m3_f8e5m2_8192",
    "C4 fp8 E4M3xE4M3 8192^3, K-contiguous A and B": "gemm_f8e4m3_8192_kcontig",
    "C5 f16 pack+GEMM+unpack 4096x4096x14336": "pipeline_f16_4096x4096x14336",
    "C5 pack A": "pack_e16_4096sq",
    "C5 pack B": "pack_e16_4096x14336_row_panels",
    "C5 unpack C": "unpack_e32_4096x14336",
    "C4 cvt f32->E4M3": "cvt_f32_f8e4m3_8192sq",
    "target int8 8192^3": "gemm_i8_8192",
}
# Which probe is the measured ceiling of a workload's kind.
MEASURED_PEAK_OF = {"hbm": "peak_hbm_read", "i8": "peak_mfma_i8_random", "f8": "peak_mfma_f8_random",
                    "bf16": "peak_mfma_bf16_random", "f16": "peak_mfma_bf16_random"}

# HBM bytes per call from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (KiB per dispatch, summed over the call's
# kernels), FETCH_SIZE scaled by 1.998 (what it under-reads on a 64 MiB copy), WRITE_SIZE by 1.000; the runs are
# summarised in profiles/gemv_cvt_gemm_hbm_traffic.pmc.txt.
TRAFFIC_SOURCE = "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs summarised in profiles/gemv_cvt_gemm_hbm_traffic.pmc.txt"
MEASURED_TRAFFIC_BYTES = {
    "gemv_i8": int((22060.5 * 1.998 + 817.0) * 1024),
    "cvt_f32_f8e4m3_8192sq": int((131136.6 * 1.998 + 65536.0) * 1024),
    "gemm_i8_8192": int((393337.8 * 1.998 + 262443.1) * 1024),
    "gemm_f8e4m3_8192_kcontig": int((393391.2 * 1.998 + 262875.0) * 1024),
    "copy_u32_4096sq": int((32800.9 * 1.998 + 65536) * 1024),
    "gemm_i8_16x4096x11008": int((22349.1 * 1.998 + 6192.0) * 1024),
    "gemv_f8e4m3_f4_1x4096x11008": int((11060.0 * 1.998 + 43.0) * 1024),
    "gemm_i8_p4x1c_112x4096x11008": int((23911.7 * 1.998 + 4816.0) * 1024),
}


def measure(lib, key, steps=None, warmup=None, seed=0x5EED0000):
    builder, dsteps, dwarm, calls = WORKLOADS[key]
    steps = steps or dsteps
    warmup = dwarm if warmup is None else warmup
    rng = np.random.default_rng(seed)
    wl = builder(lib, rng)
    wall_ms, ev_ms = Timer(lib).run(wl["fn"], steps, warmup, calls, min_warm_ms=MFMA_WARM_MS if wl["bound"] == "mfma" else 0.0)
    out = dict(workload=key, name=wl["name"], steps=steps, warmup=warmup, calls_per_step=calls, ms_per_step=wall_ms,
               event_ms_per_call=ev_ms, dtype=wl["dtype"])
    sec, wall_sec = ev_ms * 1e-3, wall_ms * 1e-3 / calls
    if wl["bound"] == "hbm":
        gbs = wl["bytes"] / sec / 1e9
        out.update(value=wl["bytes"] / wall_sec / 1e9, unit="GB/s",
                   roofline=dict(bound="hbm", achieved=gbs, peak=HBM_PEAK_GBS, unit="GB/s", frac=gbs / HBM_PEAK_GBS,
                                 traffic=None, kernel=wl["kernel"], algorithmic_bytes=wl["bytes"]))
    else:
        tops = wl["ops"] / sec / 1e12
        peak = MFMA_PEAK_TOPS[wl["dtype"]]
        unit = "TOP/s" if wl["dtype"] == "i8" else "TFLOP/s"
        out.update(value=wl["ops"] / wall_sec / 1e12, unit=unit,
                   roofline=dict(bound="mfma", achieved=tops, peak=peak, unit=unit, frac=tops / peak, traffic=None,
                                 kernel=wl["kernel"], ops=wl["ops"]))
    out["roofline"]["traffic"] = MEASURED_TRAFFIC_BYTES.get(key)
    if key in MEASURED_TRAFFIC_BYTES:
        out["roofline"]["traffic_source"] = TRAFFIC_SOURCE
    out["buffers_rotated"] = wl.get("nbuf", 1)
    out["peak_kind"] = "hbm" if wl["bound"] == "hbm" else wl["dtype"]
    for buf in _flatten(wl["keep"]):
        buf.free()
    return out


def _flatten(x):
    for item in x:
        if isinstance(item, (list, tuple)):
            yield from _flatten(item)
        else:
            yield item


def cpu_baseline(budget_s=12.0):
    """The reference's scalar int8 GEMM (ref/gemm/gemm_i8rc_i8rc_i32rc.c) on the
    headline shape, one thread, repeated until about `budget_s` seconds are spent."""
    from oracle import loader
    ref = loader.load_ref()
    kind = "reference"
    if ref is None:
        ref, kind = loader.load_oracle(), "port"
    fn = ref.skl_gemm_i8rc_i8rc_i32rc_ref if kind == "reference" else ref.skl_gemm_i8rc_i8rc_i32rc_oracle
    k, n = 4096, 11008
    rng = np.random.default_rng(0x5EED0021)
    x, w, y = rand_i8(rng, k), rand_i8(rng, k * n), np.zeros(n, np.int32)
    reps, t0 = 0, time.perf_counter()
    while True:
        fn(1, n, k, 1, x, k, 1, w, n, 1, 0, y, n, 1)
        reps += 1
        el = time.perf_counter() - t0
        if el > budget_s or reps >= 4096:
            break
    byts = k * n + k + 4 * n
    out = dict(value=byts * reps / el / 1e9, unit="GB/s", cores=1, kind=kind,
               sample=f"{reps} full calls of the 1x4096x11008 int8 GEMV ({el:.1f} s, one thread)",
               host_cpus=os.cpu_count())
    # The same unmodified function on disjoint column panels of W and y from one thread per core of the box's
    # CPU share: the same result, the reference's path at its best on this host.
    import threading
    cores = min(16, os.cpu_count() or 1)
    panel = n // 16 * (16 // cores)  # 688 columns with 16 threads
    y_all = np.zeros(n, np.int32)
    rounds = max(1, int(0.3 * budget_s * (reps / el) * cores))  # about a third of the budget if the cores scale

    def worker(t):
        j0 = t * panel
        for _ in range(rounds):
            fn(1, panel, k, 1, x, k, 1, w[j0:], n, 1, 0, y_all[j0:], n, 1)

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(cores)]
    t0 = time.perf_counter()
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    el_all = time.perf_counter() - t0
    if np.array_equal(y_all, y):
        out["all_cores"] = dict(value=byts * rounds / el_all / 1e9, unit="GB/s", cores=cores,
                                sample=f"{rounds} GEMVs, each as {cores} column panels of {panel} on {cores} threads "
                                       f"({el_all:.1f} s)")
    return out


def vendor_blas():
    """What the vendor's BLAS reaches on this device for three of the table's products, through torch (measurement
    only: nothing of the library calls it). The same data distributions and the same sustained-clock warm-up as
    the library's rows; microseconds per call from torch's events on torch's stream."""
    import torch
    dev = "cuda"
    out = {}

    def timed(fn, flops, key, calls=20):
        try:
            t0 = time.perf_counter()
            while (time.perf_counter() - t0) * 1e3 < MFMA_WARM_MS:
                for _ in range(4):
                    fn()
                torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(calls):
                fn()
            e1.record()
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) / calls * 1e3
            out[key] = {"us": round(us, 2), "achieved": round(flops / us * 1e-6, 1)}
        except Exception as e:  # a product this torch build does not offer
            out[key] = {"error": str(e)[:80]}

    n = 8192
    try:
        a8 = torch.randint(-128, 128, (n, n), device=dev, dtype=torch.int8)
        b8 = torch.randint(-128, 128, (n, n), device=dev, dtype=torch.int8)
        timed(lambda: torch._int_mm(a8, b8), 2.0 * n ** 3, "int8 8192^3 (row-major A and B)")
        del a8, b8
    except Exception as e:
        out["int8 8192^3 (row-major A and B)"] = {"error": str(e)[:80]}
    try:
        af = torch.randn(n, n, device=dev).to(torch.float8_e4m3fn)
        bf = torch.randn(n, n, device=dev).to(torch.float8_e4m3fn).t()   # K-contiguous B
        one = torch.tensor(1.0, device=dev)
        timed(lambda: torch._scaled_mm(af, bf, scale_a=one, scale_b=one, out_dtype=torch.float32), 2.0 * n ** 3,
              "fp8 E4M3 8192^3 (K-contiguous A and B, fp32 out)")
        del af, bf
    except Exception as e:
        out["fp8 E4M3 8192^3 (K-contiguous A and B, fp32 out)"] = {"error": str(e)[:80]}
    a = torch.randn(2048, 4096, device=dev, dtype=torch.bfloat16)
    b = (torch.randn(4096, 4096, device=dev) * 0.02).to(torch.bfloat16)
    c = torch.randn(2048, 4096, device=dev, dtype=torch.float32)
    timed(lambda: torch.addmm(c.to(torch.bfloat16), a, b), 2.0 * 2048 * 4096 * 4096, "bf16 2048x4096x4096 (bf16 out, beta=1)", calls=80)
    return out


def config_rows(records, probes):
    """`roofline.configs`: one short row per benchmark configuration - workload key, microseconds per call (HIP
    events), achieved rate, fraction of the published peak and of the ceiling measured on this device."""
    rows = {}
    for label, key in CONFIG_TABLE.items():
        r = records.get(key)
        if r is None:
            continue
        if "error" in r:
            rows[label] = {"key": key, "error": str(r["error"])[:80]}
            continue
        roof = r["roofline"]
        probe = probes.get(MEASURED_PEAK_OF.get(r["peak_kind"]))
        rows[label] = {"key": key, "us": round(r["event_ms_per_call"] * 1e3, 2), "achieved": round(roof["achieved"], 1),
                       "unit": roof["unit"], "frac": round(roof["frac"], 4),
                       "frac_of_measured": round(roof["achieved"] / probe["roofline"]["achieved"], 4) if probe else None}
    return rows


def compact_result(head, records, cpu, device):
    """The record of the final stdout line: the headline, its roofline with the measured ceilings and the table of
    benchmark configurations, the CPU baseline and the device. Everything else goes to the results file. `records`
    maps workload keys to measure() records (or {"error": ...})."""
    probes = {k: r for k, r in records.items() if k.startswith("peak_") and "error" not in r}
    roof = dict(head["roofline"])
    probe = probes.get(MEASURED_PEAK_OF.get(head["peak_kind"]))
    if probe and not head["workload"].startswith("peak_"):
        roof["measured_peak"] = {"value": round(probe["roofline"]["achieved"], 1), "unit": probe["roofline"]["unit"],
                                 "workload": probe["workload"]}
        roof["frac_of_measured"] = round(roof["achieved"] / probe["roofline"]["achieved"], 4)
    roof["measured_peaks"] = {k: {"value": round(r["roofline"]["achieved"], 1), "unit": r["roofline"]["unit"]}
                              for k, r in probes.items()}
    rows = config_rows(records, probes)
    if rows:
        roof["configs"] = rows
    result = {
        "metric": METRIC,
        "value": head["value"],
        "unit": head["unit"],
        "n_gpus": 1,
        "steps": head["steps"],
        "warmup": head["warmup"],
        "ms_per_step": head["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": head["dtype"],
        "data": "synthetic",
        "config": {"workload": head["name"], "key": head["workload"], "resident": "HBM",
                   "calls_per_step": head["calls_per_step"], "event_us_per_call": round(head["event_ms_per_call"] * 1e3, 3),
                   "weight_buffers_rotated": head.get("buffers_rotated", 1)},
        "roofline": roof,
    }
    if cpu is not None:
        result["cpu_baseline"] = cpu
    result["device"] = device
    return result


def device_description(lib):
    import ctypes
    name, cus, mhz = ctypes.create_string_buffer(128), ctypes.c_int(0), ctypes.c_int(0)
    lib.skl_hip_device_info(name, 128, ctypes.byref(cus), ctypes.byref(mhz))
    return f"{name.value.decode().strip()}, {cus.value} CUs, {mhz.value} MHz"


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None)
    ap.add_argument("--warmup", type=int, default=None)
    ap.add_argument("--workload", default=HEADLINE, choices=sorted(WORKLOADS))
    ap.add_argument("--no-extra", action="store_true", help="only the chosen workload: no table of configurations")
    ap.add_argument("--full", action="store_true", help="also run every other workload (records go to the results file)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--vendor-only", action="store_true",
                    help="time the vendor BLAS (through torch) on three of the table's products and print that alone: a process "
                         "of its own, since torch brings its own HIP runtime")
    ap.add_argument("--out", default=os.path.join(ROOT, "gpurun_out", "bench_full.json"),
                    help="file that receives the full records of everything measured")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this library runs on one GPU; --gpus must be 1 (no multi-GPU path exists)")

    if args.vendor_only:
        print(json.dumps({"vendor_blas": vendor_blas()}, separators=(",", ":")), flush=True)
        return
    lib = skl_amd.load()
    if lib.skl_hip_init(0) != 0:
        sys.exit("bench.py: no GPU: " + lib.skl_hip_last_error_string().decode())
    lib.skl_hip_set_pointer_mode(1)  # device pointers only: no per-call pointer queries

    records = {args.workload: measure(lib, args.workload, args.steps, args.warmup)}
    head = records[args.workload]

    def measured(key):
        if key not in records:
            try:
                records[key] = measure(lib, key)
            except Exception as e:  # a failing extra must not hide the headline
                records[key] = {"workload": key, "error": str(e)}

    if head["peak_kind"] in MEASURED_PEAK_OF:
        measured(MEASURED_PEAK_OF[head["peak_kind"]])
    if not args.no_extra:
        for key in list(CONFIG_TABLE.values()) + sorted(set(MEASURED_PEAK_OF.values())):
            measured(key)
    if args.full:
        for key in WORKLOADS:
            measured(key)
    cpu = None if args.no_cpu else cpu_baseline()
    result = compact_result(head, records, cpu, device_description(lib))
    try:
        os.makedirs(os.path.dirname(args.out), exist_ok=True)
        with open(args.out, "w") as f:
            json.dump({"line": result, "records": records}, f, indent=1)
        result["full_results"] = os.path.relpath(args.out, ROOT)
    except OSError:
        pass
    print(json.dumps(result, separators=(",", ":")), flush=True)


if __name__ == "__main__":
    main()
