"""A decode loop captured into a HIP graph: the entry points called with device pointers only enqueue kernels on
the calling thread's stream (no allocation, no memset, no synchronisation once the per-device scratch exists), so a
sequence of them can be captured once and replayed. Each replay is checked against the CPU checker (int8, bit for
bit) or the eager result (bf16), with new inputs written between the replays."""
import numpy as np
import pytest

import skl_amd
import support
from support import rowmajor_case, run_oracle_gemm

pytestmark = pytest.mark.gpu


def _hip():
    """The HIP runtime the library itself is linked against (already loaded with it)."""
    import ctypes
    hip = ctypes.CDLL("libamdhip64.so.7")
    for name in ("hipStreamCreate", "hipStreamBeginCapture", "hipStreamEndCapture", "hipGraphInstantiate", "hipGraphLaunch",
                 "hipStreamSynchronize", "hipGraphExecDestroy", "hipGraphDestroy", "hipStreamDestroy"):
        getattr(hip, name).restype = ctypes.c_int
    return hip, ctypes


def test_decode_loop_replays_from_a_graph(gpu):
    hip, ct = _hip()
    rng = np.random.default_rng(2024)
    layers, n, k = 6, 2048, 1024
    B = skl_amd.DeviceBuffer
    hw = [rng.integers(-128, 128, (k, n), dtype=np.int8) for _ in range(layers)]
    hwt = rng.integers(-128, 128, (n, k), dtype=np.int8)        # stored [n][k]: K contiguous
    hw16 = rng.integers(-128, 128, (4096, n), dtype=np.int8)    # 16 rows against it: few tiles, long K - K is shared
    hwb = support.ETYPES["bf16"].gen(rng, k * n)
    w = [B.from_array(h) for h in hw]
    wt, w16, wb = B.from_array(hwt), B.from_array(hw16), B.from_array(hwb)
    x, xs, a16, xb = B(k), B(4 * k), B(16 * 4096), B(2 * k)
    y = [B(4 * n) for _ in range(layers)]
    yt, ys, y16, yb = B(4 * n), B(16 * n), B(64 * n), B(4 * n)
    # MXFP4 weights stored [n][k] with one scale per 32 k, E4M3 activations in {1, 2, 4}: every sum is exact
    import ofp4_support as f4
    codes4 = rng.integers(0, 16, size=n * k, dtype=np.uint8)
    hs4 = rng.integers(125, 130, size=n * (k // 32), dtype=np.uint8)
    w4, s4, x4, y4 = B.from_array(f4.pack_nibbles(codes4)), B.from_array(hs4), B(k), B(4 * n)
    W4 = f4.E2M1_VALUES[codes4].reshape(n, k) * np.ldexp(1.0, hs4.reshape(n, k // 32).astype(np.int64) - 127).repeat(32, axis=1)

    def enqueue():
        for l in range(layers):
            gpu.skl_gemm_i8_i8_i32_gfx950(1, n, k, 1, x, k, w[l], n, 0, y[l], n)
        gpu.skl_gemm_i8rc_i8rc_i32rc_gfx950(1, n, k, 1, x, k, 1, wt, 1, k, 0, yt, n, 1)
        gpu.skl_gemm_i8_i8_i32_gfx950(4, n, k, 1, xs, k, w[0], n, 0, ys, n)
        gpu.skl_gemm_i8_i8_i32_gfx950(16, n, 4096, 1, a16, 4096, w16, n, 0, y16, n)
        gpu.skl_gemm_bf16_bf16_f32_gfx950(1, n, k, 1.0, xb, k, wb, n, 0.0, yb, n)
        gpu.skl_gemm_f8e4m3rc_mxf4e2m1c_f32rc_gfx950(1, n, k, 1.0, x4, k, 1, w4, k, s4, k // 32, 0.0, y4, n, 1)

    stream, graph, executable = ct.c_void_p(), ct.c_void_p(), ct.c_void_p()
    assert hip.hipStreamCreate(ct.byref(stream)) == 0
    gpu.skl_hip_set_pointer_mode(1)  # device pointers promised: no runtime queries inside the capture
    gpu.skl_hip_set_stream(stream.value)
    try:
        for buf, nbytes in ((x, k), (xs, 4 * k), (a16, 16 * 4096), (xb, 2 * k), (x4, k)):
            gpu.skl_hip_memset(buf, 0, nbytes)
        enqueue()  # eager once: creates the library's scratch blocks and configures the kernels
        assert gpu.skl_hip_synchronize() == 0
        skl_amd.check_error()
        assert hip.hipStreamBeginCapture(stream, 0) == 0
        enqueue()
        assert hip.hipStreamEndCapture(stream, ct.byref(graph)) == 0
        skl_amd.check_error()
        assert hip.hipGraphInstantiate(ct.byref(executable), graph, None, None, ct.c_size_t(0)) == 0
        for rep in range(4):
            hx = rng.integers(-128, 128, k, dtype=np.int8)
            hxs = rng.integers(-128, 128, (4, k), dtype=np.int8)
            ha = rng.integers(-128, 128, (16, 4096), dtype=np.int8)
            hb = support.ETYPES["bf16"].gen(rng, k)
            hx4 = rng.choice(np.array([0x38, 0x40, 0x48], np.uint8), k)
            x.upload(hx), xs.upload(hxs), a16.upload(ha), xb.upload(hb), x4.upload(hx4)
            for t, count in [(t, n) for t in y] + [(yt, n), (ys, 4 * n), (y16, 16 * n), (yb, n), (y4, n)]:
                gpu.skl_hip_memset(t, 0x5A, 4 * count)  # a replay must rewrite every output
            assert hip.hipGraphLaunch(executable, stream) == 0
            assert hip.hipStreamSynchronize(stream) == 0
            wide = lambda a: a.astype(np.int64)
            for l in range(layers):
                assert np.array_equal(y[l].download(np.int32), (wide(hx) @ wide(hw[l])).astype(np.int32)), (rep, l)
            assert np.array_equal(yt.download(np.int32), (wide(hwt) @ wide(hx)).astype(np.int32)), rep
            assert np.array_equal(ys.download(np.int32), (wide(hxs) @ wide(hw[0])).astype(np.int32).ravel()), rep
            assert np.array_equal(y16.download(np.int32), (wide(ha) @ wide(hw16)).astype(np.int32).ravel()), rep
            xv, wv = support.ETYPES["bf16"].widen(hb), support.ETYPES["bf16"].widen(hwb).reshape(k, n)
            bound = 2 * ((1 + 2.0 ** -24) ** (k + 2) - 1) * (np.abs(xv) @ np.abs(wv)) + 1e-30
            assert np.all(np.abs(yb.download(np.float32) - xv @ wv) <= bound), rep
            assert np.array_equal(y4.download(np.float32).astype(np.float64), W4 @ support.decode_table("f8e4m3")[hx4]), rep
    finally:
        gpu.skl_hip_set_stream(None)
        gpu.skl_hip_set_pointer_mode(0)
        if executable:
            hip.hipGraphExecDestroy(executable)
        if graph:
            hip.hipGraphDestroy(graph)
        gpu.skl_hip_release_stream(stream.value)
        hip.hipStreamDestroy(stream)
        for d in w + y + [wt, w16, wb, x, xs, a16, xb, yt, ys, y16, yb, w4, s4, x4, y4]:
            d.free()
    # the integer products used above are what the checker computes (one layer)
    case = rowmajor_case("i8", 1, n, k, alpha=1, beta=0)
    a_, b_, c_ = case.make_inputs(5)
    assert np.array_equal(run_oracle_gemm(case, a_, b_, c_)[:n],
                          (a_[:k].astype(np.int64) @ b_[:k * n].reshape(k, n).astype(np.int64)).astype(np.int32))
