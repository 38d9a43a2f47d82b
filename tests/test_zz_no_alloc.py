"""skl_gemm_i8_i8_i32_noalloc_gfx950: the int8 decode call that allocates nothing (its shared sums live in a static
device array of 65536 slots) must give the bits of skl_gemm_i8_i8_i32_gfx950 - which the other tests compare with
the CPU checker - on calls in a row, the later ones smaller than the first, and must reject what it cannot serve."""
import numpy as np
import pytest

import skl_amd
from skl_amd import DeviceBuffer

pytestmark = pytest.mark.gpu


def _both(lib, m, n, k, alpha, beta, seed, rsb=None, rsc=None):
    """The same call through both entry points on device buffers; returns (no-alloc C, ordinary C), whole buffers."""
    rng = np.random.default_rng(seed)
    rsb, rsc = rsb or n, rsc or n
    a = rng.integers(-128, 128, size=m * k, dtype=np.int8)
    b = rng.integers(-128, 128, size=k * rsb, dtype=np.int8)
    c = rng.integers(-2 ** 31, 2 ** 31, size=m * rsc).astype(np.int32)
    da, db = DeviceBuffer.from_array(a), DeviceBuffer.from_array(b)
    out = []
    for name in ("skl_gemm_i8_i8_i32_noalloc_gfx950", "skl_gemm_i8_i8_i32_gfx950"):
        dc = DeviceBuffer.from_array(c)
        getattr(lib, name)(m, n, k, alpha, da, k, db, rsb, beta, dc, rsc)
        assert lib.skl_hip_synchronize() == 0
        skl_amd.check_error()
        out.append(dc.download(np.int32, c.size))
        dc.free()
    da.free()
    db.free()
    return out


def test_two_calls_in_a_row_the_second_smaller(gpu):
    # 4096 x 11008: eight workgroups share every column through the static slots; then a smaller problem on the
    # slots the first one used, then a batch of rows, then the first shape again
    for seed, (m, n, k, alpha, beta) in enumerate(((1, 11008, 4096, 1, 0), (1, 2048, 1536, -3, 1), (5, 4096, 2048, 2, -7),
                                                    (8, 8192, 1024, 1, 0), (1, 11008, 4096, 0x01010101, 5))):
        got, want = _both(gpu, m, n, k, alpha, beta, 900 + seed)
        assert np.array_equal(got, want), (m, n, k, alpha, beta)


def test_padded_strides_and_ragged_k(gpu):
    got, want = _both(gpu, 1, 4112, 1000, 1, 1, 950, rsb=4112 + 16, rsc=4112 + 3)
    assert np.array_equal(got, want)
    got, want = _both(gpu, 3, 1040, 520, -1, 0, 951, rsb=1040 + 32, rsc=1040 + 1)
    assert np.array_equal(got, want)


def test_rejects_what_the_static_scratch_cannot_hold(gpu):
    lib = gpu
    n, k = 65536 + 16, 64
    da, db, dc = DeviceBuffer(k), DeviceBuffer(k * n), DeviceBuffer.from_array(np.full(n, 7, np.int32))
    for (m, nn, kk) in ((1, n, k), (9, 1024, 64), (1, 1000, 64), (2, 65536, 64)):  # too wide, too many rows, ragged N, M * N
        lib.skl_gemm_i8_i8_i32_noalloc_gfx950(m, nn, kk, 1, da, kk, db, nn, 0, dc, nn)
        assert lib.skl_hip_last_error() == -2, (m, nn, kk)
        assert b"noalloc" in lib.skl_hip_last_error_string()
    assert lib.skl_hip_synchronize() == 0
    assert np.all(dc.download(np.int32, n) == 7)  # nothing was written
    # the widest call it takes
    got, want = _both(gpu, 1, 65536, 512, 1, 0, 960)
    assert np.array_equal(got, want)
    for d in (da, db, dc):
        d.free()


def test_allocates_nothing_and_replays_from_a_graph(gpu):
    """What the entry point exists for: on a stream that holds no scratch slot of the library, the call changes
    nothing about the device's free memory, it can be recorded into a HIP graph, and every replay - with new
    activations written in between and eager work of the process around it - gives the ordinary entry point's bits.
    A spoiled array of sums is put right by skl_hip_noalloc_reset()."""
    import ctypes as ct

    lib = gpu
    hip = ct.CDLL("libamdhip64.so.7")
    for name in ("hipStreamCreate", "hipStreamBeginCapture", "hipStreamEndCapture", "hipGraphInstantiate", "hipGraphLaunch",
                 "hipStreamSynchronize", "hipGraphExecDestroy", "hipGraphDestroy", "hipStreamDestroy", "hipMemGetInfo"):
        getattr(hip, name).restype = ct.c_int

    def free_bytes():
        free, total = ct.c_size_t(), ct.c_size_t()
        assert hip.hipMemGetInfo(ct.byref(free), ct.byref(total)) == 0
        return free.value

    m, n, k = 3, 4096, 2048
    rng = np.random.default_rng(77)
    b = rng.integers(-128, 128, size=k * n, dtype=np.int8)
    c0 = rng.integers(-1000, 1000, size=m * n).astype(np.int32)
    da, db, dc, dref = DeviceBuffer(m * k), DeviceBuffer.from_array(b), DeviceBuffer.from_array(c0), DeviceBuffer.from_array(c0)
    stream, graph, executable = ct.c_void_p(), ct.c_void_p(), ct.c_void_p()
    assert hip.hipStreamCreate(ct.byref(stream)) == 0
    lib.skl_hip_set_pointer_mode(1)
    try:
        lib.skl_hip_set_stream(stream.value)
        a = rng.integers(-128, 128, size=m * k, dtype=np.int8)
        lib.skl_hip_memcpy_h2d(da, a, a.nbytes)
        before = free_bytes()
        lib.skl_gemm_i8_i8_i32_noalloc_gfx950(m, n, k, 2, da, k, db, n, 1, dc, n)     # eager, on the fresh stream
        assert lib.skl_hip_synchronize() == 0 and lib.skl_hip_last_error() == 0
        assert free_bytes() == before                                              # no scratch block, no workspace
        assert hip.hipStreamBeginCapture(stream, 0) == 0
        lib.skl_gemm_i8_i8_i32_noalloc_gfx950(m, n, k, 2, da, k, db, n, 1, dc, n)
        assert hip.hipStreamEndCapture(stream, ct.byref(graph)) == 0
        assert lib.skl_hip_last_error() == 0
        assert hip.hipGraphInstantiate(ct.byref(executable), graph, None, None, 0) == 0
        expected = None
        for replay in range(3):
            a = rng.integers(-128, 128, size=m * k, dtype=np.int8)
            lib.skl_hip_memcpy_h2d(da, a, a.nbytes)
            lib.skl_hip_memcpy_h2d(dc, c0, c0.nbytes)
            assert hip.hipGraphLaunch(executable, stream) == 0
            assert hip.hipStreamSynchronize(stream) == 0
            lib.skl_hip_set_stream(None)                                           # the ordinary call, eagerly, on the default stream
            lib.skl_hip_memcpy_h2d(dref, c0, c0.nbytes)
            lib.skl_gemm_i8_i8_i32_gfx950(m, n, k, 2, da, k, db, n, 1, dref, n)
            assert lib.skl_hip_synchronize() == 0
            lib.skl_hip_set_stream(stream.value)
            expected = dref.download(np.int32, c0.size)
            assert np.array_equal(dc.download(np.int32, c0.size), expected), replay
        # sums left behind (as overlapping calls would) spoil the next result; the reset puts them right
        assert lib.skl_hip_noalloc_reset() == 0
        lib.skl_hip_memcpy_h2d(dc, c0, c0.nbytes)
        lib.skl_gemm_i8_i8_i32_noalloc_gfx950(m, n, k, 2, da, k, db, n, 1, dc, n)
        assert lib.skl_hip_synchronize() == 0 and lib.skl_hip_last_error() == 0
        assert np.array_equal(dc.download(np.int32, c0.size), expected)
    finally:
        lib.skl_hip_set_stream(None)
        lib.skl_hip_set_pointer_mode(0)
        if executable:
            hip.hipGraphExecDestroy(executable)
        if graph:
            hip.hipGraphDestroy(graph)
        lib.skl_hip_release_stream(stream.value)
        hip.hipStreamDestroy(stream)
        for d in (da, db, dc, dref):
            d.free()
        lib.skl_hip_last_error()
