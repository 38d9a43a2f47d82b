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
