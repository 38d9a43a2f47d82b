"""GPU parity of the conversion kernels with the CPU checker: bit-exact on the
reference's test inputs (test/cvt/cvt_f32_f8.c:29-35 and the suites' tables),
on structured bit patterns, with scales, tails and misaligned pointers."""
import numpy as np
import pytest

import skl_amd
import support
from gpu_support import MODES, run_inout
from support import oracle
from test_oracle_cvt import _structured_f32_patterns, reference_cvt_input

pytestmark = pytest.mark.gpu
FMTS = ("f8e4m3", "f8e5m2")


def both(gpu, stem, src, dst, extra, mode):
    """Runs <stem>_oracle on the host and <stem>_gfx950 through the library."""
    n = dst.size - 8  # callers leave 8 poison elements at the end
    want = dst.copy()
    getattr(oracle(), stem + "_oracle")(want, src, *extra, n)
    got = run_inout(gpu, stem + "_gfx950", lambda s, d: (d, s, *extra, n), src, dst, mode)
    return got, want


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("row", support.table_rows("test/cvt/cvt_f32_f8_zvfofp8min.c", ("TEST", "BENCH")),
                         ids=lambda r: f"L{r['line']}")
def test_f32_reference_table(gpu, row, mode):
    fmt = "f8e4m3" if row["kind"].endswith("E4M3") else "f8e5m2"
    stem = f"skl_cvt_{'sat_' if row['saturation'] else ''}f32_{fmt}"
    x = reference_cvt_input(row["len"], row["line"])
    got, want = both(gpu, stem, x, np.full(row["len"] + 8, 0xAA, np.uint8), (float(row["scale"]),), mode)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("row", support.table_rows("test/cvt/cvt_bf16_f8_zvfofp8min_zvfbfmin.c", ("TEST", "BENCH")),
                         ids=lambda r: f"L{r['line']}")
def test_bf16_reference_table(gpu, row, mode):
    fmt = "f8e4m3" if row["kind"].endswith("E4M3") else "f8e5m2"
    stem = f"skl_cvt_{'sat_' if row['saturation'] else ''}bf16_{fmt}"
    x = support.f32_to_bf16_bits(np.random.default_rng(row["line"]).uniform(-512, 512, row["len"]).astype(np.float32))
    x[:3] = [0x7FC0, 0x7F80, 0xFF80]
    got, want = both(gpu, stem, x, np.full(row["len"] + 8, 0xAA, np.uint8), (float(row["scale"]),), mode)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("sat", (False, True))
@pytest.mark.parametrize("fmt", FMTS)
def test_f32_bit_patterns(gpu, fmt, sat):
    """2^16 upper halves x 8 lower halves + 2M random fp32 patterns."""
    x = _structured_f32_patterns()
    stem = f"skl_cvt_{'sat_' if sat else ''}f32_{fmt}"
    got, want = both(gpu, stem, x, np.full(x.size + 8, 0xAA, np.uint8), (1.0,), "device")
    bad = np.nonzero(got != want)[0]
    assert bad.size == 0, [(hex(x.view(np.uint32)[i]), hex(got[i]), hex(want[i])) for i in bad[:5]]


@pytest.mark.parametrize("scale", (1.5, 2.0 ** 100, 2.0 ** -100, 3.0e38, -0.75))
@pytest.mark.parametrize("fmt", FMTS)
def test_f32_scaled(gpu, fmt, scale):
    rng = np.random.default_rng(5)
    x = np.concatenate([
        rng.uniform(-512, 512, 4096).astype(np.float32),
        rng.integers(0, 1 << 23, 4096, dtype=np.uint32).view(np.float32),  # fp32 subnormals must not be flushed
        (rng.integers(0, 1 << 23, 4096, dtype=np.uint32) | np.uint32(0x80000000)).view(np.float32),
        np.float32([np.nan, np.inf, -np.inf, 0.0, -0.0]),
    ])
    for sat in (False, True):
        stem = f"skl_cvt_{'sat_' if sat else ''}f32_{fmt}"
        got, want = both(gpu, stem, x, np.full(x.size + 8, 0xAA, np.uint8), (float(scale),), "device")
        assert np.array_equal(got, want)


@pytest.mark.parametrize("scale", (1.0, 1.5, 1e30))
@pytest.mark.parametrize("sat", (False, True))
@pytest.mark.parametrize("fmt", FMTS)
def test_bf16_all_patterns(gpu, fmt, sat, scale):
    x = np.arange(1 << 16, dtype=np.uint16)
    stem = f"skl_cvt_{'sat_' if sat else ''}bf16_{fmt}"
    got, want = both(gpu, stem, x, np.full(x.size + 8, 0xAA, np.uint8), (float(scale),), "device")
    assert np.array_equal(got, want)


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("fmt", FMTS)
def test_f8_to_bf16_all_codes(gpu, fmt, mode):
    x = np.tile(np.arange(256, dtype=np.uint8), 5)[:1027]
    got, want = both(gpu, f"skl_cvt_{fmt}_bf16", x, np.full(x.size + 8, 0xAAAA, np.uint16), (), mode)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("n", (0, 1, 2, 7, 31, 32, 33, 511, 512, 4099))
def test_f4_to_f8(gpu, n, mode):
    x = np.tile(np.arange(256, dtype=np.uint8), 9)[:(n + 1) // 2 + 1]
    got, want = both(gpu, "skl_cvt_f4e2m1_f8e4m3", x, np.full(n + 8, 0xAA, np.uint8), (), mode)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("n", (0, 1, 5, 8, 9, 255, 256, 257, 1000))
@pytest.mark.parametrize("src_off,dst_off", ((0, 0), (1, 0), (0, 3), (3, 5)))
def test_tails_and_misaligned_pointers(gpu, n, src_off, dst_off):
    """Element-aligned but not vector-aligned pointers, every tail length; the
    bytes before and after the destination range must stay untouched."""
    x = reference_cvt_input(n + 8, n)[:n + 8]
    dsrc = skl_amd.DeviceBuffer.from_array(np.concatenate([np.zeros(src_off, np.float32), x]))
    ddst = skl_amd.DeviceBuffer.from_array(np.full(n + 32, 0xAA, np.uint8))
    gpu.skl_cvt_sat_f32_f8e4m3_gfx950(ddst.offset(dst_off), dsrc.offset(4 * src_off), 1.5, n)
    gpu.skl_hip_synchronize()
    skl_amd.check_error()
    got = ddst.download(np.uint8)
    want = np.full(n + 32, 0xAA, np.uint8)
    tmp = np.zeros(max(n, 1), np.uint8)
    oracle().skl_cvt_sat_f32_f8e4m3_oracle(tmp, x, 1.5, n)
    want[dst_off:dst_off + n] = tmp[:n]
    assert np.array_equal(got, want)


def test_config4_operand_preparation(gpu):
    """fp32 ~ N(0,1) -> E4M3 / E5M2 with saturation, scale 1 (benchmark configuration 4's
    input preparation), 4M elements, against the checker."""
    x = np.random.default_rng(0x5EED0040).normal(size=1 << 22).astype(np.float32)
    for fmt in FMTS:
        got, want = both(gpu, f"skl_cvt_sat_f32_{fmt}", x, np.full(x.size + 8, 0xAA, np.uint8), (1.0,), "device")
        assert np.array_equal(got, want)


def test_mixed_pointers_are_refused(gpu):
    x = np.zeros(16, np.float32)
    d = skl_amd.DeviceBuffer(16)
    gpu.skl_cvt_f32_f8e4m3_gfx950(d, x, 1.0, 16)
    assert gpu.skl_hip_last_error() == -1
    assert b"mixed" in gpu.skl_hip_last_error_string()


@pytest.mark.parametrize("sat", (False, True))
@pytest.mark.parametrize("fmt", FMTS)
def test_f32_every_bit_pattern(gpu, fmt, sat):
    """All 2^32 fp32 bit patterns through the GPU kernel against the CPU checker (which is itself compared with the
    compiled reference over the same 2^32 inputs by test_oracle_cvt's exhaustive sweep). The checker runs on a pool of
    threads while the GPU converts the next chunk: about four seconds per variant on the GPU host."""
    from concurrent.futures import ThreadPoolExecutor
    stem = f"skl_cvt_{'sat_' if sat else ''}f32_{fmt}"
    chunk = 1 << 24
    src, dst = skl_amd.DeviceBuffer(4 * chunk), skl_amd.DeviceBuffer(chunk)

    def chunk_input(c):
        return (np.arange(chunk, dtype=np.uint32) | np.uint32(c << 24)).view(np.float32)

    def checker(c):
        want = np.empty(chunk, np.uint8)
        getattr(oracle(), stem + "_oracle")(want, chunk_input(c), 1.0, chunk)
        return want

    with ThreadPoolExecutor(max_workers=12) as pool:
        window = 24
        pending = {c: pool.submit(checker, c) for c in range(window)}
        for c in range(256):
            src.upload(chunk_input(c))
            getattr(gpu, stem + "_gfx950")(dst, src, 1.0, chunk)
            assert gpu.skl_hip_synchronize() == 0
            got = dst.download(np.uint8)
            want = pending.pop(c).result()
            if c + window < 256:
                pending[c + window] = pool.submit(checker, c + window)
            bad = np.nonzero(got != want)[0]
            assert bad.size == 0, (c, [(hex(int(chunk_input(c).view(np.uint32)[i])), hex(got[i]), hex(want[i])) for i in bad[:5]])
            if c % 32 == 31:
                print(f"{stem}: {c + 1} / 256 chunks equal", flush=True)
    src.free(), dst.free()
