"""GPU parity of pack / unpack / transpose / panel pack with the CPU checker
over the reference's test tables (whole destination buffers compared, so the
stride gaps are a clobber check), plus the benchmark configuration 5 shapes checked
through the closed-form index map."""
import numpy as np
import pytest

import skl_amd
import support
from gpu_support import MODES, run_inout
from support import oracle
from test_oracle_pack import DT, PACK_ROWS, numpy_pack, pack_case_buffers

pytestmark = pytest.mark.gpu
PAD = {8: 0xFF, 16: 0xFFFF, 32: 0xFFFFFFFF}


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("w", (8, 16, 32))
def test_pack_reference_table(gpu, w, mode):
    for row in PACK_ROWS[w]:
        src, dst = pack_case_buffers(row, w, row["line"])
        tail = (row["m0"], row["n0"])
        strides = (row["rs0"], row["cs0"], row["rs1"], row["cs1"], PAD[w])
        want = dst.copy()
        getattr(oracle(), f"skl_pack_e{w}rc_e{w}rcprc_oracle")(row["m"], row["n"], src, row["rs"], row["cs"], *tail,
                                                                want, *strides)
        got = run_inout(gpu, f"skl_pack_e{w}rc_e{w}rcprc_gfx950",
                        lambda s, d: (row["m"], row["n"], s, row["rs"], row["cs"], *tail, d, *strides), src, dst, mode)
        assert np.array_equal(got, want), row


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("w", (8, 16, 32))
def test_unpack_reference_table(gpu, w, mode):
    for row in support.table_rows("test/pack/rvv/skl_unpack_e8rcprc_e8rc_zve32x.c", ("TEST", "BENCH")):
        plain, packed = pack_case_buffers(row, w, row["line"] + 7)
        blk = (row["m0"], row["n0"])
        bs = (row["rs0"], row["cs0"], row["rs1"], row["cs1"])
        want = plain.copy()
        getattr(oracle(), f"skl_unpack_e{w}rcprc_e{w}rc_oracle")(*blk, packed, *bs, row["m"], row["n"], want,
                                                                  row["rs"], row["cs"])
        got = run_inout(gpu, f"skl_unpack_e{w}rcprc_e{w}rc_gfx950",
                        lambda s, d: (*blk, s, *bs, row["m"], row["n"], d, row["rs"], row["cs"]), packed, plain, mode)
        assert np.array_equal(got, want), row


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("w", (8, 16, 32))
def test_transpose_reference_table(gpu, w, mode):
    rows = support.table_rows(f"test/pack/rvv/skl_transpose_e{w}_zve32x.c", ("TEST", "BENCH")) + \
        support.table_rows(f"test/pack/xsfmm/skl_transpose_e{w}_xsfmmbase.c", ("TEST", "BENCH"))
    for row in rows:
        m, n = row["m"], row["n"]
        rsa, rsat = row.get("rsa") or n, row.get("rsat") or m
        rng = np.random.default_rng(row["line"])
        a = rng.integers(0, 1 << w, size=max(m * rsa, 1), dtype=np.uint64).astype(DT[w])
        at = rng.integers(0, 1 << w, size=max(n * rsat, 1), dtype=np.uint64).astype(DT[w])
        want = at.copy()
        getattr(oracle(), f"skl_transpose_e{w}_oracle")(m, n, a, rsa, want, rsat)
        got = run_inout(gpu, f"skl_transpose_e{w}_gfx950", lambda s, d: (m, n, s, rsa, d, rsat), a, at, mode)
        assert np.array_equal(got, want), row


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("w", (8, 16, 32))
def test_panel_pack_reference_table(gpu, w, mode):
    te = support.TE
    src_w = 16 if w == 8 else w   # the reference has no 8-bit panel suite: reuse the 16-bit table
    for row in support.table_rows(f"test/pack/xsfmm/skl_pack_e{src_w}_e{src_w}rcptex1c_xsfmmbase.c", ("TEST", "BENCH")):
        m, n = row["m"], row["n"]
        rs = row.get("rs") or n
        cs1 = row.get("cs1") or te
        rs1 = row.get("rs1") or n * cs1
        full = dict(m=m, n=n, rs=rs, cs=1, m0=te, n0=1, rs0=1, cs0=te, rs1=rs1, cs1=cs1)
        src, dst = pack_case_buffers(full, w, row["line"])
        want = dst.copy()
        getattr(oracle(), f"skl_pack_e{w}rc_e{w}rcprc_oracle")(m, n, src, rs, 1, te, 1, want, 1, 0, rs1, cs1, PAD[w])
        got = run_inout(gpu, f"skl_pack_e{w}_e{w}rcptex1c_gfx950",
                        lambda s, d: (m, n, s, rs, d, rs1, cs1, PAD[w]), src, dst, mode)
        assert np.array_equal(got, want), row


def test_zero_extents_touch_nothing(gpu):
    src = np.arange(64, dtype=np.uint8)
    for (m, n, m0, n0) in ((0, 4, 2, 2), (4, 0, 2, 2), (4, 4, 0, 2), (4, 4, 2, 0)):
        dst = np.full(64, 0xAA, np.uint8)
        gpu.skl_pack_e8rc_e8rcprc_gfx950(m, n, src, 4, 1, m0, n0, dst, 1, 2, 8, 4, 0)
        gpu.skl_unpack_e8rcprc_e8rc_gfx950(m0, n0, src, 1, 2, 8, 4, m, n, dst, 4, 1)
        skl_amd.check_error()
        assert np.all(dst == 0xAA)


def test_config5_pipeline_shapes(gpu):
    """benchmark configuration 5: pack A (4096x4096 f16 -> TE x 1 panels), pack B
    (4096x14336 f16 -> 1 x TE panels), unpack C (TE x TE f32 blocks -> row-major
    4096x14336). Full size, device resident, checked against the closed-form
    index map (numpy) and by pack -> unpack round trip."""
    te = support.TE
    rng = np.random.default_rng(0x5EED0050)
    m, k, n = 4096, 4096, 14336
    # A -> A_p[i/64][k][i%64]
    a = rng.integers(0, 1 << 16, size=m * k, dtype=np.uint16)
    da, dap = skl_amd.DeviceBuffer.from_array(a), skl_amd.DeviceBuffer(2 * m * k)
    gpu.skl_pack_e16_e16rcptex1c_gfx950(m, k, da, k, dap, k * te, te, 0)
    gpu.skl_hip_synchronize()
    got = dap.download(np.uint16).reshape(m // te, k, te)
    assert np.array_equal(got, a.reshape(m // te, te, k).transpose(0, 2, 1))
    da.free(), dap.free()
    # B -> B_p[j/64][k][j%64]
    b = rng.integers(0, 1 << 16, size=k * n, dtype=np.uint16)
    db, dbp = skl_amd.DeviceBuffer.from_array(b), skl_amd.DeviceBuffer(2 * k * n)
    gpu.skl_pack_e16rc_e16rcprc_gfx950(k, n, db, n, 1, 1, te, dbp, te, 1, te, k * te, 0)
    gpu.skl_hip_synchronize()
    got = dbp.download(np.uint16).reshape(n // te, k, te)
    assert np.array_equal(got, b.reshape(k, n // te, te).transpose(1, 0, 2))
    # round trip of B through unpack
    dbu = skl_amd.DeviceBuffer(2 * k * n)
    gpu.skl_unpack_e16rcprc_e16rc_gfx950(1, te, dbp, te, 1, te, k * te, k, n, dbu, n, 1)
    gpu.skl_hip_synchronize()
    assert np.array_equal(dbu.download(np.uint16), b)
    db.free(), dbp.free(), dbu.free()
    # C blocks [I][J][64][64] -> row-major
    c = rng.integers(0, 1 << 32, size=m * n, dtype=np.uint32)
    dc, dcu = skl_amd.DeviceBuffer.from_array(c), skl_amd.DeviceBuffer(4 * m * n)
    gpu.skl_unpack_e32rcprc_e32rc_gfx950(te, te, dc, te, 1, (n // te) * te * te, te * te, m, n, dcu, n, 1)
    gpu.skl_hip_synchronize()
    skl_amd.check_error()
    got = dcu.download(np.uint32).reshape(m, n)
    want = c.reshape(m // te, n // te, te, te).transpose(0, 2, 1, 3).reshape(m, n)
    assert np.array_equal(got, want)
    dc.free(), dcu.free()


def _vector_layouts(w):
    """Layouts whose unit-stride runs are whole 16-byte vectors on both sides: dense along the same
    direction (vector copy) and along different directions (vector transpose through LDS). Extents cross
    tile edges, rows and columns are padded, and every leading dimension leaves a gap."""
    v = 128 // w
    out = []
    # plain dense along c, blocks dense along c
    m, n, m0, n0 = 203, 21 * v, 5, 4 * v
    n1 = -(-n // n0)
    rs0, cs1 = n0 + v, m0 * (n0 + v) + v
    out.append(dict(m=m, n=n, rs=n + v, cs=1, m0=m0, n0=n0, rs0=rs0, cs0=1, cs1=cs1, rs1=n1 * cs1 + v))
    # plain dense along r, blocks dense along r
    m, n, m0, n0 = 19 * v, 150, 2 * v, 3
    m1 = -(-m // m0)
    cs0, rs1 = m0 + v, n0 * (m0 + v)
    out.append(dict(m=m, n=n, rs=1, cs=m + v, m0=m0, n0=n0, rs0=1, cs0=cs0, rs1=rs1, cs1=m1 * rs1 + v))
    # plain dense along c, blocks dense along r: the TE x 1 panel packer's shape (n0 = 1) and a 3-wide one
    for n0 in (1, 3):
        m, n, m0 = 200, 19 * v, 64
        cs0 = m0 + v
        cs1 = n0 * cs0
        n1 = -(-n // n0)
        out.append(dict(m=m, n=n, rs=n + 2 * v, cs=1, m0=m0, n0=n0, rs0=1, cs0=cs0, cs1=cs1, rs1=n1 * cs1 + v))
    # plain dense along r, blocks dense along c
    m, n, m0, n0 = 18 * v, 170, 3, 2 * v
    rs0 = n0 + v
    rs1 = m0 * rs0
    m1 = -(-m // m0)
    out.append(dict(m=m, n=n, rs=1, cs=m + v, m0=m0, n0=n0, rs0=rs0, cs0=1, rs1=rs1, cs1=m1 * rs1 + 2 * v))
    return out


@pytest.mark.parametrize("w", (8, 16, 32))
def test_vector_paths_pack_and_unpack(gpu, w):
    for i, row in enumerate(_vector_layouts(w)):
        src, dst = pack_case_buffers(row, w, 900 + i)
        tail = (row["m0"], row["n0"])
        bs = (row["rs0"], row["cs0"], row["rs1"], row["cs1"])
        want = dst.copy()
        getattr(oracle(), f"skl_pack_e{w}rc_e{w}rcprc_oracle")(row["m"], row["n"], src, row["rs"], row["cs"], *tail,
                                                                want, *bs, PAD[w] ^ 0x5A)
        got = run_inout(gpu, f"skl_pack_e{w}rc_e{w}rcprc_gfx950",
                        lambda s, d: (row["m"], row["n"], s, row["rs"], row["cs"], *tail, d, *bs, PAD[w] ^ 0x5A),
                        src, dst, "device")
        assert np.array_equal(got, want), ("pack", row)
        packed, plain = want, src.copy()
        plain[:] = np.arange(plain.size).astype(plain.dtype)
        want_u = plain.copy()
        getattr(oracle(), f"skl_unpack_e{w}rcprc_e{w}rc_oracle")(*tail, packed, *bs, row["m"], row["n"], want_u,
                                                                  row["rs"], row["cs"])
        got_u = run_inout(gpu, f"skl_unpack_e{w}rcprc_e{w}rc_gfx950",
                          lambda s, d: (*tail, s, *bs, row["m"], row["n"], d, row["rs"], row["cs"]),
                          packed, plain, "device")
        assert np.array_equal(got_u, want_u), ("unpack", row)


@pytest.mark.parametrize("mode", MODES)
def test_block4x8x4_packers(gpu, mode):
    """The four packers of the 4 x 8 / 8 x 4 / 4 x 4 block layouts (src/pack/README.md:172-178) against the checker's
    general pack / unpack with those block sizes and strides, and against numpy's reshape of the packed buffer;
    partial blocks padded, gaps between block rows untouched; pack -> unpack returns the matrix."""
    rng = np.random.default_rng(4848)
    for (m, n, gap) in ((4, 8, 0), (8, 8, 0), (7, 13, 5), (64, 96, 0), (129, 130, 32), (1, 1, 3)):
        for name, w, (m0, n0) in (("skl_pack_e8_e8p4x8", 8, (4, 8)), ("skl_pack_e8_e8p8x4", 8, (8, 4)),
                                  ("skl_pack_e32_e32p4x4", 32, (4, 4))):
            m1, n1 = -(-m // m0), -(-n // n0)
            rs, rs1 = n + 3, n1 * m0 * n0 + gap
            src = rng.integers(0, 1 << w, size=m * rs, dtype=np.uint64).astype(DT[w])
            dst = rng.integers(0, 1 << w, size=m1 * rs1, dtype=np.uint64).astype(DT[w])
            want = dst.copy()
            getattr(oracle(), f"skl_pack_e{w}rc_e{w}rcprc_oracle")(m, n, src, rs, 1, m0, n0, want, n0, 1, rs1, m0 * n0, PAD[w])
            got = run_inout(gpu, name + "_gfx950", lambda s, d: (m, n, s, rs, d, rs1, PAD[w]), src, dst, mode)
            assert np.array_equal(got, want), (name, m, n, gap)
            blocks = np.stack([got[i * rs1:i * rs1 + n1 * m0 * n0] for i in range(m1)]).reshape(m1, n1, m0, n0)
            dense = np.full((m1 * m0, n1 * n0), PAD[w], DT[w])
            dense[:m, :n] = src.reshape(m, rs)[:, :n]
            assert np.array_equal(blocks.transpose(0, 2, 1, 3).reshape(m1 * m0, n1 * n0), dense)
            if name == "skl_pack_e32_e32p4x4":
                back = rng.integers(0, 1 << 32, size=m * rs, dtype=np.uint64).astype(np.uint32)
                want_back = back.copy()
                want_back.reshape(m, rs)[:, :n] = src.reshape(m, rs)[:, :n]
                got_back = run_inout(gpu, "skl_unpack_e32p4x4_e32_gfx950", lambda s, d: (m, n, s, rs1, d, rs), got, back, mode)
                assert np.array_equal(got_back, want_back), (m, n, gap)
