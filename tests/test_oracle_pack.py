"""Pins the CPU checker's pack / unpack / transpose: the worked examples of the
reference's documentation as known answers, the closed-form index map in
numpy, round trips, and the reference's own library over the reference's test
tables (whole destination buffers compared, as test/pack/pack_e8rc_e8rcprc.c:61-88 does).
"""
import numpy as np
import pytest

import support
from support import oracle, ref

DT = {8: np.uint8, 16: np.uint16, 32: np.uint32}


def pack(lib, suffix, w, m, n, src, rs, cs, m0, n0, dst, rs0, cs0, rs1, cs1, pad):
    getattr(lib, f"skl_pack_e{w}rc_e{w}rcprc{suffix}")(m, n, src, rs, cs, m0, n0, dst, rs0, cs0, rs1, cs1, pad)


def test_doc_example_p4x1c():
    # src/pack/README.md:81-106
    src = np.arange(32, dtype=np.uint8)
    dst = np.zeros(32, np.uint8)
    pack(oracle(), "_oracle", 8, 8, 4, src, 4, 1, 4, 1, dst, 1, 0, 16, 4, 0)
    assert dst[:24].tolist() == [0, 4, 8, 12, 1, 5, 9, 13, 2, 6, 10, 14, 3, 7, 11, 15,
                                 16, 20, 24, 28, 17, 21, 25, 29]


def test_doc_example_cp1x4():
    # src/pack/README.md:109-138
    src = np.arange(32, dtype=np.uint8)
    dst = np.zeros(32, np.uint8)
    pack(oracle(), "_oracle", 8, 4, 8, src, 8, 1, 1, 4, dst, 0, 1, 4, 16, 0)
    assert dst[:24].tolist() == [0, 1, 2, 3, 8, 9, 10, 11, 16, 17, 18, 19, 24, 25, 26, 27,
                                 4, 5, 6, 7, 12, 13, 14, 15]


def test_doc_example_p2x2c():
    # src/pack/README.md:141-162
    src = np.arange(16, dtype=np.uint8)
    dst = np.zeros(16, np.uint8)
    pack(oracle(), "_oracle", 8, 4, 4, src, 4, 1, 2, 2, dst, 1, 2, 8, 4, 0)
    assert dst.tolist() == [0, 4, 1, 5, 2, 6, 3, 7, 8, 12, 9, 13, 10, 14, 11, 15]


def test_doc_example_7x6_blocks_3x4():
    # src/gemm/packed-gemm.md:34-68: rs0 = 4, cs0 = 1, rs1 = 24, cs1 = 12, zero padding
    src = (np.arange(42) + 1).astype(np.uint16)           # c_ij = 6 i + j + 1 (non-zero)
    dst = np.full(72, 999, np.uint16)
    pack(oracle(), "_oracle", 16, 7, 6, src, 6, 1, 3, 4, dst, 4, 1, 24, 12, 0)
    c = lambda i, j: 6 * i + j + 1
    blk00 = [c(0, 0), c(0, 1), c(0, 2), c(0, 3), c(1, 0), c(1, 1), c(1, 2), c(1, 3), c(2, 0), c(2, 1), c(2, 2), c(2, 3)]
    blk01 = [c(0, 4), c(0, 5), 0, 0, c(1, 4), c(1, 5), 0, 0, c(2, 4), c(2, 5), 0, 0]
    blk20 = [c(6, 0), c(6, 1), c(6, 2), c(6, 3)] + [0] * 8
    blk21 = [c(6, 4), c(6, 5), 0, 0] + [0] * 8
    assert dst[0:12].tolist() == blk00 and dst[12:24].tolist() == blk01
    assert dst[48:60].tolist() == blk20 and dst[60:72].tolist() == blk21


def numpy_pack(m, n, src, rs, cs, m0, n0, dst, rs0, cs0, rs1, cs1, pad):
    out = dst.copy()
    m1, n1 = -(-m // m0), -(-n // n0)
    offs = support.blocked_offsets(m1, n1, m0, n0, rs0, cs0, rs1, cs1)
    r, c = np.meshgrid(np.arange(m1 * m0), np.arange(n1 * n0), indexing="ij")
    inside = (r < m) & (c < n)
    vals = np.full(offs.shape, pad, dtype=dst.dtype)
    vals[inside] = src[(r * rs + c * cs)[inside]]
    out[offs.ravel()] = vals.ravel()
    return out


def pack_case_buffers(row, w, seed):
    m, n, m0, n0 = row["m"], row["n"], row["m0"], row["n0"]
    m1, n1 = -(-m // m0), -(-n // n0)
    rng = np.random.default_rng(seed)
    ns = support.span((m, n), (row["rs"], row["cs"]))
    nd = support.span((m1, n1, m0, n0), (row["rs1"], row["cs1"], row["rs0"], row["cs0"]))
    src = rng.integers(0, 1 << w, size=max(ns, 1), dtype=np.uint64).astype(DT[w])
    dst = rng.integers(0, 1 << w, size=max(nd, 1), dtype=np.uint64).astype(DT[w])
    return src, dst


PACK_ROWS = {w: support.table_rows(f"test/pack/rvv/skl_pack_e{w}rc_e{w}rcprc_zve32x.c", ("TEST", "BENCH"))
             for w in (8, 16, 32)}


@pytest.mark.parametrize("w", (8, 16, 32))
def test_pack_reference_table(w):
    pad = {8: 0xFF, 16: 0xFFFF, 32: 0xFFFFFFFF}[w]     # test/pack/pack_e8rc_e8rcprc.h:49-51
    for row in PACK_ROWS[w]:
        src, dst = pack_case_buffers(row, w, row["line"])
        args = (row["m"], row["n"], src, row["rs"], row["cs"], row["m0"], row["n0"])
        strides = (row["rs0"], row["cs0"], row["rs1"], row["cs1"], pad)
        a = dst.copy()
        pack(oracle(), "_oracle", w, *args, a, *strides)
        want = numpy_pack(row["m"], row["n"], src, row["rs"], row["cs"], row["m0"], row["n0"], dst, *strides)
        assert np.array_equal(a, want), row
        if ref() is not None:
            b = dst.copy()
            pack(ref(), "_ref", w, *args, b, *strides)
            assert np.array_equal(a, b), row


@pytest.mark.parametrize("w", (8, 16, 32))
def test_unpack_inverts_pack_and_matches_reference(w):
    for row in support.table_rows("test/pack/rvv/skl_unpack_e8rcprc_e8rc_zve32x.c", ("TEST", "BENCH")):
        src, packed = pack_case_buffers(row, w, row["line"] + 1000)
        pack(oracle(), "_oracle", w, row["m"], row["n"], src, row["rs"], row["cs"], row["m0"], row["n0"], packed,
             row["rs0"], row["cs0"], row["rs1"], row["cs1"], 0)
        poison = np.random.default_rng(1).integers(0, 1 << w, size=src.size, dtype=np.uint64).astype(DT[w])
        out = poison.copy()
        getattr(oracle(), f"skl_unpack_e{w}rcprc_e{w}rc_oracle")(
            row["m0"], row["n0"], packed, row["rs0"], row["cs0"], row["rs1"], row["cs1"], row["m"], row["n"], out,
            row["rs"], row["cs"])
        r, c = np.meshgrid(np.arange(row["m"]), np.arange(row["n"]), indexing="ij")
        addressed = (r * row["rs"] + c * row["cs"]).ravel()
        assert np.array_equal(out[addressed], src[addressed]), row
        mask = np.ones(out.size, bool)
        mask[addressed] = False
        assert np.array_equal(out[mask], poison[mask]), row      # gaps untouched
        if ref() is not None and w == 8:
            b = poison.copy()
            ref().skl_unpack_e8rcprc_e8rc_ref(row["m0"], row["n0"], packed, row["rs0"], row["cs0"], row["rs1"],
                                              row["cs1"], row["m"], row["n"], b, row["rs"], row["cs"])
            assert np.array_equal(out, b), row


def test_unpack_zero_block_is_noop():
    src = np.arange(16, dtype=np.uint8)
    out = np.full(16, 0xAA, np.uint8)
    oracle().skl_unpack_e8rcprc_e8rc_oracle(0, 4, src, 1, 1, 1, 1, 4, 4, out, 4, 1)  # ref/pack/unpack_e8rcprc_e8rc.c:16-18
    oracle().skl_unpack_e8rcprc_e8rc_oracle(4, 0, src, 1, 1, 1, 1, 4, 4, out, 4, 1)
    assert np.all(out == 0xAA)


@pytest.mark.parametrize("w", (8, 16, 32))
def test_transpose_reference_table(w):
    rows = support.table_rows(f"test/pack/rvv/skl_transpose_e{w}_zve32x.c", ("TEST", "BENCH")) + \
        support.table_rows(f"test/pack/xsfmm/skl_transpose_e{w}_xsfmmbase.c", ("TEST", "BENCH"))
    for row in rows:
        m, n = row["m"], row["n"]
        rsa, rsat = row.get("rsa") or n, row.get("rsat") or m
        rng = np.random.default_rng(row["line"])
        a = rng.integers(0, 1 << w, size=max(m * rsa, 1), dtype=np.uint64).astype(DT[w])
        at0 = rng.integers(0, 1 << w, size=max(n * rsat, 1), dtype=np.uint64).astype(DT[w])
        got = at0.copy()
        getattr(oracle(), f"skl_transpose_e{w}_oracle")(m, n, a, rsa, got, rsat)
        want = at0.copy()
        if m and n:
            want.reshape(-1)[(np.arange(n)[:, None] * rsat + np.arange(m)[None, :]).ravel()] = \
                a[(np.arange(m)[None, :] * rsa + np.arange(n)[:, None]).ravel()]
        assert np.array_equal(got, want), row
        # transpose == pack of one m x n block with strides (1, rsat): src/transpose/README.md:3-9
        if m and n:
            via_pack = at0.copy()
            pack(oracle(), "_oracle", w, m, n, a, rsa, 1, m, n, via_pack, 1, rsat, 0, 0, 0)
            assert np.array_equal(via_pack, want), row
        if ref() is not None:
            b = at0.copy()
            getattr(ref(), f"skl_transpose_e{w}_ref")(m, n, a, rsa, b, rsat)
            assert np.array_equal(got, b), row


@pytest.mark.parametrize("w", (16, 32))
def test_panel_pack_reference_table(w):
    """TE x 1 column panels = pack(m, n, src, rs, 1, TE, 1, dst, 1, 0, rs1, cs1, pad)
    (src/pack/pack_e16_xsfmmbase.h:34-43); defaults of the suite's main()."""
    te = support.TE
    for row in support.table_rows(f"test/pack/xsfmm/skl_pack_e{w}_e{w}rcptex1c_xsfmmbase.c", ("TEST", "BENCH")):
        m, n = row["m"], row["n"]
        rs = row.get("rs") or n
        cs1 = row.get("cs1") or te
        rs1 = row.get("rs1") or n * cs1
        full = dict(m=m, n=n, rs=rs, cs=1, m0=te, n0=1, rs0=1, cs0=te, rs1=rs1, cs1=cs1, line=row["line"])
        src, dst = pack_case_buffers(full, w, row["line"])
        a = dst.copy()
        pack(oracle(), "_oracle", w, m, n, src, rs, 1, te, 1, a, 1, 0, rs1, cs1, 0)
        want = numpy_pack(m, n, src, rs, 1, te, 1, dst, 1, 0, rs1, cs1, 0)
        assert np.array_equal(a, want), row
        if ref() is not None:
            b = dst.copy()
            pack(ref(), "_ref", w, m, n, src, rs, 1, te, 1, b, 1, 0, rs1, cs1, 0)
            assert np.array_equal(a, b), row
