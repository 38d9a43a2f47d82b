"""Randomised differential test of pack / unpack / transpose: random element width, shape, block sizes, layouts
(row- or column-major source, blocks stored row- or column-major, with padding and stride gaps) against the CPU
checker over the whole destination buffer (pad values, untouched gaps). The copy-speed vector kernels have
eligibility rules (16-byte runs, alignment); this test walks their borders."""
import numpy as np
import pytest

from gpu_support import run_inout
from support import oracle
from test_oracle_pack import DT

pytestmark = pytest.mark.gpu


def _layouts(rng, m, n, w):
    vec = 16 // (w // 8)  # elements per 16 bytes
    m0 = int(rng.choice([1, 2, 3, 4, 8, 16, 64, vec, 2 * vec]))
    n0 = int(rng.choice([1, 2, 3, 4, 8, 16, 64, vec, 2 * vec]))
    m1, n1 = -(-m // m0), -(-n // n0)
    pad = int(rng.choice([0, 0, 1, vec]))
    if rng.integers(2):   # blocks stored row-major
        cs0, rs0 = 1, n0 + pad
        block = m0 * rs0
    else:                 # blocks stored column-major
        rs0, cs0 = 1, m0 + pad
        block = n0 * cs0
    block += int(rng.choice([0, 0, 3, vec]))
    if rng.integers(2):
        cs1, rs1 = block, n1 * block
    else:
        rs1, cs1 = block, m1 * block
    if rng.integers(2):   # row-major plain matrix
        rs, cs = n + int(rng.choice([0, 1, vec])), 1
    else:
        rs, cs = 1, m + int(rng.choice([0, 1, vec]))
    plain_len = (m - 1) * rs + (n - 1) * cs + 1
    packed_len = (m1 - 1) * rs1 + (n1 - 1) * cs1 + (m0 - 1) * rs0 + (n0 - 1) * cs0 + 1
    return (m0, n0, rs0, cs0, rs1, cs1, rs, cs), plain_len, packed_len


@pytest.mark.parametrize("chunk", range(12))
def test_random_pack_unpack_transpose(gpu, chunk):
    rng = np.random.default_rng(7000 + chunk)
    for _ in range(40):
        w = int(rng.choice([8, 16, 32]))
        m = int(rng.choice([int(rng.integers(1, 50)), 16 * int(rng.integers(1, 12)), 64 * int(rng.integers(1, 4))]))
        n = int(rng.choice([int(rng.integers(1, 50)), 16 * int(rng.integers(1, 12)), 64 * int(rng.integers(1, 4))]))
        (m0, n0, rs0, cs0, rs1, cs1, rs, cs), plain_len, packed_len = _layouts(rng, m, n, w)
        mode = "device" if rng.integers(4) else "host"
        plain = rng.integers(0, 1 << w, size=plain_len, dtype=np.uint64).astype(DT[w])
        packed = rng.integers(0, 1 << w, size=packed_len, dtype=np.uint64).astype(DT[w])
        padv = int(rng.integers(0, 1 << w))
        what = (w, m, n, m0, n0, rs0, cs0, rs1, cs1, rs, cs, mode)
        # pack
        want = packed.copy()
        getattr(oracle(), f"skl_pack_e{w}rc_e{w}rcprc_oracle")(m, n, plain, rs, cs, m0, n0, want, rs0, cs0, rs1, cs1, padv)
        got = run_inout(gpu, f"skl_pack_e{w}rc_e{w}rcprc_gfx950",
                        lambda s, d: (m, n, s, rs, cs, m0, n0, d, rs0, cs0, rs1, cs1, padv), plain, packed, mode)
        assert np.array_equal(got, want), ("pack",) + what
        # unpack of what was packed gives the matrix back; gaps of the destination stay
        back = rng.integers(0, 1 << w, size=plain_len, dtype=np.uint64).astype(DT[w])
        want_back = back.copy()
        getattr(oracle(), f"skl_unpack_e{w}rcprc_e{w}rc_oracle")(m0, n0, want, rs0, cs0, rs1, cs1, m, n, want_back, rs, cs)
        got_back = run_inout(gpu, f"skl_unpack_e{w}rcprc_e{w}rc_gfx950",
                             lambda s, d: (m0, n0, s, rs0, cs0, rs1, cs1, m, n, d, rs, cs), want, back, mode)
        assert np.array_equal(got_back, want_back), ("unpack",) + what
        # transpose (both row-major, padded)
        rsa, rsat = n + int(rng.choice([0, 1, 16])), m + int(rng.choice([0, 1, 16]))
        a = rng.integers(0, 1 << w, size=m * rsa, dtype=np.uint64).astype(DT[w])
        at = rng.integers(0, 1 << w, size=n * rsat, dtype=np.uint64).astype(DT[w])
        want_t = at.copy()
        getattr(oracle(), f"skl_transpose_e{w}_oracle")(m, n, a, rsa, want_t, rsat)
        got_t = run_inout(gpu, f"skl_transpose_e{w}_gfx950", lambda s, d: (m, n, s, rsa, d, rsat), a, at, mode)
        assert np.array_equal(got_t, want_t), ("transpose", w, m, n, rsa, rsat, mode)
