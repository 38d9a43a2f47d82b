// skl_pack.hip - pack / unpack (and, as special cases, transpose and the TE x 1
// panel packers) for 8-, 16- and 32-bit elements on gfx950.
//
// Semantics: ref/pack/pack_e8rc_e8rcprc.c:10-35 (pack: blocked copy with
// padding, gaps untouched) and ref/pack/unpack_e8rcprc_e8rc.c:10-37 (unpack:
// inverse gather, only in-range elements written). The plain matrix is
// addressed r*rs + c*cs; the blocked one (r/m0)*rs1 + (r%m0)*rs0 + (c/n0)*cs1 +
// (c%n0)*cs0 - both separable into a row term plus a column term. A workgroup
// moves one 64x64 tile: the two terms are tabulated once per tile (one integer
// division per row/column instead of per element), the tile is read with lanes
// running along the source's denser direction, staged in LDS, and written with
// lanes running along the destination's denser direction, so that both sides
// are coalesced even when the copy transposes.
#include <hip/hip_runtime.h>

#include "skl_device.hpp"

namespace {

constexpr int kTile = 64;
constexpr int kThreads = 256;

struct PackArgs {
  size_t m, n;      // extent of the plain matrix
  size_t rows, cols;  // extent of the iteration space (padded for pack, m x n for unpack)
  size_t rs, cs;    // plain strides
  size_t m0, n0, rs0, cs0, rs1, cs1;  // blocked layout
  unsigned pad;
  unsigned tiles_x;  // tiles per tile-row (the grid is one-dimensional)
  int plain_along_c;    // lanes run along columns when touching the plain matrix
  int blocked_along_c;  // lanes run along columns when touching the blocked matrix
};

template <typename T, bool PACK>
__global__ void __launch_bounds__(kThreads) pack_tile_kernel(const T *__restrict__ src, T *__restrict__ dst, PackArgs p) {
  __shared__ T tile[kTile][kTile + (sizeof(T) == 4 ? 1 : sizeof(T) == 2 ? 2 : 4)];
  __shared__ size_t plain_r[kTile], plain_c[kTile], blk_r[kTile], blk_c[kTile];

  const size_t r0 = (size_t)(blockIdx.x / p.tiles_x) * kTile, c0 = (size_t)(blockIdx.x % p.tiles_x) * kTile;
  const int t = threadIdx.x;
  if (t < kTile) {
    const size_t r = r0 + t;
    plain_r[t] = r * p.rs;
    blk_r[t] = (r / p.m0) * p.rs1 + (r % p.m0) * p.rs0;
  } else if (t < 2 * kTile) {
    const size_t c = c0 + (t - kTile);
    plain_c[t - kTile] = c * p.cs;
    blk_c[t - kTile] = (c / p.n0) * p.cs1 + (c % p.n0) * p.cs0;
  }
  __syncthreads();

  const int lane64 = t & 63, grp = t >> 6;  // 4 groups of 64 lanes
  const bool src_along_c = PACK ? p.plain_along_c : p.blocked_along_c;
  const bool dst_along_c = PACK ? p.blocked_along_c : p.plain_along_c;

#pragma unroll 4
  for (int i = 0; i < kTile / 4; ++i) {
    const int tr = src_along_c ? grp + 4 * i : lane64;
    const int tc = src_along_c ? lane64 : grp + 4 * i;
    const size_t r = r0 + tr, c = c0 + tc;
    if (r < p.rows && c < p.cols) {
      T v;
      if (PACK) {
        v = (r < p.m && c < p.n) ? src[plain_r[tr] + plain_c[tc]] : (T)p.pad;
      } else {
        v = src[blk_r[tr] + blk_c[tc]];
      }
      tile[tr][tc] = v;
    }
  }
  __syncthreads();
#pragma unroll 4
  for (int i = 0; i < kTile / 4; ++i) {
    const int tr = dst_along_c ? grp + 4 * i : lane64;
    const int tc = dst_along_c ? lane64 : grp + 4 * i;
    const size_t r = r0 + tr, c = c0 + tc;
    if (r < p.rows && c < p.cols) {
      if (PACK)
        dst[blk_r[tr] + blk_c[tc]] = tile[tr][tc];
      else
        dst[plain_r[tr] + plain_c[tc]] = tile[tr][tc];
    }
  }
}

template <typename T>
int launch(bool pack, const void *src, void *dst, PackArgs p) {
  if (p.rows == 0 || p.cols == 0) return 0;
  const size_t gx = (p.cols + kTile - 1) / kTile, gy = (p.rows + kTile - 1) / kTile;
  if (gx * gy > 0x7FFFFFFFu) {
    skl_hip_record_error(-2, "pack: matrix too large for one launch");
    return -2;
  }
  p.tiles_x = (unsigned)gx;
  const unsigned grid = (unsigned)(gx * gy);
  if (pack)
    pack_tile_kernel<T, true><<<grid, kThreads, 0, skl_current_stream()>>>((const T *)src, (T *)dst, p);
  else
    pack_tile_kernel<T, false><<<grid, kThreads, 0, skl_current_stream()>>>((const T *)src, (T *)dst, p);
  return skl_check_launch(pack ? "pack" : "unpack");
}

int dispatch(int esize, bool pack, const void *src, void *dst, const PackArgs &p) {
  switch (esize) {
    case 1: return launch<uint8_t>(pack, src, dst, p);
    case 2: return launch<uint16_t>(pack, src, dst, p);
    case 4: return launch<uint32_t>(pack, src, dst, p);
    default:
      skl_hip_record_error(-2, "pack: element size");
      return -2;
  }
}

}  // namespace

extern "C" {

int skl_hip_launch_pack(int esize, size_t m, size_t n, const void *src, size_t rs, size_t cs, size_t m0, size_t n0,
                        void *dst, size_t rs0, size_t cs0, size_t rs1, size_t cs1, uint32_t pad) {
  if (m == 0 || n == 0 || m0 == 0 || n0 == 0) return 0;
  PackArgs p;
  p.m = m;
  p.n = n;
  p.rows = (m + m0 - 1) / m0 * m0;
  p.cols = (n + n0 - 1) / n0 * n0;
  p.rs = rs;
  p.cs = cs;
  p.m0 = m0;
  p.n0 = n0;
  p.rs0 = rs0;
  p.cs0 = cs0;
  p.rs1 = rs1;
  p.cs1 = cs1;
  p.pad = pad;
  p.plain_along_c = cs <= rs;
  // Within a block the denser direction decides; a 1-wide block dimension has no stride of its own.
  const size_t eff_rs0 = m0 > 1 ? rs0 : rs1, eff_cs0 = n0 > 1 ? cs0 : cs1;
  p.blocked_along_c = eff_cs0 <= eff_rs0;
  return dispatch(esize, true, src, dst, p);
}

int skl_hip_launch_unpack(int esize, size_t m0, size_t n0, const void *src, size_t rs0, size_t cs0, size_t rs1,
                          size_t cs1, size_t m, size_t n, void *dst, size_t rs, size_t cs) {
  if (m == 0 || n == 0 || m0 == 0 || n0 == 0) return 0;
  PackArgs p;
  p.m = m;
  p.n = n;
  p.rows = m;
  p.cols = n;
  p.rs = rs;
  p.cs = cs;
  p.m0 = m0;
  p.n0 = n0;
  p.rs0 = rs0;
  p.cs0 = cs0;
  p.rs1 = rs1;
  p.cs1 = cs1;
  p.pad = 0;
  p.plain_along_c = cs <= rs;
  const size_t eff_rs0 = m0 > 1 ? rs0 : rs1, eff_cs0 = n0 > 1 ? cs0 : cs1;
  p.blocked_along_c = eff_cs0 <= eff_rs0;
  return dispatch(esize, false, src, dst, p);
}

}  // extern "C"
