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

#include <cstdlib>

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

// Blocked source of a realigning copy: element (x, p) at (x/x0)*s1 + (x%x0)*s0 + (p/k0)*sk1 + (p%k0)*sk0.
struct RealignSource {
  size_t x0, s0, s1, k0, sk0, sk1;
};

template <typename T>
__global__ void __launch_bounds__(kThreads) realign_kernel(const T *__restrict__ src, T *__restrict__ dst, size_t x, size_t k,
                                                           size_t kp, RealignSource f, unsigned tiles_p, int along_x) {
  __shared__ T tile[kTile][kTile + 3];  // [p][x]
  const size_t x_base = (size_t)(blockIdx.x / tiles_p) * kTile, p_base = (size_t)(blockIdx.x % tiles_p) * kTile;
  const int fast = threadIdx.x % kTile, slow = threadIdx.x / kTile;
  for (int it = slow; it < kTile; it += kThreads / kTile) {
    const int xi = along_x ? fast : it, pi = along_x ? it : fast;
    const size_t xx = x_base + xi, pp = p_base + pi;
    tile[pi][xi] = (xx < x && pp < k)
                       ? src[(xx / f.x0) * f.s1 + (xx % f.x0) * f.s0 + (pp / f.k0) * f.sk1 + (pp % f.k0) * f.sk0]
                       : T(0);
  }
  __syncthreads();
  for (int it = slow; it < kTile; it += kThreads / kTile) {
    const size_t xx = x_base + it, pp = p_base + fast;
    if (xx < x && pp < kp) dst[xx * kp + pp] = tile[fast][it];
  }
}

// The two common sources of a realigning copy, with 16-byte stores on the aligned side. Flat K (k0 == 1).
//
// Source rows contiguous in K: one thread per 16-byte piece of a destination row, fetched with the widest loads
// the source's alignment allows (VEC bytes: 16, 4, or one element).
template <int ES, int VEC>
__global__ void __launch_bounds__(kThreads) realign_rows_kernel(const char *__restrict__ src, char *__restrict__ dst, size_t x,
                                                                size_t kbytes, size_t pitch, RealignSource f) {
  const size_t pieces_per_row = pitch / 16;
  const size_t idx = (size_t)blockIdx.x * kThreads + threadIdx.x;
  if (idx >= x * pieces_per_row) return;
  const size_t xx = idx / pieces_per_row, off = (idx % pieces_per_row) * 16;
  const char *row = src + ((xx / f.x0) * f.s1 + (xx % f.x0) * f.s0) * ES;
  uint4 v = make_uint4(0, 0, 0, 0);
  if (off + 16 <= kbytes) {
    if constexpr (VEC == 16) {
      v = *reinterpret_cast<const uint4 *>(row + off);
    } else if constexpr (VEC == 4) {
      const unsigned *w = reinterpret_cast<const unsigned *>(row + off);
      v = make_uint4(w[0], w[1], w[2], w[3]);
    } else {
      unsigned char b[16];
#pragma unroll
      for (int i = 0; i < 16; i += ES) {
        if constexpr (ES == 1) b[i] = (unsigned char)row[off + i];
        else *reinterpret_cast<uint16_t *>(b + i) = *reinterpret_cast<const uint16_t *>(row + off + i);
      }
      v = *reinterpret_cast<const uint4 *>(b);
    }
  } else if (off < kbytes) {  // the piece that holds the end of K: element by element, zero beyond
    unsigned char b[16] = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    for (size_t i = 0; off + i < kbytes; ++i) b[i] = (unsigned char)row[off + i];
    v = *reinterpret_cast<const uint4 *>(b);
  }
  *reinterpret_cast<uint4 *>(dst + xx * pitch + off) = v;
}

// Source blocked along K with the block's k contiguous in runs of a whole number of 8-byte pieces (the 4 x 8 blocks
// of src/gemm/packed-gemm.md:270-298: four rows of eight k in 32 bytes): one thread per 16-byte piece of a destination
// row, gathered from 8-byte pieces of the source. The rows of one block of x0 rows are neighbouring threads, so a
// wave reads whole lines of the source and writes 16-byte pieces that the next lanes continue.
template <int ES>
__global__ void __launch_bounds__(kThreads) realign_kruns_kernel(const char *__restrict__ src, char *__restrict__ dst, size_t x,
                                                                 size_t kbytes, size_t pitch, RealignSource f, size_t lanes_x) {
  const size_t pieces_per_row = pitch / 16;
  const size_t idx = (size_t)blockIdx.x * kThreads + threadIdx.x;
  // lanes_x rows (a power of two dividing x0, at most 64) x pieces, rows fastest
  const size_t in_group = idx % lanes_x, rest = idx / lanes_x;
  const size_t piece = rest % pieces_per_row, xx = (rest / pieces_per_row) * lanes_x + in_group;
  if (xx >= x) return;
  const char *row = src + ((xx / f.x0) * f.s1 + (xx % f.x0) * f.s0) * ES;
  uint2 half[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const size_t off = piece * 16 + 8 * h, p = off / ES;
    half[h] = off < kbytes ? *reinterpret_cast<const uint2 *>(row + ((p / f.k0) * f.sk1 + (p % f.k0)) * ES) : make_uint2(0, 0);
  }
  *reinterpret_cast<uint4 *>(dst + xx * pitch + piece * 16) = make_uint4(half[0].x, half[0].y, half[1].x, half[1].y);
}

// 8-bit source in blocks of k0 k-rows of four contiguous x (the 8 x 4 blocks of src/gemm/packed-gemm.md:270-298):
// a thread takes eight k-rows of one block - 32 contiguous bytes -, turns them into eight k-bytes for each of the
// four x (byte permutes) and stores them to the four destination rows. Four neighbouring blocks along x and 64
// k-groups per workgroup: a wave reads 128 contiguous bytes per k-group when the blocks lie side by side and writes
// 128 contiguous bytes per destination row.
__global__ void __launch_bounds__(kThreads) realign_x4_kernel(const char *__restrict__ src, char *__restrict__ dst, size_t x,
                                                              size_t k, size_t pitch, RealignSource f, unsigned tiles_p) {
  const size_t xb = (size_t)(blockIdx.x / tiles_p) * 4 + (threadIdx.x & 3);   // block of four x
  const size_t kg = (size_t)(blockIdx.x % tiles_p) * 64 + (threadIdx.x >> 2);  // group of eight k
  if (xb * 4 >= x || kg * 8 >= pitch) return;
  unsigned v[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  if (kg * 8 < k) {
    const size_t p = kg * 8;
    const uint4 *from = reinterpret_cast<const uint4 *>(src + xb * f.s1 + (p / f.k0) * f.sk1 + (p % f.k0) * 4);
    const uint4 lo = from[0], hi = from[1];
    v[0] = lo.x, v[1] = lo.y, v[2] = lo.z, v[3] = lo.w, v[4] = hi.x, v[5] = hi.y, v[6] = hi.z, v[7] = hi.w;
  }
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const unsigned pick = 0x0C0C0000u | ((4u + c) << 8) | (unsigned)c;   // byte c of the low, then of the high operand
    const unsigned k01 = __builtin_amdgcn_perm(v[1], v[0], pick), k23 = __builtin_amdgcn_perm(v[3], v[2], pick);
    const unsigned k45 = __builtin_amdgcn_perm(v[5], v[4], pick), k67 = __builtin_amdgcn_perm(v[7], v[6], pick);
    *reinterpret_cast<uint2 *>(dst + (xb * 4 + c) * pitch + kg * 8) =
        make_uint2(__builtin_amdgcn_perm(k23, k01, 0x05040100u), __builtin_amdgcn_perm(k67, k45, 0x05040100u));
  }
}

// Any other source (contiguous along x, blocked in K, no unit stride at all): a 64 x 64 tile is read with lanes
// along the source's denser direction, kept in LDS with K contiguous (row pitch 64 elements + 4 bytes: lanes along
// x hit distinct banks), and written as 16-byte pieces of the destination rows.
// VECX > 1: the source is contiguous along x in runs that 4-byte loads can take (lanes along x, VECX elements each).
template <typename T, int VECX>
__global__ void __launch_bounds__(kThreads) realign_tile_kernel(const T *__restrict__ src, char *__restrict__ dst, size_t x,
                                                                size_t k, size_t pitch, RealignSource f, unsigned tiles_p,
                                                                int along_x) {
  constexpr int kRowBytes = kTile * (int)sizeof(T), kLdsPitch = kRowBytes + 4;
  __shared__ __attribute__((aligned(16))) char tile[kTile * kLdsPitch];
  const size_t x_base = (size_t)(blockIdx.x / tiles_p) * kTile, p_base = (size_t)(blockIdx.x % tiles_p) * kTile;
  auto at = [&](size_t xx, size_t pp) {
    return (xx / f.x0) * f.s1 + (xx % f.x0) * f.s0 + (pp / f.k0) * f.sk1 + (pp % f.k0) * f.sk0;
  };
  if constexpr (VECX > 1) {
    constexpr int kLanesX = kTile / VECX, kRowsPerPass = kThreads / kLanesX;
    const int xi = (threadIdx.x % kLanesX) * VECX, pr = threadIdx.x / kLanesX;
#pragma unroll
    for (int pi = pr; pi < kTile; pi += kRowsPerPass) {
      const size_t xx = x_base + xi, pp = p_base + pi;
      T v[VECX];
      if (xx + VECX <= x && pp < k) {
        const unsigned w = *reinterpret_cast<const unsigned *>(src + at(xx, pp));
#pragma unroll
        for (int e = 0; e < VECX; ++e) v[e] = (T)(w >> (8 * sizeof(T) * e));
      } else {
#pragma unroll
        for (int e = 0; e < VECX; ++e) v[e] = (xx + e < x && pp < k) ? src[at(xx + e, pp)] : T(0);
      }
#pragma unroll
      for (int e = 0; e < VECX; ++e) *reinterpret_cast<T *>(tile + (xi + e) * kLdsPitch + pi * (int)sizeof(T)) = v[e];
    }
  } else {
    const int fast = threadIdx.x % kTile, slow = threadIdx.x / kTile;
#pragma unroll 4
    for (int it = slow; it < kTile; it += kThreads / kTile) {
      const int xi = along_x ? fast : it, pi = along_x ? it : fast;
      const size_t xx = x_base + xi, pp = p_base + pi;
      const T v = (xx < x && pp < k) ? src[at(xx, pp)] : T(0);
      *reinterpret_cast<T *>(tile + xi * kLdsPitch + pi * (int)sizeof(T)) = v;
    }
  }
  __syncthreads();
  constexpr int kPiecesPerRow = kRowBytes / 16, kPieces = kTile * kPiecesPerRow;
#pragma unroll
  for (int piece = threadIdx.x; piece < kPieces; piece += kThreads) {
    const int xi = piece / kPiecesPerRow, off = (piece % kPiecesPerRow) * 16;
    const size_t xx = x_base + xi, byte = p_base * sizeof(T) + off;
    if (xx >= x || byte >= pitch) continue;  // the pitch is a whole number of 16-byte pieces
    const unsigned *w = reinterpret_cast<const unsigned *>(tile + xi * kLdsPitch + off);
    *reinterpret_cast<uint4 *>(dst + xx * pitch + byte) = make_uint4(w[0], w[1], w[2], w[3]);
  }
}

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

// ---- 16-byte vector variants -------------------------------------------------------------------
// When each side has a unit-stride direction whose runs are whole 16-byte vectors, a lane moves a
// vector instead of an element. If both sides are dense along the same direction the tile is a
// straight vector copy with table-driven addresses; if they are dense along different directions
// (the TE x 1 panel packer of a row-major matrix, transposes) the tile goes through LDS: written
// as vectors along the source's direction, gathered element by element into vectors along the
// destination's. The 16-byte chunks of an LDS line are XOR-swizzled by (line / V) so that the
// gather (lanes V lines apart) and the vector writes are both free of bank conflicts.
typedef int v4i __attribute__((ext_vector_type(4)));

// Development switch: SKL_PACK_ELEMENTWISE=1 forces the element kernel.
bool skl_pack_vectorise() {
  static const bool on = [] {
    const char *e = getenv("SKL_PACK_ELEMENTWISE");
    return !(e && e[0] == '1');
  }();
  return on;
}

template <int ES>
struct VecShape {
  static constexpr int V = 16 / ES;            // elements per vector
  static constexpr int T = ES == 1 ? 128 : 64;  // tile edge in elements
  static constexpr int NV = T / V;              // vectors per tile line
};

template <int ES> struct ElemOf;
template <> struct ElemOf<1> { typedef uint8_t type; };
template <> struct ElemOf<2> { typedef uint16_t type; };
template <> struct ElemOf<4> { typedef uint32_t type; };

template <int ES, bool PACK, bool TRANSPOSE>
__global__ void __launch_bounds__(kThreads) pack_vec_kernel(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst,
                                                            PackArgs p) {
  typedef typename ElemOf<ES>::type E;
  constexpr int V = VecShape<ES>::V, T = VecShape<ES>::T, NV = VecShape<ES>::NV;
  constexpr int kIters = T * NV / kThreads;
  __shared__ size_t plain_r[T], plain_c[T], blk_r[T], blk_c[T];
  __shared__ v4i stage[TRANSPOSE ? T * NV : 1];

  const size_t r0 = (size_t)(blockIdx.x / p.tiles_x) * T, c0 = (size_t)(blockIdx.x % p.tiles_x) * T;
  const int t = threadIdx.x;
  for (int i = t; i < 2 * T; i += kThreads) {
    if (i < T) {
      const size_t r = r0 + i;
      plain_r[i] = r * p.rs;
      blk_r[i] = (r / p.m0) * p.rs1 + (r % p.m0) * p.rs0;
    } else {
      const size_t c = c0 + (i - T);
      plain_c[i - T] = c * p.cs;
      blk_c[i - T] = (c / p.n0) * p.cs1 + (c % p.n0) * p.cs0;
    }
  }
  __syncthreads();

  const bool in_along_c = PACK ? p.plain_along_c : p.blocked_along_c;
  v4i padv;
  {
    unsigned w = p.pad;
    if (ES == 1) w = (w & 0xFF) * 0x01010101u;
    if (ES == 2) w = (w & 0xFFFF) * 0x00010001u;
    padv = (v4i)((int)w);
  }

#pragma unroll
  for (int it = 0; it < kIters; ++it) {
    const int idx = it * kThreads + t;
    const int wv = idx % NV, u = idx / NV;  // vector within the line, line
    const int tr = in_along_c ? u : wv * V, tc = in_along_c ? wv * V : u;
    const size_t r = r0 + tr, c = c0 + tc;
    if (r < p.rows && c < p.cols) {
      v4i v;
      if (PACK)
        v = (r < p.m && c < p.n) ? *(const v4i *)(src + (plain_r[tr] + plain_c[tc]) * ES) : padv;
      else
        v = *(const v4i *)(src + (blk_r[tr] + blk_c[tc]) * ES);
      if (TRANSPOSE)
        stage[u * NV + (wv ^ ((u / V) & (NV - 1)))] = v;
      else
        *(v4i *)(dst + (PACK ? blk_r[tr] + blk_c[tc] : plain_r[tr] + plain_c[tc]) * ES) = v;
    }
  }
  if (!TRANSPOSE) return;
  __syncthreads();

  const uint8_t *bytes = (const uint8_t *)stage;
#pragma unroll
  for (int it = 0; it < kIters; ++it) {
    const int idx = it * kThreads + t;
    const int uv = idx % NV, w = idx / NV;  // vector of V source lines, position along the source's direction
    const int tr = in_along_c ? uv * V : w, tc = in_along_c ? w : uv * V;
    const size_t r = r0 + tr, c = c0 + tc;
    if (r < p.rows && c < p.cols) {
      const int chunk = (w * ES) >> 4, within = (w * ES) & 15;
      const uint8_t *col = bytes + (size_t)(((uv * V) * NV + (chunk ^ uv)) * 16 + within);
      E e[V];
#pragma unroll
      for (int i = 0; i < V; ++i) e[i] = *(const E *)(col + i * NV * 16);
      v4i v;
      __builtin_memcpy(&v, e, 16);
      *(v4i *)(dst + (PACK ? blk_r[tr] + blk_c[tc] : plain_r[tr] + plain_c[tc]) * ES) = v;
    }
  }
}

// 0: element kernel; 1: vector copy; 2: vector transpose. Sets the lane directions for the vector kernels.
int vector_plan(int es, bool pack, const void *src, const void *dst, PackArgs &p) {
  const size_t V = 16 / es;
  if ((((uintptr_t)src | (uintptr_t)dst) & 15) != 0) return 0;
  const bool use_rs0 = p.m0 > 1, use_cs0 = p.n0 > 1, use_rs1 = p.rows > p.m0, use_cs1 = p.cols > p.n0;
  auto mult = [&](bool used, size_t s) { return !used || s % V == 0; };
  const bool plain_c = p.cs == 1 && p.n % V == 0 && (p.m == 1 || p.rs % V == 0);
  const bool plain_r = p.rs == 1 && p.m % V == 0 && (p.n == 1 || p.cs % V == 0);
  const bool blk_c = use_cs0 && p.cs0 == 1 && p.n0 % V == 0 && mult(use_rs0, p.rs0) && mult(use_rs1, p.rs1) &&
                     mult(use_cs1, p.cs1);
  const bool blk_r = use_rs0 && p.rs0 == 1 && p.m0 % V == 0 && mult(use_cs0, p.cs0) && mult(use_rs1, p.rs1) &&
                     mult(use_cs1, p.cs1);
  if (plain_c && blk_c) { p.plain_along_c = 1; p.blocked_along_c = 1; return 1; }
  if (plain_r && blk_r) { p.plain_along_c = 0; p.blocked_along_c = 0; return 1; }
  // Unpack reads only in-range elements (the caller's last block may be cut short), so the source
  // vectors of a transposing unpack - V rows (columns) of a block - must lie inside m (n) as well.
  if (plain_c && blk_r && (pack || p.m % V == 0)) { p.plain_along_c = 1; p.blocked_along_c = 0; return 2; }
  if (plain_r && blk_c && (pack || p.n % V == 0)) { p.plain_along_c = 0; p.blocked_along_c = 1; return 2; }
  return 0;
}

template <int ES>
int launch_vec(bool pack, bool transpose, const void *src, void *dst, PackArgs p) {
  constexpr int T = VecShape<ES>::T;
  const size_t gx = (p.cols + T - 1) / T, gy = (p.rows + T - 1) / T;
  if (gx * gy > 0x7FFFFFFFu) {
    skl_hip_record_error(-2, "pack: matrix too large for one launch");
    return -2;
  }
  p.tiles_x = (unsigned)gx;
  const unsigned grid = (unsigned)(gx * gy);
  hipStream_t st = skl_current_stream();
  const uint8_t *s = (const uint8_t *)src;
  uint8_t *d = (uint8_t *)dst;
  if (pack && transpose) pack_vec_kernel<ES, true, true><<<grid, kThreads, 0, st>>>(s, d, p);
  else if (pack) pack_vec_kernel<ES, true, false><<<grid, kThreads, 0, st>>>(s, d, p);
  else if (transpose) pack_vec_kernel<ES, false, true><<<grid, kThreads, 0, st>>>(s, d, p);
  else pack_vec_kernel<ES, false, false><<<grid, kThreads, 0, st>>>(s, d, p);
  return skl_check_launch(pack ? "pack" : "unpack");
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

int dispatch(int esize, bool pack, const void *src, void *dst, PackArgs p) {
  if (p.rows == 0 || p.cols == 0) return 0;
  if (esize == 1 || esize == 2 || esize == 4) {
    const int plan = skl_pack_vectorise() ? vector_plan(esize, pack, src, dst, p) : 0;
    if (plan) {
      switch (esize) {
        case 1: return launch_vec<1>(pack, plan == 2, src, dst, p);
        case 2: return launch_vec<2>(pack, plan == 2, src, dst, p);
        default: return launch_vec<4>(pack, plan == 2, src, dst, p);
      }
    }
  }
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

// A GEMM operand in the reference's blocked description - element (x, p), x along M or N and p along K, at
// (x/x0)*s1 + (x%x0)*s0 + (p/k0)*sk1 + (p%k0)*sk0 - copied into rows contiguous in K: dst[x*kp + p], zero for
// k <= p < kp. 64 x 64 tiles through LDS, read with lanes along x when the source is contiguous there and along p
// otherwise, written along p.
int skl_hip_launch_realign(int esize, size_t x, size_t k, const void *src, size_t x0, size_t s0, size_t s1, size_t k0,
                           size_t sk0, size_t sk1, void *dst, size_t kp) {
  if (x == 0 || kp == 0) return 0;
  const size_t tiles_p = (kp + kTile - 1) / kTile, tiles = ((x + kTile - 1) / kTile) * tiles_p;
  if (tiles > 0x7FFFFFFFu || (esize != 1 && esize != 2) || x0 == 0 || k0 == 0) {
    skl_hip_record_error(-2, "realign: bad problem");
    return -2;
  }
  const RealignSource f = {x0, s0, s1, k0, sk0, sk1};
  const size_t step_x = x0 > 1 ? s0 : s1, step_p = k0 > 1 ? sk0 : sk1;
  const int along_x = step_x == 1 && step_p != 1;
  hipStream_t st = skl_current_stream();
  const size_t es = (size_t)esize, pitch = kp * es;
  if (k0 == 1 && pitch % 16 == 0 && ((uintptr_t)dst & 15) == 0) {
    if (sk1 == 1) {  // rows contiguous in K
      const size_t blocks = (x * (pitch / 16) + kThreads - 1) / kThreads;
      if (blocks <= 0x7FFFFFFFu) {
        const uintptr_t align = (uintptr_t)src | (x0 > 1 ? s0 * es : 0) | (s1 * es);
        const char *s8 = (const char *)src;
        char *d8 = (char *)dst;
        const unsigned grid = (unsigned)blocks;
        if (esize == 1) {
          if (align % 16 == 0) realign_rows_kernel<1, 16><<<grid, kThreads, 0, st>>>(s8, d8, x, k * es, pitch, f);
          else if (align % 4 == 0) realign_rows_kernel<1, 4><<<grid, kThreads, 0, st>>>(s8, d8, x, k * es, pitch, f);
          else realign_rows_kernel<1, 1><<<grid, kThreads, 0, st>>>(s8, d8, x, k * es, pitch, f);
        } else {
          if (align % 16 == 0) realign_rows_kernel<2, 16><<<grid, kThreads, 0, st>>>(s8, d8, x, k * es, pitch, f);
          else if (align % 4 == 0) realign_rows_kernel<2, 4><<<grid, kThreads, 0, st>>>(s8, d8, x, k * es, pitch, f);
          else realign_rows_kernel<2, 2><<<grid, kThreads, 0, st>>>(s8, d8, x, k * es, pitch, f);
        }
        return skl_check_launch("realign_rows");
      }
    }
  }
  if (esize == 1 && x0 == 1 && s1 == 4 && k0 == 4 && sk0 == 1 && sk1 % 16 == 0 && k % 16 == 0 && kp == k && x % 4 == 0 &&
      (((uintptr_t)src | (uintptr_t)dst) & 15) == 0) {
    // K in groups of four bytes per x, the groups of neighbouring x side by side (the K-packed B of the dot-product
    // GEMM, src/gemm/packed-gemm.md:178-219): as 32-bit elements that is a (k / 4) x x matrix with unit column
    // stride, and the copy is its transpose - the vectorised transposing pack kernel with one block of k / 4 rows.
    return skl_hip_launch_pack(4, k / 4, x, src, sk1 / 4, 1, k / 4, 1, dst, 1, 0, 0, kp / 4, 0);
  }
  if (k0 > 1 && sk0 == 1 && (k0 * es) % 8 == 0 && pitch % 16 == 0 && ((uintptr_t)dst & 15) == 0 && k % k0 == 0 &&
      (((uintptr_t)src | (x0 > 1 ? s0 * es : 0) | (s1 * es) | (sk1 * es)) & 7) == 0) {
    // K in blocks whose k are contiguous: 8-byte pieces
    size_t lanes_x = 1;
    while (lanes_x < 64 && x0 % (lanes_x * 2) == 0) lanes_x *= 2;
    const size_t groups = (x + lanes_x - 1) / lanes_x, blocks = (groups * lanes_x * (pitch / 16) + kThreads - 1) / kThreads;
    if (blocks <= 0x7FFFFFFFu) {
      if (esize == 1) realign_kruns_kernel<1><<<(unsigned)blocks, kThreads, 0, st>>>((const char *)src, (char *)dst, x, k * es, pitch, f, lanes_x);
      else realign_kruns_kernel<2><<<(unsigned)blocks, kThreads, 0, st>>>((const char *)src, (char *)dst, x, k * es, pitch, f, lanes_x);
      return skl_check_launch("realign_kruns");
    }
  }
  if (esize == 1 && x0 == 4 && s0 == 1 && sk0 == 4 && k0 % 8 == 0 && k % k0 == 0 && x % 4 == 0 && pitch % 8 == 0 &&
      ((uintptr_t)dst & 7) == 0 && (((uintptr_t)src | s1 | sk1) & 15) == 0) {
    // blocks of k0 k-rows of four contiguous x
    const size_t tp = (pitch / 8 + 63) / 64, blocks = ((x / 4 + 3) / 4) * tp;
    if (blocks <= 0x7FFFFFFFu) {
      realign_x4_kernel<<<(unsigned)blocks, kThreads, 0, st>>>((const char *)src, (char *)dst, x, k, pitch, f, (unsigned)tp);
      return skl_check_launch("realign_x4");
    }
  }
  if (pitch % 16 == 0 && ((uintptr_t)dst & 15) == 0) {
    // lanes along K when that is the source's denser direction (a unit or the smaller step), else along x
    const int lanes_along_x = step_x < step_p;
    // 4-byte loads along x: unit stride there in runs of a multiple of 4 bytes, everything else 4-byte aligned
    const size_t run = x0 > 1 ? x0 : (size_t)1 << 20;  // x0 == 1 with s1 == 1 is one long run
    const size_t other = ((uintptr_t)src) | (x0 > 1 ? s1 * es : 0) | (k0 > 1 ? sk0 * es : 0) | (sk1 * es);
    const bool wide = lanes_along_x && step_x == 1 && (run * es) % 4 == 0 && other % 4 == 0;
    const unsigned grid = (unsigned)tiles, tp = (unsigned)tiles_p;
    if (esize == 1) {
      if (wide) realign_tile_kernel<uint8_t, 4><<<grid, kThreads, 0, st>>>((const uint8_t *)src, (char *)dst, x, k, pitch, f, tp, 1);
      else realign_tile_kernel<uint8_t, 1><<<grid, kThreads, 0, st>>>((const uint8_t *)src, (char *)dst, x, k, pitch, f, tp, lanes_along_x);
    } else {
      if (wide) realign_tile_kernel<uint16_t, 2><<<grid, kThreads, 0, st>>>((const uint16_t *)src, (char *)dst, x, k, pitch, f, tp, 1);
      else realign_tile_kernel<uint16_t, 1><<<grid, kThreads, 0, st>>>((const uint16_t *)src, (char *)dst, x, k, pitch, f, tp, lanes_along_x);
    }
    return skl_check_launch("realign_tile");
  }
  if (esize == 1)
    realign_kernel<uint8_t><<<(unsigned)tiles, kThreads, 0, st>>>((const uint8_t *)src, (uint8_t *)dst, x, k, kp, f,
                                                                (unsigned)tiles_p, along_x);
  else
    realign_kernel<uint16_t><<<(unsigned)tiles, kThreads, 0, st>>>((const uint16_t *)src, (uint16_t *)dst, x, k, kp, f,
                                                                 (unsigned)tiles_p, along_x);
  return skl_check_launch("realign");
}

}  // extern "C"
