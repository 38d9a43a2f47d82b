// skl_gemv.hip - the M == 1 ("decode") path: y = beta*y + alpha * x*B, a pure
// HBM stream over B. No matrix cores: the kernel is bound by how fast B's bytes
// arrive, so the design is about memory-level parallelism and coalescing.
//
// The reference has no separate GEMV API: M == 1 is a branch inside its GEMM
// dispatchers (src/gemm/gemm_bf16_bf16_f32_zvfbfwma_x390.c:1220-1224,
// src/gemm/gemm_i8rcp1x4_i8p4x1c_i32_xsfvqdotq.c:645-660) and, for row-major
// int8, the one-row remainder loop (src/gemm/gemm_i8_i8_i32_zve32x_x390.c:532-600);
// the arithmetic is ref/gemm/gemm_i8rc_i8rc_i32rc.c:10-26 with m = 1.
//
// Work decomposition (row-major B, int8): a lane owns 16 consecutive columns
// (one 128-bit load per row) and ROWS_PER_LANE consecutive rows; eight lanes
// cover one 128-byte line of a row and the eight lane-groups of a wave take
// different row ranges, so a workgroup streams a 128-column strip of
// kRowsPerGroup rows with every load instruction touching eight full lines and
// all loads of a wave in flight before the first use. Four rows at a time are
// transposed in registers (v_perm_b32) so that v_dot4_i32_i8 multiplies four
// k-values of one column with four packed x bytes. The 32 partial sums per
// column of a workgroup meet in LDS; the few workgroups that share a column
// strip (K / kRowsPerGroup of them) meet in a zero-initialised int32 accumulator
// in device memory through relaxed device-scope atomics (integer adds: exact in
// any order). A ticket counter per strip tells the workgroup that arrives last
// to apply alpha and beta, write y and put accumulator and ticket back to zero.
// Only atomics carry data between workgroups, so ordering needs no cache
// write-back: a wait for the workgroup's outstanding atomics before the ticket
// is taken is enough (a device-scope fence would flush the whole L2 and costs
// ten times the kernel).
#include <hip/hip_runtime.h>

#include <mutex>

#include "skl_device.hpp"

namespace {

constexpr int kColsPerLane = 16;
constexpr int kColLanes = 8;                           // lanes side by side along a row
constexpr int kRowLanes = 64 / kColLanes;              // lane groups taking different rows
constexpr int kTileCols = kColLanes * kColsPerLane;    // 128 columns = one 128-byte line per row
constexpr int kRowsPerLane = 16;
constexpr int kWaves = 4;
constexpr int kPartials = kWaves * kRowLanes;          // partial sums per column in a workgroup
constexpr int kRowsPerGroup = kPartials * kRowsPerLane;  // 512 rows (k) per workgroup

// Zero-initialised per-device scratch: int32/float accumulators + tickets.
constexpr size_t kMaxCols = size_t(1) << 22;  // 4 Mi columns
constexpr size_t kMaxTiles = kMaxCols / kTileCols;
struct Reduction {
  void *acc = nullptr;      // kMaxCols 32-bit accumulators
  unsigned *tickets = nullptr;  // kMaxTiles counters
};
std::mutex g_mutex;
Reduction g_reduction[16];

bool reduction_scratch(Reduction *out) {
  int dev = 0;
  if (skl_check_hip(hipGetDevice(&dev), "hipGetDevice") != 0 || dev >= 16) return false;
  std::lock_guard<std::mutex> lock(g_mutex);
  Reduction &r = g_reduction[dev];
  if (!r.acc) {
    const size_t bytes = kMaxCols * 4 + kMaxTiles * sizeof(unsigned);
    void *p = nullptr;
    if (skl_check_hip(hipMalloc(&p, bytes), "gemv scratch") != 0) return false;
    if (skl_check_hip(hipMemset(p, 0, bytes), "gemv scratch clear") != 0) return false;
    r.acc = p;
    r.tickets = (unsigned *)((char *)p + kMaxCols * 4);
  }
  *out = r;
  return true;
}

struct GemvArgs {
  const int8_t *x;
  size_t x_sk;
  int x_vec;  // x is contiguous and 16-byte aligned
  const int8_t *b;
  size_t b_sk;  // stride between k rows (bytes = elements)
  size_t b_s1;  // stride between 64-column blocks
  int32_t *y;
  size_t y_s;
  size_t n, k;
  int32_t alpha, beta;
  int32_t *acc;
  unsigned *tickets;
  unsigned tiles, slabs;
};

// 4x4 byte transpose: in r[j] byte i  ->  out t[i] byte j.
__device__ __forceinline__ void transpose4x4(unsigned r0, unsigned r1, unsigned r2, unsigned r3, unsigned &t0,
                                             unsigned &t1, unsigned &t2, unsigned &t3) {
  // v_perm_b32(a, b, sel): bytes 0-3 index b, 4-7 index a.
  const unsigned lo01 = __builtin_amdgcn_perm(r1, r0, 0x05010400u);  // r0.b0 r1.b0 r0.b1 r1.b1
  const unsigned hi01 = __builtin_amdgcn_perm(r1, r0, 0x07030602u);  // r0.b2 r1.b2 r0.b3 r1.b3
  const unsigned lo23 = __builtin_amdgcn_perm(r3, r2, 0x05010400u);
  const unsigned hi23 = __builtin_amdgcn_perm(r3, r2, 0x07030602u);
  t0 = __builtin_amdgcn_perm(lo23, lo01, 0x05040100u);  // r0.b0 r1.b0 r2.b0 r3.b0
  t1 = __builtin_amdgcn_perm(lo23, lo01, 0x07060302u);
  t2 = __builtin_amdgcn_perm(hi23, hi01, 0x05040100u);
  t3 = __builtin_amdgcn_perm(hi23, hi01, 0x07060302u);
}

__global__ void __launch_bounds__(kWaves * 64) gemv_i8_rowmajor_kernel(GemvArgs p) {
  __shared__ int red[kPartials][kTileCols + 4];
  __shared__ unsigned ticket_s;

  const unsigned tile = blockIdx.x % p.tiles, slab = blockIdx.x / p.tiles;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int cl = lane % kColLanes, rl = lane / kColLanes;
  const int part = wave * kRowLanes + rl;
  const size_t k0 = (size_t)slab * kRowsPerGroup + (size_t)part * kRowsPerLane;
  const size_t col = (size_t)tile * kTileCols + (size_t)cl * kColsPerLane;

  int acc[kColsPerLane];
#pragma unroll
  for (int j = 0; j < kColsPerLane; ++j) acc[j] = 0;

  if (col < p.n && k0 < p.k) {
    // All of the lane's rows are requested before anything is consumed.
    const int8_t *wp = p.b + (col >> 6) * p.b_s1 + (col & 63) + k0 * p.b_sk;
    uint4 rows[kRowsPerLane];
#pragma unroll
    for (int r = 0; r < kRowsPerLane; ++r) {
      if (k0 + r < p.k)
        rows[r] = *reinterpret_cast<const uint4 *>(wp + (size_t)r * p.b_sk);
      else
        rows[r] = make_uint4(0, 0, 0, 0);
    }
    // Four x bytes per group of four rows; rows at or beyond K were loaded as zero.
    int xw[kRowsPerLane / 4];
    if (p.x_vec && k0 + kRowsPerLane <= p.k) {
      const int4 *xp = reinterpret_cast<const int4 *>(p.x + k0);
#pragma unroll
      for (int q = 0; q < kRowsPerLane / 16; ++q) {
        const int4 v = xp[q];
        xw[4 * q] = v.x, xw[4 * q + 1] = v.y, xw[4 * q + 2] = v.z, xw[4 * q + 3] = v.w;
      }
    } else {
#pragma unroll
      for (int g = 0; g < kRowsPerLane / 4; ++g) {
        unsigned w = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const size_t k = k0 + 4 * g + i;
          const unsigned byte = k < p.k ? (unsigned)(uint8_t)p.x[k * p.x_sk] : 0u;
          w |= byte << (8 * i);
        }
        xw[g] = (int)w;
      }
    }
#pragma unroll
    for (int g = 0; g < kRowsPerLane / 4; ++g) {
      const uint4 r0 = rows[4 * g], r1 = rows[4 * g + 1], r2 = rows[4 * g + 2], r3 = rows[4 * g + 3];
      const unsigned a0[4] = {r0.x, r0.y, r0.z, r0.w}, a1[4] = {r1.x, r1.y, r1.z, r1.w};
      const unsigned a2[4] = {r2.x, r2.y, r2.z, r2.w}, a3[4] = {r3.x, r3.y, r3.z, r3.w};
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        unsigned t0, t1, t2, t3;
        transpose4x4(a0[d], a1[d], a2[d], a3[d], t0, t1, t2, t3);
        acc[4 * d + 0] = __builtin_amdgcn_sdot4((int)t0, xw[g], acc[4 * d + 0], false);
        acc[4 * d + 1] = __builtin_amdgcn_sdot4((int)t1, xw[g], acc[4 * d + 1], false);
        acc[4 * d + 2] = __builtin_amdgcn_sdot4((int)t2, xw[g], acc[4 * d + 2], false);
        acc[4 * d + 3] = __builtin_amdgcn_sdot4((int)t3, xw[g], acc[4 * d + 3], false);
      }
    }
  }
  // The workgroup's partial sums meet in LDS.
#pragma unroll
  for (int j = 0; j < kColsPerLane; j += 4)
    *reinterpret_cast<int4 *>(&red[part][cl * kColsPerLane + j]) = make_int4(acc[j], acc[j + 1], acc[j + 2], acc[j + 3]);
  __syncthreads();
  const size_t tile_col0 = (size_t)tile * kTileCols;
  const bool owner = threadIdx.x < kTileCols && tile_col0 + threadIdx.x < p.n;
  int sum = 0;
  if (owner) {
#pragma unroll
    for (int w = 0; w < kPartials; ++w) sum += red[w][threadIdx.x];
  }
  if (p.slabs == 1) {  // the strip is complete inside this workgroup
    if (owner) {
      int32_t *y = p.y + (tile_col0 + threadIdx.x) * p.y_s;
      *y = (int32_t)((uint32_t)p.beta * (uint32_t)*y + (uint32_t)p.alpha * (uint32_t)sum);
    }
    return;
  }
  if (owner) atomicAdd(&p.acc[tile_col0 + threadIdx.x], sum);
  // Wait until this wave's atomics have been performed, then take a ticket.
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
  if (threadIdx.x == 0) ticket_s = atomicAdd(&p.tickets[tile], 1u);
  __syncthreads();
  if (ticket_s != p.slabs - 1) return;
  if (owner) {
    const size_t j = tile_col0 + threadIdx.x;
    const int total = atomicExch(&p.acc[j], 0);  // read the total and leave zero behind
    int32_t *y = p.y + j * p.y_s;
    *y = (int32_t)((uint32_t)p.beta * (uint32_t)*y + (uint32_t)p.alpha * (uint32_t)total);
  }
  if (threadIdx.x == 0) atomicExch(&p.tickets[tile], 0u);
}

inline bool aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }

}  // namespace

extern "C" int skl_hip_gemv_supported(const skl_gemm_canon *g, int layout) {
  if (layout != 0) return 0;
  if (g->ta != SKL_DT_I8 || g->tb != SKL_DT_I8) return 0;
  if (g->m != 1 || g->k == 0 || g->n == 0) return 0;
  if (g->b_s0 != 1 || (g->n % kColsPerLane) != 0 || g->n > kMaxCols) return 0;
  if (!aligned16(g->b) || (g->b_sk % 16) != 0 || (g->b_s1 % 16) != 0) return 0;
  if (g->csc1 != 64 * g->csc0) return 0;  // y must be a flat strided vector
  return 1;
}

extern "C" int skl_hip_launch_gemv(const skl_gemm_canon *g, int layout) {
  if (!skl_hip_gemv_supported(g, layout)) {
    skl_hip_record_error(-2, "gemv: unsupported problem");
    return -2;
  }
  Reduction red;
  if (!reduction_scratch(&red)) return -4;
  GemvArgs p;
  p.x = (const int8_t *)g->a;
  p.x_sk = g->a_sk;
  p.x_vec = (g->a_sk == 1 && aligned16(g->a)) ? 1 : 0;
  p.b = (const int8_t *)g->b;
  p.b_sk = g->b_sk;
  p.b_s1 = g->b_s1;
  p.y = (int32_t *)g->c;
  p.y_s = g->csc0;
  p.n = g->n;
  p.k = g->k;
  p.alpha = g->alpha.i;
  p.beta = g->beta.i;
  p.acc = (int32_t *)red.acc;
  p.tickets = red.tickets;
  p.tiles = skl_div_up(g->n, kTileCols);
  p.slabs = skl_div_up(g->k, kRowsPerGroup);
  const size_t grid = (size_t)p.tiles * p.slabs;
  if (grid > 0x7FFFFFFFu) {
    skl_hip_record_error(-2, "gemv: grid too large");
    return -2;
  }
  gemv_i8_rowmajor_kernel<<<(unsigned)grid, kWaves * 64, 0, skl_current_stream()>>>(p);
  return skl_check_launch("gemv_i8_rowmajor");
}
