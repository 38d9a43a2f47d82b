// skl_gemv.hip - the M == 1 ("decode") path: y = beta*y + alpha * x*B, a pure
// HBM stream over B. The one-row kernels use no matrix cores: they are bound by how
// fast B's bytes arrive, so the design is about memory-level parallelism and coalescing.
// The kernels: gemv_kernel (M = 1, row-major or K-packed B; described below),
// gemv_rows_kernel (a few rows of A against a row-major B), gemv_mfma_rows_kernel (up to
// 16 rows of A against a row-major or K-packed B: the same stream, B transposed in registers
// and multiplied on the matrix cores), gemv_rowgroups_kernel (the same with B held in
// registers for several groups of 16 rows), gemv_k4_wholek_kernel (K-packed B with K <= 4096:
// one workgroup per column tile takes all of K) and gemv_kc_kernel (1 to 4 rows of A against
// a B with K contiguous), each introduced where it is defined. Decode batches on a B with K
// contiguous: skl_gemv_kcrows.hip; 4-bit weights: skl_gemv_f4.hip.
//
// The reference has no separate GEMV API: M == 1 is a branch inside its GEMM
// dispatchers (src/gemm/gemm_bf16_bf16_f32_zvfbfwma_x390.c:1220-1224,
// src/gemm/gemm_i8rcp1x4_i8p4x1c_i32_xsfvqdotq.c:645-660) and, for row-major
// int8, the one-row remainder loop (src/gemm/gemm_i8_i8_i32_zve32x_x390.c:532-600);
// the arithmetic is ref/gemm/gemm_i8rc_i8rc_i32rc.c:10-26 with m = 1.
//
// Work decomposition (row-major B, int8): a lane owns 16 consecutive columns
// (one 128-bit load per row) and ROWS_PER_LANE consecutive rows; a pair of lanes
// reads 32 adjacent bytes of a row, the four pairs of a wave that sit at the same
// place in the four rows of 16 lanes cover one 128-byte line, and the eight row
// groups of a wave sit inside each row of 16 lanes. A workgroup (eight waves)
// streams a 128-column strip of kRowsPerGroup rows with all loads of every lane
// in flight before the first use. Four rows at a time are transposed in
// registers (v_perm_b32) so that v_dot4_i32_i8 multiplies four k-values of one
// column with four packed x bytes. The eight row groups of a wave are summed in
// registers with three DPP rotations; one partial sum per wave and column goes
// through LDS. The few workgroups that share a column strip (K / kRowsPerGroup
// of them) meet in a zero-initialised accumulator in device memory through
// relaxed device-scope atomics (integer adds: exact in any order). The slot is
// 64 bits wide: the sum lives in the high word and an arrival count in the low
// word, one atomic add carries both and returns the previous value, so the lane
// whose add completes the count knows the total, applies alpha and beta - the
// old y was asked for when the kernel started - writes y and puts the slot back
// to zero: one round trip to memory after the last byte of B has arrived.
// Floating-point sums depend on their order, so those modes do not add into a
// shared slot: every workgroup stores its sums to a plane of its own, and the
// one that draws the last ticket of the strip adds the planes in slab order
// (ordered_sum_over_slabs): the same bits on every run. Ordering needs no cache
// write-back: a wait for the workgroup's own stores before the ticket is taken
// is enough; a device-scope fence would flush the whole L2 and costs ten times
// the kernel.
//
// The same skeleton serves more operand kinds: OCP fp8 weights and x (E4M3, E5M2 and E4M3 x with E5M2
// weights; a lane owns 16 columns, the hardware conversions decode to fp32), bf16 and f16 weights
// (a lane owns 8 columns, fp32 accumulation with v_fma) and the K-packed int8 layout of the dot4
// entry point (B(4P+p, j) at P*rsb1 + 4j + p: a 128-bit load holds four columns times four
// k, which v_dot4_i32_i8 consumes without any byte shuffling).
#include <hip/hip_runtime.h>

#include <atomic>

#include <type_traits>

#include <mutex>

#include "skl_device.hpp"
#include "skl_fp8.hpp"

// Scratch of the entry point that allocates nothing (skl_gemm_i8_i8_i32_noalloc_gfx950, at the end of this file):
// the 64-bit sum + count slots of the int8 kernels in a static array of a fixed size instead of the block the
// library allocates per stream. Each GPU the library runs on holds its own copy until the process ends. The
// array is zero when the module is loaded, and every kernel puts the slots it used back to zero.
constexpr size_t kNoAllocSlots = size_t(1) << 16;  // 512 KiB
static __device__ __align__(256) unsigned long long scratch[kNoAllocSlots];

namespace {

// Kernel modes.
enum { kI8RowMajor = 0, kI8K4 = 1, kBF16 = 2, kF16 = 3, kF8E4M3 = 4, kF8E5M2 = 5, kF8Mixed = 6 /* E4M3 x, E5M2 B */ };

constexpr int kColLanes = 8;                 // lanes side by side along a row: 8 x 16 B = one 128-byte line
constexpr int kRowLanes = 64 / kColLanes;    // lane groups taking different rows
constexpr int kLoadsPerLane = 8;             // 128-bit loads in flight per lane
constexpr int kWaves = 8;
constexpr int kPartials = kWaves * kRowLanes;  // partial sums per column in a workgroup

template <int MODE>
struct Mode {
  static constexpr bool kFp8 = MODE == kF8E4M3 || MODE == kF8E5M2 || MODE == kF8Mixed;
  static constexpr int kCols = (MODE == kI8RowMajor || kFp8) ? 16 : MODE == kI8K4 ? 4 : 8;  // columns per lane
  static constexpr int kTileCols = kColLanes * kCols;                              // columns per workgroup
  static constexpr int kKPerLoad = MODE == kI8K4 ? 4 : 1;                          // k values per 128-bit load
  static constexpr int kKPerLane = kLoadsPerLane * kKPerLoad;
  static constexpr int kKPerGroup = kPartials * kKPerLane;                         // k per workgroup
  static constexpr int kES = (MODE == kBF16 || MODE == kF16) ? 2 : 1;
  using Acc = typename std::conditional<(MODE == kBF16 || MODE == kF16 || kFp8), float, int>::type;
};

// Zero-initialised scratch of the launching stream: one 64-bit slot per column (the floating-point modes use the
// first 32 bits of the region as an fp32 array) + tickets.
constexpr size_t kMaxCols = size_t(1) << 22;  // 4 Mi columns
constexpr size_t kMaxTiles = kMaxCols / 32;
struct Reduction {
  void *acc = nullptr;          // kMaxCols 64-bit slots
  unsigned *tickets = nullptr;  // kMaxTiles counters
};

// One block per stream and device: launches on different streams may run at the same time.
bool reduction_scratch(Reduction *out) {
  void *p = skl_zeroed_scratch(kMaxCols * 8 + kMaxTiles * sizeof(unsigned));
  if (!p) return false;
  out->acc = p;
  out->tickets = (unsigned *)((char *)p + kMaxCols * 8);
  return true;
}

struct GemvArgs {
  const char *x;
  size_t x_sk;  // elements
  int x_vec;    // x is contiguous and 16-byte aligned
  const char *b;
  size_t b_sk;  // bytes between consecutive k rows (K4 layout: between groups of four k)
  size_t b_s1;  // bytes between 64-column blocks (row-major modes)
  char *y;
  size_t y_s;   // elements
  size_t n, k;
  skl_scalar alpha, beta;
  void *acc;         // integer kinds: one zero-initialised 64-bit slot per column
  unsigned *tickets; // floating point: one zero-initialised counter per strip ...
  float *planes;     // ... and `slabs` planes of n sums (the stream's workspace)
  unsigned tiles, slabs;
  const char *bias;  // FUSED kernels: the steps behind alpha / beta (bias and maximum of y's type, or null) ...
  char *max;
  skl_requant rq;    // ... activation and 8-bit copy
};

// B is read once: a non-temporal 128-bit load.
typedef unsigned u4v __attribute__((ext_vector_type(4)));
typedef float v2f __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint4 stream_load(const char *p) {
  const u4v v = __builtin_nontemporal_load(reinterpret_cast<const u4v *>(p));
  return make_uint4(v.x, v.y, v.z, v.w);
}

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

__device__ __forceinline__ float widen16(unsigned bits16, bool is_bf16) {
  if (is_bf16) return __uint_as_float(bits16 << 16);
  _Float16 h = __builtin_bit_cast(_Float16, (unsigned short)bits16);
  return (float)h;
}


// Sum over the eight lanes of a row of 16 that share a column group (same lane parity), in every lane:
// three DPP rotations inside the row, no LDS crossbar. A fixed order, also for floats.
__device__ __forceinline__ int sum_over_row_groups(int v) {
  v += __builtin_amdgcn_update_dpp(0, v, 0x128 /* row_ror:8 */, 0xF, 0xF, false);
  v += __builtin_amdgcn_update_dpp(0, v, 0x124 /* row_ror:4 */, 0xF, 0xF, false);
  v += __builtin_amdgcn_update_dpp(0, v, 0x122 /* row_ror:2 */, 0xF, 0xF, false);
  return v;
}

__device__ __forceinline__ float sum_over_row_groups(float v) {
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128, 0xF, 0xF, false));
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x124, 0xF, 0xF, false));
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x122, 0xF, 0xF, false));
  return v;
}

// Floating-point sums of the workgroups that share columns. Each workgroup leaves its sums in its own plane of
// `planes` (element `idx` of plane `slab`, planes `plane_elems` apart) with stores that go through to memory, waits
// until they have been performed and takes a ticket; the workgroup that draws the last ticket reads every plane
// back - with read-modify-write atomics, which are performed where the stores went and never see a stale cache
// line - and adds them in slab order: the same bits on every run, whichever workgroup finishes last. Returns
// true in that workgroup, with the total of the caller's element in `total`. `mine` says whether the calling
// thread owns an element at all; every thread of the workgroup must call.
__device__ __forceinline__ bool ordered_sum_over_slabs(float *planes, size_t plane_elems, size_t idx, unsigned slab,
                                                       unsigned slabs, unsigned *ticket, unsigned *ticket_s, bool mine,
                                                       float sum, float &total) {
  if (mine) __hip_atomic_store(planes + (size_t)slab * plane_elems + idx, sum, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_s_waitcnt(0);  // this wave's stores have been performed
  __syncthreads();
  if (threadIdx.x == 0) *ticket_s = __hip_atomic_fetch_add(ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __syncthreads();
  if (*ticket_s != slabs - 1) return false;
  if (threadIdx.x == 0) __hip_atomic_store(ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // zero for the next call
  if (mine) {
    // eight planes are requested before the first is used; the sum still runs over the planes in order
    unsigned *words = reinterpret_cast<unsigned *>(planes) + idx;
    float t = 0.0f;
    for (unsigned q0 = 0; q0 < slabs; q0 += 8) {
      unsigned v[8];
#pragma unroll
      for (unsigned u = 0; u < 8; ++u)
        v[u] = q0 + u < slabs ? __hip_atomic_fetch_or(words + (size_t)(q0 + u) * plane_elems, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0u;
#pragma unroll
      for (unsigned u = 0; u < 8; ++u)
        if (q0 + u < slabs) t = (q0 + u == 0) ? __uint_as_float(v[u]) : __fadd_rn(t, __uint_as_float(v[u]));
    }
    total = t;
  }
  return true;
}

// LOADS: 128-bit loads in flight per lane = rows of B (K-packed layout: groups of four rows) a lane takes.
// Lane pairs read 32 adjacent bytes of a row and the eight row groups of a wave sit inside each row of 16 lanes
// (column lane = pair member + 2 * row of 16), so that the lanes that share columns are summed with DPP rotations
// and only one partial sum per wave and column goes through LDS.
// FUSED: the thread that completes a column applies the fused steps (bias, activation, 8-bit copy, maximum) to it.
// WHOLE: the strips and row ranges divide the matrix evenly (n a multiple of the strip's columns, k of a workgroup's
// rows); a 2-D grid (strip, row range). No load is guarded, and the rows are dealt out the other way round: load r
// of a lane is row r * 64 + (its place among the workgroup's 64 row lanes), so that load r of the eight waves covers
// 64 consecutive rows of the strip - the order in which a plain read walks memory. On config 2's row pitch (86 lines)
// a read-only kernel in this order takes 8.3 us per 45 MB where eight consecutive rows per lane take 8.8 us (a plain
// read: 8.0 us), and the kernel as a whole 9.6 us against 10.3 us.
template <int MODE, int LOADS, bool FUSED = false, bool WHOLE = false>
__global__ void __launch_bounds__(kWaves * 64) gemv_kernel(GemvArgs p) {
  using Md = Mode<MODE>;
  static_assert(!WHOLE || Md::kKPerLoad == 1, "one row per load");
  constexpr int kKPerLaneL = LOADS * Md::kKPerLoad, kKPerGroupL = kPartials * kKPerLaneL;
  constexpr size_t kRowStep = WHOLE ? kPartials : 1;  // rows from one load of a lane to its next
  using Acc = typename Md::Acc;
  constexpr int kCols = Md::kCols;
  __shared__ __attribute__((aligned(16))) Acc red[kWaves][Md::kTileCols + 4];
  __shared__ unsigned ticket_s;

  const unsigned tile = WHOLE ? blockIdx.x : blockIdx.x % p.tiles, slab = WHOLE ? blockIdx.y : blockIdx.x / p.tiles;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int cl = (lane & 1) + 2 * (lane >> 4), rl = (lane >> 1) & 7;
  const int part = wave * kRowLanes + rl;
  const size_t k0 = (size_t)slab * kKPerGroupL + (WHOLE ? (size_t)part : (size_t)part * kKPerLaneL);  // the lane's first row
  const size_t col = (size_t)tile * Md::kTileCols + (size_t)cl * kCols;

  Acc acc[kCols];
#pragma unroll
  for (int j = 0; j < kCols; ++j) acc[j] = 0;

  // The thread that will write column tile_col0 + threadIdx.x asks for its old value now, so that it is there
  // when the sums are: no memory round trip behind the last byte of B.
  const size_t tile_col0 = (size_t)tile * Md::kTileCols;
  const bool owner = threadIdx.x < Md::kTileCols && tile_col0 + threadIdx.x < p.n;
  Acc *yv = reinterpret_cast<Acc *>(p.y);
  const bool y_is_read = !skl_beta_is_zero<Acc>(p.beta);
  Acc y_old = 0;

  {
    // All of the lane's loads are requested before anything is consumed. Without WHOLE they are clamped into B
    // rather than guarded (a guard is a branch, and the compiler waits for the loads in flight at a branch it
    // cannot prove uniform): a lane beyond N reads column 0 and writes nothing, a row beyond K is read as row 0 and
    // meets a zero of x - or, in the floating-point kinds, where 0 * NaN would not be 0, is zeroed itself.
    const size_t colc = (WHOLE || col < p.n) ? col : 0;
    const char *wp;
    if constexpr (MODE == kI8K4)
      wp = p.b + colc * 4;
    else
      wp = p.b + (colc >> 6) * p.b_s1 + (colc & 63) * Md::kES;
    uint4 rows[LOADS];
#pragma unroll
    for (int r = 0; r < LOADS; ++r) {
      const size_t kr = k0 + (size_t)r * kRowStep * Md::kKPerLoad;
      const bool inside = WHOLE || kr < p.k;
      rows[r] = stream_load(wp + ((inside ? kr : 0) / Md::kKPerLoad) * p.b_sk);
      if constexpr (!WHOLE && MODE != kI8RowMajor && MODE != kI8K4) {
        rows[r].x = inside ? rows[r].x : 0u, rows[r].y = inside ? rows[r].y : 0u;
        rows[r].z = inside ? rows[r].z : 0u, rows[r].w = inside ? rows[r].w : 0u;
      }
    }
    if (owner && y_is_read) y_old = yv[(tile_col0 + threadIdx.x) * p.y_s];
    if constexpr (MODE == kI8RowMajor || MODE == kI8K4) {
      // x as packed bytes, four k per dword; k at or beyond K contributes zero.
      constexpr int kWords = kKPerLaneL / 4;
      int xw[kWords];
      const int8_t *x = reinterpret_cast<const int8_t *>(p.x);
      if constexpr (WHOLE) {  // the lane's rows are kRowStep apart: its x bytes one by one (cache hits, behind B's loads)
#pragma unroll
        for (int g = 0; g < kWords; ++g) {
          unsigned w = 0;
#pragma unroll
          for (int i = 0; i < 4; ++i) w |= (unsigned)(uint8_t)x[(k0 + (size_t)(4 * g + i) * kRowStep) * p.x_sk] << (8 * i);
          xw[g] = (int)w;
        }
      } else if (p.x_vec && k0 + kKPerLaneL <= p.k) {
        const int *xp = reinterpret_cast<const int *>(x + k0);  // k0 is a multiple of kKPerLane: aligned
#pragma unroll
        for (int q = 0; q < kWords; ++q) xw[q] = xp[q];
      } else {
#pragma unroll
        for (int g = 0; g < kWords; ++g) {
          unsigned w = 0;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const size_t k = k0 + 4 * g + i;
            const unsigned byte = k < p.k ? (unsigned)(uint8_t)x[k * p.x_sk] : 0u;
            w |= byte << (8 * i);
          }
          xw[g] = (int)w;
        }
      }
      if constexpr (MODE == kI8RowMajor) {
#pragma unroll
        for (int g = 0; g < LOADS / 4; ++g) {
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
      } else {  // K4: each dword already holds four k of one column
#pragma unroll
        for (int r = 0; r < LOADS; ++r) {
          acc[0] = __builtin_amdgcn_sdot4((int)rows[r].x, xw[r], acc[0], false);
          acc[1] = __builtin_amdgcn_sdot4((int)rows[r].y, xw[r], acc[1], false);
          acc[2] = __builtin_amdgcn_sdot4((int)rows[r].z, xw[r], acc[2], false);
          acc[3] = __builtin_amdgcn_sdot4((int)rows[r].w, xw[r], acc[3], false);
        }
      }
    } else if constexpr (Md::kFp8) {
      // OCP fp8 weights and x: the hardware conversions decode every code but the NaNs exactly as the
      // reference's decode does (a NaN comes out with its sign set; it is a NaN either way), and the
      // product of two fp8 values is exact in fp32, so a fused multiply-add rounds like multiply, then add.
      constexpr bool x_e5m2 = MODE == kF8E5M2, b_e5m2 = MODE != kF8E4M3;
      const uint8_t *x = reinterpret_cast<const uint8_t *>(p.x);
#pragma unroll
      for (int r = 0; r < LOADS; ++r) {
        const size_t k = k0 + r * kRowStep;
        const bool inside = WHOLE || k < p.k;
        const int xl = (int)x[(inside ? k : 0) * p.x_sk];
        const int xb = inside ? xl : 0;  // code 0 is +0.0 in both formats
        const float xv = x_e5m2 ? __builtin_amdgcn_cvt_f32_bf8(xb, 0) : __builtin_amdgcn_cvt_f32_fp8(xb, 0);
        const unsigned w[4] = {rows[r].x, rows[r].y, rows[r].z, rows[r].w};
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          v2f lo, hi;  // bytes 0, 1 and bytes 2, 3 of the dword: four consecutive columns
          if constexpr (b_e5m2) {
            lo = __builtin_amdgcn_cvt_pk_f32_bf8((int)w[d], false);
            hi = __builtin_amdgcn_cvt_pk_f32_bf8((int)w[d], true);
          } else {
            lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[d], false);
            hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[d], true);
          }
          acc[4 * d + 0] = __fmaf_rn(xv, lo.x, acc[4 * d + 0]);
          acc[4 * d + 1] = __fmaf_rn(xv, lo.y, acc[4 * d + 1]);
          acc[4 * d + 2] = __fmaf_rn(xv, hi.x, acc[4 * d + 2]);
          acc[4 * d + 3] = __fmaf_rn(xv, hi.y, acc[4 * d + 3]);
        }
      }
    } else {
      constexpr bool bf = MODE == kBF16;
      const unsigned short *x = reinterpret_cast<const unsigned short *>(p.x);
#pragma unroll
      for (int r = 0; r < LOADS; ++r) {
        const size_t k = k0 + r * kRowStep;
        const bool inside = WHOLE || k < p.k;
        const float xl = widen16(x[(inside ? k : 0) * p.x_sk], bf);
        const float xv = inside ? xl : 0.0f;
        const unsigned w[4] = {rows[r].x, rows[r].y, rows[r].z, rows[r].w};
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          acc[2 * d] = __fmaf_rn(xv, widen16(w[d] & 0xFFFFu, bf), acc[2 * d]);
          acc[2 * d + 1] = __fmaf_rn(xv, widen16(w[d] >> 16, bf), acc[2 * d + 1]);
        }
      }
    }
  }
  // The eight row groups of a wave are summed in registers (every lane takes part); the first hands the wave's
  // sums to LDS, where the eight waves meet.
#pragma unroll
  for (int j = 0; j < kCols; ++j) acc[j] = sum_over_row_groups(acc[j]);
  if (rl == 0) {  // 16-byte stores: a row of `red` is a multiple of 16 bytes, a lane's columns start on one
    typedef Acc acc4 __attribute__((ext_vector_type(4)));
#pragma unroll
    for (int j = 0; j < kCols; j += 4) *reinterpret_cast<acc4 *>(&red[wave][cl * kCols + j]) = acc4{acc[j], acc[j + 1], acc[j + 2], acc[j + 3]};
  }
  __syncthreads();
  Acc sum = 0;
  if (owner) {
    sum = red[0][threadIdx.x];
#pragma unroll
    for (int w = 1; w < kWaves; ++w) sum += red[w][threadIdx.x];
  }
  // `total` is complete: the alpha/beta step with the old value that was asked for at the start (the initialising
  // mode reads it only now, and only where alpha * total is a zero).
  Acc largest = skl_lowest<Acc>();  // FUSED: what this thread wrote, for the maximum
  auto finish = [&](Acc total) {
    Acc *y = yv + (tile_col0 + threadIdx.x) * p.y_s;
    Acc v = y_is_read ? skl_combine(total, y_old, p.alpha, p.beta) : skl_initialise(total, y, p.alpha, p.beta);
    if constexpr (FUSED) {
      const size_t j = tile_col0 + threadIdx.x;
      if (p.bias) v = skl_add_bias(v, reinterpret_cast<const Acc *>(p.bias)[j]);
      v = skl_activate(v, p.rq.act);
      if (!p.rq.q_only) *y = v;
      skl_emit_requantised(p.rq, v, 0, j);
      if (v > largest) largest = v;
    } else {
      *y = v;
    }
  };
  // FUSED: every thread of the workgroup comes here once it has finished what it finishes (most finish nothing);
  // one atomic per wave that wrote something.
  auto report_maximum = [&]() {
    if constexpr (FUSED) {
      if (!p.max) return;
      const Acc best = skl_wave_max(largest);
      if ((threadIdx.x & 63) == 0 && best > skl_lowest<Acc>()) skl_atomic_max(reinterpret_cast<Acc *>(p.max), best);
    }
  };
  if (p.slabs == 1) {  // the strip is complete inside this workgroup
    if (owner) finish(sum);
    report_maximum();
    return;
  }
  if constexpr (std::is_same<Acc, int>::value) {
    // Integer strips: sum and arrival count travel in one 64-bit atomic (sum in the high word, where
    // it wraps like int32; count in the low word). The add returns the previous value, so the lane
    // whose add completes the count holds the total: no ticket, no read-back.
    if (owner) {
      const size_t j = tile_col0 + threadIdx.x;
      unsigned long long *slot = reinterpret_cast<unsigned long long *>(p.acc) + j;
      const unsigned long long mine = ((unsigned long long)(unsigned)sum << 32) | 1ull;
      const unsigned long long now = atomicAdd(slot, mine) + mine;
      if ((unsigned)now == p.slabs) {
        __hip_atomic_store(slot, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // zero for the next call
        finish((int)(unsigned)(now >> 32));
      }
    }
  } else {
    float total = 0.0f;
    if (ordered_sum_over_slabs(p.planes, p.n, tile_col0 + threadIdx.x, slab, p.slabs, &p.tickets[tile], &ticket_s,
                               owner, sum, total) && owner)
      finish(total);
  }
  report_maximum();
}


// ---------------------------------------------------------------------------
// 2 <= M <= 8 rows of A against a row-major B ("decode" with a small batch): still a stream over
// B, so the M = 1 decomposition is kept - same strips, same loads, same 4x4 byte transposes - and every
// transposed dword is multiplied with the packed x bytes of each of the MR rows (the transposes are shared:
// (8 + 4 MR) / 16 VALU operations per byte of B). The rows are taken four at a time over the bytes held in
// registers (64 sums per lane: two workgroups per compute unit). The eight row groups of a wave are laid
// out inside each row of 16 lanes, so their sums are combined with three DPP rotations; the eight waves
// meet in LDS, and the workgroups of a strip meet in one 64-bit slot per (row, column) like the M = 1 kernel.
// The floating-point kinds (bf16, f16, fp8) run on the same skeleton: a loaded row of B is widened once and
// multiplied with the x value of every row, fp32 sums; between workgroups the sums travel in planes that the
// last workgroup of a strip adds in slab order, as in the M = 1 kernel (the same bits on every run).
// ---------------------------------------------------------------------------
constexpr int kMaxRows = 8;

struct GemvRowsArgs {
  const char *x;   // MR rows of K bytes, x_row bytes apart (4-byte aligned)
  size_t x_row;
  const char *b;
  size_t b_sk, b_s1;
  char *y;         // element (i, j) at i * y_row + j * y_s (elements)
  size_t y_row, y_s;
  size_t n, k;
  skl_scalar alpha, beta;
  void *acc;       // int8: MR * n 64-bit slots, zero between calls
  unsigned *tickets;  // floating point: one counter per strip, zero between calls ...
  float *planes;      // ... and `slabs` planes of MR * n sums (the stream's workspace)
  unsigned tiles, slabs;
};

constexpr int kRowChunk = 4;  // rows of A multiplied per pass over the loaded bytes of B: 64 sums per lane

template <int MR, int MODE>
__global__ void __launch_bounds__(kWaves * 64, 2) gemv_rows_kernel(GemvRowsArgs p) {
  using Md = Mode<MODE>;
  using Acc = typename Md::Acc;
  constexpr int kCols = Md::kCols, kWords = Md::kKPerLane / 4;
  constexpr bool kInt = MODE == kI8RowMajor;
  __shared__ Acc red[kWaves][MR][Md::kTileCols];
  __shared__ unsigned ticket_s;

  const unsigned tile = blockIdx.x % p.tiles, slab = blockIdx.x / p.tiles;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  // Lane pairs read 32 adjacent bytes of a row; the eight row groups sit inside a row of 16 lanes, so that
  // the lanes that share columns can be summed with DPP rotations: column lane = pair member + 2 * row of 16.
  const int cl = (lane & 1) + 2 * (lane >> 4), rl = (lane >> 1) & 7;
  const int part = wave * kRowLanes + rl;
  const size_t k0 = (size_t)slab * Md::kKPerGroup + (size_t)part * Md::kKPerLane;
  const size_t col = (size_t)tile * Md::kTileCols + (size_t)cl * kCols;
  const bool live = col < p.n && k0 < p.k;

  // B's bytes are loaded once and stay in registers for all passes. The loads are clamped into B, not guarded (a
  // guard is a branch, and the compiler waits for the loads in flight at a branch it cannot prove uniform): a lane
  // beyond N reads column 0, a row beyond K row 0, and what they read is zeroed afterwards.
  uint4 rows[kLoadsPerLane];
  {
    const size_t colc = col < p.n ? col : 0;
    const char *wp = p.b + (colc >> 6) * p.b_s1 + (colc & 63) * Md::kES;
#pragma unroll
    for (int r = 0; r < kLoadsPerLane; ++r) {
      const bool inside = col < p.n && k0 + (size_t)r < p.k;
      rows[r] = stream_load(wp + (inside ? k0 + (size_t)r : 0) * p.b_sk);
      rows[r].x = inside ? rows[r].x : 0u, rows[r].y = inside ? rows[r].y : 0u;
      rows[r].z = inside ? rows[r].z : 0u, rows[r].w = inside ? rows[r].w : 0u;
    }
  }
#pragma unroll
  for (int i0 = 0; i0 < MR; i0 += kRowChunk) {
    Acc acc[kRowChunk][kCols];
#pragma unroll
    for (int i = 0; i < kRowChunk; ++i)
#pragma unroll
      for (int j = 0; j < kCols; ++j) acc[i][j] = 0;
    if (live) {
      if constexpr (kInt) {
        // x bytes of the lane's k range, four per dword, for the rows of this pass; k at or beyond K
        // contributes zero
        int xw[kRowChunk][kWords];
#pragma unroll
        for (int i = 0; i < kRowChunk; ++i) {
          if (i0 + i >= MR) continue;
          const int8_t *x = reinterpret_cast<const int8_t *>(p.x + (size_t)(i0 + i) * p.x_row);
          if (k0 + Md::kKPerLane <= p.k) {
            const int *xp = reinterpret_cast<const int *>(x + k0);  // k0 is a multiple of 8, rows are 4-byte aligned
#pragma unroll
            for (int q = 0; q < kWords; ++q) xw[i][q] = xp[q];
          } else {
#pragma unroll
            for (int g = 0; g < kWords; ++g) {
              unsigned w = 0;
#pragma unroll
              for (int b = 0; b < 4; ++b) {
                const size_t k = k0 + 4 * g + b;
                w |= (k < p.k ? (unsigned)(uint8_t)x[k] : 0u) << (8 * b);
              }
              xw[i][g] = (int)w;
            }
          }
        }
#pragma unroll
        for (int g = 0; g < kLoadsPerLane / 4; ++g) {
          const uint4 r0 = rows[4 * g], r1 = rows[4 * g + 1], r2 = rows[4 * g + 2], r3 = rows[4 * g + 3];
          const unsigned a0[4] = {r0.x, r0.y, r0.z, r0.w}, a1[4] = {r1.x, r1.y, r1.z, r1.w};
          const unsigned a2[4] = {r2.x, r2.y, r2.z, r2.w}, a3[4] = {r3.x, r3.y, r3.z, r3.w};
#pragma unroll
          for (int d = 0; d < 4; ++d) {
            unsigned t[4];
            transpose4x4(a0[d], a1[d], a2[d], a3[d], t[0], t[1], t[2], t[3]);
#pragma unroll
            for (int i = 0; i < kRowChunk; ++i) {
              if (i0 + i >= MR) continue;
#pragma unroll
              for (int c = 0; c < 4; ++c)
                acc[i][4 * d + c] = __builtin_amdgcn_sdot4((int)t[c], xw[i][g], acc[i][4 * d + c], false);
            }
          }
        }
      } else {
        // Floating-point kinds: a loaded row of B is widened once and multiplied with the x value of every row.
#pragma unroll
        for (int r = 0; r < kLoadsPerLane; ++r) {
          const size_t k = k0 + r;
          const unsigned w[4] = {rows[r].x, rows[r].y, rows[r].z, rows[r].w};
          float wide[kCols];
          if constexpr (Md::kFp8) {
            constexpr bool b_e5m2 = MODE != kF8E4M3;
#pragma unroll
            for (int d = 0; d < 4; ++d) {
              const v2f lo = b_e5m2 ? __builtin_amdgcn_cvt_pk_f32_bf8((int)w[d], false) : __builtin_amdgcn_cvt_pk_f32_fp8((int)w[d], false);
              const v2f hi = b_e5m2 ? __builtin_amdgcn_cvt_pk_f32_bf8((int)w[d], true) : __builtin_amdgcn_cvt_pk_f32_fp8((int)w[d], true);
              wide[4 * d] = lo.x, wide[4 * d + 1] = lo.y, wide[4 * d + 2] = hi.x, wide[4 * d + 3] = hi.y;
            }
          } else {
#pragma unroll
            for (int d = 0; d < 4; ++d) {
              wide[2 * d] = widen16(w[d] & 0xFFFFu, MODE == kBF16);
              wide[2 * d + 1] = widen16(w[d] >> 16, MODE == kBF16);
            }
          }
#pragma unroll
          for (int i = 0; i < kRowChunk; ++i) {
            if (i0 + i >= MR) continue;
            const char *xr = p.x + (size_t)(i0 + i) * p.x_row;
            float xv;  // loaded from inside the row, zeroed beyond K: no branch between the loads
            const size_t kc = k < p.k ? k : 0;
            if constexpr (Md::kFp8) {
              const int xb = (int)reinterpret_cast<const uint8_t *>(xr)[kc];
              xv = MODE == kF8E5M2 ? __builtin_amdgcn_cvt_f32_bf8(xb, 0) : __builtin_amdgcn_cvt_f32_fp8(xb, 0);
            } else {
              xv = widen16(reinterpret_cast<const unsigned short *>(xr)[kc], MODE == kBF16);
            }
            xv = k < p.k ? xv : 0.0f;
#pragma unroll
            for (int c = 0; c < kCols; ++c) acc[i][c] = __fmaf_rn(xv, wide[c], acc[i][c]);
          }
        }
      }
    }
    // The eight row groups of the wave hold sums of the same columns (every lane takes part);
    // the first group hands the wave's sums to LDS.
#pragma unroll
    for (int i = 0; i < kRowChunk; ++i) {
      if (i0 + i >= MR) continue;
#pragma unroll
      for (int j = 0; j < kCols; ++j) acc[i][j] = sum_over_row_groups(acc[i][j]);
      if (rl == 0) {
#pragma unroll
        for (int j = 0; j < kCols; ++j) red[wave][i0 + i][cl * kCols + j] = acc[i][j];
      }
    }
  }
  __syncthreads();
  const size_t tile_col0 = (size_t)tile * Md::kTileCols;
  // thread t: column t % kTileCols, rows t / kTileCols, + kRowStep, ...
  constexpr int kRowStep = kWaves * 64 / Md::kTileCols, kPasses = (MR + kRowStep - 1) / kRowStep;
  const int c = threadIdx.x % Md::kTileCols, row0 = threadIdx.x / Md::kTileCols;
  const size_t j = tile_col0 + c;
  const bool valid = j < p.n;
  Acc *yv = reinterpret_cast<Acc *>(p.y);
  Acc sum[kPasses];
#pragma unroll
  for (int q = 0; q < kPasses; ++q) {
    const int i = row0 + kRowStep * q;
    sum[q] = 0;
    if (i < MR) {
#pragma unroll
      for (int w = 0; w < kWaves; ++w) sum[q] += red[w][i][c];
    }
  }
  if (p.slabs == 1) {
#pragma unroll
    for (int q = 0; q < kPasses; ++q) {
      const int i = row0 + kRowStep * q;
      if (valid && i < MR) skl_update(sum[q], yv + (size_t)i * p.y_row + j * p.y_s, p.alpha, p.beta);
    }
    return;
  }
  if constexpr (kInt) {
    // all of the thread's atomics go out before the first result is looked at
    unsigned long long now[kPasses];
#pragma unroll
    for (int q = 0; q < kPasses; ++q) {
      const int i = row0 + kRowStep * q;
      if (valid && i < MR) {
        unsigned long long *slot = reinterpret_cast<unsigned long long *>(p.acc) + (size_t)i * p.n + j;
        const unsigned long long mine = ((unsigned long long)(unsigned)sum[q] << 32) | 1ull;
        now[q] = atomicAdd(slot, mine) + mine;
      }
    }
#pragma unroll
    for (int q = 0; q < kPasses; ++q) {
      const int i = row0 + kRowStep * q;
      if (valid && i < MR && (unsigned)now[q] == p.slabs) {
        unsigned long long *slot = reinterpret_cast<unsigned long long *>(p.acc) + (size_t)i * p.n + j;
        __hip_atomic_store(slot, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // zero for the next call
        skl_update((int)(unsigned)(now[q] >> 32), yv + (size_t)i * p.y_row + j * p.y_s, p.alpha, p.beta);
      }
    }
  } else {
    // one plane of sums per workgroup of the strip, added in slab order by the one that finishes last, as in the
    // M = 1 kernel (at most three rows of A here: one element per thread)
    static_assert(kPasses == 1 || kInt, "the floating-point kinds take at most kRowStep rows");
    const int i = row0;
    const bool mine = valid && i < MR;
    float total = 0.0f;
    if (ordered_sum_over_slabs(p.planes, (size_t)MR * p.n, (size_t)i * p.n + j, slab, p.slabs, &p.tickets[tile], &ticket_s,
                               mine, sum[0], total) && mine)
      skl_update(total, yv + (size_t)i * p.y_row + j * p.y_s, p.alpha, p.beta);
  }
}


// ---------------------------------------------------------------------------
// 4 <= M <= 16 rows of int8 A (other kinds, below: from two rows) against a row-major B: still one pass over B
// at the speed it arrives, with the multiply-adds on the matrix cores so that their number does not grow with the rows of A
// (v_mfma_i32_16x16x64_i8: a 16 x 64 block of A times a 64 x 16 block of B). B never goes through LDS: a lane
// loads 16 consecutive rows of 16 consecutive columns (128-bit non-temporal loads, 16 lanes side by side cover
// 256 columns, the four lane groups of a wave take four ranges of 16 rows), transposes the 16 x 16 bytes in
// registers (v_perm_b32) and then holds, for each of its 16 columns, the 16 consecutive k the instruction wants
// from one lane. Instruction c of a block multiplies column c of every lane, i.e. the 16 columns 16 j + c of the
// 256: which 16 columns share an instruction is free, and so is the order of k inside it as long as A's lanes
// hold the same k in the same bytes - A's rows are contiguous in K, so one 128-bit load per block gives exactly
// that. A wave takes two blocks of 64 rows with all 32 loads in flight before the first use, the four waves
// of a workgroup take consecutive k ranges of the same 256 columns and meet in LDS.
// Workgroups that share columns meet in C itself: a first kernel scales C by beta (beta == 0: writes zeros, C is
// not read), and every workgroup adds alpha times its partial sums with atomics that return nothing. int32
// arithmetic wraps, so beta*c + alpha*s1 + alpha*s2 + ... equals beta*c + alpha*(s1 + s2 + ...) bit for bit.
// (Partial sums in planes and a second kernel that adds them: 19 us for 16 x 4096 x 11008; 64-bit atomics that
// carry an arrival count like the M = 1 kernel's: 19 us; this: 15 us, and 13 us for 5 rows.)
// OCP fp8 (E4M3, E5M2, E4M3 A with E5M2 B) runs on the same skeleton: every E4M3 / E5M2 value is an f16 value, so
// the bytes are widened in registers (exactly) and multiplied with v_mfma_f32_16x16x32_f16, whose products are
// exact and whose sums are fp32 - the fp8 matrix-core instructions drop bits below the largest product of an
// instruction, and here the arithmetic is free (8 values of K per lane and instruction: two per column and block).
// Floating-point sums depend on their order and the reference's epilogue rounds beta*c + alpha*acc in one place, so
// here each workgroup stores its raw sums to its own plane of the stream's workspace and a second kernel adds the
// planes in order, applies alpha / beta and the fused steps: deterministic.
// bf16 / f16: a 128-bit load holds 8 columns and v_mfma_f32_16x16x32_{bf16,f16} wants 8 consecutive k per lane, so a
// lane loads 8 rows of 8 columns and transposes 8 x 8 halfwords (one v_perm_b32 per dword of the result); 16 lanes
// cover 128 columns, the four lane groups 32 rows, a wave takes four such blocks. Raw sums in planes like fp8.
// ---------------------------------------------------------------------------
constexpr int kMfmaMinRowsInt8 = 4, kMfmaMaxRows = 16, kMfmaWaves = 4;
// The K-packed int8 layout of the dot4 entry point (B(4P + p, j) at P * b_sk + 4 j + p) needs no transposes at all:
// a 128-bit load holds four columns times four k, so four loads at consecutive P give a lane the 16 consecutive k
// of four columns, dword c of the four loads being the operand of column c. 16 lanes cover 64 columns (256 bytes
// of a row of groups), a block is 64 k by 64 columns and four instructions, a wave takes four blocks.
template <int ES, bool K4 = false>
struct MfmaShape {
  static constexpr int kLaneCols = K4 ? 4 : 16 / ES;  // columns in a 128-bit load = instructions per block
  static constexpr int kLaneRows = K4 ? 4 : 16 / ES;  // loads of a lane per block
  static constexpr int kKPerLoad = K4 ? 4 : 1;        // k a load covers: kLaneRows * kKPerLoad = k per lane and block
  static constexpr int kBlockK = 4 * kLaneRows * kKPerLoad;  // 64 or 32
  static constexpr int kIters = K4 ? 4 : 32 / kLaneRows;  // blocks per wave: 32 loads in flight per lane (K-packed: 16 -
                                                          // with 32 the kernel needs 378 registers, one wave per SIMD)
  static constexpr int kTileCols = 16 * kLaneCols;    // 256, 128 or 64
  static constexpr int kKPerGroup = kMfmaWaves * kIters * kBlockK;  // 512 (K-packed: 1024)
  static constexpr int kPitch = kTileCols + 4;        // 4-byte words per row of the LDS block
  static constexpr size_t kLds = (size_t)kMfmaWaves * 16 * kPitch * 4;
};

struct GemvMfmaArgs {
  const char *a;   // rows of A: K contiguous elements, a_row bytes apart, 16-byte aligned
  size_t a_row;
  const char *b;   // B(k, j) at (j / 64) * b_s1 + (j % 64) * elemsize + k * b_sk (bytes)
  size_t b_sk, b_s1;
  int *c;          // element (i, j) at i * c_row + j * c_s
  size_t c_row, c_s;
  size_t m, n, k;
  skl_scalar alpha, beta;
  unsigned tiles, slabs;
  float *planes;        // floating point: slabs planes of m x n raw sums
  const float *bias;    // floating point: fused steps of the second pass, or null
  float *max;
  skl_requant rq;       // ... activation, requantised int8 copy
};

__global__ void __launch_bounds__(256) gemv_mfma_scale_c_kernel(GemvMfmaArgs p) {
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= p.m * p.n) return;
  int *c = p.c + (idx / p.n) * p.c_row + (idx % p.n) * p.c_s;
  *c = p.beta.i == 0 ? 0 : (int)((unsigned)p.beta.i * (unsigned)*c);
}

// C = beta*C + alpha * (sum of the planes, in order), then bias and maximum: the second pass of the floating-point kinds.
__global__ void __launch_bounds__(256) gemv_mfma_add_planes_kernel(GemvMfmaArgs p) {
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= p.m * p.n) return;
  // Eight planes are requested before the first is used (one memory round trip per eight, not per plane); the
  // sum still runs over the planes in order, starting from plane 0 itself.
  const float *plane = p.planes + idx;
  const size_t mn = p.m * p.n;
  float sum = plane[0];
  for (unsigned q0 = 1; q0 < p.slabs; q0 += 8) {
    float v[8];
#pragma unroll
    for (unsigned u = 0; u < 8; ++u) v[u] = q0 + u < p.slabs ? plane[(size_t)(q0 + u) * mn] : 0.0f;
#pragma unroll
    for (unsigned u = 0; u < 8; ++u)
      if (q0 + u < p.slabs) sum = __fadd_rn(sum, v[u]);
  }
  const size_t col = idx % p.n;
  float *c = reinterpret_cast<float *>(p.c) + (idx / p.n) * p.c_row + col * p.c_s;
  float v = skl_beta_is_zero<float>(p.beta) ? skl_initialise(sum, c, p.alpha, p.beta) : skl_combine(sum, *c, p.alpha, p.beta);
  if (p.bias) v = skl_add_bias(v, p.bias[col]);
  v = skl_activate(v, p.rq.act);
  if (!p.rq.q_only) *c = v;
  skl_emit_requantised(p.rq, v, idx / p.n, col);
  if (p.max && v > skl_lowest<float>()) skl_atomic_max(p.max, v);
}

// WHOLE: n is a whole number of column tiles and k of workgroup ranges (checked by the launcher), so no load is
// guarded - the guarded kernel's compares and selects on 32 addresses per lane cost 1.5 to 2 us of a 13 us call.
template <int MODE, bool WHOLE = false>
__global__ void __launch_bounds__(kMfmaWaves * 64) gemv_mfma_rows_kernel(GemvMfmaArgs p) {
  constexpr bool kInt = MODE == kI8RowMajor || MODE == kI8K4, k16 = MODE == kBF16 || MODE == kF16;
  constexpr bool kPacked = MODE == kI8K4;
  constexpr int ES = k16 ? 2 : 1;
  using Sh = MfmaShape<ES, kPacked>;
  constexpr int LC = Sh::kLaneCols, LR = Sh::kLaneRows, ITERS = Sh::kIters;
  using Acc = typename Mode<MODE>::Acc;  // int or float: 4 bytes either way
  typedef Acc v4acc __attribute__((ext_vector_type(4)));
  typedef int v4i __attribute__((ext_vector_type(4)));
  extern __shared__ __attribute__((aligned(16))) int mfma_red_raw[];
  Acc(*red)[16][Sh::kPitch] = reinterpret_cast<Acc(*)[16][Sh::kPitch]>(mfma_red_raw);
  const unsigned tile = blockIdx.x % p.tiles, slab = blockIdx.x / p.tiles;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int jl = lane & 15, g = lane >> 4;
  const size_t col = (size_t)tile * Sh::kTileCols + (size_t)jl * LC;  // the lane's columns: inside one block of 64
  const size_t kwave = ((size_t)slab * kMfmaWaves + wave) * (Sh::kBlockK * ITERS);
  const bool col_ok = WHOLE || col < p.n;  // n is a multiple of the columns per lane
  const char *bp = kPacked ? p.b + col * 4 : p.b + (col >> 6) * p.b_s1 + (col & 63) * ES;
  constexpr int kLaneK = LR * Sh::kKPerLoad;  // k of a lane per block: 16 bytes of A

  uint4 rows[ITERS][LR];
  v4i xa[ITERS];
  // A's pieces are requested ahead of B's: loads come back in the order of their requests, so with A behind B the
  // first block's multiplications would wait for the last block's rows (0.75 us of a 15 us call).
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    // k is a multiple of a lane's k per block: a 16-byte piece of a row of A is inside or outside
    const size_t k0 = kwave + (size_t)it * Sh::kBlockK + (size_t)g * kLaneK;
    if ((size_t)jl < p.m && (WHOLE || k0 < p.k))
      xa[it] = *reinterpret_cast<const v4i *>(p.a + (size_t)jl * p.a_row + k0 * ES);
    else
      xa[it] = v4i{0, 0, 0, 0};
  }
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const size_t k0 = kwave + (size_t)it * Sh::kBlockK + (size_t)g * kLaneK;
#pragma unroll
    for (int r = 0; r < LR; ++r) {
      if (WHOLE || (col_ok && k0 + (size_t)r * Sh::kKPerLoad < p.k))
        rows[it][r] = stream_load(bp + (k0 / Sh::kKPerLoad + r) * p.b_sk);
      else
        rows[it][r] = make_uint4(0, 0, 0, 0);
    }
  }
  v4acc acc[LC];
#pragma unroll
  for (int c = 0; c < LC; ++c) acc[c] = v4acc{0, 0, 0, 0};
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    unsigned t[4][LC];  // [dword of the operand][column]: the lane's k of one column, ascending
    if constexpr (kPacked) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        t[q][0] = rows[it][q].x, t[q][1] = rows[it][q].y, t[q][2] = rows[it][q].z, t[q][3] = rows[it][q].w;
      }
    } else if constexpr (k16) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {  // rows 2q and 2q + 1 of the block
        const uint4 lo = rows[it][2 * q], hi = rows[it][2 * q + 1];
        const unsigned l4[4] = {lo.x, lo.y, lo.z, lo.w}, h4[4] = {hi.x, hi.y, hi.z, hi.w};
#pragma unroll
        for (int d = 0; d < 4; ++d) {  // dword d holds columns 2d and 2d + 1
          t[q][2 * d] = __builtin_amdgcn_perm(h4[d], l4[d], 0x05040100u);      // low halves: row 2q, row 2q + 1
          t[q][2 * d + 1] = __builtin_amdgcn_perm(h4[d], l4[d], 0x07060302u);  // high halves
        }
      }
    } else {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const uint4 r0 = rows[it][4 * q], r1 = rows[it][4 * q + 1], r2 = rows[it][4 * q + 2], r3 = rows[it][4 * q + 3];
        const unsigned a0[4] = {r0.x, r0.y, r0.z, r0.w}, a1[4] = {r1.x, r1.y, r1.z, r1.w};
        const unsigned a2[4] = {r2.x, r2.y, r2.z, r2.w}, a3[4] = {r3.x, r3.y, r3.z, r3.w};
#pragma unroll
        for (int d = 0; d < 4; ++d)
          transpose4x4(a0[d], a1[d], a2[d], a3[d], t[q][4 * d], t[q][4 * d + 1], t[q][4 * d + 2], t[q][4 * d + 3]);
      }
    }
#pragma unroll
    for (int c = 0; c < LC; ++c) {
      const v4i bw = {(int)t[0][c], (int)t[1][c], (int)t[2][c], (int)t[3][c]};
      if constexpr (kInt) {
        acc[c] = __builtin_amdgcn_mfma_i32_16x16x64_i8(xa[it], bw, acc[c], 0, 0, 0);
      } else if constexpr (MODE == kBF16) {
        typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
        acc[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, xa[it]), __builtin_bit_cast(v8bf, bw),
                                                         acc[c], 0, 0, 0);
      } else if constexpr (MODE == kF16) {
        typedef _Float16 v8h __attribute__((ext_vector_type(8)));
        acc[c] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, xa[it]), __builtin_bit_cast(v8h, bw),
                                                        acc[c], 0, 0, 0);
      } else {
        // OCP fp8: both operands are widened to f16 in registers - every E4M3 and E5M2 value is an f16 value - and
        // multiplied by the f16 instruction: exact products, fp32 sums, so the reference's own error bound holds.
        // (The fp8 instructions align the products of one instruction to a common exponent and drop what falls
        // about 12 bits below the largest: more than that bound allows when K is small. The conversions cost one
        // VALU operation per two bytes, which this kernel has to spare.) 8 k per lane and instruction: the lane's
        // 16 k in two halves, A's bytes split the same way.
        constexpr bool a_e5m2 = MODE == kF8E5M2, b_e5m2 = MODE != kF8E4M3;
        acc[c] = __builtin_amdgcn_mfma_f32_16x16x32_f16(skl_fp8::widen8_to_f16<a_e5m2>((unsigned)xa[it].x, (unsigned)xa[it].y),
                                                        skl_fp8::widen8_to_f16<b_e5m2>(t[0][c], t[1][c]), acc[c], 0, 0, 0);
        acc[c] = __builtin_amdgcn_mfma_f32_16x16x32_f16(skl_fp8::widen8_to_f16<a_e5m2>((unsigned)xa[it].z, (unsigned)xa[it].w),
                                                        skl_fp8::widen8_to_f16<b_e5m2>(t[2][c], t[3][c]), acc[c], 0, 0, 0);
      }
    }
  }
  // acc[c][r] is row 4 g + r of C, column LC jl + c of the tile.
#pragma unroll
  for (int r = 0; r < 4; ++r)
#pragma unroll
    for (int c4 = 0; c4 < LC / 4; ++c4)
      *reinterpret_cast<v4acc *>(&red[wave][4 * g + r][LC * jl + 4 * c4]) =
          v4acc{acc[4 * c4][r], acc[4 * c4 + 1][r], acc[4 * c4 + 2][r], acc[4 * c4 + 3][r]};
  __syncthreads();
  // 256 threads: one column each (two rows of C at a time for the 128-column tiles)
  constexpr int kRowStep = kMfmaWaves * 64 / Sh::kTileCols;
  const int tc = threadIdx.x % Sh::kTileCols;
  const size_t j = (size_t)tile * Sh::kTileCols + tc;
  if (!WHOLE && j >= p.n) return;
  // All rows' sums are read from LDS before the first goes out (a loop over the rows of A would pay an LDS round
  // trip per row).
  constexpr int kPasses = kMfmaMaxRows / kRowStep;
  const int i0 = threadIdx.x / Sh::kTileCols;
  Acc sums[kPasses];
#pragma unroll
  for (int q = 0; q < kPasses; ++q) {
    const int i = i0 + q * kRowStep;
    if constexpr (kInt) {
      unsigned sum = 0;
#pragma unroll
      for (int w = 0; w < kMfmaWaves; ++w) sum += (unsigned)red[w][i][tc];
      sums[q] = (int)((unsigned)p.alpha.i * sum);
    } else {
      float sum = red[0][i][tc];
#pragma unroll
      for (int w = 1; w < kMfmaWaves; ++w) sum = __fadd_rn(sum, red[w][i][tc]);
      sums[q] = sum;
    }
  }
  if constexpr (kInt) {
    int *cp = p.c + (size_t)i0 * p.c_row + j * p.c_s;
#pragma unroll
    for (int q = 0; q < kPasses; ++q)
      if ((size_t)(i0 + q * kRowStep) < p.m)
        (void)__hip_atomic_fetch_add(cp + (size_t)q * kRowStep * p.c_row, sums[q], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  } else {
    // past the compute die's L2: the second kernel runs on every die, and lines left dirty here would have to be
    // written back between the two kernels (16 x 4096 x 11008: 1 us of a 16 us call)
    float *plane = p.planes + (size_t)slab * p.m * p.n + (size_t)i0 * p.n + j;
#pragma unroll
    for (int q = 0; q < kPasses; ++q)
      if ((size_t)(i0 + q * kRowStep) < p.m) __builtin_nontemporal_store(sums[q], plane + (size_t)q * kRowStep * p.n);
  }
}


// ---------------------------------------------------------------------------
// 17 to 128 rows of int8 A: the kernel above with RG groups of 16 rows, for the K-packed B (any K beyond what the
// whole-K kernel below takes) and for the row-major B. B's bytes are loaded once - and, row-major, transposed once -
// and stay in registers while the row groups take their turns (a pass over B per 16 rows, as chunked calls of the
// kernel above cost, is what this saves: K-packed 112 x 4096 x 11008 took 110 us in seven passes; the tile kernels
// take 29 / 31 us for 32 / 64 rows against a row-major B). The A fragment of a row group - 16 bytes per lane and
// block, from L2 - is requested two groups ahead; the sums of a group go through the same LDS block as above, one
// group at a time, and meet the other workgroups' in C.
// ---------------------------------------------------------------------------
constexpr int kK4MaxRowGroups = 8;
constexpr int kRowMajorMaxRows = 32;  // row-major B: rows of A up to which the row groups beat the tile kernels (4096 x 11008 weights: 32
                                      // rows 19.5 against 20.3 us, 64 rows 27.4 against 24.1, 128 rows 42.5 against 28.8)

template <int MODE, int RG>
__global__ void __launch_bounds__(kMfmaWaves * 64, 2) gemv_rowgroups_kernel(GemvMfmaArgs p) {
  constexpr bool kPacked = MODE == kI8K4;
  static_assert(kPacked || MODE == kI8RowMajor, "int8 only");
  using Sh = MfmaShape<1, kPacked>;
  constexpr int LC = Sh::kLaneCols, LR = Sh::kLaneRows, ITERS = Sh::kIters;
  constexpr int kLaneK = LR * Sh::kKPerLoad;  // 16
  typedef int v4i __attribute__((ext_vector_type(4)));
  extern __shared__ __attribute__((aligned(16))) int mfma_red_raw[];
  int(*red)[16][Sh::kPitch] = reinterpret_cast<int(*)[16][Sh::kPitch]>(mfma_red_raw);
  const unsigned tile = blockIdx.x % p.tiles, slab = blockIdx.x / p.tiles;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int jl = lane & 15, g = lane >> 4;
  const size_t col = (size_t)tile * Sh::kTileCols + (size_t)jl * LC;
  const size_t kwave = ((size_t)slab * kMfmaWaves + wave) * (Sh::kBlockK * ITERS);
  const size_t colc = col < p.n ? col : 0;  // n is a multiple of the columns per lane: a lane is inside or outside
  const char *bp = kPacked ? p.b + colc * 4 : p.b + (colc >> 6) * p.b_s1 + (colc & 63);

  // The lane's 16 k of row 16 rg + jl, for each of the wave's blocks: loaded from inside A, zeroed beyond M and K
  // (k is a multiple of 16) - which is also what makes the rows of B beyond K, read as row 0, count for nothing.
  auto fragment_of = [&](int rg, v4i(&xa)[ITERS]) {
    const size_t row = (size_t)rg * 16 + jl;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const size_t k0 = kwave + (size_t)it * Sh::kBlockK + (size_t)g * kLaneK;
      const bool inside = row < p.m && k0 < p.k;
      const v4i v = *reinterpret_cast<const v4i *>(p.a + (row < p.m ? row : p.m - 1) * p.a_row + (k0 < p.k ? k0 : 0));
      xa[it] = v4i{inside ? v.x : 0, inside ? v.y : 0, inside ? v.z : 0, inside ? v.w : 0};
    }
  };
  v4i xa[3][ITERS];
  fragment_of(0, xa[0]);  // ahead of B: loads come back in the order of their requests
  uint4 rows[ITERS][LR];
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const size_t k0 = kwave + (size_t)it * Sh::kBlockK + (size_t)g * kLaneK;
#pragma unroll
    for (int r = 0; r < LR; ++r) {
      const size_t kr = k0 + (size_t)r * Sh::kKPerLoad;
      rows[it][r] = stream_load(bp + ((kr < p.k ? kr : 0) / Sh::kKPerLoad) * p.b_sk);  // clamped, not guarded
    }
  }
  if constexpr (RG > 1) fragment_of(1, xa[1]);
  __builtin_amdgcn_sched_barrier(0);  // every request is out before the first use
  // t[it][q][c]: dword q of the operand of column c in block it - the lane's 16 k of that column, ascending
  unsigned t[ITERS][4][LC];
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    if constexpr (kPacked) {
#pragma unroll
      for (int q = 0; q < 4; ++q) t[it][q][0] = rows[it][q].x, t[it][q][1] = rows[it][q].y, t[it][q][2] = rows[it][q].z, t[it][q][3] = rows[it][q].w;
    } else {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const uint4 r0 = rows[it][4 * q], r1 = rows[it][4 * q + 1], r2 = rows[it][4 * q + 2], r3 = rows[it][4 * q + 3];
        const unsigned a0[4] = {r0.x, r0.y, r0.z, r0.w}, a1[4] = {r1.x, r1.y, r1.z, r1.w};
        const unsigned a2[4] = {r2.x, r2.y, r2.z, r2.w}, a3[4] = {r3.x, r3.y, r3.z, r3.w};
#pragma unroll
        for (int d = 0; d < 4; ++d)
          transpose4x4(a0[d], a1[d], a2[d], a3[d], t[it][q][4 * d], t[it][q][4 * d + 1], t[it][q][4 * d + 2], t[it][q][4 * d + 3]);
      }
    }
  }
  constexpr int kRowStep = kMfmaWaves * 64 / Sh::kTileCols;  // 4 (K-packed), 1 (row-major)
  constexpr int kPasses = 16 / kRowStep;
  const int tc = threadIdx.x % Sh::kTileCols, i0 = threadIdx.x / Sh::kTileCols;
  const size_t j = (size_t)tile * Sh::kTileCols + tc;
#pragma unroll
  for (int rg = 0; rg < RG; ++rg) {
    if (rg + 2 < RG) fragment_of(rg + 2, xa[(rg + 2) % 3]);
    if ((size_t)rg * 16 >= p.m) break;  // the same for every thread of the workgroup
    v4i acc[LC];
#pragma unroll
    for (int c = 0; c < LC; ++c) acc[c] = v4i{0, 0, 0, 0};
#pragma unroll
    for (int it = 0; it < ITERS; ++it)
#pragma unroll
      for (int c = 0; c < LC; ++c) {
        const v4i bw = {(int)t[it][0][c], (int)t[it][1][c], (int)t[it][2][c], (int)t[it][3][c]};
        acc[c] = __builtin_amdgcn_mfma_i32_16x16x64_i8(xa[rg % 3][it], bw, acc[c], 0, 0, 0);
      }
    // acc[c][r] is row 16 rg + 4 g + r of C, column LC jl + c of the tile.
    if (rg > 0) __syncthreads();  // the previous group's sums have been read
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
      for (int c4 = 0; c4 < LC / 4; ++c4)
        *reinterpret_cast<v4i *>(&red[wave][4 * g + r][LC * jl + 4 * c4]) = v4i{acc[4 * c4][r], acc[4 * c4 + 1][r], acc[4 * c4 + 2][r], acc[4 * c4 + 3][r]};
    __syncthreads();
    // all of the thread's sums are read from LDS before the first goes out
    int sums[kPasses];
#pragma unroll
    for (int q = 0; q < kPasses; ++q) {
      unsigned sum = 0;
#pragma unroll
      for (int w = 0; w < kMfmaWaves; ++w) sum += (unsigned)red[w][i0 + q * kRowStep][tc];
      sums[q] = (int)((unsigned)p.alpha.i * sum);
    }
    if (j < p.n) {
      int *cp = p.c + ((size_t)rg * 16 + i0) * p.c_row + j * p.c_s;
#pragma unroll
      for (int q = 0; q < kPasses; ++q)
        if ((size_t)rg * 16 + i0 + q * kRowStep < p.m)
          (void)__hip_atomic_fetch_add(cp + (size_t)q * kRowStep * p.c_row, sums[q], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

// ---------------------------------------------------------------------------
// The K-packed B again, K <= 4096 and 2 to 128 rows of A: one workgroup of eight waves per 64 columns takes ALL of K
// (512 k per wave: 32 loads per lane, the whole of B in flight from the start), so the sums of a column tile never
// leave the workgroup - they meet in LDS, C is written once with the alpha / beta step applied in place, and neither
// the kernel that scales C in front nor the atomic adds into C (one per element and quarter of K above: 19.7 MB next
// to 45 MB of weights for 112 x 4096 x 11008) are needed. Loads are clamped into the operands instead of guarded -
// a guard is a branch, and the compiler waits for every earlier load at a branch it cannot prove uniform; rows
// beyond K meet zeros of A, columns beyond N are computed and not written.
// Up to three row groups: the waves write their 16 x 64 sums side by side, one barrier per group (two blocks take
// turns). From four groups on the waves add into one plane with LDS atomics and meet once at the end: barriers would
// keep them in step, and out of step they hide each other's waits for the next group's pieces of A (an L2 round trip
// each - every workgroup reads all of A, which is what bounds this kernel from about 64 rows on).
// 4096 x 11008 weights: 16 rows 11.2 us (13.4 with the kernels above), 32 rows 13.0 (18.4), 112 rows 24.1 (30.4).
// ---------------------------------------------------------------------------
constexpr int kK4WholeWaves = 8, kK4WholeIters = 8, kK4WholePitch = 68;
constexpr size_t kK4WholeMaxK = (size_t)kK4WholeWaves * kK4WholeIters * 64;
constexpr size_t k4_whole_lds(int rg) {
  return (rg >= 4 ? (size_t)rg * 16 : (size_t)2 * kK4WholeWaves * 16) * kK4WholePitch * sizeof(int);
}

template <int RG>
__global__ void __launch_bounds__(kK4WholeWaves * 64) gemv_k4_wholek_kernel(GemvMfmaArgs p) {
  constexpr bool kOnePlane = RG >= 4;
  constexpr int ITERS = kK4WholeIters, W = kK4WholeWaves, PITCH = kK4WholePitch;
  typedef int v4i __attribute__((ext_vector_type(4)));
  extern __shared__ __attribute__((aligned(16))) int mfma_red_raw[];
  const unsigned tile = blockIdx.x;
  // A second grid dimension deals the groups of RG * 16 rows out to workgroups of their own (problems with so few
  // column tiles that the chip is empty otherwise: B is small then, and read once per workgroup).
  const size_t row0 = (size_t)blockIdx.y * (RG * 16), m = p.m - row0;
  const char *const a = p.a + row0 * p.a_row;
  int *const c = p.c + row0 * p.c_row;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int jl = lane & 15, g = lane >> 4;
  const size_t col = (size_t)tile * 64 + (size_t)jl * 4;
  const char *bp = p.b + (col < p.n ? col : p.n - 4) * 4;  // n is a multiple of four
  const size_t kwave = (size_t)wave * (64 * ITERS);
  // The lane's 16 k of row 16 rg + jl for each of the wave's blocks: loaded from inside A, zeroed beyond M and K.
  auto fragment_of = [&](int rg, v4i(&xa)[ITERS]) {
    const size_t row = (size_t)rg * 16 + jl;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const size_t k0 = kwave + (size_t)it * 64 + (size_t)g * 16;
      const bool inside = row < m && k0 < p.k;  // k is a multiple of 16
      const v4i v = *reinterpret_cast<const v4i *>(a + (row < m ? row : m - 1) * p.a_row + (k0 < p.k ? k0 : p.k - 16));
      xa[it] = v4i{inside ? v.x : 0, inside ? v.y : 0, inside ? v.z : 0, inside ? v.w : 0};
    }
  };
  v4i xa[2][ITERS];
  fragment_of(0, xa[0]);  // ahead of B: loads come back in the order of their requests
  uint4 rows[ITERS][4];
  const size_t groups = p.k / 4;
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const size_t k0 = kwave + (size_t)it * 64 + (size_t)g * 16;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const size_t group = k0 / 4 + r;
      rows[it][r] = stream_load(bp + (group < groups ? group : groups - 1) * p.b_sk);
    }
  }
  if constexpr (RG > 1) fragment_of(1, xa[1]);
  __builtin_amdgcn_sched_barrier(0);  // every request is out before the first use (the scheduler would otherwise
                                      // sink loads to their uses to save registers: 12 in flight instead of 32)
  int(*plane)[PITCH] = reinterpret_cast<int(*)[PITCH]>(mfma_red_raw);
  if constexpr (kOnePlane) {  // zeroed while the loads are under way
    for (int idx = threadIdx.x; idx < RG * 16 * PITCH / 4; idx += W * 64) reinterpret_cast<v4i *>(mfma_red_raw)[idx] = v4i{0, 0, 0, 0};
    __syncthreads();
  }
  const int tc = threadIdx.x & 63;
  const size_t j = (size_t)tile * 64 + tc;
#pragma unroll
  for (int rg = 0; rg < RG; ++rg) {
    if ((size_t)rg * 16 >= m) break;  // the same for every thread of the workgroup
    v4i acc[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) acc[c] = v4i{0, 0, 0, 0};
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const unsigned t[4][4] = {{rows[it][0].x, rows[it][0].y, rows[it][0].z, rows[it][0].w},
                                {rows[it][1].x, rows[it][1].y, rows[it][1].z, rows[it][1].w},
                                {rows[it][2].x, rows[it][2].y, rows[it][2].z, rows[it][2].w},
                                {rows[it][3].x, rows[it][3].y, rows[it][3].z, rows[it][3].w}};
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const v4i bw = {(int)t[0][c], (int)t[1][c], (int)t[2][c], (int)t[3][c]};
        acc[c] = __builtin_amdgcn_mfma_i32_16x16x64_i8(xa[rg & 1][it], bw, acc[c], 0, 0, 0);
      }
    }
    if (rg + 2 < RG) fragment_of(rg + 2, xa[rg & 1]);
    // acc[c][r] is row 16 rg + 4 g + r of C, column 4 jl + c of the tile.
    if constexpr (kOnePlane) {
#pragma unroll
      for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int c = 0; c < 4; ++c)
          (void)__hip_atomic_fetch_add(&plane[rg * 16 + 4 * g + r][4 * jl + c], acc[c][r], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    } else {
      // two blocks take turns: the next group's barrier stands between this group's readers and the writers of
      // the group after it
      int(*red)[16][PITCH] = reinterpret_cast<int(*)[16][PITCH]>(mfma_red_raw + (rg & 1) * W * 16 * PITCH);
#pragma unroll
      for (int r = 0; r < 4; ++r) *reinterpret_cast<v4i *>(&red[wave][4 * g + r][4 * jl]) = v4i{acc[0][r], acc[1][r], acc[2][r], acc[3][r]};
      __syncthreads();
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        const int il = (threadIdx.x >> 6) + W * q;
        const size_t i = (size_t)rg * 16 + il;
        unsigned sum = 0;
#pragma unroll
        for (int w = 0; w < W; ++w) sum += (unsigned)red[w][il][tc];
        if (i < m && j < p.n) skl_update((int)sum, c + i * p.c_row + j * p.c_s, p.alpha, p.beta);
      }
    }
  }
  if constexpr (kOnePlane) {
    __syncthreads();
    if (j >= p.n) return;
#pragma unroll
    for (int q = 0; q < RG * 16 / W; ++q) {
      const size_t i = (size_t)(threadIdx.x >> 6) + (size_t)q * W;
      if (i < m) skl_update(plane[i][tc], c + i * p.c_row + j * p.c_s, p.alpha, p.beta);
    }
  }
}

// ---------------------------------------------------------------------------
// B with K contiguous (column j is K consecutive elements, columns a fixed distance apart - how a linear
// layer's weight [out][in] is stored): every output is a dot product over contiguous memory. A wave owns
// two or four columns and walks K one KiB (64 lanes x 16 bytes) at a time, kKcUnroll KiB per column in
// flight; the x values of a KiB are loaded once per row of A (1 to 4 rows) and reused by the columns.
// The lanes' sums are combined inside the wave (DPP rotations, then two cross-lane exchanges), and
// lane 0 writes the results: no sums between workgroups, no scratch, a fixed summation order.
// ---------------------------------------------------------------------------
constexpr int kKcUnroll = 4, kKcWaves = 4, kKcMaxRows = 4;
// Columns per wave: two with one row of A (twice the waves in flight measured 8.4 us against 11.2 us with four
// on the 45 MB case), four with more rows, where the x values a wave loads are shared by more columns.
constexpr int kc_cols(int rows) { return rows == 1 ? 2 : 4; }

struct GemvKcArgs {
  const char *x;   // rows of A: K contiguous elements, x_row bytes apart
  size_t x_row;
  const char *b;   // column j at b + j * b_col (bytes)
  size_t b_col;
  char *y;         // element (i, j) at i * y_row + j * y_s (elements)
  size_t y_row, y_s;
  size_t n, kbytes;
  skl_scalar alpha, beta;
  const char *bias;  // FUSED kernels: the steps behind alpha / beta (bias and maximum of y's type, or null) ...
  char *max;
  skl_requant rq;    // ... activation and 8-bit copy
};

template <typename T>
__device__ __forceinline__ T wave_sum(T v) {
  // rows of 16 lanes: four DPP rotations leave the row's sum in every lane; the four rows are then combined
  // through the cross-lane network (two exchanges per value, once per wave). The row-swap instructions
  // (v_permlane16_swap / v_permlane32_swap) are not used: given the same value for both operands the
  // compiler folds the sum of their two results into twice the first one.
  unsigned u;
#define SKL_ROTATE_ADD(ctrl)                                                              \
  u = (unsigned)__builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, 0xF, 0xF, false); \
  v += __builtin_bit_cast(T, u);
  SKL_ROTATE_ADD(0x128)
  SKL_ROTATE_ADD(0x124)
  SKL_ROTATE_ADD(0x122)
  SKL_ROTATE_ADD(0x121)
#undef SKL_ROTATE_ADD
  v += __shfl_xor(v, 16, 64);
  v += __shfl_xor(v, 32, 64);
  return v;
}

// acc += sum over the 16 bytes of w and x (elements of kind MODE)
template <int MODE>
__device__ __forceinline__ void dot16(const uint4 &w, const uint4 &x, typename Mode<MODE>::Acc &acc) {
  const unsigned ww[4] = {w.x, w.y, w.z, w.w}, xx[4] = {x.x, x.y, x.z, x.w};
  if constexpr (MODE == kI8RowMajor) {
#pragma unroll
    for (int d = 0; d < 4; ++d) acc = __builtin_amdgcn_sdot4((int)ww[d], (int)xx[d], acc, false);
  } else if constexpr (Mode<MODE>::kFp8) {
    constexpr bool x_e5m2 = MODE == kF8E5M2, b_e5m2 = MODE != kF8E4M3;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const v2f w_lo = b_e5m2 ? __builtin_amdgcn_cvt_pk_f32_bf8((int)ww[d], false) : __builtin_amdgcn_cvt_pk_f32_fp8((int)ww[d], false);
      const v2f w_hi = b_e5m2 ? __builtin_amdgcn_cvt_pk_f32_bf8((int)ww[d], true) : __builtin_amdgcn_cvt_pk_f32_fp8((int)ww[d], true);
      const v2f x_lo = x_e5m2 ? __builtin_amdgcn_cvt_pk_f32_bf8((int)xx[d], false) : __builtin_amdgcn_cvt_pk_f32_fp8((int)xx[d], false);
      const v2f x_hi = x_e5m2 ? __builtin_amdgcn_cvt_pk_f32_bf8((int)xx[d], true) : __builtin_amdgcn_cvt_pk_f32_fp8((int)xx[d], true);
      acc = __fmaf_rn(x_lo.x, w_lo.x, acc);
      acc = __fmaf_rn(x_lo.y, w_lo.y, acc);
      acc = __fmaf_rn(x_hi.x, w_hi.x, acc);
      acc = __fmaf_rn(x_hi.y, w_hi.y, acc);
    }
  } else {
    constexpr bool bf = MODE == kBF16;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      acc = __fmaf_rn(widen16(xx[d] & 0xFFFFu, bf), widen16(ww[d] & 0xFFFFu, bf), acc);
      acc = __fmaf_rn(widen16(xx[d] >> 16, bf), widen16(ww[d] >> 16, bf), acc);
    }
  }
}

// FUSED: the lane that writes an element applies the fused steps (bias, activation, 8-bit copy, maximum) to it.
template <int MODE, int MR, bool FUSED = false>
__global__ void __launch_bounds__(kKcWaves * 64) gemv_kc_kernel(GemvKcArgs p) {
  using Acc = typename Mode<MODE>::Acc;
  constexpr int kKcCols = kc_cols(MR);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const size_t col0 = ((size_t)blockIdx.x * kKcWaves + wave) * kKcCols;
  if (col0 >= p.n) return;  // whole waves leave; no barrier follows
  Acc acc[MR][kKcCols];
#pragma unroll
  for (int i = 0; i < MR; ++i)
#pragma unroll
    for (int c = 0; c < kKcCols; ++c) acc[i][c] = 0;
  const char *col_ptr[kKcCols];
#pragma unroll
  for (int c = 0; c < kKcCols; ++c) {
    const size_t col = col0 + c < p.n ? col0 + c : p.n - 1;  // a column past the end repeats the last one; not written
    col_ptr[c] = p.b + col * p.b_col;
  }
  const uint4 zero = make_uint4(0, 0, 0, 0);
  for (size_t base = 0; base < p.kbytes; base += (size_t)kKcUnroll * 1024) {
    uint4 w[kKcUnroll][kKcCols], xs[kKcUnroll][MR];
    if (base + (size_t)kKcUnroll * 1024 <= p.kbytes) {  // the whole block is inside K: no per-load checks
#pragma unroll
      for (int u = 0; u < kKcUnroll; ++u) {
        const size_t off = base + (size_t)u * 1024 + (size_t)lane * 16;
#pragma unroll
        for (int c = 0; c < kKcCols; ++c) w[u][c] = stream_load(col_ptr[c] + off);
#pragma unroll
        for (int i = 0; i < MR; ++i) xs[u][i] = *reinterpret_cast<const uint4 *>(p.x + (size_t)i * p.x_row + off);
      }
    } else {
#pragma unroll
      for (int u = 0; u < kKcUnroll; ++u) {
        const size_t off = base + (size_t)u * 1024 + (size_t)lane * 16;
        const bool in = off < p.kbytes;  // K bytes are a multiple of 16: a 16-byte piece is inside or outside
#pragma unroll
        for (int c = 0; c < kKcCols; ++c) w[u][c] = in ? stream_load(col_ptr[c] + off) : zero;
#pragma unroll
        for (int i = 0; i < MR; ++i) xs[u][i] = in ? *reinterpret_cast<const uint4 *>(p.x + (size_t)i * p.x_row + off) : zero;
      }
    }
#pragma unroll
    for (int u = 0; u < kKcUnroll; ++u)
#pragma unroll
      for (int i = 0; i < MR; ++i)
#pragma unroll
        for (int c = 0; c < kKcCols; ++c) dot16<MODE>(w[u][c], xs[u][i], acc[i][c]);
  }
#pragma unroll
  for (int i = 0; i < MR; ++i)
#pragma unroll
    for (int c = 0; c < kKcCols; ++c) acc[i][c] = wave_sum(acc[i][c]);
  if (lane == 0) {
    Acc *yv = reinterpret_cast<Acc *>(p.y);
    Acc largest = skl_lowest<Acc>();
#pragma unroll
    for (int i = 0; i < MR; ++i)
#pragma unroll
      for (int c = 0; c < kKcCols; ++c) {
        if (col0 + c >= p.n) continue;
        Acc *y = yv + (size_t)i * p.y_row + (col0 + c) * p.y_s;
        if constexpr (FUSED) {
          Acc v = skl_beta_is_zero<Acc>(p.beta) ? skl_initialise(acc[i][c], y, p.alpha, p.beta) : skl_combine(acc[i][c], *y, p.alpha, p.beta);
          if (p.bias) v = skl_add_bias(v, reinterpret_cast<const Acc *>(p.bias)[col0 + c]);
          v = skl_activate(v, p.rq.act);
          if (!p.rq.q_only) *y = v;
          skl_emit_requantised(p.rq, v, (size_t)i, col0 + c);
          if (v > largest) largest = v;
        } else {
          skl_update(acc[i][c], y, p.alpha, p.beta);
        }
      }
    if constexpr (FUSED) {
      if (p.max && largest > skl_lowest<Acc>()) skl_atomic_max(reinterpret_cast<Acc *>(p.max), largest);  // one per wave
    }
  }
}

inline bool aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }

int mode_of(const skl_gemm_canon *g, int layout) {
  if (layout == 1) return (g->ta == SKL_DT_I8 && g->tb == SKL_DT_I8) ? kI8K4 : -1;
  if (g->ta == SKL_DT_F8E4M3 && g->tb == SKL_DT_F8E5M2) return kF8Mixed;
  if (g->ta != g->tb) return -1;
  switch (g->ta) {
    case SKL_DT_I8: return kI8RowMajor;
    case SKL_DT_BF16: return kBF16;
    case SKL_DT_F16: return kF16;
    case SKL_DT_F8E4M3: return kF8E4M3;
    case SKL_DT_F8E5M2: return kF8E5M2;
    default: return -1;
  }
}

template <int MODE>
int launch(const skl_gemm_canon *g, const Reduction &red) {
  using Md = Mode<MODE>;
  GemvArgs p;
  p.x = (const char *)g->a;
  p.x_sk = g->a_sk;
  p.x_vec = (g->a_sk == 1 && aligned16(g->a)) ? 1 : 0;
  p.b = (const char *)g->b;
  p.b_sk = g->b_sk * Md::kES;
  p.b_s1 = g->b_s1 * Md::kES;
  p.y = (char *)g->c;
  p.y_s = g->csc0;
  p.n = g->n;
  p.k = g->k;
  p.alpha = g->alpha;
  p.beta = g->beta;
  p.acc = red.acc;
  p.tickets = red.tickets;
  p.tiles = skl_div_up(g->n, Md::kTileCols);
  // Eight loads per lane put every workgroup of a 45 MB stream on the chip at once (688 of 1024 places); a stream
  // with more than two rounds of workgroups runs 4 % shorter with sixteen (1 x 8192 x 28672: 44.5 -> 42.5 us),
  // the 45 MB one 10 % longer.
  const size_t groups8 = (size_t)p.tiles * skl_div_up(g->k, kPartials * 8 * Md::kKPerLoad);
  const int loads = groups8 > 2048 ? 16 : 8;
  p.slabs = skl_div_up(g->k, (size_t)kPartials * loads * Md::kKPerLoad);
  const size_t grid = (size_t)p.tiles * p.slabs;
  if (grid > 0x7FFFFFFFu) {
    skl_hip_record_error(-2, "gemv: grid too large");
    return -2;
  }
  p.planes = nullptr;
  if constexpr (!std::is_same<typename Md::Acc, int>::value) {
    if (p.slabs > 1 && !(p.planes = (float *)skl_workspace((size_t)p.slabs * p.n * sizeof(float)))) return -4;
  }
  p.bias = (const char *)g->bias, p.max = (char *)g->max;
  p.rq = g->rq;
  const bool fused = g->bias || g->max || g->rq.act || g->rq.q;
  if constexpr (MODE == kI8RowMajor || MODE == kBF16 || MODE == kF16) {
    // strips and row ranges that divide the matrix evenly: the kernel without guards, rows dealt 64 at a time
    // (1 x 4096 x 11008: int8 10.3 -> 9.9 us, bf16 21.2 -> 19.9 us; the fp8 kinds measured slower that way, 13.5
    // against 12.0 us, and stay on the guarded kernel)
    if (loads == 8 && g->n % Md::kTileCols == 0 && g->k % (size_t)(kPartials * 8) == 0 && p.slabs <= 65535) {
      const dim3 grid2(p.tiles, p.slabs);
      if (fused)
        gemv_kernel<MODE, 8, true, true><<<grid2, kWaves * 64, 0, skl_current_stream()>>>(p);
      else
        gemv_kernel<MODE, 8, false, true><<<grid2, kWaves * 64, 0, skl_current_stream()>>>(p);
      return skl_check_launch("gemv");
    }
  }
  if (fused && loads == 16)
    gemv_kernel<MODE, 16, true><<<(unsigned)grid, kWaves * 64, 0, skl_current_stream()>>>(p);
  else if (fused)
    gemv_kernel<MODE, 8, true><<<(unsigned)grid, kWaves * 64, 0, skl_current_stream()>>>(p);
  else if (loads == 16)
    gemv_kernel<MODE, 16><<<(unsigned)grid, kWaves * 64, 0, skl_current_stream()>>>(p);
  else
    gemv_kernel<MODE, 8><<<(unsigned)grid, kWaves * 64, 0, skl_current_stream()>>>(p);
  return skl_check_launch("gemv");
}


template <int MR, int MODE>
int launch_rows(const skl_gemm_canon *g, const Reduction &red) {
  using Md = Mode<MODE>;
  GemvRowsArgs p;
  p.x = (const char *)g->a;
  p.x_row = g->a_s0 * Md::kES;
  p.b = (const char *)g->b;
  p.b_sk = g->b_sk * Md::kES;
  p.b_s1 = g->b_s1 * Md::kES;
  p.y = (char *)g->c;
  p.y_row = g->rsc0;
  p.y_s = g->csc0;
  p.n = g->n;
  p.k = g->k;
  p.alpha = g->alpha;
  p.beta = g->beta;
  p.acc = red.acc;
  p.tickets = red.tickets;
  p.tiles = skl_div_up(g->n, Md::kTileCols);
  p.slabs = skl_div_up(g->k, Md::kKPerGroup);
  const size_t grid = (size_t)p.tiles * p.slabs;
  if (grid > 0x7FFFFFFFu) {
    skl_hip_record_error(-2, "gemv: grid too large");
    return -2;
  }
  p.planes = nullptr;
  if constexpr (MODE != kI8RowMajor) {
    if (p.slabs > 1 && !(p.planes = (float *)skl_workspace((size_t)p.slabs * MR * p.n * sizeof(float)))) return -4;
  }
  gemv_rows_kernel<MR, MODE><<<(unsigned)grid, kWaves * 64, 0, skl_current_stream()>>>(p);
  return skl_check_launch("gemv_rows");
}

// The floating-point kinds pay one multiply-add per element of B and row (there is no dot instruction over
// k for them) and are bound by that from four rows on, where the tile kernels are faster: they stop at three.
constexpr int kMaxRowsFloat = 3;

template <int MODE>
int launch_rows_of(const skl_gemm_canon *g, const Reduction &red) {
  if constexpr (MODE != kI8RowMajor) {
    return g->m == 2 ? launch_rows<2, MODE>(g, red) : launch_rows<3, MODE>(g, red);
  } else
  switch (g->m) {
    case 2: return launch_rows<2, MODE>(g, red);
    case 3: return launch_rows<3, MODE>(g, red);
    case 4: return launch_rows<4, MODE>(g, red);
    case 5: return launch_rows<5, MODE>(g, red);
    case 6: return launch_rows<6, MODE>(g, red);
    case 7: return launch_rows<7, MODE>(g, red);
    default: return launch_rows<8, MODE>(g, red);
  }
}


template <int MODE, int MR>
int launch_kc(const skl_gemm_canon *g) {
  constexpr size_t es = Mode<MODE>::kES;
  GemvKcArgs p;
  p.x = (const char *)g->a;
  p.x_row = g->a_s0 * es;
  p.b = (const char *)g->b;
  p.b_col = g->b_s0 * es;
  p.y = (char *)g->c;
  p.y_row = g->rsc0;
  p.y_s = g->csc0;
  p.n = g->n;
  p.kbytes = g->k * es;
  p.alpha = g->alpha;
  p.beta = g->beta;
  const size_t grid = (g->n + kKcWaves * kc_cols(MR) - 1) / (kKcWaves * kc_cols(MR));
  if (grid > 0x7FFFFFFFu) {
    skl_hip_record_error(-2, "gemv: grid too large");
    return -2;
  }
  p.bias = (const char *)g->bias, p.max = (char *)g->max;
  p.rq = g->rq;
  if (g->bias || g->max || g->rq.act || g->rq.q)
    gemv_kc_kernel<MODE, MR, true><<<(unsigned)grid, kKcWaves * 64, 0, skl_current_stream()>>>(p);
  else
    gemv_kc_kernel<MODE, MR><<<(unsigned)grid, kKcWaves * 64, 0, skl_current_stream()>>>(p);
  return skl_check_launch("gemv_kc");
}

template <int MODE>
int launch_kc_of(const skl_gemm_canon *g) {
  switch (g->m) {
    case 1: return launch_kc<MODE, 1>(g);
    case 2: return launch_kc<MODE, 2>(g);
    case 3: return launch_kc<MODE, 3>(g);
    default: return launch_kc<MODE, 4>(g);
  }
}

}  // namespace

extern "C" int skl_hip_gemv_supported(const skl_gemm_canon *g, int layout) {
  const int mode = mode_of(g, layout);
  if (mode < 0) return 0;
  if (g->c_row_shift != 6 || g->c_col_shift != 6) return 0;  // C in blocks of 64 (or flat) only
  if (g->m != 1 || g->k == 0 || g->n == 0 || g->n > kMaxCols) return 0;
  const size_t es = (mode == kBF16 || mode == kF16) ? 2 : 1;
  const size_t cols = (mode == kI8RowMajor || mode >= kF8E4M3) ? 16 : mode == kI8K4 ? 4 : 8;
  if ((g->n % cols) != 0 || !aligned16(g->b) || ((g->b_sk * es) % 16) != 0) return 0;
  if (mode != kI8K4 && (g->b_s0 != 1 || ((g->b_s1 * es) % 16) != 0)) return 0;
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
  switch (mode_of(g, layout)) {
    case kI8RowMajor: return launch<kI8RowMajor>(g, red);
    case kI8K4: return launch<kI8K4>(g, red);
    case kBF16: return launch<kBF16>(g, red);
    case kF16: return launch<kF16>(g, red);
    case kF8E4M3: return launch<kF8E4M3>(g, red);
    case kF8E5M2: return launch<kF8E5M2>(g, red);
    default: return launch<kF8Mixed>(g, red);
  }
}

// 2 <= M <= 8 (int8) or 2 <= M <= 3 (bf16, f16, fp8), row-major B: rows of A contiguous in K (int8: 4-byte
// aligned), C rows inside one block of 64.
extern "C" int skl_hip_gemv_rows_supported(const skl_gemm_canon *g) {
  const int mode = mode_of(g, 0);
  if (mode < 0) return 0;
  if (g->c_row_shift != 6 || g->c_col_shift != 6) return 0;  // C in blocks of 64 (or flat) only
  if (g->m < 2 || g->m > (size_t)(mode == kI8RowMajor ? kMaxRows : kMaxRowsFloat)) return 0;
  if (g->k == 0 || g->n == 0 || g->m * g->n > kMaxCols) return 0;
  const size_t es = (mode == kBF16 || mode == kF16) ? 2 : 1;
  const size_t cols = es == 2 ? 8 : 16;
  if (g->a_sk != 1) return 0;
  if (mode == kI8RowMajor && ((((uintptr_t)g->a) & 3) != 0 || (g->a_s0 & 3) != 0)) return 0;
  if ((g->n % cols) != 0 || !aligned16(g->b) || ((g->b_sk * es) % 16) != 0) return 0;
  if (g->b_s0 != 1 || ((g->b_s1 * es) % 16) != 0) return 0;
  if (g->csc1 != 64 * g->csc0) return 0;
  return 1;
}

extern "C" int skl_hip_launch_gemv_rows(const skl_gemm_canon *g) {
  if (!skl_hip_gemv_rows_supported(g)) {
    skl_hip_record_error(-2, "gemv_rows: unsupported problem");
    return -2;
  }
  Reduction red;
  if (!reduction_scratch(&red)) return -4;
  switch (mode_of(g, 0)) {
    case kI8RowMajor: return launch_rows_of<kI8RowMajor>(g, red);
    case kBF16: return launch_rows_of<kBF16>(g, red);
    case kF16: return launch_rows_of<kF16>(g, red);
    case kF8E4M3: return launch_rows_of<kF8E4M3>(g, red);
    case kF8E5M2: return launch_rows_of<kF8E5M2>(g, red);
    default: return launch_rows_of<kF8Mixed>(g, red);
  }
}

// 4 <= M <= 16 (int8) or 2 <= M <= 16 (fp8, bf16, f16), row-major B (flat or in panels of 64 columns), rows of A contiguous in K and
// 16-byte aligned, K and N multiples of 16 bytes of elements, C rows inside one block of 64 and its columns a fixed
// distance apart. Small problems are left to the kernels that need one launch.
// Bytes of B from which the two launches of this path beat the one launch of gemv_rows_kernel (measured on
// 2048^2, 4096^2, 8192 x 1024, 4096 x 8192 and 4096 x 11008: e.g. int8 with 4 rows 8.0 against 8.9 us at 16 MiB,
// 13.9 against 13.3 us at 43 MiB; bf16 with 2 rows 6.9 against 8.5 us at 8 MiB, 9.7 against 9.3 us at 16 MiB). Row
// counts the other kernel does not take (int8 above 8, floating point above 3) come here from 1 MiB on.
namespace {
size_t mfma_rows_min_bytes(int mode, size_t m) {
  constexpr size_t MiB = size_t(1) << 20;
  if (mode == kI8RowMajor) return m == 4 ? 40 * MiB : m == 5 ? 12 * MiB : m <= 7 ? 4 * MiB : MiB;
  if (mode == kBF16 || mode == kF16) return m <= 3 ? 12 * MiB : MiB;
  return m == 2 ? 12 * MiB : MiB;  // fp8
}
}  // namespace

extern "C" int skl_hip_gemv_mfma_rows_supported(const skl_gemm_canon *g, int layout) {
  const int mode = mode_of(g, layout);
  if (mode < 0) return 0;
  if (mode == kI8K4) {
    // B(4P + p, j) at P * b_sk + 4 j + p; 2 to 128 rows (no other kernel reads this layout with more than one row)
    if (g->c_row_shift != 6 || g->c_col_shift != 6 || g->bias || g->max || g->rq.act || g->rq.q) return 0;
    if (g->m < 2 || g->m > (size_t)(16 * kK4MaxRowGroups) || g->k == 0 || g->n == 0) return 0;
    if ((g->k % 16) != 0 || (g->n % 4) != 0) return 0;
    // A small B (under 1 MiB) only where the whole-K kernel runs a workgroup per column tile and group of 16 rows:
    // elsewhere the tile kernels are faster on it.
    const bool side_by_side = g->k <= kK4WholeMaxK && skl_div_up(g->n, (size_t)64) * ((g->m + 15) / 16) <= 256;
    if (g->k * g->n < (size_t(1) << 20) && !side_by_side) return 0;
    if (g->a_sk != 1 || !aligned16(g->a) || (g->a_s0 % 16) != 0) return 0;
    if (!aligned16(g->b) || (g->b_sk % 16) != 0) return 0;
    return g->csc1 == 64 * g->csc0;
  }
  const size_t es = (mode == kBF16 || mode == kF16) ? 2 : 1, piece = 16 / es;  // elements in 16 bytes
  if (g->c_row_shift != 6 || g->c_col_shift != 6) return 0;
  // Fewest rows from which this kernel is the faster one for 1 x 4096 x 11008 weights: int8 13.1 us whatever the
  // rows against 11.2 / 12.9 / 14.6 us for 2 / 3 / 4 rows on the kernel that shares the byte transposes; fp8 13.7 us
  // against 17.9 us for 2 rows; bf16 20.5 us against 27.1 us. (One row: int8 12.8 against 10.3 us, fp8 13.5 against
  // 11.5 us, bf16 20.4 against 21.6 us - left to the M = 1 kernel, which uses no matrix cores.)
  // A fused floating-point call with one row that the M = 1 kernel does not take (its own conditions on B and y)
  // still streams here rather than on the tile kernels: 13.5 / 20.4 us plus the pass over the planes for fp8 / bf16
  // weights of 4096 x 11008, on the tile kernels twice that.
  const bool fused_single_row = mode != kI8RowMajor && g->m == 1 && (g->bias || g->max || g->rq.act || g->rq.q);
  const size_t min_rows = mode == kI8RowMajor ? kMfmaMinRowsInt8 : fused_single_row ? 1 : 2;
  // int8 against a row-major B: beyond 16 rows in groups of 16 with B held in registers
  const size_t max_rows = mode == kI8RowMajor && !(g->bias || g->max || g->rq.act || g->rq.q) ? (size_t)kRowMajorMaxRows : (size_t)kMfmaMaxRows;
  if (g->m < min_rows || g->m > max_rows || g->k == 0 || g->n == 0) return 0;
  if (g->m > 64 && (g->a_s1 != 64 * g->a_s0 || g->rsc1 != 64 * g->rsc0)) return 0;  // rows a fixed distance apart
  const size_t min_bytes = fused_single_row ? size_t(1) << 20 : mfma_rows_min_bytes(mode, g->m);
  if ((g->k % piece) != 0 || (g->n % piece) != 0 || g->k * g->n * es < min_bytes) return 0;
  if (g->a_sk != 1 || !aligned16(g->a) || (g->a_s0 % piece) != 0) return 0;
  if (g->b_s0 != 1 || !aligned16(g->b) || (g->b_sk % piece) != 0 || (g->b_s1 % piece) != 0) return 0;
  if (g->csc1 != 64 * g->csc0) return 0;
  if (mode == kI8RowMajor && (g->bias || g->max || g->rq.act || g->rq.q)) return 0;  // the fused steps ride on the second pass (floating point)
  // floating point: one plane of raw sums per 512 k, inside the workspace's usual 64 MiB
  const size_t slabs = (g->k + MfmaShape<1>::kKPerGroup - 1) / MfmaShape<1>::kKPerGroup;
  static_assert(MfmaShape<1>::kKPerGroup == MfmaShape<2>::kKPerGroup, "one group length for every floating-point kind");
  if (mode != kI8RowMajor && slabs * g->m * g->n * sizeof(float) > (size_t(64) << 20)) return 0;
  return 1;
}

namespace {

template <int MODE>
int launch_mfma_rows(const GemvMfmaArgs &args) {
  using Sh = MfmaShape<(MODE == kBF16 || MODE == kF16) ? 2 : 1, MODE == kI8K4>;
  constexpr size_t kMfmaLds = Sh::kLds;
  const bool whole = args.n % Sh::kTileCols == 0 && args.k % Sh::kKPerGroup == 0;
  auto kernel = whole ? gemv_mfma_rows_kernel<MODE, true> : gemv_mfma_rows_kernel<MODE, false>;
  static std::atomic<bool> configured{false};  // per instantiation; racing threads set the same values
  if (!configured.load(std::memory_order_acquire)) {
    for (auto k : {gemv_mfma_rows_kernel<MODE, true>, gemv_mfma_rows_kernel<MODE, false>}) {
      int rc = skl_check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(k),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMfmaLds),
                             "gemv_mfma_rows: LDS size");
      if (rc != 0) return rc;
    }
    configured.store(true, std::memory_order_release);
  }
  GemvMfmaArgs p = args;
  p.tiles = skl_div_up(p.n, Sh::kTileCols);
  p.slabs = skl_div_up(p.k, Sh::kKPerGroup);
  const size_t grid = (size_t)p.tiles * p.slabs, cells = (p.m * p.n + 255) / 256;
  if (grid > 0x7FFFFFFFu || cells > 0x7FFFFFFFu) {
    skl_hip_record_error(-2, "gemv_mfma_rows: grid too large");
    return -2;
  }
  if constexpr (MODE == kI8K4) {
    if (p.k <= kK4WholeMaxK) {  // all of K inside one workgroup: no sums between workgroups
      const unsigned tiles = (unsigned)skl_div_up(p.n, (size_t)64);
      hipStream_t st = skl_current_stream();
      constexpr unsigned threads = kK4WholeWaves * 64;
      static std::atomic<bool> whole_configured{false};
      if (!whole_configured.load(std::memory_order_acquire)) {  // the kinds with two blocks of sums pass 64 KiB
        for (const void *f : {reinterpret_cast<const void *>(gemv_k4_wholek_kernel<1>), reinterpret_cast<const void *>(gemv_k4_wholek_kernel<2>),
                              reinterpret_cast<const void *>(gemv_k4_wholek_kernel<3>)}) {
          int rc = skl_check_hip(hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, (int)k4_whole_lds(1)), "gemv_k4_wholek: LDS size");
          if (rc != 0) return rc;
        }
        whole_configured.store(true, std::memory_order_release);
      }
      const unsigned row_groups = (unsigned)((p.m + 15) / 16);
      if (row_groups > 1 && (size_t)tiles * row_groups <= 256) {
        // So few column tiles that all row groups side by side still leave compute units free: a workgroup per
        // column tile and group of 16 rows (B is small then; each workgroup reads its 64 columns of it).
        gemv_k4_wholek_kernel<1><<<dim3(tiles, row_groups), threads, k4_whole_lds(1), st>>>(p);
        return skl_check_launch("gemv_k4_wholek");
      }
      switch (row_groups) {
        case 1: gemv_k4_wholek_kernel<1><<<tiles, threads, k4_whole_lds(1), st>>>(p); break;
        case 2: gemv_k4_wholek_kernel<2><<<tiles, threads, k4_whole_lds(2), st>>>(p); break;
        case 3: gemv_k4_wholek_kernel<3><<<tiles, threads, k4_whole_lds(3), st>>>(p); break;
        case 4: gemv_k4_wholek_kernel<4><<<tiles, threads, k4_whole_lds(4), st>>>(p); break;
        case 5: gemv_k4_wholek_kernel<5><<<tiles, threads, k4_whole_lds(5), st>>>(p); break;
        case 6: gemv_k4_wholek_kernel<6><<<tiles, threads, k4_whole_lds(6), st>>>(p); break;
        case 7: gemv_k4_wholek_kernel<7><<<tiles, threads, k4_whole_lds(7), st>>>(p); break;
        default: gemv_k4_wholek_kernel<8><<<tiles, threads, k4_whole_lds(8), st>>>(p); break;
      }
      return skl_check_launch("gemv_k4_wholek");
    }
  }
  if constexpr (MODE == kI8RowMajor || MODE == kI8K4) {
    if (p.beta.i != 1) {  // beta == 1: C is the starting value as it is
      gemv_mfma_scale_c_kernel<<<(unsigned)cells, 256, 0, skl_current_stream()>>>(p);
      int rc = skl_check_launch("gemv_mfma_scale_c");
      if (rc != 0) return rc;
    }
    if (p.m > (size_t)kMfmaMaxRows) {  // more than one group of 16 rows: one pass over B for all of them
      constexpr unsigned threads = kMfmaWaves * 64;
      hipStream_t st = skl_current_stream();
      static std::atomic<bool> groups_configured{false};
      if (!groups_configured.load(std::memory_order_acquire)) {
        for (const void *f : {reinterpret_cast<const void *>(gemv_rowgroups_kernel<MODE, 2>), reinterpret_cast<const void *>(gemv_rowgroups_kernel<MODE, 3>),
                              reinterpret_cast<const void *>(gemv_rowgroups_kernel<MODE, 4>), reinterpret_cast<const void *>(gemv_rowgroups_kernel<MODE, 5>),
                              reinterpret_cast<const void *>(gemv_rowgroups_kernel<MODE, 6>), reinterpret_cast<const void *>(gemv_rowgroups_kernel<MODE, 7>),
                              reinterpret_cast<const void *>(gemv_rowgroups_kernel<MODE, 8>)}) {
          int rc = skl_check_hip(hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMfmaLds), "gemv_rowgroups: LDS size");
          if (rc != 0) return rc;
        }
        groups_configured.store(true, std::memory_order_release);
      }
      switch ((p.m + 15) / 16) {
        case 2: gemv_rowgroups_kernel<MODE, 2><<<(unsigned)grid, threads, kMfmaLds, st>>>(p); break;
        case 3: gemv_rowgroups_kernel<MODE, 3><<<(unsigned)grid, threads, kMfmaLds, st>>>(p); break;
        case 4: gemv_rowgroups_kernel<MODE, 4><<<(unsigned)grid, threads, kMfmaLds, st>>>(p); break;
        case 5: gemv_rowgroups_kernel<MODE, 5><<<(unsigned)grid, threads, kMfmaLds, st>>>(p); break;
        case 6: gemv_rowgroups_kernel<MODE, 6><<<(unsigned)grid, threads, kMfmaLds, st>>>(p); break;
        case 7: gemv_rowgroups_kernel<MODE, 7><<<(unsigned)grid, threads, kMfmaLds, st>>>(p); break;
        default: gemv_rowgroups_kernel<MODE, 8><<<(unsigned)grid, threads, kMfmaLds, st>>>(p); break;
      }
      return skl_check_launch("gemv_rowgroups");
    }
    kernel<<<(unsigned)grid, kMfmaWaves * 64, kMfmaLds, skl_current_stream()>>>(p);
    return skl_check_launch("gemv_mfma_rows");
  } else {
    // The planes travel from the first kernel to the second through the stream's workspace: other host threads
    // on this stream must not get in between.
    skl_hip_sequence_begin();
    int rc = -4;
    p.planes = (float *)skl_workspace((size_t)p.slabs * p.m * p.n * sizeof(float));
    if (p.planes) {
      kernel<<<(unsigned)grid, kMfmaWaves * 64, kMfmaLds, skl_current_stream()>>>(p);
      rc = skl_check_launch("gemv_mfma_rows");
      if (rc == 0) {
        gemv_mfma_add_planes_kernel<<<(unsigned)cells, 256, 0, skl_current_stream()>>>(p);
        rc = skl_check_launch("gemv_mfma_add_planes");
      }
    }
    skl_hip_sequence_end();
    return rc;
  }
}

}  // namespace

extern "C" int skl_hip_launch_gemv_mfma_rows(const skl_gemm_canon *g, int layout) {
  if (!skl_hip_gemv_mfma_rows_supported(g, layout)) {
    skl_hip_record_error(-2, "gemv_mfma_rows: unsupported problem");
    return -2;
  }
  GemvMfmaArgs p;
  p.a = (const char *)g->a;
  const int mode = mode_of(g, layout);
  const size_t es = (mode == kBF16 || mode == kF16) ? 2 : 1;
  p.a_row = g->a_s0 * es;
  p.b = (const char *)g->b;
  p.b_sk = g->b_sk * es;
  p.b_s1 = g->b_s1 * es;
  p.c = (int *)g->c;
  p.c_row = g->rsc0;
  p.c_s = g->csc0;
  p.m = g->m;
  p.n = g->n;
  p.k = g->k;
  p.alpha = g->alpha;
  p.beta = g->beta;
  p.tiles = p.slabs = 0;  // set per kind
  p.planes = nullptr;
  p.bias = (const float *)g->bias;
  p.max = (float *)g->max;
  p.rq = g->rq;
  switch (mode) {
    case kI8RowMajor: return launch_mfma_rows<kI8RowMajor>(p);
    case kI8K4: return launch_mfma_rows<kI8K4>(p);
    case kBF16: return launch_mfma_rows<kBF16>(p);
    case kF16: return launch_mfma_rows<kF16>(p);
    case kF8E4M3: return launch_mfma_rows<kF8E4M3>(p);
    case kF8E5M2: return launch_mfma_rows<kF8E5M2>(p);
    default: return launch_mfma_rows<kF8Mixed>(p);
  }
}

// 1 <= M <= 4 against a B whose columns are contiguous in K (16-byte aligned columns and rows of A, K bytes a
// multiple of 16, columns a fixed distance apart).
extern "C" int skl_hip_gemv_kc_supported(const skl_gemm_canon *g) {
  const int mode = mode_of(g, 0);
  if (mode < 0) return 0;
  if (g->c_row_shift != 6 || g->c_col_shift != 6) return 0;  // C in blocks of 64 (or flat) only
  if (g->m < 1 || g->m > (size_t)kKcMaxRows || g->k == 0 || g->n == 0) return 0;
  const size_t es = (mode == kBF16 || mode == kF16) ? 2 : 1;
  if (g->b_sk != 1 || g->a_sk != 1 || ((g->k * es) % 16) != 0) return 0;
  if (!aligned16(g->b) || ((g->b_s0 * es) % 16) != 0 || (g->n > 64 && g->b_s1 != 64 * g->b_s0)) return 0;
  if (!aligned16(g->a) || (g->m > 1 && ((g->a_s0 * es) % 16) != 0)) return 0;
  if (g->n > 64 && g->csc1 != 64 * g->csc0) return 0;
  return 1;
}

extern "C" int skl_hip_launch_gemv_kc(const skl_gemm_canon *g) {
  if (!skl_hip_gemv_kc_supported(g)) {
    skl_hip_record_error(-2, "gemv_kc: unsupported problem");
    return -2;
  }
  switch (mode_of(g, 0)) {
    case kI8RowMajor: return launch_kc_of<kI8RowMajor>(g);
    case kBF16: return launch_kc_of<kBF16>(g);
    case kF16: return launch_kc_of<kF16>(g);
    case kF8E4M3: return launch_kc_of<kF8E4M3>(g);
    case kF8E5M2: return launch_kc_of<kF8E5M2>(g);
    default: return launch_kc_of<kF8Mixed>(g);
  }
}

// ---------------------------------------------------------------------------
// The entry point that allocates nothing: int8 decode calls (1 to 8 rows of A against a row-major B) on the same
// kernels as skl_hip_launch_gemv / skl_hip_launch_gemv_rows, with the static array at the top of this file as the
// slots. The array's name is only a handle on the host; its address on a device comes from hipGetSymbolAddress,
// asked once per device (skl_hip_init does it, else the first call here) and kept.
// ---------------------------------------------------------------------------
namespace {
constexpr int kNoAllocMaxDevices = 16;
unsigned long long *g_noalloc_slots[kNoAllocMaxDevices];  // per device: where `scratch` lives there
std::mutex g_noalloc_mutex;

unsigned long long *noalloc_slots_of_current_device() {
  int dev = 0;
  if (skl_check_hip(hipGetDevice(&dev), "hipGetDevice") != 0) return nullptr;
  if (dev < 0 || dev >= kNoAllocMaxDevices) {
    skl_hip_record_error(-2, "noalloc: device index beyond 15");
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(g_noalloc_mutex);
  if (!g_noalloc_slots[dev]) {
    void *ptr = nullptr;
    if (skl_check_hip(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)), "noalloc: address of the static scratch") != 0)
      return nullptr;
    g_noalloc_slots[dev] = static_cast<unsigned long long *>(ptr);
  }
  return g_noalloc_slots[dev];
}
}  // namespace

// The block of sums as an int32 matrix that is zero between calls: what a decode batch may add its product into
// without a kernel in front that zeroes it, provided whoever reads the product puts the zeros back. NULL when the
// product is larger than the block (or there is no block).
extern "C" void *skl_hip_zeroed_sums(size_t bytes) {
  Reduction red;
  if (bytes > kMaxCols * 8 || !reduction_scratch(&red)) return nullptr;
  return red.acc;
}

extern "C" int skl_hip_gemv_reserve_scratch(void) {
  Reduction red;
  return reduction_scratch(&red) ? 0 : -4;  // SKL_HIP_ERR_WORKSPACE
}

extern "C" int skl_hip_noalloc_setup(void) { return noalloc_slots_of_current_device() ? 0 : -2; }

extern "C" size_t skl_hip_noalloc_max_sums(void) { return kNoAllocSlots; }

// Puts the static sums back to zero on the current device, enqueued on the calling thread's stream: the way out
// after no-alloc calls overlapped (or one was aborted) and left slots that are not zero - every later call would add
// to them. Not for use under graph capture (a memset node); allocates nothing.
extern "C" int skl_hip_noalloc_reset(void) {
  unsigned long long *slots = noalloc_slots_of_current_device();
  if (!slots) return -2;
  return skl_check_hip(hipMemsetAsync(slots, 0, kNoAllocSlots * sizeof(unsigned long long), skl_current_stream()), "skl_hip_noalloc_reset");
}

extern "C" int skl_hip_launch_gemv_noalloc(const skl_gemm_canon *g) {
  if (g->ta != SKL_DT_I8 || g->tb != SKL_DT_I8 || g->m < 1 || g->m > (size_t)kMaxRows ||
      (g->m == 1 ? !skl_hip_gemv_supported(g, 0) : !skl_hip_gemv_rows_supported(g))) {
    skl_hip_record_error(-2, "noalloc: not an int8 decode call (1 to 8 rows of A contiguous in K, row-major B with "
                             "16-byte aligned rows, N a multiple of 16, K > 0)");
    return -2;
  }
  if (g->m * g->n > kNoAllocSlots) {
    skl_hip_record_error(-2, "noalloc: M * N exceeds the 65536 sums of the static scratch");
    return -2;
  }
  Reduction red;
  red.acc = noalloc_slots_of_current_device();
  if (!red.acc) return -2;
  return g->m == 1 ? launch<kI8RowMajor>(g, red) : launch_rows_of<kI8RowMajor>(g, red);
}
