// skl_gemv_f4.hip - decode against OFP4 (E2M1) weights: up to 16 rows of E4M3 A times a B whose columns are
// contiguous in K and hold two 4-bit values per byte (element 2i in the low nibble of byte i, as
// ref/cvt/cvt_ofp4.c:59-68 unpacks them). The reference has no GEMM over 4-bit weights; it converts them
// (skl_cvt_f4e2m1_f8e4m3, ref/cvt/cvt_ofp4.c:59-68 - exact, every E2M1 value is an E4M3 value) and multiplies
// the result (ref/gemm/gemm_f8rc_f8rc_f32rc.c with rsb = 1, csb = ldb): that composition defines the result
// here. The point of doing it in one kernel is the stream: the weights cross HBM at half a byte per element.
// Optionally every 32 consecutive k of a column carry a scale, a power of two stored as its biased exponent (E8M0:
// 2^(s - 127)) - the OCP microscaling format MXFP4. The reference has no notion of it; the result is then defined as
// the fp32 GEMM (ref/gemm/gemm_f32rc_f32rc_f32rc.c:9-24) of the decoded operands, B's values times their scales.
//
// Decomposition: a workgroup of four waves owns 16 columns and all of K. In a chunk of 256 k a lane (column
// lane % 16, k group lane / 16) loads 32 consecutive bytes of its column - the four groups cover one 128-byte
// line - and 64 bytes of row lane % 16 of A, the same k. These are the operands of two 16x16x128 matrix-core
// instructions whose B format is FP4 (v_mfma_scale_f32_16x16x128_f8f6f4 with unit scales: the conversion is the
// instruction's), or - for short K, where that instruction's internal alignment of the 128 products loses more
// than the reference's error bound allows - of eight v_mfma_f32_16x16x32_bf16 on operands widened to bf16 in
// registers, B's with its scale (every E4M3 value and every scaled E2M1 value is a bf16 value: exact products, fp32
// sums). A lane's 32 values of B are exactly one scale's block, which is how the scaled instruction takes scales: one
// per lane. Which k of a chunk meet in which instruction is free as long as A's and
// B's lanes hold the same ones. For the f16 instructions that is each lane's own 8 k. The scaled instruction counts
// k differently for its two formats (found by reading single products back): an FP4 operand holds k = 32 g + t in
// nibble t of lane group g, an FP8 operand k = 16 g + t in byte t < 16 and 64 + 16 g + (t - 16) above - so A's lanes
// load the two 16-byte pieces that B's layout puts there. The four waves take the chunks in turn and meet in LDS,
// added in wave order: no sums between workgroups, no scratch, the same bits on every run.
#include <hip/hip_runtime.h>

#include "skl_device.hpp"
#include "skl_fp8.hpp"

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));

constexpr int kWaves = 4, kCols = 16, kMaxRows = 16;
constexpr int kChunk = 256;       // k per wave and step: 64 per lane group
constexpr int kInFlight = 4;      // chunks a wave requests before it multiplies the first
constexpr size_t kExactMaxK = 2304;  // up to here the bf16 instructions (the bound of the reference grows with K)

struct F4Args {
  const char *a;  // E4M3, row i at a + i * a_row, K contiguous
  size_t a_row;
  const char *b;  // E2M1 pairs, column j at b + j * b_col (bytes), K contiguous
  size_t b_col;
  const uint8_t *s;  // E8M0 scales, one per 32 k: column j's at s + j * s_col; null: none
  size_t s_col;
  int s_pairs;       // K is a multiple of 64 and every column's scales start on a 2-byte boundary: a lane's two scales
                     // of a chunk in one load
  float *c;       // element (i, j) at c + i * c_row + j * c_col
  size_t c_row, c_col;
  size_t m, n, k;
  skl_scalar alpha, beta;
};

__device__ __forceinline__ v4i load16(const char *p) { return __builtin_nontemporal_load(reinterpret_cast<const v4i *>(p)); }

// Eight E2M1 values (one dword, low nibble first) times `scale` (a power of two) as eight bf16 values: exact.
__device__ __forceinline__ v8bf widen_f4(unsigned w, float scale) {
  const v2bf p0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scale, 0), p1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scale, 1);
  const v2bf p2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scale, 2), p3 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scale, 3);
  return v8bf{p0.x, p0.y, p1.x, p1.y, p2.x, p2.y, p3.x, p3.y};
}
// Eight E4M3 values (two dwords, ascending) as eight bf16 values: exact.
__device__ __forceinline__ v8bf widen_e4m3(unsigned lo, unsigned hi) {
  const v2bf p0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(lo, 1.0f, false), p1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(lo, 1.0f, true);
  const v2bf p2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(hi, 1.0f, false), p3 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(hi, 1.0f, true);
  return v8bf{p0.x, p0.y, p1.x, p1.y, p2.x, p2.y, p3.x, p3.y};
}

// CG groups of 16 columns per workgroup: a wave's pieces of A serve CG instructions each. With one group, 16 rows of
// A make every workgroup pull 64 KB of A through its L1 for 32 KB of weights (12.2 us for 16 x 4096 x 11008 against
// 7.2 us for one row); four groups quarter that. Loads are clamped into the operands rather than guarded (a guard is
// a branch, and at a branch the compiler waits for the loads before it): k beyond K meets zeros of A, rows beyond M
// and columns beyond N are computed and not written.
template <bool EXACT, int CG>
__global__ void __launch_bounds__(kWaves * 64) gemv_f4_kernel(F4Args p) {
  __shared__ float red[kWaves][kMaxRows][CG * kCols + 1];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int jl = lane & 15, g = lane >> 4;
  const char *bp[CG];
  const uint8_t *sp[CG];
#pragma unroll
  for (int cg = 0; cg < CG; ++cg) {
    const size_t col = ((size_t)blockIdx.x * CG + cg) * kCols + jl;
    bp[cg] = p.b + (col < p.n ? col : p.n - 1) * p.b_col;
    sp[cg] = p.s ? p.s + (col < p.n ? col : p.n - 1) * p.s_col : nullptr;
  }
  const bool row_ok = (size_t)jl < p.m;
  const char *ap = p.a + (row_ok ? (size_t)jl : p.m - 1) * p.a_row;
  v4f acc[CG];
#pragma unroll
  for (int cg = 0; cg < CG; ++cg) acc[cg] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
  const v4i zero = {0, 0, 0, 0};
  // K is a multiple of 32: a 16-byte piece of B (32 k) is inside or outside, and so are the two pieces of A with it.
  for (size_t k0 = (size_t)wave * kChunk; k0 < p.k; k0 += (size_t)kWaves * kChunk * kInFlight) {
    v4i b[kInFlight][CG][2], a[kInFlight][4];
    unsigned sc[kInFlight][CG][2];  // the biased exponent of the scale of b[u][cg][h]; 127 (2^0) without scales
#pragma unroll
    for (int u = 0; u < kInFlight; ++u) {
      const size_t kc = k0 + (size_t)u * kWaves * kChunk;  // chunk u of this wave
      const size_t kl = kc + (size_t)g * 64;               // this lane's 64 k of B in it
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        // A's two 16-byte pieces for the same instruction: the lane's own k (bf16 instructions), or the k that the
        // FP8 operand layout pairs with B's nibbles (see the head of the file)
        const size_t ka0 = EXACT ? kl + 32 * h : kc + 64 * (size_t)(g >> 1) + 32 * h + 16 * (size_t)(g & 1);
        const size_t ka1 = EXACT ? ka0 + 16 : ka0 + 128;
        const v4i a0 = *reinterpret_cast<const v4i *>(ap + (ka0 < p.k ? ka0 : p.k - 16));
        const v4i a1 = *reinterpret_cast<const v4i *>(ap + (ka1 < p.k ? ka1 : p.k - 16));
        a[u][2 * h] = ka0 < p.k && row_ok ? a0 : zero;
        a[u][2 * h + 1] = ka1 < p.k && row_ok ? a1 : zero;
#pragma unroll
        for (int cg = 0; cg < CG; ++cg) {
          const size_t kb = kl + 32 * h;
          b[u][cg][h] = load16(bp[cg] + (kb < p.k ? kb : p.k - 32) / 2);
        }
      }
    }
    // The scales behind the operands' requests (they are needed last, and their lines are small change next to B's).
#pragma unroll
    for (int u = 0; u < kInFlight; ++u) {
      const size_t kl = k0 + (size_t)u * kWaves * kChunk + (size_t)g * 64;
#pragma unroll
      for (int cg = 0; cg < CG; ++cg) {
        sc[u][cg][0] = sc[u][cg][1] = 127u;
        const size_t last = p.k / 32 - 1, i0 = kl / 32, i1 = kl / 32 + 1;
        if (p.s_pairs) {  // the same for every thread: K a multiple of 64, scales on 2-byte boundaries
          const unsigned two = *reinterpret_cast<const unsigned short *>(sp[cg] + (i1 < last ? i0 : last - 1));
          sc[u][cg][0] = two & 0xFFu, sc[u][cg][1] = two >> 8;
        } else if (p.s) {
          sc[u][cg][0] = sp[cg][i0 < last ? i0 : last];
          sc[u][cg][1] = sp[cg][i1 < last ? i1 : last];
        }
      }
    }
#pragma unroll
    for (int u = 0; u < kInFlight; ++u)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        if constexpr (EXACT) {
          v8bf aw[4];
#pragma unroll
          for (int q = 0; q < 4; ++q) {  // 8 k per lane and instruction: byte pairs of A, one dword of B
            const v4i &ah = a[u][2 * h + (q >> 1)];
            aw[q] = widen_e4m3((unsigned)((q & 1) ? ah.z : ah.x), (unsigned)((q & 1) ? ah.w : ah.y));
          }
#pragma unroll
          for (int cg = 0; cg < CG; ++cg) {
            const float scale = __uint_as_float(sc[u][cg][h] << 23);  // 2^(s - 127) for s = 1 .. 254
#pragma unroll
            for (int q = 0; q < 4; ++q)
              acc[cg] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(aw[q], widen_f4((unsigned)b[u][cg][h][q], scale), acc[cg], 0, 0, 0);
          }
        } else {
          const v8i av = {a[u][2 * h].x, a[u][2 * h].y, a[u][2 * h].z, a[u][2 * h].w,
                          a[u][2 * h + 1].x, a[u][2 * h + 1].y, a[u][2 * h + 1].z, a[u][2 * h + 1].w};
#pragma unroll
          for (int cg = 0; cg < CG; ++cg) {
            const v8i bv = {b[u][cg][h].x, b[u][cg][h].y, b[u][cg][h].z, b[u][cg][h].w, 0, 0, 0, 0};
            // A: E4M3 (format 0) with scale 2^0, B: E2M1 (format 4) with this lane's scale for its 32 values
            acc[cg] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(av, bv, acc[cg], 0, 4, 0, 127, 0, (int)sc[u][cg][h]);
          }
        }
      }
  }
  // acc[cg][r] is row 4 g + r of C, column 16 cg + jl of the workgroup's.
#pragma unroll
  for (int cg = 0; cg < CG; ++cg)
#pragma unroll
    for (int r = 0; r < 4; ++r) red[wave][4 * g + r][cg * kCols + jl] = acc[cg][r];
  __syncthreads();
  const int row = threadIdx.x >> 4, tc = threadIdx.x & 15;
  if ((size_t)row >= p.m) return;
  float sums[CG];
#pragma unroll
  for (int cg = 0; cg < CG; ++cg) {
    sums[cg] = red[0][row][cg * kCols + tc];
#pragma unroll
    for (int w = 1; w < kWaves; ++w) sums[cg] = __fadd_rn(sums[cg], red[w][row][cg * kCols + tc]);
  }
#pragma unroll
  for (int cg = 0; cg < CG; ++cg) {
    const size_t j = ((size_t)blockIdx.x * CG + cg) * kCols + tc;
    if (j < p.n) skl_update(sums[cg], p.c + (size_t)row * p.c_row + j * p.c_col, p.alpha, p.beta);
  }
}

// 17 to 128 rows of A: the same decomposition with B held in registers for 4096 k (one pass of the K loop above:
// four chunks per wave; a longer K takes one launch per 4096 k, the later ones adding to C) while up to eight groups of 16 rows take their turns - the 4-bit weights cross
// HBM once and never exist as a converted copy (which cost 22.5 MB read, 45 MB written and a tile GEMM behind it:
// 37 / 40 / 45 us for 32 / 64 / 128 x 4096 x 11008). Two groups of 16 columns per workgroup; a row group's pieces of A
// are requested two groups ahead; its sums go through one of two LDS blocks, added in wave order (one barrier per
// group: the next group's barrier stands between this group's readers and the writers of the group after it).
constexpr int kRowsCG = 4, kMaxRowGroups = 8;
constexpr size_t kRowsMaxK = (size_t)kWaves * kChunk * kInFlight;  // 4096

template <bool EXACT, int RG>
__global__ void __launch_bounds__(kWaves * 64) gemv_f4_rows_kernel(F4Args p) {
  constexpr int CG = kRowsCG;
  __shared__ float red[2][kWaves][kMaxRows][CG * kCols + 1];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int jl = lane & 15, g = lane >> 4;
  const v4i zero = {0, 0, 0, 0};
  // The pieces of A for row group rg: chunk u of this wave, as in the kernel above; loaded from inside A and zeroed
  // beyond M and K.
  auto fragment_of = [&](int rg, v4i(&a)[kInFlight][4]) {
    const size_t row = (size_t)rg * 16 + jl;
    const bool row_ok = row < p.m;
    const char *ap = p.a + (row_ok ? row : p.m - 1) * p.a_row;
#pragma unroll
    for (int u = 0; u < kInFlight; ++u) {
      const size_t kc = ((size_t)wave + (size_t)u * kWaves) * kChunk, kl = kc + (size_t)g * 64;
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const size_t ka0 = EXACT ? kl + 32 * h : kc + 64 * (size_t)(g >> 1) + 32 * h + 16 * (size_t)(g & 1);
        const size_t ka1 = EXACT ? ka0 + 16 : ka0 + 128;
        const v4i a0 = *reinterpret_cast<const v4i *>(ap + (ka0 < p.k ? ka0 : p.k - 16));
        const v4i a1 = *reinterpret_cast<const v4i *>(ap + (ka1 < p.k ? ka1 : p.k - 16));
        a[u][2 * h] = ka0 < p.k && row_ok ? a0 : zero;
        a[u][2 * h + 1] = ka1 < p.k && row_ok ? a1 : zero;
      }
    }
  };
  v4i a[2][kInFlight][4];
  fragment_of(0, a[0]);  // ahead of B: loads come back in the order of their requests
  v4i b[kInFlight][CG][2];
  unsigned sc[kInFlight][CG][2];
#pragma unroll
  for (int cg = 0; cg < CG; ++cg) {
    const size_t col = ((size_t)blockIdx.x * CG + cg) * kCols + jl;
    const size_t colc = col < p.n ? col : p.n - 1;
    const char *bp = p.b + colc * p.b_col;
    const uint8_t *sp = p.s ? p.s + colc * p.s_col : nullptr;
#pragma unroll
    for (int u = 0; u < kInFlight; ++u) {
      const size_t kl = ((size_t)wave + (size_t)u * kWaves) * kChunk + (size_t)g * 64;
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const size_t kb = kl + 32 * h;
        b[u][cg][h] = load16(bp + (kb < p.k ? kb : p.k - 32) / 2);
      }
      sc[u][cg][0] = sc[u][cg][1] = 127u;
      if (p.s) {  // the same for every thread
        const size_t last = p.k / 32 - 1, i0 = kl / 32, i1 = kl / 32 + 1;
        sc[u][cg][0] = sp[i0 < last ? i0 : last];
        sc[u][cg][1] = sp[i1 < last ? i1 : last];
      }
    }
  }
  if constexpr (RG > 1) fragment_of(1, a[1]);
  __builtin_amdgcn_sched_barrier(0);  // every request is out before the first use
  const int row = threadIdx.x >> 4, tc = threadIdx.x & 15;
#pragma unroll
  for (int rg = 0; rg < RG; ++rg) {
    if ((size_t)rg * 16 >= p.m) break;  // the same for every thread of the workgroup
    v4f acc[CG];
#pragma unroll
    for (int cg = 0; cg < CG; ++cg) acc[cg] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int u = 0; u < kInFlight; ++u)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const v4i(&ar)[4] = a[rg & 1][u];
        if constexpr (EXACT) {
          v8bf aw[4];
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const v4i &ah = ar[2 * h + (q >> 1)];
            aw[q] = widen_e4m3((unsigned)((q & 1) ? ah.z : ah.x), (unsigned)((q & 1) ? ah.w : ah.y));
          }
#pragma unroll
          for (int cg = 0; cg < CG; ++cg) {
            const float scale = __uint_as_float(sc[u][cg][h] << 23);
#pragma unroll
            for (int q = 0; q < 4; ++q)
              acc[cg] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(aw[q], widen_f4((unsigned)b[u][cg][h][q], scale), acc[cg], 0, 0, 0);
          }
        } else {
          const v8i av = {ar[2 * h].x, ar[2 * h].y, ar[2 * h].z, ar[2 * h].w, ar[2 * h + 1].x, ar[2 * h + 1].y, ar[2 * h + 1].z, ar[2 * h + 1].w};
#pragma unroll
          for (int cg = 0; cg < CG; ++cg) {
            const v8i bv = {b[u][cg][h].x, b[u][cg][h].y, b[u][cg][h].z, b[u][cg][h].w, 0, 0, 0, 0};
            acc[cg] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(av, bv, acc[cg], 0, 4, 0, 127, 0, (int)sc[u][cg][h]);
          }
        }
      }
    if (rg + 2 < RG) fragment_of(rg + 2, a[rg & 1]);
    // acc[cg][r] is row 16 rg + 4 g + r of C, column 16 cg + jl of the workgroup's.
    float(*block)[kMaxRows][CG * kCols + 1] = red[rg & 1];
#pragma unroll
    for (int cg = 0; cg < CG; ++cg)
#pragma unroll
      for (int r = 0; r < 4; ++r) block[wave][4 * g + r][cg * kCols + jl] = acc[cg][r];
    __syncthreads();
    const size_t i = (size_t)rg * 16 + row;
#pragma unroll
    for (int cg = 0; cg < CG; ++cg) {
      float sum = block[0][row][cg * kCols + tc];
#pragma unroll
      for (int w = 1; w < kWaves; ++w) sum = __fadd_rn(sum, block[w][row][cg * kCols + tc]);
      const size_t j = ((size_t)blockIdx.x * CG + cg) * kCols + tc;
      if (i < p.m && j < p.n) skl_update(sum, p.c + i * p.c_row + j * p.c_col, p.alpha, p.beta);
    }
  }
}

inline bool aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }

}  // namespace

// 1 to 16 rows of A (to 128 when B holds at least 2^20 values), K a multiple of 32, rows of A and columns of B on 16-byte boundaries.
extern "C" int skl_hip_gemv_f4_supported(size_t m, size_t n, size_t k, const void *a, size_t rsa, size_t csa, const void *b,
                                         size_t ldb) {
  if (m < 1 || m > (size_t)(kMaxRows * kMaxRowGroups) || n == 0 || k == 0 || (k % 32) != 0) return 0;
  // beyond 16 rows: B stays in registers for 4096 k at a time, and there must be enough of it to be worth a pass per 128 rows
  if (m > (size_t)kMaxRows && n * k < (size_t(1) << 20)) return 0;
  if (csa != 1 || !aligned16(a) || (m > 1 && (rsa % 16) != 0)) return 0;
  if (!aligned16(b) || (n > 1 && (ldb % 32) != 0)) return 0;
  return 1;
}

extern "C" int skl_hip_launch_gemv_f4(size_t m, size_t n, size_t k, skl_scalar alpha, const void *a, size_t rsa, size_t csa,
                                      const void *b, size_t ldb, const uint8_t *scales, size_t lds, skl_scalar beta, float *c,
                                      size_t rsc, size_t csc) {
  if (!skl_hip_gemv_f4_supported(m, n, k, a, rsa, csa, b, ldb)) {
    skl_hip_record_error(-2, "gemv_f4: unsupported problem");
    return -2;
  }
  if (m > (size_t)kMaxRows) {
    const size_t grid = (n + (size_t)kRowsCG * kCols - 1) / ((size_t)kRowsCG * kCols);
    if (grid > 0x7FFFFFFFu) {
      skl_hip_record_error(-2, "gemv_f4: grid too large");
      return -2;
    }
    hipStream_t st = skl_current_stream();
    const unsigned blocks = (unsigned)grid, threads = kWaves * 64;
    // A K beyond what the registers hold goes in passes of 4096 k: the first applies the caller's beta, the others
    // add to C (beta = 1) - launches on one stream, in order; the same bits on every run.
    for (size_t k0 = 0; k0 < k; k0 += kRowsMaxK) {
      const size_t kk = k - k0 < kRowsMaxK ? k - k0 : kRowsMaxK;
      skl_scalar pass_beta = beta;
      if (k0 != 0) pass_beta.fz.value = 1.0f, pass_beta.fz.skip_c_read = 0;
      F4Args p = {(const char *)a + k0, rsa, (const char *)b + k0 / 2, ldb / 2, scales ? scales + k0 / 32 : nullptr, lds, 0,
                  c, rsc, csc, m, n, kk, alpha, pass_beta};
      const bool exact = kk <= kExactMaxK;
#define SKL_F4_ROWS(RG)                                                           \
  case RG:                                                                        \
    if (exact) gemv_f4_rows_kernel<true, RG><<<blocks, threads, 0, st>>>(p);      \
    else gemv_f4_rows_kernel<false, RG><<<blocks, threads, 0, st>>>(p);           \
    break;
      switch ((m + 15) / 16) {
        SKL_F4_ROWS(2) SKL_F4_ROWS(3) SKL_F4_ROWS(4) SKL_F4_ROWS(5) SKL_F4_ROWS(6) SKL_F4_ROWS(7)
        default:
          if (exact) gemv_f4_rows_kernel<true, 8><<<blocks, threads, 0, st>>>(p);
          else gemv_f4_rows_kernel<false, 8><<<blocks, threads, 0, st>>>(p);
      }
#undef SKL_F4_ROWS
      const int rc = skl_check_launch("gemv_f4_rows");
      if (rc != 0) return rc;
    }
    return 0;
  }
  // Four groups of 16 columns per workgroup from three rows of A on, where that still leaves at least 128
  // workgroups: the pieces of A are what a wave loads most of then.
  const int cg = m >= 3 && n >= 128 * 4 * kCols ? 4 : 1;
  const size_t grid = (n + (size_t)cg * kCols - 1) / ((size_t)cg * kCols);
  if (grid > 0x7FFFFFFFu) {
    skl_hip_record_error(-2, "gemv_f4: grid too large");
    return -2;
  }
  const int s_pairs = scales && (k % 64) == 0 && ((uintptr_t)scales & 1) == 0 && (n == 1 || (lds & 1) == 0);
  F4Args p = {(const char *)a, rsa, (const char *)b, ldb / 2, scales, lds, s_pairs, c, rsc, csc, m, n, k, alpha, beta};
  hipStream_t st = skl_current_stream();
  if (k <= kExactMaxK) {
    if (cg == 4) gemv_f4_kernel<true, 4><<<(unsigned)grid, kWaves * 64, 0, st>>>(p);
    else gemv_f4_kernel<true, 1><<<(unsigned)grid, kWaves * 64, 0, st>>>(p);
  } else {
    if (cg == 4) gemv_f4_kernel<false, 4><<<(unsigned)grid, kWaves * 64, 0, st>>>(p);
    else gemv_f4_kernel<false, 1><<<(unsigned)grid, kWaves * 64, 0, st>>>(p);
  }
  return skl_check_launch("gemv_f4");
}
