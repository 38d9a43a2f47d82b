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
  int s_pairs;       // every column's scales start on a 2-byte boundary: a lane's two scales of a chunk in one load
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

template <bool EXACT>
__global__ void __launch_bounds__(kWaves * 64) gemv_f4_kernel(F4Args p) {
  __shared__ float red[kWaves][kMaxRows][kCols + 1];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int jl = lane & 15, g = lane >> 4;
  const size_t col = (size_t)blockIdx.x * kCols + jl;
  const bool col_ok = col < p.n, row_ok = (size_t)jl < p.m;
  const char *bp = p.b + (col_ok ? col : 0) * p.b_col;
  const uint8_t *sp = p.s ? p.s + (col_ok ? col : 0) * p.s_col : nullptr;
  const char *ap = p.a + (row_ok ? (size_t)jl : 0) * p.a_row;
  v4f acc = {0.0f, 0.0f, 0.0f, 0.0f};
  const v4i zero = {0, 0, 0, 0};
  // K is a multiple of 32: a 16-byte piece of B (32 k) is inside or outside, and so are the two pieces of A with it.
  for (size_t k0 = (size_t)wave * kChunk; k0 < p.k; k0 += (size_t)kWaves * kChunk * kInFlight) {
    v4i b[kInFlight][2], a[kInFlight][4];
    unsigned sc[kInFlight][2];  // the biased exponent of the scale of b[u][h]; 127 (2^0) without scales
#pragma unroll
    for (int u = 0; u < kInFlight; ++u) {
      const size_t kc = k0 + (size_t)u * kWaves * kChunk;  // chunk u of this wave
      const size_t kl = kc + (size_t)g * 64;               // this lane's 64 k of B in it
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        b[u][h] = (kl + 32 * h < p.k && col_ok) ? load16(bp + (kl + 32 * h) / 2) : zero;
        // A's two 16-byte pieces for the same instruction: the lane's own k (f16 instructions), or the k that the
        // FP8 operand layout pairs with B's nibbles (see the head of the file)
        const size_t ka0 = EXACT ? kl + 32 * h : kc + 64 * (size_t)(g >> 1) + 32 * h + 16 * (size_t)(g & 1);
        const size_t ka1 = EXACT ? ka0 + 16 : ka0 + 128;
        a[u][2 * h] = (ka0 < p.k && row_ok) ? *reinterpret_cast<const v4i *>(ap + ka0) : zero;
        a[u][2 * h + 1] = (ka1 < p.k && row_ok) ? *reinterpret_cast<const v4i *>(ap + ka1) : zero;
      }
    }
    // The scales behind the operands' requests (they are needed last, and their lines are small change next to B's):
    // a lane's two of a chunk are neighbours.
#pragma unroll
    for (int u = 0; u < kInFlight; ++u) {
      const size_t kl = k0 + (size_t)u * kWaves * kChunk + (size_t)g * 64;
      sc[u][0] = sc[u][1] = 127u;
      if (sp && col_ok && kl < p.k) {
        if (p.s_pairs && kl + 32 < p.k) {
          const unsigned two = *reinterpret_cast<const unsigned short *>(sp + kl / 32);
          sc[u][0] = two & 0xFFu, sc[u][1] = two >> 8;
        } else {
          sc[u][0] = sp[kl / 32];
          if (kl + 32 < p.k) sc[u][1] = sp[kl / 32 + 1];
        }
      }
    }
#pragma unroll
    for (int u = 0; u < kInFlight; ++u)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        if constexpr (EXACT) {
          const float scale = __uint_as_float(sc[u][h] << 23);  // 2^(s - 127) for s = 1 .. 254
#pragma unroll
          for (int q = 0; q < 4; ++q) {  // 8 k per lane and instruction: byte pairs of A, one dword of B
            const v4i &ah = a[u][2 * h + (q >> 1)];
            const unsigned lo = (unsigned)((q & 1) ? ah.z : ah.x), hi = (unsigned)((q & 1) ? ah.w : ah.y);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(widen_e4m3(lo, hi), widen_f4((unsigned)b[u][h][q], scale), acc, 0, 0, 0);
          }
        } else {
          const v8i av = {a[u][2 * h].x, a[u][2 * h].y, a[u][2 * h].z, a[u][2 * h].w,
                          a[u][2 * h + 1].x, a[u][2 * h + 1].y, a[u][2 * h + 1].z, a[u][2 * h + 1].w};
          const v8i bv = {b[u][h].x, b[u][h].y, b[u][h].z, b[u][h].w, 0, 0, 0, 0};
          // A: E4M3 (format 0) with scale 2^0, B: E2M1 (format 4) with this lane's scale for its 32 values
          acc = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(av, bv, acc, 0, 4, 0, 127, 0, (int)sc[u][h]);
        }
      }
  }
  // acc[r] is row 4 g + r of C, column jl of the workgroup's 16.
#pragma unroll
  for (int r = 0; r < 4; ++r) red[wave][4 * g + r][jl] = acc[r];
  __syncthreads();
  const int row = threadIdx.x >> 4, tc = threadIdx.x & 15;
  const size_t j = (size_t)blockIdx.x * kCols + tc;
  if ((size_t)row >= p.m || j >= p.n) return;
  float sum = red[0][row][tc];
#pragma unroll
  for (int w = 1; w < kWaves; ++w) sum = __fadd_rn(sum, red[w][row][tc]);
  skl_update(sum, p.c + (size_t)row * p.c_row + j * p.c_col, p.alpha, p.beta);
}

inline bool aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }

}  // namespace

// 1 to 16 rows of A, K a multiple of 32, rows of A and columns of B on 16-byte boundaries.
extern "C" int skl_hip_gemv_f4_supported(size_t m, size_t n, size_t k, const void *a, size_t rsa, size_t csa, const void *b,
                                         size_t ldb) {
  if (m < 1 || m > (size_t)kMaxRows || n == 0 || k == 0 || (k % 32) != 0) return 0;
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
  const size_t grid = (n + kCols - 1) / kCols;
  if (grid > 0x7FFFFFFFu) {
    skl_hip_record_error(-2, "gemv_f4: grid too large");
    return -2;
  }
  const int s_pairs = scales && ((uintptr_t)scales & 1) == 0 && (n == 1 || (lds & 1) == 0);
  F4Args p = {(const char *)a, rsa, (const char *)b, ldb / 2, scales, lds, s_pairs, c, rsc, csc, m, n, k, alpha, beta};
  if (k <= kExactMaxK)
    gemv_f4_kernel<true><<<(unsigned)grid, kWaves * 64, 0, skl_current_stream()>>>(p);
  else
    gemv_f4_kernel<false><<<(unsigned)grid, kWaves * 64, 0, skl_current_stream()>>>(p);
  return skl_check_launch("gemv_f4");
}
