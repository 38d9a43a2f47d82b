// skl_gemm_mfma.hip - the entry points of the matrix-core GEMM: which problems it takes, and the dispatch to the
// operand kind's translation unit (skl_gemm_mfma_<kind>.hip; the kernels live in skl_gemm_mfma_impl.hpp and are
// compiled one kind per file, side by side).
#include "skl_gemm_mfma_impl.hpp"

SKL_MFMA_DECLARE_KIND(i8)
SKL_MFMA_DECLARE_KIND(bf16)
SKL_MFMA_DECLARE_KIND(f16)
SKL_MFMA_DECLARE_KIND(f8e4m3)
SKL_MFMA_DECLARE_KIND(f8e5m2)
SKL_MFMA_DECLARE_KIND(f8e4m3_f8e5m2)
SKL_MFMA_DECLARE_KIND(f8e5m2_f8e4m3)

extern "C" int skl_hip_gemm_mfma_supported(const skl_gemm_canon *g) {
  if (g->m == 0 || g->n == 0 || g->k == 0) return 0;
  const bool fp8a = g->ta == SKL_DT_F8E4M3 || g->ta == SKL_DT_F8E5M2;
  const bool fp8b = g->tb == SKL_DT_F8E4M3 || g->tb == SKL_DT_F8E5M2;
  if (!(g->ta == g->tb || (fp8a && fp8b))) return 0;
  const size_t es = (g->ta == SKL_DT_BF16 || g->ta == SKL_DT_F16) ? 2 : 1;
  if (!operand_ok(g->a, es, g->a_s1, g->a_s0, g->a_sk, g->m, g->k)) return 0;
  if (!operand_ok(g->b, es, g->b_s1, g->b_s0, g->b_sk, g->n, g->k)) return 0;
  if (((uintptr_t)g->c & 3) != 0) return 0;
  if (g->c_row_shift < 2 || g->c_row_shift > 6 || g->c_col_shift < 1 || g->c_col_shift > 6) return 0;
  return 1;
}

namespace {

// Would the problem, as it lies in memory, run on the streaming kernel? (The rule of launch_tile.)
bool streams_in_place(const skl_gemm_canon *g, size_t es) {
  if (!skl_hip_gemm_mfma_supported(g) || g->m % 256 != 0 || (g->k * es) % 128 != 0) return false;
  const size_t tiles_m = g->m / 256;
  return (g->n % 256 == 0 && tiles_m * (g->n / 256) >= 200) || (g->n % 128 == 0 && tiles_m * (g->n / 128) >= 96);
}

}  // namespace

// Would the streaming kernel take this int8 problem as it lies and write its C 16 bytes per lane (C in blocks of 4
// to 16 columns with contiguous rows)? Then a blocked C costs no more than a row-major one.
extern "C" int skl_hip_gemm_mfma_streams_c_quads(const skl_gemm_canon *g) {
  if (g->ta != SKL_DT_I8 || g->tb != SKL_DT_I8 || g->a_sk != 1 || g->b_sk != 1 || !streams_in_place(g, 1)) return 0;
  MfmaArgs p;
  p.c = (char *)g->c;
  p.rsc0 = g->rsc0, p.csc0 = g->csc0, p.rsc1 = g->rsc1, p.csc1 = g->csc1;
  p.crs = g->c_row_shift, p.ccs = g->c_col_shift;
  p.bias = (const char *)g->bias, p.max = (char *)g->max;
  p.rq = g->rq;
  return c_in_row_quads(p);
}

// A problem the streaming kernel does not take as it lies in memory - ragged M, N or K, operands off the 16-byte
// rule - can still run on it from copies of A and B padded to whole tiles (rows contiguous in K, `*kp` elements
// apart, `*mp` / `*np` of them, K zero-filled to whole slice pairs) while C stays where it is. Returns the tile
// width (256 or 128) when that is worth it: enough tiles to fill the chip, at most 30 % of padding, and not a
// problem that streams in place anyway; else 0.
extern "C" int skl_hip_gemm_mfma_padded_plan(const skl_gemm_canon *g, size_t *mp, size_t *np, size_t *kp) {
  if (g->m == 0 || g->n == 0 || g->k == 0 || g->ta > SKL_DT_F8E5M2 || g->tb > SKL_DT_F8E5M2) return 0;
  const bool fp8a = g->ta >= SKL_DT_F8E4M3, fp8b = g->tb >= SKL_DT_F8E4M3;
  if (!(g->ta == g->tb || (fp8a && fp8b)) || ((uintptr_t)g->c & 3) != 0) return 0;
  const size_t es = (g->ta == SKL_DT_BF16 || g->ta == SKL_DT_F16) ? 2 : 1;
  if (streams_in_place(g, es)) return 0;
  if (g->rq.act || g->rq.q) return 0;  // the streaming kernel over padded copies has no activation / requantisation steps
  if (fp8a && g->k <= kF8ExactMaxK) return 0;  // short K: the exact fp8 product, which the streaming kernel does not have
  const size_t tiles_m = (g->m + 255) / 256;
  int tile_cols = 0;
  if (tiles_m * ((g->n + 255) / 256) >= 200) tile_cols = 256;
  else if (tiles_m * ((g->n + 127) / 128) >= 96) tile_cols = 128;
  if (!tile_cols) return 0;
  *mp = tiles_m * 256;
  *np = (g->n + tile_cols - 1) / tile_cols * tile_cols;
  *kp = (g->k * es + 127) / 128 * 128 / es;
  const double padded = (double)*mp * (double)*np * (double)*kp, exact = (double)g->m * (double)g->n * (double)g->k;
  if (padded > 1.3 * exact || *kp * es * 256 >= (size_t(1) << 31)) return 0;  // offsets inside a tile stay in 32 bits
  return tile_cols;
}

// `g` describes the padded copies (a_sk == b_sk == 1, rows kp apart in flat blocks of 64, k == kp) and the true
// m, n and C; `tile_cols` is what the plan returned.
extern "C" int skl_hip_launch_gemm_mfma_padded(const skl_gemm_canon *g, int tile_cols) {
  const size_t es = (g->ta == SKL_DT_BF16 || g->ta == SKL_DT_F16) ? 2 : 1;
  if ((tile_cols != 256 && tile_cols != 128) || g->a_sk != 1 || g->b_sk != 1 || (g->k * es) % 128 != 0 ||
      g->a_s1 != 64 * g->a_s0 || g->b_s1 != 64 * g->b_s0 || ((g->a_s0 * es) & 15) != 0 || ((g->b_s0 * es) & 15) != 0 ||
      ((uintptr_t)g->a & 15) != 0 || ((uintptr_t)g->b & 15) != 0 || ((uintptr_t)g->c & 3) != 0) {
    skl_hip_record_error(-2, "gemm_mfma_padded: not a padded problem");
    return -2;
  }
  MfmaArgs p;
  p.a = (const char *)g->a;
  p.b = (const char *)g->b;
  p.c = (char *)g->c;
  p.m = g->m, p.n = g->n, p.k = g->k;
  p.a_s1 = g->a_s1, p.a_s0 = g->a_s0, p.a_sk = g->a_sk;
  p.b_s1 = g->b_s1, p.b_s0 = g->b_s0, p.b_sk = g->b_sk;
  p.rsc0 = g->rsc0, p.csc0 = g->csc0, p.rsc1 = g->rsc1, p.csc1 = g->csc1;
  p.crs = g->c_row_shift, p.ccs = g->c_col_shift;
  p.alpha = g->alpha, p.beta = g->beta;
  p.bias = (const char *)g->bias, p.max = (char *)g->max;
  p.rq = g->rq;
  p.tiles_m = p.tiles_n = 0;
  p.splits = 1, p.slices_per_split = 0, p.partial = nullptr;
  switch (g->ta * 8 + g->tb) {
    case SKL_DT_I8 * 8 + SKL_DT_I8: return skl_mfma_launch_padded_i8(p, tile_cols);
    case SKL_DT_BF16 * 8 + SKL_DT_BF16: return skl_mfma_launch_padded_bf16(p, tile_cols);
    case SKL_DT_F16 * 8 + SKL_DT_F16: return skl_mfma_launch_padded_f16(p, tile_cols);
    case SKL_DT_F8E4M3 * 8 + SKL_DT_F8E4M3: return skl_mfma_launch_padded_f8e4m3(p, tile_cols);
    case SKL_DT_F8E5M2 * 8 + SKL_DT_F8E5M2: return skl_mfma_launch_padded_f8e5m2(p, tile_cols);
    case SKL_DT_F8E4M3 * 8 + SKL_DT_F8E5M2: return skl_mfma_launch_padded_f8e4m3_f8e5m2(p, tile_cols);
    case SKL_DT_F8E5M2 * 8 + SKL_DT_F8E4M3: return skl_mfma_launch_padded_f8e5m2_f8e4m3(p, tile_cols);
    default:
      skl_hip_record_error(-2, "gemm_mfma_padded: operand type pair");
      return -2;
  }
}

// C = beta*C + alpha*P, then the fused steps (bias, activation, 8-bit copy, maximum), for a product P that another
// kernel has left as a row-major M x N matrix of C's type in scratch memory: the pass that adds the shares of K,
// given one share. What a streaming kernel without fused steps needs to serve a fused call (int32 C: the detour is
// exact).
namespace {
// The epilogue pass on a product that lives in the stream's block of sums: the same steps, and the element read is
// put back to zero (the block is zero between calls).
__global__ void __launch_bounds__(256) gemm_epilogue_zeroing_kernel(MfmaArgs p) {
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= p.m * p.n) return;
  const size_t row = idx / p.n, col = idx % p.n;
  int *product = reinterpret_cast<int *>(p.partial) + idx;
  const int sum = *product;
  *product = 0;
  int *c = reinterpret_cast<int *>(p.c) + (row >> p.crs) * p.rsc1 + (row & ((size_t(1) << p.crs) - 1)) * p.rsc0 +
           (col >> p.ccs) * p.csc1 + (col & ((size_t(1) << p.ccs) - 1)) * p.csc0;
  int v = skl_beta_is_zero<int>(p.beta) ? skl_initialise(sum, c, p.alpha, p.beta) : skl_combine(sum, *c, p.alpha, p.beta);
  if (p.bias) v = skl_add_bias(v, reinterpret_cast<const int *>(p.bias)[col]);
  v = skl_activate(v, p.rq.act);
  if (!p.rq.q_only) *c = v;
  skl_emit_requantised(p.rq, v, row, col);
  if (p.max && v > skl_lowest<int>()) skl_atomic_max(reinterpret_cast<int *>(p.max), v);
}
int launch_epilogue(const skl_gemm_canon *g, const void *product, bool zeroing);
}  // namespace

extern "C" int skl_hip_launch_gemm_epilogue(const skl_gemm_canon *g, const void *product) { return launch_epilogue(g, product, false); }
extern "C" int skl_hip_launch_gemm_epilogue_zeroing(const skl_gemm_canon *g, void *product) { return launch_epilogue(g, product, true); }

namespace {
int launch_epilogue(const skl_gemm_canon *g, const void *product, bool zeroing) {
  if (g->ta != SKL_DT_I8 || g->tb != SKL_DT_I8 || g->m == 0 || g->n == 0 || !product || ((uintptr_t)g->c & 3) != 0 ||
      ((uintptr_t)product & 3) != 0 || g->c_row_shift > 6 || g->c_col_shift > 6) {
    skl_hip_record_error(-2, "gemm_epilogue: unsupported problem");
    return -2;
  }
  MfmaArgs p;
  p.a = p.b = nullptr;
  p.c = (char *)g->c;
  p.m = g->m, p.n = g->n, p.k = g->k;
  p.a_s1 = p.a_s0 = p.a_sk = p.b_s1 = p.b_s0 = p.b_sk = 0;
  p.rsc0 = g->rsc0, p.csc0 = g->csc0, p.rsc1 = g->rsc1, p.csc1 = g->csc1;
  p.crs = g->c_row_shift, p.ccs = g->c_col_shift;
  p.alpha = g->alpha, p.beta = g->beta;
  p.bias = (const char *)g->bias, p.max = (char *)g->max;
  p.rq = g->rq;
  p.tiles_m = p.tiles_n = 0;
  p.splits = 1, p.slices_per_split = 0, p.partial = (char *)product;
  const size_t blocks = (p.m * p.n + 255) / 256;
  if (blocks > 0x7FFFFFFFu) {
    skl_hip_record_error(-2, "gemm_epilogue: grid too large");
    return -2;
  }
  if (zeroing)
    gemm_epilogue_zeroing_kernel<<<(unsigned)blocks, 256, 0, skl_current_stream()>>>(p);
  else
    gemm_split_reduce_kernel<int><<<(unsigned)blocks, 256, 0, skl_current_stream()>>>(p);
  return skl_check_launch("gemm_epilogue");
}
}  // namespace

extern "C" int skl_hip_launch_gemm_mfma(const skl_gemm_canon *g) {
  if (!skl_hip_gemm_mfma_supported(g)) {
    skl_hip_record_error(-2, "gemm_mfma: unsupported problem");
    return -2;
  }
  MfmaArgs p;
  p.a = (const char *)g->a;
  p.b = (const char *)g->b;
  p.c = (char *)g->c;
  p.m = g->m, p.n = g->n, p.k = g->k;
  p.a_s1 = g->a_s1, p.a_s0 = g->a_s0, p.a_sk = g->a_sk;
  p.b_s1 = g->b_s1, p.b_s0 = g->b_s0, p.b_sk = g->b_sk;
  p.rsc0 = g->rsc0, p.csc0 = g->csc0, p.rsc1 = g->rsc1, p.csc1 = g->csc1;
  p.crs = g->c_row_shift, p.ccs = g->c_col_shift;
  p.alpha = g->alpha, p.beta = g->beta;
  p.bias = (const char *)g->bias, p.max = (char *)g->max;
  p.rq = g->rq;
  p.tiles_m = p.tiles_n = 0;
  p.splits = 1, p.slices_per_split = 0, p.partial = nullptr;
  switch (g->ta * 8 + g->tb) {
    case SKL_DT_I8 * 8 + SKL_DT_I8: return skl_mfma_launch_i8(p);
    case SKL_DT_BF16 * 8 + SKL_DT_BF16: return skl_mfma_launch_bf16(p);
    case SKL_DT_F16 * 8 + SKL_DT_F16: return skl_mfma_launch_f16(p);
    case SKL_DT_F8E4M3 * 8 + SKL_DT_F8E4M3: return skl_mfma_launch_f8e4m3(p);
    case SKL_DT_F8E5M2 * 8 + SKL_DT_F8E5M2: return skl_mfma_launch_f8e5m2(p);
    case SKL_DT_F8E4M3 * 8 + SKL_DT_F8E5M2: return skl_mfma_launch_f8e4m3_f8e5m2(p);
    case SKL_DT_F8E5M2 * 8 + SKL_DT_F8E4M3: return skl_mfma_launch_f8e5m2_f8e4m3(p);
    default:
      skl_hip_record_error(-2, "gemm_mfma: operand type pair");
      return -2;
  }
}
