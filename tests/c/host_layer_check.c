/* host_layer_check.c - the C host layer (skl_amd/csrc/skl_api.c) under AddressSanitizer and
 * UndefinedBehaviorSanitizer, on the CPU, without a GPU.
 *
 * Built by `make -C skl_amd/csrc asan`: skl_api.c is compiled with -fsanitize=address,undefined and linked with
 * the library's real objects, so that the questions the host layer asks ("would this kernel take the problem?",
 * the padded-tile plan) get the real answers - but every function that would touch the GPU (launchers, buffers,
 * copies, pointer queries) is redirected here with the linker's --wrap. The stand-ins
 *   - check that every element a descriptor addresses lies inside a buffer the caller (or the host layer, for its
 *     scratch copies) owns: the registry below, on top of what the sanitizer's red zones catch;
 *   - check that the launcher's own "supported" predicate holds for what it is handed;
 *   - carry the operation out with plain loops over the descriptor, so that the result of the whole call - through
 *     canonicalisation, operand copies, padded tiles, row chunks, staging of host buffers - can be compared with
 *     loops over the caller's original arguments.
 * Operands hold small integers (exact in every element kind and in any summation order), so results must be equal.
 * The cases are drawn at random: every GEMM form and element kind, both pointer modes, blocked layouts with the four
 * index levels nested in a random order and padded, pack / unpack / transpose and the conversions. */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "skl-gfx950.h"
#include "../../skl_amd/csrc/skl_launch.h"

/* ------------------------------------------------------------------ registry of owned byte ranges */
typedef struct {
  const char *lo, *hi;
  int device; /* what skl_hip_pointer_is_device answers for addresses inside */
} range_t;
static range_t g_ranges[256];
static int g_nranges;
static long g_checked, g_launches;
static int g_failures;
/* how often each stand-in ran: the summary shows which routes of the dispatch the cases reached */
enum { P_GENERIC, P_TILED, P_MFMA, P_PADDED, P_EPILOGUE, P_GEMV, P_GEMV_K4, P_ROWS, P_MFMA_ROWS, P_MFMA_ROWS_K4, P_KC, P_REALIGN, P_PACK, P_UNPACK, P_CVT, P_F4, P_SCARCE, P_COUNT };
static const char *const kPathNames[P_COUNT] = {"any-stride", "register-tiled", "matrix-core", "padded tiles", "epilogue pass", "GEMV", "GEMV K-packed", "few rows",
                                                "decode batch", "decode batch K-packed", "dot-product GEMV", "operand copy", "pack", "unpack", "cvt", "4-bit weights",
                                                "declined: no scratch"};
static long g_path[P_COUNT];

static void range_add(const void *p, size_t bytes, int device) {
  if (g_nranges == 256) abort();
  g_ranges[g_nranges++] = (range_t){(const char *)p, (const char *)p + bytes, device};
}
static void range_remove(const void *p) {
  for (int i = 0; i < g_nranges; ++i)
    if (g_ranges[i].lo == (const char *)p) {
      g_ranges[i] = g_ranges[--g_nranges];
      return;
    }
}
static const range_t *range_of(const void *p) {
  for (int i = 0; i < g_nranges; ++i)
    if ((const char *)p >= g_ranges[i].lo && (const char *)p < g_ranges[i].hi) return &g_ranges[i];
  return NULL;
}
static void fail(const char *what) {
  fprintf(stderr, "FAIL: %s\n", what);
  ++g_failures;
}
/* [p + first*es, p + (last+1)*es) must lie in one owned range */
static void must_own(const void *p, size_t first, size_t last, size_t es, const char *what) {
  const char *lo = (const char *)p + first * es, *hi = (const char *)p + (last + 1) * es;
  const range_t *r = range_of(lo);
  ++g_checked;
  if (!r || hi > r->hi) {
    fprintf(stderr, "FAIL: %s addresses bytes outside the caller's buffer\n", what);
    ++g_failures;
  }
}

/* ------------------------------------------------------------------ element kinds */
static size_t esize(int dt) {
  return dt == SKL_DT_F64 ? 8 : dt == SKL_DT_F32 ? 4 : (dt == SKL_DT_BF16 || dt == SKL_DT_F16 || dt == SKL_DT_F16H) ? 2 : 1;
}
static size_t c_esize(int dt) { return dt == SKL_DT_F64 ? 8 : dt == SKL_DT_F16H ? 2 : 4; }

static double f8_value(unsigned code, int ebits) { /* finite codes only */
  const int mbits = 7 - ebits, bias = (1 << (ebits - 1)) - 1;
  const int e = (int)((code & 0x7F) >> mbits), m = (int)(code & ((1u << mbits) - 1));
  const double mag = e ? ldexp(1.0 + m / (double)(1 << mbits), e - bias) : ldexp(m / (double)(1 << mbits), 1 - bias);
  return (code & 0x80) ? -mag : mag;
}
/* x as an OCP fp8 code by search over the codes: the nearest value, a tie to the code with an even last bit, and one
 * value beyond the largest (480 / 65536) standing for overflow, which gives the largest finite code when saturating,
 * else E4M3's NaN without a sign or E5M2's infinity (ref/cvt/cvt_ofp8.c:97-172). Finite x only. */
static uint8_t f8_encode(double x, int ebits, int sat) {
  const unsigned top = ebits == 4 ? 0x7F : 0x7C;
  const uint8_t sign = signbit(x) ? 0x80 : 0;
  const double mag = fabs(x), beyond = ebits == 4 ? 480.0 : 65536.0;
  unsigned best = 0;
  double best_d = mag;
  for (unsigned code = 1; code <= top; ++code) {
    const double d = fabs((code == top ? beyond : f8_value(code, ebits)) - mag);
    if (d < best_d || (d == best_d && !(code & 1))) best = code, best_d = d;
  }
  if (best == top || mag > beyond) return sat ? (uint8_t)(sign | (top - 1)) : ebits == 4 ? 0x7F : (uint8_t)(sign | 0x7C);
  return (uint8_t)(sign | best);
}
static double load_elem(int dt, const void *base, size_t i) {
  switch (dt) {
    case SKL_DT_I8: return ((const int8_t *)base)[i];
    case SKL_DT_BF16: {
      const uint32_t bits = (uint32_t)((const uint16_t *)base)[i] << 16;
      float f;
      memcpy(&f, &bits, 4);
      return f;
    }
    case SKL_DT_F16:
    case SKL_DT_F16H: return (double)((const _Float16 *)base)[i];
    case SKL_DT_F8E4M3: return f8_value(((const uint8_t *)base)[i], 4);
    case SKL_DT_F8E5M2: return f8_value(((const uint8_t *)base)[i], 5);
    case SKL_DT_F32: return ((const float *)base)[i];
    default: return ((const double *)base)[i];
  }
}
/* small integers -2 .. 2 in every kind */
static void store_small(int dt, void *base, size_t i, int v) {
  static const uint16_t bf[5] = {0xC000, 0xBF80, 0x0000, 0x3F80, 0x4000};
  static const uint8_t e4[5] = {0xC0, 0xB8, 0x00, 0x38, 0x40}, e5[5] = {0xC0, 0xBC, 0x00, 0x3C, 0x40};
  switch (dt) {
    case SKL_DT_I8: ((int8_t *)base)[i] = (int8_t)v; break;
    case SKL_DT_BF16: ((uint16_t *)base)[i] = bf[v + 2]; break;
    case SKL_DT_F16:
    case SKL_DT_F16H: ((_Float16 *)base)[i] = (_Float16)v; break;
    case SKL_DT_F8E4M3: ((uint8_t *)base)[i] = e4[v + 2]; break;
    case SKL_DT_F8E5M2: ((uint8_t *)base)[i] = e5[v + 2]; break;
    case SKL_DT_F32: ((float *)base)[i] = (float)v; break;
    default: ((double *)base)[i] = v; break;
  }
}
static double load_c(int dt, const void *c, size_t i) {
  if (dt == SKL_DT_I8) return ((const int32_t *)c)[i];
  if (dt == SKL_DT_F64) return ((const double *)c)[i];
  if (dt == SKL_DT_F16H) return (double)((const _Float16 *)c)[i];
  return ((const float *)c)[i];
}
static void store_c(int dt, void *c, size_t i, double v) {
  if (dt == SKL_DT_I8) ((int32_t *)c)[i] = (int32_t)v;
  else if (dt == SKL_DT_F64) ((double *)c)[i] = v;
  else if (dt == SKL_DT_F16H) ((_Float16 *)c)[i] = (_Float16)v;
  else ((float *)c)[i] = (float)v;
}
static double scalar_of(int dt, skl_scalar s) { return dt == SKL_DT_I8 ? s.i : dt == SKL_DT_F64 ? s.d : s.f; }

/* ------------------------------------------------------------------ plain loops over the two descriptors */
/* A floating-point call that writes only the 8-bit copy, with beta == 0, neither writes nor reads C: the old C counts
 * as +0 (include/skl-gfx950.h). `marked`: what the host layer put next to beta for the kernels (checked where the
 * descriptor comes from the host layer). */
static int c_is_unread(int dt, const skl_requant *rq, double beta, int from_host_layer, skl_scalar raw_beta, const char *who) {
  const int unread = rq->q && rq->q_only && beta == 0 && dt != SKL_DT_I8 && dt != SKL_DT_F64 && dt != SKL_DT_F32 && dt != SKL_DT_F16H;
  if (from_host_layer && unread != (dt != SKL_DT_I8 && dt != SKL_DT_F64 && raw_beta.fz.skip_c_read == 2)) {
    fprintf(stderr, "FAIL: %s: beta is not marked as the call asks (C untouched: %d)\n", who, unread);
    ++g_failures;
  }
  return unread;
}
/* The fused steps behind the alpha/beta step for element (i, j) of value v (include/skl-gfx950.h): bias, activation,
 * C unless q_only, the requantised copy, the maximum. Scales are powers of two and values small integers here, so
 * double arithmetic gives the float result exactly. */
static void fused_steps(int dt, void *c, size_t idx, size_t i, size_t j, double v, const void *bias, void *max, const skl_requant *rq,
                        const char *who) {
  if (bias) v += load_c(dt, bias, j);
  if (rq->act == 1 && !(v > 0)) v = 0;
  if (!rq->q_only) store_c(dt, c, idx, v);
  if (rq->q) {
    const size_t at = i * rq->rsq + j * rq->csq;
    double r;
    long t;
    must_own(rq->q, at, at, 1, who);
    must_own(rq->q_scale, rq->q_per_column ? j : 0, rq->q_per_column ? j : 0, sizeof(float), who);
    if (g_failures) return;
    if (rq->q_fmt) {
      rq->q[at] = (int8_t)f8_encode(v * (double)rq->q_scale[rq->q_per_column ? j : 0], rq->q_fmt <= 2 ? 4 : 5, rq->q_fmt == 2 || rq->q_fmt == 4);
    } else {
      r = nearbyint(v * (double)rq->q_scale[rq->q_per_column ? j : 0]);
      t = (long)(r > 1e9 ? 1e9 : r < -1e9 ? -1e9 : r) + rq->q_zero;
      rq->q[at] = (int8_t)(t < -128 ? -128 : t > 127 ? 127 : t);
    }
  }
  if (max && v > load_c(dt, max, 0)) store_c(dt, max, 0, v);
}

static void gemm_over_desc(const skl_gemm_desc *d, int check, const char *who) {
  const size_t esa = esize(d->ta), esb = esize(d->tb), esc = c_esize(d->ta);
  const size_t K = d->k0 * d->k1;
  if (check) {
    if (K) {
      must_own(d->a, 0, (d->m1 - 1) * d->rsa1 + (d->k1 - 1) * d->csa1 + (d->m0 - 1) * d->rsa0 + (d->k0 - 1) * d->csa0, esa, who);
      must_own(d->b, 0, (d->k1 - 1) * d->rsb1 + (d->n1 - 1) * d->csb1 + (d->k0 - 1) * d->rsb0 + (d->n0 - 1) * d->csb0, esb, who);
    }
  }
  const double alpha = scalar_of(d->ta, d->alpha), beta = scalar_of(d->ta, d->beta);
  const int c_unread = c_is_unread(d->ta, &d->rq, beta, check, d->beta, who);
  if (check && !c_unread) /* a C that is neither written nor read need not exist */
    must_own(d->c, 0, (d->m1 - 1) * d->rsc1 + (d->n1 - 1) * d->csc1 + (d->m0 - 1) * d->rsc0 + (d->n0 - 1) * d->csc0, esc, who);
  for (size_t I = 0; I < d->m1; ++I)
    for (size_t i = 0; i < d->m0; ++i)
      for (size_t J = 0; J < d->n1; ++J)
        for (size_t j = 0; j < d->n0; ++j) {
          double acc = 0;
          if (d->ta == SKL_DT_I8 && d->k0 == 1 && d->k1 != 0) { /* the common case without the per-element dispatch (K = 0: A and B may be null) */
            const int8_t *ap = (const int8_t *)d->a + I * d->rsa1 + i * d->rsa0, *bp = (const int8_t *)d->b + J * d->csb1 + j * d->csb0;
            long sum = 0;
            for (size_t P = 0; P < d->k1; ++P) sum += (long)ap[P * d->csa1] * bp[P * d->rsb1];
            acc = (double)sum;
          } else {
            for (size_t P = 0; P < d->k1; ++P)
              for (size_t p = 0; p < d->k0; ++p)
                acc += load_elem(d->ta, d->a, I * d->rsa1 + P * d->csa1 + i * d->rsa0 + p * d->csa0) *
                       load_elem(d->tb, d->b, P * d->rsb1 + J * d->csb1 + p * d->rsb0 + j * d->csb0);
          }
          const size_t idx = I * d->rsc1 + J * d->csc1 + i * d->rsc0 + j * d->csc0;
          fused_steps(d->ta, d->c, idx, I * d->m0 + i, J * d->n0 + j, beta * (c_unread ? 0.0 : load_c(d->ta, d->c, idx)) + alpha * acc, d->bias,
                      d->max, &d->rq, who);
        }
}

/* layout: 0 the canonical form of skl_launch.h, 1 the K-packed int8 B (rows of A contiguous in K, a_s0 apart) */
static void gemm_over_canon(const skl_gemm_canon *g, int layout, const char *who) {
  const size_t esa = esize(g->ta), esb = esize(g->tb), esc = c_esize(g->ta);
  const size_t rmask = ((size_t)1 << g->c_row_shift) - 1, cmask = ((size_t)1 << g->c_col_shift) - 1;
  const double alpha = scalar_of(g->ta, g->alpha), beta = scalar_of(g->ta, g->beta);
  const int c_unread = c_is_unread(g->ta, &g->rq, beta, 1, g->beta, who);
  size_t a_max = 0, b_max = 0, c_max = 0;
  ++g_launches;
  for (size_t i = 0; i < g->m; ++i)
    for (size_t j = 0; j < g->n; ++j) {
      double acc = 0;
      if (g->ta == SKL_DT_I8 && layout == 0 && (i || j) && g->k) { /* corners were checked at (0, 0); plain int8 loop */
        const int8_t *ap = (const int8_t *)g->a + (i / 64) * g->a_s1 + (i % 64) * g->a_s0, *bp = (const int8_t *)g->b + (j / 64) * g->b_s1 + (j % 64) * g->b_s0;
        long sum = 0;
        for (size_t p = 0; p < g->k; ++p) sum += (long)ap[p * g->a_sk] * bp[p * g->b_sk];
        acc = (double)sum;
        if ((size_t)(ap - (const int8_t *)g->a) + (g->k - 1) * g->a_sk > a_max) a_max = (size_t)(ap - (const int8_t *)g->a) + (g->k - 1) * g->a_sk;
        if ((size_t)(bp - (const int8_t *)g->b) + (g->k - 1) * g->b_sk > b_max) b_max = (size_t)(bp - (const int8_t *)g->b) + (g->k - 1) * g->b_sk;
      } else
      for (size_t p = 0; p < g->k; ++p) {
        const size_t ia = layout == 1 ? i * g->a_s0 + p : (i / 64) * g->a_s1 + (i % 64) * g->a_s0 + p * g->a_sk;
        const size_t ib = layout == 1 ? (p / 4) * g->b_sk + j * 4 + p % 4 : (j / 64) * g->b_s1 + (j % 64) * g->b_s0 + p * g->b_sk;
        if (ia > a_max) a_max = ia;
        if (ib > b_max) b_max = ib;
        if (i == 0 && j == 0 && p == 0) { /* the far corners first: a wild descriptor is reported, not dereferenced */
          const size_t i9 = g->m - 1, j9 = g->n - 1, p9 = g->k - 1;
          must_own(g->a, 0, layout == 1 ? i9 * g->a_s0 + p9 : (i9 / 64) * g->a_s1 + (i9 % 64) * g->a_s0 + p9 * g->a_sk, esa, who);
          must_own(g->b, 0, layout == 1 ? (p9 / 4) * g->b_sk + j9 * 4 + p9 % 4 : (j9 / 64) * g->b_s1 + (j9 % 64) * g->b_s0 + p9 * g->b_sk, esb, who);
          if (!c_unread) must_own(g->c, 0, (i9 >> g->c_row_shift) * g->rsc1 + (i9 & rmask) * g->rsc0 + (j9 >> g->c_col_shift) * g->csc1 + (j9 & cmask) * g->csc0, esc, who);
          if (g_failures) return;
        }
        acc += load_elem(g->ta, g->a, ia) * load_elem(g->tb, g->b, ib);
      }
      const size_t idx = (i >> g->c_row_shift) * g->rsc1 + (i & rmask) * g->rsc0 + (j >> g->c_col_shift) * g->csc1 + (j & cmask) * g->csc0;
      if (idx > c_max) c_max = idx;
      if (g->k == 0 && i == 0 && j == 0 && !c_unread) must_own(g->c, 0, 0, esc, who);
      fused_steps(g->ta, g->c, idx, i, j, beta * (c_unread ? 0.0 : load_c(g->ta, g->c, idx)) + alpha * acc, g->bias, g->max, &g->rq, who);
    }
  if (g->k) {
    must_own(g->a, 0, a_max, esa, who);
    must_own(g->b, 0, b_max, esb, who);
  }
  if (!c_unread) must_own(g->c, 0, c_max, esc, who);
}

/* ------------------------------------------------------------------ the redirected GPU layer */
/* Scratch memory runs out: every kernel that would use some reports so before launching anything, as the real
 * launchers do, and the copies of operands get no memory either. The call must then end on a kernel that needs
 * none, with the right result and no error left recorded. */
static int g_scarce;
#define SCARCE(what)                                          \
  do {                                                        \
    if (g_scarce) {                                           \
      ++g_path[P_SCARCE];                                     \
      skl_hip_record_error(SKL_HIP_ERR_WORKSPACE, what);      \
      return SKL_HIP_ERR_WORKSPACE;                           \
    }                                                         \
  } while (0)
int __wrap_skl_hip_gemv_reserve_scratch(void) {
  SCARCE("reserve (stand-in)");
  return 0;
}

#define EXPECT(cond, what) \
  do {                     \
    if (!(cond)) fail(what); \
  } while (0)

int __wrap_skl_hip_launch_gemm_generic(const skl_gemm_desc *d) {
  ++g_launches, ++g_path[P_GENERIC];
  gemm_over_desc(d, 1, "any-stride GEMM");
  return 0;
}
int __wrap_skl_hip_launch_gemm_tiled(const skl_gemm_canon *g) {
  EXPECT(skl_hip_gemm_tiled_supported(g), "register-tiled GEMM handed a problem it does not support");
  ++g_path[P_TILED];
  gemm_over_canon(g, 0, "register-tiled GEMM");
  return 0;
}
int __wrap_skl_hip_launch_gemm_mfma(const skl_gemm_canon *g) {
  SCARCE("matrix-core GEMM (stand-in)");
  EXPECT(skl_hip_gemm_mfma_supported(g), "matrix-core GEMM handed a problem it does not support");
  ++g_path[P_MFMA];
  gemm_over_canon(g, 0, "matrix-core GEMM");
  return 0;
}
/* C = beta*C + alpha*product and the fused steps, the product a row-major m x n int32 matrix in scratch memory. */
static int epilogue_pass(const skl_gemm_canon *g, const void *product) {
  const size_t rmask = ((size_t)1 << g->c_row_shift) - 1, cmask = ((size_t)1 << g->c_col_shift) - 1;
  const double alpha = scalar_of(g->ta, g->alpha), beta = scalar_of(g->ta, g->beta);
  EXPECT(g->ta == SKL_DT_I8 && g->tb == SKL_DT_I8 && g->m && g->n, "epilogue pass: int8 problems only");
  ++g_launches, ++g_path[P_EPILOGUE];
  must_own(product, 0, g->m * g->n - 1, 4, "epilogue pass (product)");
  must_own(g->c, 0, ((g->m - 1) >> g->c_row_shift) * g->rsc1 + ((g->m - 1) & rmask) * g->rsc0 + ((g->n - 1) >> g->c_col_shift) * g->csc1 +
                        ((g->n - 1) & cmask) * g->csc0, 4, "epilogue pass (C)");
  if (g_failures) return 0;
  for (size_t i = 0; i < g->m; ++i)
    for (size_t j = 0; j < g->n; ++j) {
      const size_t idx = (i >> g->c_row_shift) * g->rsc1 + (i & rmask) * g->rsc0 + (j >> g->c_col_shift) * g->csc1 + (j & cmask) * g->csc0;
      fused_steps(g->ta, g->c, idx, i, j, beta * load_c(g->ta, g->c, idx) + alpha * (double)((const int32_t *)product)[i * g->n + j], g->bias, g->max,
                  &g->rq, "epilogue pass");
    }
  return 0;
}
int __wrap_skl_hip_launch_gemm_epilogue(const skl_gemm_canon *g, const void *product) { return epilogue_pass(g, product); }
/* The stream's block of sums, zero between calls: handed out for a product only while it is zero, and whoever reads
 * the product has to leave it zero again. */
static int32_t *g_zeroed_sums;
static size_t g_zeroed_sums_bytes;
void *__wrap_skl_hip_zeroed_sums(size_t bytes) {
  if (g_scarce) return NULL;
  if (bytes > g_zeroed_sums_bytes) {
    if (g_zeroed_sums) {
      range_remove(g_zeroed_sums);
      free(g_zeroed_sums);
    }
    g_zeroed_sums = calloc(1, bytes);
    g_zeroed_sums_bytes = bytes;
    range_add(g_zeroed_sums, bytes, 1);
  }
  for (size_t i = 0; i < g_zeroed_sums_bytes / 4; ++i) EXPECT(g_zeroed_sums[i] == 0, "block of sums handed out while not zero");
  return g_zeroed_sums;
}
int __wrap_skl_hip_launch_gemm_epilogue_zeroing(const skl_gemm_canon *g, void *product) {
  EXPECT(product == (void *)g_zeroed_sums, "zeroing epilogue pass on a product outside the block of sums");
  const int rc = epilogue_pass(g, product);
  if (!g_failures) memset(product, 0, g->m * g->n * 4);
  return rc;
}
int __wrap_skl_hip_launch_gemm_mfma_padded(const skl_gemm_canon *g, int tile_cols) {
  SCARCE("padded GEMM (stand-in)");
  const size_t es = esize(g->ta);
  EXPECT(tile_cols == 256 || tile_cols == 128, "padded GEMM: tile width");
  EXPECT(g->a_sk == 1 && g->b_sk == 1 && (g->k * es) % 128 == 0, "padded GEMM: K not padded to whole slice pairs");
  /* the kernel reads whole tiles of the copies: the padded rows must exist */
  must_own(g->a, 0, ((g->m + 255) / 256 * 256 - 1) * g->a_s0 + g->k - 1, es, "padded GEMM (rows of A up to the tile edge)");
  must_own(g->b, 0, ((g->n + (size_t)tile_cols - 1) / (size_t)tile_cols * (size_t)tile_cols - 1) * g->b_s0 + g->k - 1, es,
           "padded GEMM (rows of B up to the tile edge)");
  ++g_path[P_PADDED];
  gemm_over_canon(g, 0, "padded GEMM");
  return 0;
}
int __wrap_skl_hip_launch_gemv(const skl_gemm_canon *g, int layout) {
  SCARCE("GEMV (stand-in)");
  EXPECT(skl_hip_gemv_supported(g, layout), "GEMV handed a problem it does not support");
  ++g_path[layout ? P_GEMV_K4 : P_GEMV];
  gemm_over_canon(g, layout, "GEMV");
  return 0;
}
int __wrap_skl_hip_launch_gemv_rows(const skl_gemm_canon *g) {
  SCARCE("few-rows GEMV (stand-in)");
  EXPECT(skl_hip_gemv_rows_supported(g), "few-rows GEMV handed a problem it does not support");
  ++g_path[P_ROWS];
  gemm_over_canon(g, 0, "few-rows GEMV");
  return 0;
}
int __wrap_skl_hip_launch_gemv_mfma_rows(const skl_gemm_canon *g, int layout) {
  SCARCE("decode batch (stand-in)");
  EXPECT(skl_hip_gemv_mfma_rows_supported(g, layout), "decode-batch kernel handed a problem it does not support");
  ++g_path[layout ? P_MFMA_ROWS_K4 : P_MFMA_ROWS];
  gemm_over_canon(g, layout, "decode-batch kernel");
  return 0;
}
int __wrap_skl_hip_launch_gemv_kc(const skl_gemm_canon *g) {
  SCARCE("dot-product GEMV (stand-in)");
  EXPECT(skl_hip_gemv_kc_supported(g), "dot-product GEMV handed a problem it does not support");
  ++g_path[P_KC];
  gemm_over_canon(g, 0, "dot-product GEMV");
  return 0;
}
int __wrap_skl_hip_launch_gemv_kc_rows(const skl_gemm_canon *g) {
  SCARCE("decode batch on K-contiguous weights (stand-in)");
  EXPECT(skl_hip_gemv_kc_rows_supported(g), "decode batch on K-contiguous weights handed a problem it does not support");
  ++g_path[P_KC];
  gemm_over_canon(g, 0, "decode batch on K-contiguous weights");
  return 0;
}
int __wrap_skl_hip_launch_gemv_noalloc(const skl_gemm_canon *g) {
  if (g->m < 1 || g->m > 8 || g->m * g->n > 65536 || (g->m == 1 ? !skl_hip_gemv_supported(g, 0) : !skl_hip_gemv_rows_supported(g))) {
    skl_hip_record_error(SKL_HIP_ERR_BAD_ARGUMENT, "noalloc (stand-in)");
    return SKL_HIP_ERR_BAD_ARGUMENT;
  }
  gemm_over_canon(g, 0, "decode call without allocation");
  return 0;
}

int __wrap_skl_hip_launch_realign(int es, size_t x, size_t k, const void *src, size_t x0, size_t s0, size_t s1, size_t k0,
                                  size_t sk0, size_t sk1, void *dst, size_t kp) {
  ++g_launches, ++g_path[P_REALIGN];
  EXPECT(kp >= k && x0 > 0 && k0 > 0, "operand copy: pitch below K");
  if (x == 0) return 0;
  must_own(dst, 0, x * kp - 1, (size_t)es, "operand copy (destination)");
  if (k) must_own(src, 0, ((x - 1) / x0) * s1 + ((x - 1) % x0) * s0 + ((k - 1) / k0) * sk1 + ((k - 1) % k0) * sk0, (size_t)es, "operand copy (source corner)");
  if (g_failures) return 0;
  for (size_t i = 0; i < x; ++i)
    for (size_t p = 0; p < kp; ++p) {
      char *to = (char *)dst + (i * kp + p) * (size_t)es;
      if (p < k)
        memcpy(to, (const char *)src + ((i / x0) * s1 + (i % x0) * s0 + (p / k0) * sk1 + (p % k0) * sk0) * (size_t)es, (size_t)es);
      else
        memset(to, 0, (size_t)es);
    }
  return 0;
}

/* ref/pack/pack_e8rc_e8rcprc.c:10-35 and ref/pack/unpack_e8rcprc_e8rc.c:10-37, restated */
static void pack_loops(int es, size_t m, size_t n, const void *src, size_t rs, size_t cs, size_t m0, size_t n0, void *dst,
                       size_t rs0, size_t cs0, size_t rs1, size_t cs1, uint32_t pad, int check) {
  const size_t m1 = (m + m0 - 1) / m0, n1 = (n + n0 - 1) / n0;
  if (check) {
    must_own(src, 0, (m - 1) * rs + (n - 1) * cs, (size_t)es, "pack (source)");
    must_own(dst, 0, (m1 - 1) * rs1 + (n1 - 1) * cs1 + (m0 - 1) * rs0 + (n0 - 1) * cs0, (size_t)es, "pack (destination)");
    if (g_failures) return;
  }
  for (size_t i1 = 0; i1 < m1; ++i1)
    for (size_t j1 = 0; j1 < n1; ++j1)
      for (size_t i0 = 0; i0 < m0; ++i0)
        for (size_t j0 = 0; j0 < n0; ++j0) {
          const size_t i = i1 * m0 + i0, j = j1 * n0 + j0;
          char *to = (char *)dst + (i1 * rs1 + j1 * cs1 + i0 * rs0 + j0 * cs0) * (size_t)es;
          if (i < m && j < n)
            memcpy(to, (const char *)src + (i * rs + j * cs) * (size_t)es, (size_t)es);
          else
            memcpy(to, &pad, (size_t)es);
        }
}
static void unpack_loops(int es, size_t m0, size_t n0, const void *src, size_t rs0, size_t cs0, size_t rs1, size_t cs1, size_t m,
                         size_t n, void *dst, size_t rs, size_t cs, int check) {
  if (check) {
    size_t far_src = 0;
    for (size_t i = m > m0 ? m - m0 : 0; i < m; ++i)   /* the farthest source element is in the last blocks */
      for (size_t j = n > n0 ? n - n0 : 0; j < n; ++j) {
        const size_t at = (i / m0) * rs1 + (j / n0) * cs1 + (i % m0) * rs0 + (j % n0) * cs0;
        if (at > far_src) far_src = at;
      }
    must_own(src, 0, far_src, (size_t)es, "unpack (source)");
    must_own(dst, 0, (m - 1) * rs + (n - 1) * cs, (size_t)es, "unpack (destination)");
    if (g_failures) return;
  }
  for (size_t i = 0; i < m; ++i)
    for (size_t j = 0; j < n; ++j)
      memcpy((char *)dst + (i * rs + j * cs) * (size_t)es,
             (const char *)src + ((i / m0) * rs1 + (j / n0) * cs1 + (i % m0) * rs0 + (j % n0) * cs0) * (size_t)es, (size_t)es);
}
int __wrap_skl_hip_launch_pack(int es, size_t m, size_t n, const void *src, size_t rs, size_t cs, size_t m0, size_t n0, void *dst,
                               size_t rs0, size_t cs0, size_t rs1, size_t cs1, uint32_t pad) {
  ++g_launches, ++g_path[P_PACK];
  pack_loops(es, m, n, src, rs, cs, m0, n0, dst, rs0, cs0, rs1, cs1, pad, 1);
  return 0;
}
int __wrap_skl_hip_launch_unpack(int es, size_t m0, size_t n0, const void *src, size_t rs0, size_t cs0, size_t rs1, size_t cs1,
                                 size_t m, size_t n, void *dst, size_t rs, size_t cs) {
  ++g_launches, ++g_path[P_UNPACK];
  unpack_loops(es, m0, n0, src, rs0, cs0, rs1, cs1, m, n, dst, rs, cs, 1);
  return 0;
}
/* conversions: the spans only (what the kernels compute is pinned elsewhere); dst gets a mark */
static int cvt_spans(void *dst, size_t dbytes, const void *src, size_t sbytes, const char *who) {
  ++g_launches, ++g_path[P_CVT];
  must_own(src, 0, sbytes - 1, 1, who);
  must_own(dst, 0, dbytes - 1, 1, who);
  if (!g_failures) memset(dst, 0x5A, dbytes);
  return 0;
}
int __wrap_skl_hip_launch_cvt_f32_f8(int fmt, int sat, uint8_t *dst, const float *src, float scale, size_t n) {
  (void)fmt, (void)sat, (void)scale;
  return cvt_spans(dst, n, src, 4 * n, "cvt f32 -> fp8");
}
int __wrap_skl_hip_launch_cvt_bf16_f8(int fmt, int sat, uint8_t *dst, const uint16_t *src, float scale, size_t n) {
  (void)fmt, (void)sat, (void)scale;
  return cvt_spans(dst, n, src, 2 * n, "cvt bf16 -> fp8");
}
int __wrap_skl_hip_launch_cvt_f8_bf16(int fmt, uint16_t *dst, const uint8_t *src, size_t n) {
  const int rc = cvt_spans(dst, 2 * n, src, n, "cvt fp8 -> bf16");
  if (!g_failures) /* the GEMM over scaled 4-bit weights multiplies what this writes (finite codes: exact) */
    for (size_t i = 0; i < n; ++i) {
      const float v = (float)f8_value(src[i], fmt == SKL_DT_F8E4M3 ? 4 : 5);
      uint32_t bits;
      memcpy(&bits, &v, 4);
      dst[i] = (uint16_t)(bits >> 16);
    }
  return rc;
}
/* E2M1 code -> the E4M3 byte of the same value (ref/cvt/cvt_ofp4.c:59-68 is exact) */
static const uint8_t kE2M1AsE4M3[16] = {0x00, 0x30, 0x38, 0x3C, 0x40, 0x44, 0x48, 0x4C, 0x80, 0xB0, 0xB8, 0xBC, 0xC0, 0xC4, 0xC8, 0xCC};
static unsigned nibble_of(const uint8_t *b, size_t i) { return (i & 1) ? (unsigned)(b[i / 2] >> 4) : (unsigned)(b[i / 2] & 0xF); }
int __wrap_skl_hip_launch_cvt_f4_f8e4m3(uint8_t *dst, const uint8_t *src, size_t n) {
  const int rc = cvt_spans(dst, n, src, (n + 1) / 2, "cvt fp4 -> fp8");
  if (!g_failures) /* the GEMM over 4-bit weights multiplies what this writes */
    for (size_t i = 0; i < n; ++i) dst[i] = kE2M1AsE4M3[nibble_of(src, i)];
  return rc;
}
static double scale_of(const uint8_t *scales, size_t lds, size_t j, size_t p) { return scales ? ldexp(1.0, (int)scales[j * lds + p / 32] - 127) : 1.0; }
int __wrap_skl_hip_launch_cvt_mxf4_bf16(uint16_t *dst, const uint8_t *src, const uint8_t *scales, size_t lds, size_t n, size_t k, size_t ldb) {
  const char *who = "cvt scaled fp4 -> bf16";
  ++g_launches, ++g_path[P_CVT];
  must_own(dst, 0, (n - 1) * ldb + k - 1, 2, who);
  must_own(src, 0, ((n - 1) * ldb + k - 1) / 2, 1, who);
  must_own(scales, 0, (n - 1) * lds + (k - 1) / 32, 1, who);
  if (g_failures) return 0;
  for (size_t j = 0; j < n; ++j)
    for (size_t p = 0; p < k; ++p) { /* exact in float, and a float with at most two significant bits is a bf16 */
      const float v = (float)(f8_value(kE2M1AsE4M3[nibble_of(src, j * ldb + p)], 4) * scale_of(scales, lds, j, p));
      uint32_t bits;
      memcpy(&bits, &v, 4);
      dst[j * ldb + p] = (uint16_t)(bits >> 16);
    }
  return 0;
}
int __wrap_skl_hip_launch_gemv_f4(size_t m, size_t n, size_t k, skl_scalar alpha, const void *a, size_t rsa, size_t csa, const void *b,
                                  size_t ldb, const uint8_t *scales, size_t lds, skl_scalar beta, float *c, size_t rsc, size_t csc) {
  const char *who = "4-bit-weight decode kernel";
  EXPECT(skl_hip_gemv_f4_supported(m, n, k, a, rsa, csa, b, ldb), "4-bit-weight decode kernel handed a problem it does not support");
  ++g_launches, ++g_path[P_F4];
  must_own(a, 0, (m - 1) * rsa + (k - 1) * csa, 1, who);
  must_own(b, 0, ((n - 1) * ldb + k - 1) / 2, 1, who);
  must_own(c, 0, (m - 1) * rsc + (n - 1) * csc, sizeof(float), who);
  if (scales) must_own(scales, 0, (n - 1) * lds + (k - 1) / 32, 1, who);
  if (g_failures) return 0;
  for (size_t i = 0; i < m; ++i)
    for (size_t j = 0; j < n; ++j) {
      double acc = 0;
      for (size_t p = 0; p < k; ++p)
        acc += f8_value(((const uint8_t *)a)[i * rsa + p * csa], 4) * f8_value(kE2M1AsE4M3[nibble_of((const uint8_t *)b, j * ldb + p)], 4) *
               scale_of(scales, lds, j, p);
      c[i * rsc + j * csc] = (float)((double)beta.f * c[i * rsc + j * csc] + (double)alpha.f * acc);
    }
  return 0;
}
static void *g_converted_scratch;
void *__wrap_skl_hip_converted_scratch(size_t bytes) {
  if (g_scarce) return NULL;
  if (g_converted_scratch) {
    range_remove(g_converted_scratch);
    free(g_converted_scratch);
  }
  g_converted_scratch = malloc(bytes ? bytes : 1);
  range_add(g_converted_scratch, bytes ? bytes : 1, 1);
  memset(g_converted_scratch, 0xEE, bytes);
  return g_converted_scratch;
}

/* "device" memory is host memory the registry knows as device memory */
void *__wrap_skl_hip_malloc(size_t bytes) {
  void *p = malloc(bytes ? bytes : 1);
  range_add(p, bytes ? bytes : 1, 1);
  return p;
}
static long g_synchronized;
int __wrap_skl_hip_synchronize(void) {
  ++g_synchronized;
  return 0;
}
void __wrap_skl_hip_free(void *p) {
  if (!p) return;
  range_remove(p);
  free(p);
}
static int copy_checked(void *dst, const void *src, size_t bytes, const char *who) {
  if (bytes == 0) return 0;
  must_own(src, 0, bytes - 1, 1, who);
  must_own(dst, 0, bytes - 1, 1, who);
  if (!g_failures) memcpy(dst, src, bytes);
  return 0;
}
int __wrap_skl_hip_memcpy_h2d(void *dst, const void *src, size_t bytes) { return copy_checked(dst, src, bytes, "host to device copy"); }
int __wrap_skl_hip_memcpy_d2h(void *dst, const void *src, size_t bytes) { return copy_checked(dst, src, bytes, "device to host copy"); }
int __wrap_skl_hip_pointer_is_device(const void *p) {
  const range_t *r = range_of(p);
  return r ? r->device : 0;
}
static void *g_operand_scratch;
static size_t g_operand_scratch_bytes;
void *__wrap_skl_hip_operand_scratch(size_t bytes) {
  if (g_scarce) return NULL; /* not an error: the caller goes on to a kernel that needs no copy */
  if (bytes > g_operand_scratch_bytes) { /* like the library's block: grows, the address may change */
    if (g_operand_scratch) {
      range_remove(g_operand_scratch);
      free(g_operand_scratch);
    }
    g_operand_scratch = malloc(bytes);
    g_operand_scratch_bytes = bytes;
    range_add(g_operand_scratch, bytes, 1);
  }
  memset(g_operand_scratch, 0xEE, g_operand_scratch_bytes); /* stale contents must not matter */
  return g_operand_scratch;
}
void __wrap_skl_hip_sequence_begin(void) {}
void __wrap_skl_hip_sequence_end(void) {}

/* ------------------------------------------------------------------ random cases */
static uint64_t g_rng = 0x9E3779B97F4A7C15ull;
static uint32_t rnd(void) {
  g_rng ^= g_rng << 13;
  g_rng ^= g_rng >> 7;
  g_rng ^= g_rng << 17;
  return (uint32_t)(g_rng >> 32);
}
static size_t rnd_in(size_t lo, size_t hi) { return lo + rnd() % (hi - lo + 1); }
static int small(void) { return (int)(rnd() % 5) - 2; }

/* Strides of a 4-level index (extents e[0..3]) nested in a random order, each level padded at random: no two
 * index tuples share an address. Returns the number of elements spanned. */
static size_t random_layout(const size_t e[4], size_t stride[4], size_t align) {
  int order[4] = {0, 1, 2, 3};
  for (int i = 3; i > 0; --i) {
    const int j = (int)(rnd() % (unsigned)(i + 1)), t = order[i];
    order[i] = order[j], order[j] = t;
  }
  size_t run = 1;
  for (int q = 0; q < 4; ++q) {
    const int lvl = order[q];
    stride[lvl] = run;
    run *= e[lvl];
    if (q == 0 || rnd() % 3 == 0) run = (run + (rnd() % 2 ? rnd_in(0, 9) : 0) + align - 1) / align * align;
  }
  size_t span = 1;
  for (int l = 0; l < 4; ++l) span += (e[l] - 1) * stride[l];
  return span;
}

typedef struct {
  void *ptr;
  size_t bytes;
} buf_t;
static buf_t new_buf(size_t bytes, int device) {
  buf_t b = {malloc(bytes ? bytes : 1), bytes ? bytes : 1};
  range_add(b.ptr, b.bytes, device);
  return b;
}
static void drop_buf(buf_t b) {
  range_remove(b.ptr);
  free(b.ptr);
}

static const int kKinds[][2] = {{SKL_DT_I8, SKL_DT_I8},         {SKL_DT_BF16, SKL_DT_BF16},     {SKL_DT_F16, SKL_DT_F16},
                                {SKL_DT_F8E4M3, SKL_DT_F8E4M3}, {SKL_DT_F8E5M2, SKL_DT_F8E5M2}, {SKL_DT_F8E4M3, SKL_DT_F8E5M2},
                                {SKL_DT_F32, SKL_DT_F32},       {SKL_DT_F64, SKL_DT_F64},       {SKL_DT_F16H, SKL_DT_F16H}};

/* One blocked GEMM through the entry point of its kind. */
static void call_blocked(skl_gemm_desc *d, const skl_gfx950_epilogue_t *ep) {
  switch (d->ta) {
    case SKL_DT_I8:
      if (ep) {
        skl_gemm_fused_i8rcprc_i8rcprc_i32rcprc_gfx950(d->m0, d->n0, d->k0, d->m1, d->n1, d->k1, d->alpha.i, d->a, d->rsa0, d->csa0, d->rsa1,
                                                 d->csa1, d->b, d->rsb0, d->csb0, d->rsb1, d->csb1, d->beta.i, d->c, d->rsc0, d->csc0,
                                                 d->rsc1, d->csc1, ep);
        break;
      }
      skl_gemm_i8rcprc_i8rcprc_i32rcprc_gfx950(d->m0, d->n0, d->k0, d->m1, d->n1, d->k1, d->alpha.i, d->a, d->rsa0, d->csa0, d->rsa1,
                                               d->csa1, d->b, d->rsb0, d->csb0, d->rsb1, d->csb1, d->beta.i, d->c, d->rsc0, d->csc0,
                                               d->rsc1, d->csc1);
      break;
    case SKL_DT_BF16:
      if (ep) {
        skl_gemm_fused_bf16rcprc_bf16rcprc_f32rcprc_gfx950(d->m0, d->n0, d->k0, d->m1, d->n1, d->k1, d->alpha.f, d->a, d->rsa0, d->csa0, d->rsa1,
                                                     d->csa1, d->b, d->rsb0, d->csb0, d->rsb1, d->csb1, d->beta.f, d->c, d->rsc0,
                                                     d->csc0, d->rsc1, d->csc1, ep);
        break;
      }
      skl_gemm_bf16rcprc_bf16rcprc_f32rcprc_gfx950(d->m0, d->n0, d->k0, d->m1, d->n1, d->k1, d->alpha.f, d->a, d->rsa0, d->csa0, d->rsa1,
                                                   d->csa1, d->b, d->rsb0, d->csb0, d->rsb1, d->csb1, d->beta.f, d->c, d->rsc0,
                                                   d->csc0, d->rsc1, d->csc1);
      break;
    case SKL_DT_F16:
      if (ep) {
        skl_gemm_fused_f16rcprc_f16rcprc_f32rcprc_gfx950(d->m0, d->n0, d->k0, d->m1, d->n1, d->k1, d->alpha.f, d->a, d->rsa0, d->csa0, d->rsa1,
                                                   d->csa1, d->b, d->rsb0, d->csb0, d->rsb1, d->csb1, d->beta.f, d->c, d->rsc0, d->csc0,
                                                   d->rsc1, d->csc1, ep);
        break;
      }
      skl_gemm_f16rcprc_f16rcprc_f32rcprc_gfx950(d->m0, d->n0, d->k0, d->m1, d->n1, d->k1, d->alpha.f, d->a, d->rsa0, d->csa0, d->rsa1,
                                                 d->csa1, d->b, d->rsb0, d->csb0, d->rsb1, d->csb1, d->beta.f, d->c, d->rsc0, d->csc0,
                                                 d->rsc1, d->csc1);
      break;
    case SKL_DT_F8E4M3:
      if (d->tb == SKL_DT_F8E5M2) { /* the mixed pair has the strided form only */
        skl_gemm_f8e4m3rc_f8e5m2rc_f32rc_gfx950(d->m1, d->n1, d->k1, d->alpha.f, d->a, d->rsa1, d->csa1, d->b, d->rsb1, d->csb1,
                                                d->beta.f, d->c, d->rsc1, d->csc1);
        break;
      }
      if (ep) {
        skl_gemm_fused_f8e4m3rcprc_f8e4m3rcprc_f32rcprc_gfx950(d->m0, d->n0, d->k0, d->m1, d->n1, d->k1, d->alpha.f, d->a, d->rsa0, d->csa0,
                                                         d->rsa1, d->csa1, d->b, d->rsb0, d->csb0, d->rsb1, d->csb1, d->beta.f, d->c,
                                                         d->rsc0, d->csc0, d->rsc1, d->csc1, ep);
        break;
      }
      skl_gemm_f8e4m3rcprc_f8e4m3rcprc_f32rcprc_gfx950(d->m0, d->n0, d->k0, d->m1, d->n1, d->k1, d->alpha.f, d->a, d->rsa0, d->csa0,
                                                       d->rsa1, d->csa1, d->b, d->rsb0, d->csb0, d->rsb1, d->csb1, d->beta.f, d->c,
                                                       d->rsc0, d->csc0, d->rsc1, d->csc1);
      break;
    case SKL_DT_F8E5M2:
      if (ep) {
        skl_gemm_fused_f8e5m2rcprc_f8e5m2rcprc_f32rcprc_gfx950(d->m0, d->n0, d->k0, d->m1, d->n1, d->k1, d->alpha.f, d->a, d->rsa0, d->csa0,
                                                         d->rsa1, d->csa1, d->b, d->rsb0, d->csb0, d->rsb1, d->csb1, d->beta.f, d->c,
                                                         d->rsc0, d->csc0, d->rsc1, d->csc1, ep);
        break;
      }
      skl_gemm_f8e5m2rcprc_f8e5m2rcprc_f32rcprc_gfx950(d->m0, d->n0, d->k0, d->m1, d->n1, d->k1, d->alpha.f, d->a, d->rsa0, d->csa0,
                                                       d->rsa1, d->csa1, d->b, d->rsb0, d->csb0, d->rsb1, d->csb1, d->beta.f, d->c,
                                                       d->rsc0, d->csc0, d->rsc1, d->csc1);
      break;
    case SKL_DT_F32:
      skl_gemm_f32rcprc_f32rcprc_f32rcprc_gfx950(d->m0, d->n0, d->k0, d->m1, d->n1, d->k1, d->alpha.f, d->a, d->rsa0, d->csa0, d->rsa1,
                                                 d->csa1, d->b, d->rsb0, d->csb0, d->rsb1, d->csb1, d->beta.f, d->c, d->rsc0, d->csc0,
                                                 d->rsc1, d->csc1);
      break;
    case SKL_DT_F64:
      skl_gemm_f64rcprc_f64rcprc_f64rcprc_gfx950(d->m0, d->n0, d->k0, d->m1, d->n1, d->k1, d->alpha.d, d->a, d->rsa0, d->csa0, d->rsa1,
                                                 d->csa1, d->b, d->rsb0, d->csb0, d->rsb1, d->csb1, d->beta.d, d->c, d->rsc0, d->csc0,
                                                 d->rsc1, d->csc1);
      break;
    default:
      skl_gemm_f16rcprc_f16rcprc_f16rcprc_gfx950(d->m0, d->n0, d->k0, d->m1, d->n1, d->k1, (_Float16)d->alpha.f, d->a, d->rsa0, d->csa0,
                                                 d->rsa1, d->csa1, d->b, d->rsb0, d->csb0, d->rsb1, d->csb1, (_Float16)d->beta.f, d->c,
                                                 d->rsc0, d->csc0, d->rsc1, d->csc1);
      break;
  }
}

static void set_scalars(skl_gemm_desc *d, int alpha, int beta) {
  memset(&d->alpha, 0, sizeof d->alpha);
  memset(&d->beta, 0, sizeof d->beta);
  if (d->ta == SKL_DT_I8) d->alpha.i = alpha, d->beta.i = beta;
  else if (d->ta == SKL_DT_F64) d->alpha.d = alpha, d->beta.d = beta;
  else d->alpha.f = (float)alpha, d->beta.f = (float)beta;
}

/* shape classes: what the dispatcher distinguishes */
static void random_dims(int cls, size_t *m, size_t *n, size_t *k) {
  switch (cls) {
    case 0: *m = rnd_in(1, 40), *n = rnd_in(1, 40), *k = rnd_in(0, 40); break;                 /* tiny, K = 0 included */
    case 1: *m = 1, *n = 16 * rnd_in(1, 40), *k = rnd_in(1, 700); break;                        /* one row */
    case 2: *m = rnd_in(2, 16), *n = 16 * rnd_in(1, 20), *k = 16 * rnd_in(1, 40); break;        /* a few rows */
    case 3: *m = rnd_in(30, 200), *n = rnd_in(1, 8), *k = 16 * rnd_in(1, 12); break;            /* a few columns */
    case 4: *m = 64 * rnd_in(1, 3), *n = 64 * rnd_in(1, 3), *k = 16 * rnd_in(1, 6); break;      /* aligned, mid */
    default: *m = rnd_in(70, 200), *n = rnd_in(70, 200), *k = rnd_in(17, 60); break;            /* ragged, mid */
  }
}

static int run_gemm_case(int device_pointers) {
  const int kind = (int)(rnd() % 9), ta = kKinds[kind][0], tb = kKinds[kind][1];
  const int form = (int)(rnd() % 4); /* 0: strided, 1: blocked at random, 2: 64-panels, 3: K-packed int8 */
  skl_gemm_desc d;
  size_t m, n, k, sa[4], sb[4], sc[4];
  memset(&d, 0, sizeof d);
  d.ta = ta, d.tb = tb;
  random_dims((int)(rnd() % 6), &m, &n, &k);
  d.m0 = d.n0 = d.k0 = 1, d.m1 = m, d.n1 = n, d.k1 = k;
  if (form == 1 && !(ta == SKL_DT_F8E4M3 && tb == SKL_DT_F8E5M2)) {
    d.m0 = rnd_in(1, 6), d.n0 = rnd_in(1, 6), d.k0 = rnd_in(1, 6);
    if (rnd() % 3 == 0) d.m0 = 4, d.n0 = 4, d.k0 = 8;
    d.m1 = (m + d.m0 - 1) / d.m0, d.n1 = (n + d.n0 - 1) / d.n0, d.k1 = k ? (k + d.k0 - 1) / d.k0 : 0;
  } else if (form == 2 && !(ta == SKL_DT_F8E4M3 && tb == SKL_DT_F8E5M2)) {
    d.m0 = d.n0 = 64, d.m1 = rnd_in(1, 4), d.n1 = rnd_in(1, 4);
  } else if (form == 3 && ta == SKL_DT_I8) {
    d.k0 = 4, d.k1 = k ? (k + 3) / 4 : 1;
  }
  {
    const size_t align = rnd() % 2 ? 16 : 1; /* half of the cases keep the 16-byte rule */
    const size_t ea[4] = {d.m1, d.k1 ? d.k1 : 1, d.m0, d.k0}, eb[4] = {d.k1 ? d.k1 : 1, d.n1, d.k0, d.n0}, ec[4] = {d.m1, d.n1, d.m0, d.n0};
    size_t na = random_layout(ea, sa, align), nb = random_layout(eb, sb, align), nc = random_layout(ec, sc, rnd() % 2 ? 4 : 1);
    if (form == 0 && rnd() % 2) { /* plain row-major operands, as the optimized entry points take them */
      const size_t pad = rnd() % 2 ? 16 : rnd() % 4;
      sa[0] = (k ? k : 1) + pad, sa[1] = 1, na = m * sa[0];
      sb[0] = n + pad, sb[1] = 1, nb = (k ? k : 1) * sb[0];
      sc[0] = n + rnd() % 3, sc[1] = 1, nc = m * sc[0];
    }
    if (form == 3 && ta == SKL_DT_I8) { /* the dot4 entry point's layout: A rows with K contiguous, B(4P + p, j) at P*rsb1 + 4j + p */
      const size_t lda = 4 * d.k1 + 16 * (rnd() % 2), ldb = 4 * n + 16 * (rnd() % 2), ldc = n + rnd() % 3;
      sa[0] = lda, sa[1] = 4, sa[2] = 0, sa[3] = 1, na = m * lda;
      sb[0] = ldb, sb[1] = 4, sb[2] = 1, sb[3] = 0, nb = d.k1 * ldb;
      sc[0] = ldc, sc[1] = 1, sc[2] = 0, sc[3] = 0, nc = m * ldc;
    }
    d.rsa1 = sa[0], d.csa1 = sa[1], d.rsa0 = sa[2], d.csa0 = sa[3];
    d.rsb1 = sb[0], d.csb1 = sb[1], d.rsb0 = sb[2], d.csb0 = sb[3];
    d.rsc1 = sc[0], d.csc1 = sc[1], d.rsc0 = sc[2], d.csc0 = sc[3];
    const size_t esa = esize(ta), esb = esize(tb), esc = c_esize(ta);
    buf_t a = new_buf(na * esa, device_pointers), b = new_buf(nb * esb, device_pointers), c = new_buf(nc * esc, device_pointers);
    buf_t want = new_buf(nc * esc, 0);
    for (size_t i = 0; i < na; ++i) store_small(ta, a.ptr, i, small());
    for (size_t i = 0; i < nb; ++i) store_small(tb, b.ptr, i, small());
    for (size_t i = 0; i < nc; ++i) store_c(ta, c.ptr, i, small());
    memcpy(want.ptr, c.ptr, nc * esc);
    d.a = a.ptr, d.b = b.ptr, d.c = c.ptr;
    set_scalars(&d, small(), rnd() % 3 ? small() : 0);
    /* A third of the calls of the kinds that have them go through the fused entry points with a random descriptor:
     * bias, maximum, activation, a requantised copy in either orientation with one scale or one per column, q_only. */
    const int fusable = ta == tb && (ta == SKL_DT_I8 || ta == SKL_DT_BF16 || ta == SKL_DT_F16 || ta == SKL_DT_F8E4M3 || ta == SKL_DT_F8E5M2);
    const int fused = fusable && rnd() % 3 == 0;
    const size_t M = d.m0 * d.m1, N = d.n0 * d.n1;
    skl_gfx950_epilogue_t ep = SKL_GFX950_EPILOGUE_NONE;
    buf_t bias = {0}, top = {0}, q = {0}, scales = {0}, want_q = {0}, want_top = {0};
    size_t nq = 0;
    if (fused) {
      static const float kScales[4] = {0.25f, 0.5f, 1.0f, 2.0f};
      if (rnd() % 2) {
        bias = new_buf(N * esc, device_pointers);
        for (size_t j = 0; j < N; ++j) store_c(ta, bias.ptr, j, small());
        ep.bias = bias.ptr;
      }
      if (rnd() % 2) {
        top = new_buf(esc, device_pointers), want_top = new_buf(esc, 0);
        store_c(ta, top.ptr, 0, -1000), store_c(ta, want_top.ptr, 0, -1000);
        ep.max = top.ptr;
      }
      ep.activation = (int)(rnd() % 2);
      if (rnd() % 2) {
        const size_t pad = rnd() % 5;
        if (rnd() % 2) ep.rsq = N + pad, ep.csq = 1; else ep.rsq = 1, ep.csq = M + pad;
        nq = (M - 1) * ep.rsq + (N - 1) * ep.csq + 1;
        q = new_buf(nq, device_pointers), want_q = new_buf(nq, 0);
        memset(q.ptr, 0x5A, nq), memset(want_q.ptr, 0x5A, nq);
        ep.q = (int8_t *)q.ptr;
        ep.q_scale_per_column = (int)(rnd() % 2);
        scales = new_buf((ep.q_scale_per_column ? N : 1) * sizeof(float), device_pointers);
        for (size_t j = 0; j < (ep.q_scale_per_column ? N : 1); ++j) ((float *)scales.ptr)[j] = kScales[rnd() % 4];
        ep.q_scale = (const float *)scales.ptr;
        ep.q_zero = small();
        ep.q_only = rnd() % 3 == 0;
        if (rnd() % 3 == 0) ep.q_format = 1 + (int)(rnd() % 4);
      }
    }
    {
      skl_gemm_desc ref = d;
      ref.c = want.ptr;
      ref.bias = ep.bias;
      ref.max = want_top.ptr;
      ref.rq.act = ep.activation, ref.rq.q_per_column = ep.q_scale_per_column, ref.rq.q_only = ep.q_only && ep.q, ref.rq.q_zero = ep.q_zero;
      ref.rq.q = (int8_t *)want_q.ptr, ref.rq.rsq = ep.rsq, ref.rq.csq = ep.csq, ref.rq.q_scale = ep.q_scale, ref.rq.q_fmt = ep.q_format;
      { /* the reference loops read bias and scales where the caller put them: known to the registry either way */
        gemm_over_desc(&ref, 0, "reference loops");
      }
    }
    call_blocked(&d, fused ? &ep : NULL);
    if (skl_hip_last_error() != 0) fail(skl_hip_last_error_string());
    if (memcmp(want.ptr, c.ptr, nc * esc) != 0 || (nq && memcmp(want_q.ptr, q.ptr, nq) != 0) ||
        (top.ptr && memcmp(want_top.ptr, top.ptr, esc) != 0)) {
      fprintf(stderr, "FAIL: GEMM result differs: kind %d/%d form %d blocks %zu %zu %zu x %zu %zu %zu, %s pointers, fused %d (act %d, q %d, q_only %d)\n",
              ta, tb, form, d.m0, d.n0, d.k0, d.m1, d.n1, d.k1, device_pointers ? "device" : "host", fused, ep.activation, ep.q != NULL, ep.q_only);
      ++g_failures;
    }
    drop_buf(a), drop_buf(b), drop_buf(c), drop_buf(want);
    if (bias.ptr) drop_buf(bias);
    if (top.ptr) drop_buf(top), drop_buf(want_top);
    if (q.ptr) drop_buf(q), drop_buf(want_q), drop_buf(scales);
  }
  return g_failures;
}

/* E4M3 A times 4-bit B stored column by column: decode shapes on the kernel that reads the weights as they are,
 * everything else through the converted copy and the fp8 GEMM's dispatch. */
static int run_f4_case(int device_pointers) {
  const size_t m = rnd() % 3 ? rnd_in(1, 16) : rnd_in(17, 40), n = rnd_in(1, 40);
  const size_t k = rnd() % 8 == 0 ? 0 : rnd() % 2 ? 32 * rnd_in(1, 6) : rnd_in(1, 150);
  const size_t ldb = rnd() % 2 ? (k + 31) / 32 * 32 + 32 * (rnd() % 2) : k + rnd() % 5, rsa = rnd() % 2 ? (k + 15) / 16 * 16 + 16 : k + rnd() % 3 + 1;
  const size_t rsc = n + rnd() % 3, nib = k ? (n - 1) * ldb + k : 0;
  const int mx = (int)(rnd() % 2); /* with block scales 2^-2 .. 2^2: sums of small multiples of 1/8 stay exact */
  const size_t lds = (k + 31) / 32 + rnd() % 2;
  buf_t sc = new_buf(n * lds + 1, device_pointers);
  buf_t a = new_buf(m * rsa, device_pointers), b = new_buf((nib + 1) / 2 + 1, device_pointers), c = new_buf(m * rsc * sizeof(float), device_pointers);
  buf_t want = new_buf(m * rsc * sizeof(float), 0);
  const float alpha = (float)small(), beta = rnd() % 3 ? (float)small() : 0.0f;
  for (size_t i = 0; i < m * rsa; ++i) store_small(SKL_DT_F8E4M3, a.ptr, i, small());
  for (size_t i = 0; i < b.bytes; ++i) ((uint8_t *)b.ptr)[i] = (uint8_t)rnd();
  for (size_t i = 0; i < sc.bytes; ++i) ((uint8_t *)sc.ptr)[i] = (uint8_t)(125 + rnd() % 5);
  for (size_t i = 0; i < m * rsc; ++i) ((float *)c.ptr)[i] = (float)small();
  memcpy(want.ptr, c.ptr, m * rsc * sizeof(float));
  for (size_t i = 0; i < m; ++i)
    for (size_t j = 0; j < n; ++j) {
      double acc = 0;
      for (size_t p = 0; p < k; ++p)
        acc += f8_value(((const uint8_t *)a.ptr)[i * rsa + p], 4) * f8_value(kE2M1AsE4M3[nibble_of((const uint8_t *)b.ptr, j * ldb + p)], 4) *
               scale_of(mx ? (const uint8_t *)sc.ptr : NULL, lds, j, p);
      ((float *)want.ptr)[i * rsc + j] = (float)((double)beta * ((float *)want.ptr)[i * rsc + j] + (double)alpha * acc);
    }
  if (mx)
    skl_gemm_f8e4m3rc_mxf4e2m1c_f32rc_gfx950(m, n, k, alpha, (const uint8_t *)a.ptr, rsa, 1, (const uint8_t *)b.ptr, ldb, (const uint8_t *)sc.ptr,
                                             lds, beta, (float *)c.ptr, rsc, 1);
  else
    skl_gemm_f8e4m3rc_f4e2m1c_f32rc_gfx950(m, n, k, alpha, (const uint8_t *)a.ptr, rsa, 1, (const uint8_t *)b.ptr, ldb, beta, (float *)c.ptr, rsc, 1);
  if (skl_hip_last_error() != 0) fail(skl_hip_last_error_string());
  if (memcmp(want.ptr, c.ptr, m * rsc * sizeof(float)) != 0) {
    fprintf(stderr, "FAIL: 4-bit-weight GEMM differs: %zu x %zu x %zu, ldb %zu, rsa %zu, scales %d, %s pointers\n", m, n, k, ldb, rsa, mx,
            device_pointers ? "device" : "host");
    ++g_failures;
  }
  drop_buf(a), drop_buf(b), drop_buf(c), drop_buf(want), drop_buf(sc);
  return g_failures;
}

static int run_pack_case(int device_pointers) {
  static const int widths[3] = {1, 2, 4};
  const int es = widths[rnd() % 3], unpack = (int)(rnd() % 2);
  const size_t m = rnd_in(1, 150), n = rnd_in(1, 150), m0 = rnd() % 3 ? rnd_in(1, 9) : 64, n0 = rnd() % 3 ? rnd_in(1, 9) : 64;
  const size_t m1 = (m + m0 - 1) / m0, n1 = (n + n0 - 1) / n0;
  const size_t eb[4] = {m1, n1, m0, n0}, ef[4] = {m, n, 1, 1};
  size_t sb[4], sf[4];
  const size_t nb = random_layout(eb, sb, rnd() % 2 ? (size_t)(16 / es) : 1), nf = random_layout(ef, sf, rnd() % 2 ? (size_t)(16 / es) : 1);
  buf_t flat = new_buf(nf * (size_t)es, device_pointers), blocked = new_buf(nb * (size_t)es, device_pointers);
  buf_t want = new_buf((unpack ? nf : nb) * (size_t)es, 0);
  for (size_t i = 0; i < flat.bytes; ++i) ((uint8_t *)flat.ptr)[i] = (uint8_t)rnd();
  for (size_t i = 0; i < blocked.bytes; ++i) ((uint8_t *)blocked.ptr)[i] = (uint8_t)rnd();
  memcpy(want.ptr, unpack ? flat.ptr : blocked.ptr, want.bytes);
  if (unpack) {
    unpack_loops(es, m0, n0, blocked.ptr, sb[2], sb[3], sb[0], sb[1], m, n, want.ptr, sf[0], sf[1], 0);
    if (es == 1) skl_unpack_e8rcprc_e8rc_gfx950(m0, n0, blocked.ptr, sb[2], sb[3], sb[0], sb[1], m, n, flat.ptr, sf[0], sf[1]);
    if (es == 2) skl_unpack_e16rcprc_e16rc_gfx950(m0, n0, blocked.ptr, sb[2], sb[3], sb[0], sb[1], m, n, flat.ptr, sf[0], sf[1]);
    if (es == 4) skl_unpack_e32rcprc_e32rc_gfx950(m0, n0, blocked.ptr, sb[2], sb[3], sb[0], sb[1], m, n, flat.ptr, sf[0], sf[1]);
  } else {
    const uint32_t pad = rnd();
    pack_loops(es, m, n, flat.ptr, sf[0], sf[1], m0, n0, want.ptr, sb[2], sb[3], sb[0], sb[1], pad, 0);
    if (es == 1) skl_pack_e8rc_e8rcprc_gfx950(m, n, flat.ptr, sf[0], sf[1], m0, n0, blocked.ptr, sb[2], sb[3], sb[0], sb[1], (uint8_t)pad);
    if (es == 2) skl_pack_e16rc_e16rcprc_gfx950(m, n, flat.ptr, sf[0], sf[1], m0, n0, blocked.ptr, sb[2], sb[3], sb[0], sb[1], (uint16_t)pad);
    if (es == 4) skl_pack_e32rc_e32rcprc_gfx950(m, n, flat.ptr, sf[0], sf[1], m0, n0, blocked.ptr, sb[2], sb[3], sb[0], sb[1], pad);
  }
  if (skl_hip_last_error() != 0) fail(skl_hip_last_error_string());
  if (memcmp(want.ptr, unpack ? flat.ptr : blocked.ptr, want.bytes) != 0) {
    fprintf(stderr, "FAIL: %s result differs (%d-byte elements, %zu x %zu in blocks of %zu x %zu, %s pointers)\n", unpack ? "unpack" : "pack",
            es, m, n, m0, n0, device_pointers ? "device" : "host");
    ++g_failures;
  }
  drop_buf(flat), drop_buf(blocked), drop_buf(want);
  return g_failures;
}

static int run_cvt_case(int device_pointers) {
  const size_t n = rnd_in(1, 5000);
  buf_t f32 = new_buf(4 * n, device_pointers), b16 = new_buf(2 * n, device_pointers), f8 = new_buf(n, device_pointers),
        f4 = new_buf((n + 1) / 2, device_pointers);
  memset(f32.ptr, 0, f32.bytes), memset(b16.ptr, 0, b16.bytes), memset(f8.ptr, 0, f8.bytes), memset(f4.ptr, 0, f4.bytes);
  skl_cvt_sat_f32_f8e4m3_gfx950(f8.ptr, f32.ptr, 1.0f, n);
  skl_cvt_bf16_f8e5m2_gfx950(f8.ptr, b16.ptr, 0.5f, n);
  skl_cvt_f8e4m3_bf16_gfx950(b16.ptr, f8.ptr, n);
  skl_cvt_f4e2m1_f8e4m3_gfx950(f8.ptr, f4.ptr, n);
  if (skl_hip_last_error() != 0) fail(skl_hip_last_error_string());
  drop_buf(f32), drop_buf(b16), drop_buf(f8), drop_buf(f4);
  return g_failures;
}

/* Shapes the random classes do not reach: row-major problems of a given kind and size through the strided entry point. */
static void run_rowmajor(int ta, size_t m, size_t n, size_t k, size_t pad_a, size_t pad_b, size_t pad_c, int alpha, int beta, const char *what) {
  skl_gemm_desc d;
  memset(&d, 0, sizeof d);
  d.ta = d.tb = ta, d.m0 = d.n0 = d.k0 = 1, d.m1 = m, d.n1 = n, d.k1 = k;
  d.rsa1 = k + pad_a, d.csa1 = 1, d.rsb1 = n + pad_b, d.csb1 = 1, d.rsc1 = n + pad_c, d.csc1 = 1;
  const size_t esa = esize(ta), esc = c_esize(ta), na = m * d.rsa1, nb = k * d.rsb1, nc = m * d.rsc1;
  buf_t a = new_buf(na * esa, 1), b = new_buf(nb * esa, 1), c = new_buf(nc * esc, 1), want = new_buf(nc * esc, 0);
  for (size_t i = 0; i < na; ++i) store_small(ta, a.ptr, i, small());
  for (size_t i = 0; i < nb; ++i) store_small(ta, b.ptr, i, small());
  for (size_t i = 0; i < nc; ++i) store_c(ta, c.ptr, i, small());
  memcpy(want.ptr, c.ptr, c.bytes);
  d.a = a.ptr, d.b = b.ptr, d.c = want.ptr;
  set_scalars(&d, alpha, beta);
  gemm_over_desc(&d, 0, "reference loops");
  d.c = c.ptr;
  call_blocked(&d, NULL);
  if (skl_hip_last_error() != 0) fail(skl_hip_last_error_string());
  if (memcmp(want.ptr, c.ptr, c.bytes) != 0) fail(what);
  drop_buf(a), drop_buf(b), drop_buf(c), drop_buf(want);
}

/* A fused int8 call of a decode shape: bias, ReLU, the requantised copy (written next to C or alone) and the maximum. */
static void run_rowmajor_fused(size_t m, size_t n, size_t k, int alpha, int beta, int q_only, const char *what) {
  static const float kScales[4] = {0.25f, 0.5f, 1.0f, 2.0f};
  skl_gemm_desc d, ref;
  skl_gfx950_epilogue_t ep = SKL_GFX950_EPILOGUE_NONE;
  memset(&d, 0, sizeof d);
  d.ta = d.tb = SKL_DT_I8, d.m0 = d.n0 = d.k0 = 1, d.m1 = m, d.n1 = n, d.k1 = k;
  d.rsa1 = k, d.csa1 = 1, d.rsb1 = n, d.csb1 = 1, d.rsc1 = n + 4, d.csc1 = 1;
  const size_t nc = m * d.rsc1, nq = m * (n + 8);
  buf_t a = new_buf(m * k, 1), b = new_buf(k * n, 1), c = new_buf(nc * 4, 1), want = new_buf(nc * 4, 0);
  buf_t bias = new_buf(n * 4, 1), top = new_buf(4, 1), want_top = new_buf(4, 0), q = new_buf(nq, 1), want_q = new_buf(nq, 0), scales = new_buf(n * 4, 1);
  for (size_t i = 0; i < m * k; ++i) store_small(SKL_DT_I8, a.ptr, i, small());
  for (size_t i = 0; i < k * n; ++i) store_small(SKL_DT_I8, b.ptr, i, small());
  for (size_t i = 0; i < nc; ++i) store_c(SKL_DT_I8, c.ptr, i, small());
  for (size_t j = 0; j < n; ++j) store_c(SKL_DT_I8, bias.ptr, j, small()), ((float *)scales.ptr)[j] = kScales[rnd() % 4];
  store_c(SKL_DT_I8, top.ptr, 0, -1000), store_c(SKL_DT_I8, want_top.ptr, 0, -1000);
  memset(q.ptr, 0x5A, nq), memset(want_q.ptr, 0x5A, nq);
  memcpy(want.ptr, c.ptr, c.bytes);
  ep.bias = bias.ptr, ep.max = top.ptr, ep.activation = SKL_GFX950_ACT_RELU;
  ep.q = (int8_t *)q.ptr, ep.rsq = n + 8, ep.csq = 1, ep.q_scale = (const float *)scales.ptr, ep.q_scale_per_column = 1, ep.q_zero = 3, ep.q_only = q_only;
  d.a = a.ptr, d.b = b.ptr, d.c = c.ptr;
  set_scalars(&d, alpha, beta);
  ref = d;
  ref.c = want.ptr, ref.bias = ep.bias, ref.max = want_top.ptr;
  ref.rq.act = ep.activation, ref.rq.q_per_column = 1, ref.rq.q_only = q_only, ref.rq.q_zero = ep.q_zero;
  ref.rq.q = (int8_t *)want_q.ptr, ref.rq.rsq = ep.rsq, ref.rq.csq = 1, ref.rq.q_scale = ep.q_scale;
  gemm_over_desc(&ref, 0, "reference loops");
  call_blocked(&d, &ep);
  if (skl_hip_last_error() != 0) fail(skl_hip_last_error_string());
  if (memcmp(want.ptr, c.ptr, c.bytes) != 0 || memcmp(want_q.ptr, q.ptr, nq) != 0 || memcmp(want_top.ptr, top.ptr, 4) != 0) fail(what);
  drop_buf(a), drop_buf(b), drop_buf(c), drop_buf(want), drop_buf(bias), drop_buf(top), drop_buf(want_top), drop_buf(q), drop_buf(want_q), drop_buf(scales);
}

/* The same on the K-packed B of the dot-product GEMM. */
static void run_k4_fused(size_t m, size_t n, size_t k1, int alpha, int beta, int q_only, const char *what) {
  static const float kScales[4] = {0.25f, 0.5f, 1.0f, 2.0f};
  skl_gemm_desc d, ref;
  skl_gfx950_epilogue_t ep = SKL_GFX950_EPILOGUE_NONE;
  memset(&d, 0, sizeof d);
  d.ta = d.tb = SKL_DT_I8, d.m0 = d.n0 = 1, d.k0 = 4, d.m1 = m, d.n1 = n, d.k1 = k1;
  d.csa0 = 1, d.rsa1 = 4 * k1 + 16, d.csa1 = 4, d.rsb0 = 1, d.rsb1 = 4 * n, d.csb1 = 4, d.rsc1 = n + 2, d.csc1 = 1;
  const size_t nc = m * d.rsc1, nq = m * (n + 8);
  buf_t a = new_buf(m * d.rsa1, 1), b = new_buf(k1 * d.rsb1, 1), c = new_buf(nc * 4, 1), want = new_buf(nc * 4, 0);
  buf_t bias = new_buf(n * 4, 1), top = new_buf(4, 1), want_top = new_buf(4, 0), q = new_buf(nq, 1), want_q = new_buf(nq, 0), scales = new_buf(n * 4, 1);
  for (size_t i = 0; i < a.bytes; ++i) ((int8_t *)a.ptr)[i] = (int8_t)small();
  for (size_t i = 0; i < b.bytes; ++i) ((int8_t *)b.ptr)[i] = (int8_t)small();
  for (size_t i = 0; i < nc; ++i) ((int32_t *)c.ptr)[i] = small();
  for (size_t j = 0; j < n; ++j) ((int32_t *)bias.ptr)[j] = small(), ((float *)scales.ptr)[j] = kScales[rnd() % 4];
  *(int32_t *)top.ptr = *(int32_t *)want_top.ptr = -1000;
  memset(q.ptr, 0x5A, nq), memset(want_q.ptr, 0x5A, nq);
  memcpy(want.ptr, c.ptr, c.bytes);
  ep.bias = bias.ptr, ep.max = top.ptr, ep.activation = SKL_GFX950_ACT_RELU;
  ep.q = (int8_t *)q.ptr, ep.rsq = n + 8, ep.csq = 1, ep.q_scale = (const float *)scales.ptr, ep.q_scale_per_column = 1, ep.q_zero = -2, ep.q_only = q_only;
  d.a = a.ptr, d.b = b.ptr, d.c = c.ptr;
  set_scalars(&d, alpha, beta);
  ref = d;
  ref.c = want.ptr, ref.bias = ep.bias, ref.max = want_top.ptr;
  ref.rq.act = ep.activation, ref.rq.q_per_column = 1, ref.rq.q_only = q_only, ref.rq.q_zero = ep.q_zero;
  ref.rq.q = (int8_t *)want_q.ptr, ref.rq.rsq = ep.rsq, ref.rq.csq = 1, ref.rq.q_scale = ep.q_scale;
  gemm_over_desc(&ref, 0, "reference loops");
  call_blocked(&d, &ep);
  if (skl_hip_last_error() != 0) fail(skl_hip_last_error_string());
  if (memcmp(want.ptr, c.ptr, c.bytes) != 0 || memcmp(want_q.ptr, q.ptr, nq) != 0 || memcmp(want_top.ptr, top.ptr, 4) != 0) fail(what);
  drop_buf(a), drop_buf(b), drop_buf(c), drop_buf(want), drop_buf(bias), drop_buf(top), drop_buf(want_top), drop_buf(q), drop_buf(want_q), drop_buf(scales);
}

static int run_large_cases(void) {
  run_k4_fused(1, 1024, 264, 1, 0, 1, "fused int8 GEMV on K-packed B differs");
  run_k4_fused(50, 1024, 264, 2, -1, 0, "fused int8 decode batch on K-packed B differs");
  run_rowmajor_fused(1, 4096, 1536, 1, 0, 1, "fused int8 GEMV (product into scratch, then the epilogue pass) differs");
  run_rowmajor_fused(6, 2048, 2048, -1, 2, 0, "fused int8 decode batch (product into scratch, then the epilogue pass) differs");
  run_rowmajor(SKL_DT_I8, 1500, 2100, 120, 1, 5, 3, 2, -1, "large ragged int8 GEMM (tile-padded copies) differs");
  run_rowmajor(SKL_DT_BF16, 500, 600, 72, 8, 16, 1, 1, 1, "ragged mid-size bf16 GEMM differs");
  run_rowmajor(SKL_DT_I8, 3, 256, 100, 0, 0, 0, 1, 0, "int8 GEMM with three rows (few-rows kernel) differs");
  run_rowmajor(SKL_DT_I8, 6, 2048, 2048, 0, 0, 0, -1, 2, "int8 GEMM with six rows (decode batch) differs");
  run_rowmajor(SKL_DT_BF16, 4, 1024, 1024, 8, 8, 0, 2, 0, "bf16 GEMM with four rows (decode batch) differs");
  run_rowmajor(SKL_DT_F8E4M3, 2, 512, 256, 0, 0, 0, 1, 1, "fp8 GEMM with two rows differs");
  run_rowmajor(SKL_DT_I8, 1, 4096, 1536, 0, 0, 0, 1, 0, "int8 GEMV differs");
  for (size_t m = 17; m <= 50; m += 33) { /* K-packed B with more than 16 rows of A: chunks of 16 */
    const size_t n = 1024, k1 = 264;
    skl_gemm_desc d;
    memset(&d, 0, sizeof d);
    d.ta = d.tb = SKL_DT_I8, d.m0 = d.n0 = 1, d.k0 = 4, d.m1 = m, d.n1 = n, d.k1 = k1;
    d.csa0 = 1, d.rsa1 = 4 * k1 + 16, d.csa1 = 4, d.rsb0 = 1, d.rsb1 = 4 * n, d.csb1 = 4, d.rsc1 = n + 2, d.csc1 = 1;
    buf_t a = new_buf(m * d.rsa1, 1), b = new_buf(k1 * d.rsb1, 1), c = new_buf(4 * m * d.rsc1, 1), want = new_buf(4 * m * d.rsc1, 0);
    for (size_t i = 0; i < a.bytes; ++i) ((int8_t *)a.ptr)[i] = (int8_t)small();
    for (size_t i = 0; i < b.bytes; ++i) ((int8_t *)b.ptr)[i] = (int8_t)small();
    for (size_t i = 0; i < m * d.rsc1; ++i) ((int32_t *)c.ptr)[i] = small();
    memcpy(want.ptr, c.ptr, c.bytes);
    d.a = a.ptr, d.b = b.ptr, d.c = want.ptr;
    set_scalars(&d, -3, 1);
    gemm_over_desc(&d, 0, "reference loops");
    skl_gemm_i8rcp1x4_i8p4x1c_i32_gfx950(m, n, k1, -3, a.ptr, d.rsa1, 4, b.ptr, d.rsb1, 1, c.ptr, d.rsc1);
    if (skl_hip_last_error() != 0) fail(skl_hip_last_error_string());
    if (memcmp(want.ptr, c.ptr, c.bytes) != 0) fail("K-packed int8 GEMM with more than 16 rows differs");
    drop_buf(a), drop_buf(b), drop_buf(c), drop_buf(want);
  }
  return g_failures;
}

int main(int argc, char **argv) {
  const int cases = argc > 1 ? atoi(argv[1]) : 900;
  if (argc > 2) g_rng ^= strtoull(argv[2], NULL, 0);
  for (int t = 0; t < cases && !g_failures; ++t) {
    const int device_pointers = (int)(rnd() % 2);
    switch (rnd() % 8) {
      case 0: run_pack_case(device_pointers); break;
      case 1: run_cvt_case(device_pointers); break;
      case 2: run_f4_case(device_pointers); break;
      default: run_gemm_case(device_pointers); break;
    }
  }
  g_scarce = 1; /* every scratch block refused: each call must still complete, on a kernel that needs none or a buffer of its own */
  for (int t = 0; t < cases / 4 && !g_failures; ++t) run_gemm_case((int)(rnd() % 2));
  {
    const long launches = g_launches, synchronized = g_synchronized;
    for (int t = 0; t < cases / 8 && !g_failures; ++t) run_f4_case((int)(rnd() % 2));
    if (!g_failures && cases >= 64 && (g_launches == launches || g_synchronized == synchronized))
      fail("4-bit-weight GEMMs without a scratch block: no call went through a buffer of its own");
  }
  g_scarce = 0;
  if (!g_failures && argc <= 2) run_large_cases();  /* with a seed: random cases only */
  if (g_nranges != (g_operand_scratch ? 1 : 0) + (g_converted_scratch ? 1 : 0) + (g_zeroed_sums ? 1 : 0)) fail("a buffer of the host layer was not released");
  printf("%s: %d cases, %ld launches carried out, %ld address ranges checked\n", g_failures ? "host layer check FAILED" : "host layer ok",
         cases, g_launches, g_checked);
  for (int q = 0; q < P_COUNT; ++q) printf("  %-24s %ld\n", kPathNames[q], g_path[q]);
  return g_failures ? 1 : 0;
}
