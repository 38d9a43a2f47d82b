/*
 * skl_api.c - the C host layer of the gfx950 SKL library: the public entry
 * points of include/skl-gfx950.h. Like the reference's public functions
 * (src/gemm/README.md:84,113-131 - dispatchers over private kernels), each one
 * only normalises its arguments into a descriptor, stages host buffers when
 * the caller passed ordinary host memory, and picks the kernel family:
 *
 *   M == 1                          -> HBM-streaming GEMV kernels
 *   16-byte aligned canonical form  -> matrix-core (MFMA) kernels
 *   anything else                   -> any-stride kernel
 *
 * No HIP header is included here; the GPU is reached only through the C-ABI of
 * skl_launch.h and skl-hip.h.
 */
#include <stddef.h>
#include <stdint.h>
#include <string.h>

#include "../../include/skl-gfx950.h"
#include "skl_launch.h"

#define SKL_TE 64u

/* ------------------------------------------------------------------------ */
/* helpers                                                                   */
/* ------------------------------------------------------------------------ */

static size_t elem_size(int dt) {
  switch (dt) {
    case SKL_DT_BF16:
    case SKL_DT_F16:
    case SKL_DT_F16H: return 2u;
    case SKL_DT_F32: return 4u;
    case SKL_DT_F64: return 8u;
    default: return 1u;
  }
}
static size_t c_elem_size(int dt) { return dt == SKL_DT_F64 ? 8u : dt == SKL_DT_F16H ? 2u : 4u; }

/* Number of elements between the first and one past the last addressed element
 * of a 4-level strided array; 0 if any extent is 0. */
static size_t span4(size_t d0, size_t s0, size_t d1, size_t s1, size_t d2, size_t s2, size_t d3,
                    size_t s3) {
  if (d0 == 0 || d1 == 0 || d2 == 0 || d3 == 0) return 0;
  return (d0 - 1) * s0 + (d1 - 1) * s1 + (d2 - 1) * s2 + (d3 - 1) * s3 + 1;
}

/* Classifies up to three pointers (NULL entries are skipped).
 * Returns 1 all device, 0 all host, -1 mixed (error recorded). */
static int classify(const void *p0, const void *p1, const void *p2, const char *who) {
  const void *p[3];
  int n = 0, dev = 0;
  if (p0) p[n++] = p0;
  if (p1) p[n++] = p1;
  if (p2) p[n++] = p2;
  if (skl_hip_get_pointer_mode() == SKL_HIP_POINTERS_DEVICE) return 1;
  for (int i = 0; i < n; ++i) dev += skl_hip_pointer_is_device(p[i]) ? 1 : 0;
  if (dev == n) return 1;
  if (dev == 0) return 0;
  skl_hip_record_error(SKL_HIP_ERR_MIXED_POINTERS, who);
  return -1;
}

/* Device copy of a host span (NULL on failure or empty span). */
static void *stage_in(const void *host, size_t bytes) {
  void *d;
  if (bytes == 0) return NULL;
  d = skl_hip_malloc(bytes);
  if (d && skl_hip_memcpy_h2d(d, host, bytes) != 0) {
    skl_hip_free(d);
    d = NULL;
  }
  return d;
}

/* ------------------------------------------------------------------------ */
/* GEMM                                                                      */
/* ------------------------------------------------------------------------ */

/* Blocked-by-64 view of one blocked dimension (block size b0, count b1, inner
 * stride s0, block stride s1): index x = X*b0 + x0 lives at X*s1 + x0*s0. */
static int block64(size_t b0, size_t b1, size_t s0, size_t s1, size_t *o0, size_t *o1) {
  if (b0 == SKL_TE) {
    *o0 = s0;
    *o1 = s1;
  } else if (b0 == 1) {
    *o0 = s1;
    *o1 = SKL_TE * s1;
  } else if (b1 == 1 || s1 == b0 * s0) {
    *o0 = s0;
    *o1 = SKL_TE * s0;
  } else {
    return 0;
  }
  return 1;
}

/* Flat view of the K dimension (block size k0, count k1). */
static int flat_k(size_t k0, size_t k1, size_t s0, size_t s1, size_t *sk) {
  if (k0 == 1)
    *sk = s1;
  else if (k1 == 1 || s1 == k0 * s0)
    *sk = s0;
  else
    return 0;
  return 1;
}

static unsigned log2_of_power_of_two(size_t v) { /* 0 if v is not a power of two (or is 1) */
  unsigned s = 0;
  if (v < 2 || (v & (v - 1)) != 0) return 0;
  while (((size_t)1 << s) < v) ++s;
  return s;
}

/* C's part of the canonical form. With `small_blocks`, power-of-two blocks other than 64 (at least 4 rows) are
 * accepted as they are - the matrix-core epilogues index them directly. */
static int canonicalize_c(const skl_gemm_desc *d, skl_gemm_canon *g, int small_blocks) {
  g->c = d->c;
  g->c_row_shift = g->c_col_shift = 6;
  if (!block64(d->m0, d->m1, d->rsc0, d->rsc1, &g->rsc0, &g->rsc1)) {
    const unsigned s = log2_of_power_of_two(d->m0);
    if (!small_blocks || s < 2) return 0;
    g->c_row_shift = s, g->rsc0 = d->rsc0, g->rsc1 = d->rsc1;
  }
  if (!block64(d->n0, d->n1, d->csc0, d->csc1, &g->csc0, &g->csc1)) {
    const unsigned s = log2_of_power_of_two(d->n0);
    if (!small_blocks || s < 1) return 0;
    g->c_col_shift = s, g->csc0 = d->csc0, g->csc1 = d->csc1;
  }
  return 1;
}

static int canonicalize(const skl_gemm_desc *d, skl_gemm_canon *g) {
  g->ta = d->ta;
  g->tb = d->tb;
  g->m = d->m0 * d->m1;
  g->n = d->n0 * d->n1;
  g->k = d->k0 * d->k1;
  g->a = d->a;
  g->b = d->b;
  g->c = d->c;
  g->alpha = d->alpha;
  g->beta = d->beta;
  g->bias = d->bias;
  g->max = d->max;
  g->rq = d->rq;
  if (!flat_k(d->k0, d->k1, d->csa0, d->csa1, &g->a_sk)) return 0;
  if (!flat_k(d->k0, d->k1, d->rsb0, d->rsb1, &g->b_sk)) return 0;
  if (!block64(d->m0, d->m1, d->rsa0, d->rsa1, &g->a_s0, &g->a_s1)) return 0;
  if (!block64(d->n0, d->n1, d->csb0, d->csb1, &g->b_s0, &g->b_s1)) return 0;
  return canonicalize_c(d, g, 0);
}

/* The K4-interleaved int8 layout of the dot4 entry point: one row of A (`rows` == 0), or 2 to 128 rows that are
 * contiguous in K. */
static int canonicalize_k4(const skl_gemm_desc *d, skl_gemm_canon *g, int rows) {
  if (d->ta != SKL_DT_I8 || d->k0 != 4 || d->n0 != 1) return 0;
  if (rows ? (d->m0 != 1 || d->m1 < 2 || d->m1 > 128) : d->m0 * d->m1 != 1) return 0;
  if (d->rsb0 != 1 || d->csb1 != 4 || d->csa0 != 1) return 0;
  if (!(d->k1 == 1 || d->csa1 == 4)) return 0;
  memset(g, 0, sizeof *g);
  g->ta = g->tb = SKL_DT_I8;
  g->m = d->m1;
  g->a_s0 = d->rsa1;
  g->a_s1 = SKL_TE * d->rsa1;
  g->rsc0 = d->rsc1;
  g->rsc1 = SKL_TE * d->rsc1;
  g->n = d->n1;
  g->k = 4 * d->k1;
  g->a = d->a;
  g->a_sk = 1;
  g->b = d->b;
  g->b_sk = d->rsb1; /* stride between groups of four k */
  g->c = d->c;
  g->csc0 = d->csc1;
  g->csc1 = SKL_TE * d->csc1;
  g->c_row_shift = g->c_col_shift = 6;
  g->alpha = d->alpha;
  g->beta = d->beta;
  return 1;
}

/* What became of a problem offered to a kernel: TAKEN (launched), DECLINED (not its kind of problem: the next kernel
 * is tried) or FAILED (an error is recorded, nothing more is tried). A launcher that could not get its scratch
 * memory returns SKL_HIP_ERR_WORKSPACE before it has launched anything: that counts as DECLINED, so the call ends
 * on a kernel that needs no scratch, and the allocation error is withdrawn once one has taken it. */
enum { DECLINED = 0, TAKEN = 1, FAILED = -1 };
static int outcome(int rc) { return rc == 0 ? TAKEN : rc == SKL_HIP_ERR_WORKSPACE ? DECLINED : FAILED; }

/* The streaming kernels in the order they are tried. */
static int gemv_on_device(const skl_gemm_canon *g) {
  int r = DECLINED;
  if (skl_hip_gemv_kc_supported(g) && (r = outcome(skl_hip_launch_gemv_kc(g))) != DECLINED) return r;
  if (skl_hip_gemv_kc_rows_supported(g) && (r = outcome(skl_hip_launch_gemv_kc_rows(g))) != DECLINED) return r;
  if (g->m == 1 && skl_hip_gemv_supported(g, 0) && (r = outcome(skl_hip_launch_gemv(g, 0))) != DECLINED) return r;
  if (skl_hip_gemv_mfma_rows_supported(g, 0) && (r = outcome(skl_hip_launch_gemv_mfma_rows(g, 0))) != DECLINED) return r;
  if (skl_hip_gemv_rows_supported(g) && (r = outcome(skl_hip_launch_gemv_rows(g))) != DECLINED) return r;
  return DECLINED;
}

static int gemv_would_take(const skl_gemm_canon *g) {
  return skl_hip_gemv_kc_supported(g) || skl_hip_gemv_kc_rows_supported(g) || (g->m == 1 && skl_hip_gemv_supported(g, 0)) ||
         skl_hip_gemv_mfma_rows_supported(g, 0) || skl_hip_gemv_rows_supported(g);
}

/* C^T = B^T A^T: a problem with a few columns (matrix times vector, the reference's "small-N" regime,
 * src/gemm/README.md:126) is a problem with a few rows once the roles of A and B are exchanged. Products
 * commute exactly and the order of the sum over k is untouched, so the result is the same. */
static void transposed_view(const skl_gemm_canon *g, skl_gemm_canon *t) {
  *t = *g;
  t->ta = g->tb;
  t->tb = g->ta;
  t->m = g->n;
  t->n = g->m;
  t->a = g->b;
  t->a_s0 = g->b_s0;
  t->a_s1 = g->b_s1;
  t->a_sk = g->b_sk;
  t->b = g->a;
  t->b_s0 = g->a_s0;
  t->b_s1 = g->a_s1;
  t->b_sk = g->a_sk;
  t->rsc0 = g->csc0;
  t->rsc1 = g->csc1;
  t->csc0 = g->rsc0;
  t->csc1 = g->rsc1;
  t->c_row_shift = g->c_col_shift;
  t->c_col_shift = g->c_row_shift;
}

/* Offers `g` to the streaming kernels, as it is and with the roles of A and B exchanged. With `launch` == 0 only
 * asks (TAKEN: one of them would take it). */
static int gemv_paths(const skl_gemm_canon *g, int launch) {
  skl_gemm_canon t;
  int r = launch ? gemv_on_device(g) : gemv_would_take(g);
  if (r != DECLINED) return r;
  if (g->n <= 8 && g->n < g->m) {
    transposed_view(g, &t);
    r = launch ? gemv_on_device(&t) : gemv_would_take(&t);
  }
  return r;
}

/* A fused int8 call of a shape the streaming kernels take (a decode step of 2 to 16 rows; one row, and up to four on
 * a B with K contiguous, have kernels that apply the steps themselves): the plain product goes to a row-major matrix
 * in scratch memory and a second, small kernel computes beta*C + alpha*product and the steps from there - exact for
 * integers, and well below what the tile kernels take for such shapes (16 x 4096 x 11008 with bias, ReLU and int8
 * output: 17 against 28 us). */
static int gemv_then_epilogue(const skl_gemm_canon *g) {
  skl_gemm_canon h = *g;
  void *product;
  int r;
  if (g->ta != SKL_DT_I8 || g->tb != SKL_DT_I8 || g->m > 16 || g->c_row_shift > 6 || g->c_col_shift > 6) return DECLINED;
  h.c = (void *)(uintptr_t)256; /* stands for the scratch matrix while asking who would take it */
  h.rsc0 = g->n, h.rsc1 = SKL_TE * g->n, h.csc0 = 1, h.csc1 = SKL_TE;
  h.c_row_shift = h.c_col_shift = 6;
  h.alpha.i = 1, h.beta.i = 0;
  h.bias = NULL, h.max = NULL;
  memset(&h.rq, 0, sizeof h.rq);
  if (gemv_paths(&h, 0) != TAKEN) return DECLINED;
  /* The decode-batch kernel whose workgroups add into C: given the stream's block of sums - zero between calls - and
   * beta == 1 it needs no kernel in front that clears the product, and the epilogue pass puts the zeros back. (The
   * few-rows kernel keeps its own slots in that block: not for it.) */
  if (g->m > 3 && !skl_hip_gemv_kc_supported(&h) && !skl_hip_gemv_kc_rows_supported(&h) && skl_hip_gemv_mfma_rows_supported(&h, 0)) {
    skl_hip_sequence_begin();
    product = skl_hip_zeroed_sums(g->m * g->n * 4);
    if (product != NULL) {
      h.c = product;
      h.beta.i = 1;
      r = outcome(skl_hip_launch_gemv_mfma_rows(&h, 0));
      if (r == TAKEN) r = outcome(skl_hip_launch_gemm_epilogue_zeroing(g, product)) == TAKEN ? TAKEN : FAILED;
      skl_hip_sequence_end();
      return r;
    }
    skl_hip_sequence_end();
    h.beta.i = 0;
  }
  skl_hip_sequence_begin();
  product = skl_hip_operand_scratch(g->m * g->n * 4);
  r = product != NULL ? TAKEN : DECLINED;
  if (r == TAKEN) {
    h.c = product;
    r = gemv_paths(&h, 1);
  }
  if (r == TAKEN) r = outcome(skl_hip_launch_gemm_epilogue(g, product)) == TAKEN ? TAKEN : FAILED; /* C is untouched until here */
  skl_hip_sequence_end();
  return r;
}

/* The same for the K-packed B of the dot-product GEMM, which only the streaming kernels read in place (1 row, or 2
 * to 128 rows in one pass over B). */
static int k4_then_epilogue(const skl_gemm_desc *d) {
  int rows;
  for (rows = 0; rows < 2; ++rows) {
    skl_gemm_canon g, e;
    void *product;
    int r;
    if (!canonicalize_k4(d, &g, rows)) continue;
    e = g; /* the second pass's view: the caller's C and scalars, and the fused operands */
    e.bias = d->bias, e.max = d->max, e.rq = d->rq;
    g.c = (void *)(uintptr_t)256; /* stands for the scratch matrix while asking */
    g.rsc0 = g.n, g.rsc1 = SKL_TE * g.n, g.csc0 = 1, g.csc1 = SKL_TE;
    g.alpha.i = 1, g.beta.i = 0;
    if (!(rows ? skl_hip_gemv_mfma_rows_supported(&g, 1) : skl_hip_gemv_supported(&g, 1))) continue;
    skl_hip_sequence_begin();
    product = skl_hip_operand_scratch(g.m * g.n * 4);
    r = product != NULL ? TAKEN : DECLINED;
    if (r == TAKEN) {
      g.c = product;
      r = outcome(rows ? skl_hip_launch_gemv_mfma_rows(&g, 1) : skl_hip_launch_gemv(&g, 1));
    }
    if (r == TAKEN) r = outcome(skl_hip_launch_gemm_epilogue(&e, product)) == TAKEN ? TAKEN : FAILED;
    skl_hip_sequence_end();
    return r;
  }
  return DECLINED;
}

/* Streaming kernels, then the matrix-core tile kernels. */
static int gemm_fast_path(const skl_gemm_canon *g, int fused, int launch) {
  int r = DECLINED;
  if (!fused && (r = gemv_paths(g, launch)) != DECLINED) return r;
  /* the kernels for a B with K contiguous and the decode-batch kernel of the floating-point kinds apply the fused
   * steps themselves, so that a call gives the same bits with and without them */
  if (fused && skl_hip_gemv_kc_supported(g) && (r = launch ? outcome(skl_hip_launch_gemv_kc(g)) : TAKEN) != DECLINED) return r;
  if (fused && skl_hip_gemv_kc_rows_supported(g) && (r = launch ? outcome(skl_hip_launch_gemv_kc_rows(g)) : TAKEN) != DECLINED)
    return r;
  if (fused && skl_hip_gemv_mfma_rows_supported(g, 0) &&
      (r = launch ? outcome(skl_hip_launch_gemv_mfma_rows(g, 0)) : TAKEN) != DECLINED)
    return r;
  if (skl_hip_gemm_mfma_supported(g)) return launch ? outcome(skl_hip_launch_gemm_mfma(g)) : TAKEN;
  return DECLINED;
}

/* An operand in a layout that none of the kernels reads - a leading dimension that is not a multiple of 16 bytes,
 * the row-major k x n matrix of a matrix-vector product, no unit stride at all - is copied into scratch memory as
 * rows contiguous in K, 16-byte aligned, and the problem runs on the copy: B alone, A alone, or both, whichever
 * the kernels accept first. Worth a copy only when the product is not tiny. */
static int gemm_with_realigned_operands(const skl_gemm_canon *g, int fused) {
  const size_t esa = elem_size(g->ta), esb = elem_size(g->tb);
  const size_t kpa = (g->k * esa + 15) / 16 * 16 / esa, kpb = (g->k * esb + 15) / 16 * 16 / esb;
  const size_t bytes_a = (g->m * kpa * esa + 255) / 256 * 256, bytes_b = g->n * kpb * esb;
  int which, r;
  if (esa > 2 || esb > 2 || g->m * g->n * g->k < ((size_t)1 << 18)) return DECLINED;
  for (which = 1; which <= 3; ++which) { /* 1: B, 2: A, 3: both */
    skl_gemm_canon h = *g;
    const int copy_a = (which & 2) != 0, copy_b = (which & 1) != 0;
    char *scratch;
    if (copy_a) {
      h.a = (const void *)(uintptr_t)256; /* stands for the aligned copy while asking who would take it */
      h.a_sk = 1, h.a_s0 = kpa, h.a_s1 = SKL_TE * kpa;
    }
    if (copy_b) {
      h.b = (const void *)(uintptr_t)256;
      h.b_sk = 1, h.b_s0 = kpb, h.b_s1 = SKL_TE * kpb;
    }
    if (gemm_fast_path(&h, fused, 0) != TAKEN) continue;
    skl_hip_sequence_begin();
    scratch = skl_hip_operand_scratch((copy_a ? bytes_a : 0) + (copy_b ? bytes_b : 0));
    r = scratch != NULL ? TAKEN : DECLINED; /* no memory for the copies: a kernel that needs none */
    if (r == TAKEN && copy_a) {
      r = outcome(skl_hip_launch_realign((int)esa, g->m, g->k, g->a, SKL_TE, g->a_s0, g->a_s1, 1, 0, g->a_sk, scratch, kpa));
      h.a = scratch;
      scratch += bytes_a;
    }
    if (r == TAKEN && copy_b) {
      r = outcome(skl_hip_launch_realign((int)esb, g->n, g->k, g->b, SKL_TE, g->b_s0, g->b_s1, 1, 0, g->b_sk, scratch, kpb));
      h.b = scratch;
    }
    if (r == TAKEN) r = gemm_fast_path(&h, fused, 1); /* C is untouched so far: DECLINED still lets another kernel run */
    skl_hip_sequence_end();
    return r;
  }
  return DECLINED;
}

/* Ragged or misaligned problems large enough for the streaming kernel: A and B copied into scratch memory padded
 * to whole tiles (the rows beyond M and N are never written and what they hold only reaches elements of C that do
 * not exist; K is zero-filled), C updated in place. */
static int gemm_padded_to_tiles(const skl_gemm_canon *g) {
  size_t mp, np, kp;
  const int tile_cols = skl_hip_gemm_mfma_padded_plan(g, &mp, &np, &kp);
  const size_t esa = elem_size(g->ta), esb = elem_size(g->tb);
  skl_gemm_canon h = *g;
  char *scratch;
  int r;
  if (!tile_cols) return DECLINED;
  skl_hip_sequence_begin();
  scratch = skl_hip_operand_scratch(mp * kp * esa + np * kp * esb);
  r = scratch != NULL ? TAKEN : DECLINED;
  if (r == TAKEN)
    r = outcome(skl_hip_launch_realign((int)esa, g->m, g->k, g->a, SKL_TE, g->a_s0, g->a_s1, 1, 0, g->a_sk, scratch, kp));
  if (r == TAKEN)
    r = outcome(skl_hip_launch_realign((int)esb, g->n, g->k, g->b, SKL_TE, g->b_s0, g->b_s1, 1, 0, g->b_sk,
                                       scratch + mp * kp * esa, kp));
  if (r == TAKEN) {
    h.a = scratch, h.a_sk = 1, h.a_s0 = kp, h.a_s1 = SKL_TE * kp;
    h.b = scratch + mp * kp * esa, h.b_sk = 1, h.b_s0 = kp, h.b_s1 = SKL_TE * kp;
    h.k = kp;
    r = outcome(skl_hip_launch_gemm_mfma_padded(&h, tile_cols));
  }
  skl_hip_sequence_end();
  return r;
}

/* A floating-point call that writes only the 8-bit copy, with beta == 0: C is neither written nor read (gemm_run
 * marks beta so; the kernels then take +0 for the old C where the product is an exact zero). */
static int c_untouched(const skl_gemm_desc *d) {
  return d->ta != SKL_DT_I8 && d->ta != SKL_DT_F64 && d->beta.fz.skip_c_read == SKL_C_UNTOUCHED;
}

/* Any other blocking (the 4x8 / 8x4 / 4x4 blocks of src/gemm/packed-gemm.md:270-298, blocks of 32, ...): A and B
 * are copied into rows contiguous in K; C is updated where it lies when the kernels can index its blocks (below),
 * else unpacked into a row-major scratch matrix - also for beta == 0 when C is floating point, since such a call
 * still reads C where the product is an exact zero - multiplied there, and packed back. M and N are
 * whole numbers of blocks, so packing writes exactly the elements the reference writes. */
static int gemm_through_copies(const skl_gemm_desc *d, int fused) {
  const size_t M = d->m0 * d->m1, N = d->n0 * d->n1, K = d->k0 * d->k1;
  const size_t esa = elem_size(d->ta), esb = elem_size(d->tb);
  const size_t kpa = (K * esa + 15) / 16 * 16 / esa, kpb = (K * esb + 15) / 16 * 16 / esb;
  const size_t bytes_a = (M * kpa * esa + 255) / 256 * 256, bytes_b = (N * kpb * esb + 255) / 256 * 256;
  /* an integer C with beta == 0 is not read at all; a floating-point one is, where the product is an exact zero */
  const int c_is_read = !(d->ta == SKL_DT_I8 && d->beta.i == 0) && !c_untouched(d);
  skl_gemm_canon h;
  char *scratch;
  size_t flat;
  int r, c_in_place;
  if (esa > 2 || esb > 2 || M * N * K < ((size_t)1 << 18)) return DECLINED;
  memset(&h, 0, sizeof h);
  h.ta = d->ta, h.tb = d->tb;
  h.m = M, h.n = N, h.k = K;
  h.a = h.b = (const void *)(uintptr_t)256;
  h.c = (void *)(uintptr_t)256;
  h.a_sk = 1, h.a_s0 = kpa, h.a_s1 = SKL_TE * kpa;
  h.b_sk = 1, h.b_s0 = kpb, h.b_s1 = SKL_TE * kpb;
  h.rsc0 = N, h.rsc1 = SKL_TE * N, h.csc0 = 1, h.csc1 = SKL_TE;
  h.c_row_shift = h.c_col_shift = 6;
  h.alpha = d->alpha, h.beta = d->beta;
  h.bias = d->bias, h.max = d->max;
  h.rq = d->rq;
  /* C in power-of-two blocks (the 4 x 4 blocks of that format) can be updated where it is by the matrix-core
   * kernels. Small blocks make the bounds-checked kernels' stores short (16 bytes per 4 x 4 block row), so that pays
   * when C would otherwise travel three times (unpack, update, pack), not when an integer C with beta == 0 is only
   * packed - unless the streaming kernel takes the problem and writes such blocks 16 bytes per lane (8192^3: no
   * pack pass of 81 us). */
  c_in_place = canonicalize_c(d, &h, 0); /* flat or in blocks of 64: the kernels' usual C */
  if (!c_in_place && canonicalize_c(d, &h, 1)) {
    c_in_place = 1;
    if (!c_is_read) {
      h.a = h.b = (const void *)(uintptr_t)256;
      c_in_place = skl_hip_gemm_mfma_streams_c_quads(&h);
    }
  }
  if (!c_in_place) {
    h.c = (void *)(uintptr_t)256;
    h.rsc0 = N, h.rsc1 = SKL_TE * N, h.csc0 = 1, h.csc1 = SKL_TE;
    h.c_row_shift = h.c_col_shift = 6;
  }
  if (gemm_fast_path(&h, fused, 0) != TAKEN) return DECLINED;
  skl_hip_sequence_begin();
  scratch = skl_hip_operand_scratch(bytes_a + bytes_b + (c_in_place ? 0 : M * N * 4));
  r = scratch != NULL ? TAKEN : DECLINED;
  if (r == TAKEN) {
    h.a = scratch, h.b = scratch + bytes_a;
    if (!c_in_place) h.c = scratch + bytes_a + bytes_b;
    /* an operand whose K is flat in memory although the call describes it in blocks (the rows of the dot-product
     * GEMM's A: groups of four k side by side) is copied as what it is */
    if (flat_k(d->k0, d->k1, d->csa0, d->csa1, &flat))
      r = outcome(skl_hip_launch_realign((int)esa, M, K, d->a, d->m0, d->rsa0, d->rsa1, 1, 0, flat, scratch, kpa));
    else
      r = outcome(skl_hip_launch_realign((int)esa, M, K, d->a, d->m0, d->rsa0, d->rsa1, d->k0, d->csa0, d->csa1, scratch, kpa));
  }
  if (r == TAKEN) {
    if (flat_k(d->k0, d->k1, d->rsb0, d->rsb1, &flat))
      r = outcome(skl_hip_launch_realign((int)esb, N, K, d->b, d->n0, d->csb0, d->csb1, 1, 0, flat, scratch + bytes_a, kpb));
    else
      r = outcome(skl_hip_launch_realign((int)esb, N, K, d->b, d->n0, d->csb0, d->csb1, d->k0, d->rsb0, d->rsb1,
                                         scratch + bytes_a, kpb));
  }
  if (r == TAKEN && !c_in_place && c_is_read)
    r = outcome(skl_hip_launch_unpack(4, d->m0, d->n0, d->c, d->rsc0, d->csc0, d->rsc1, d->csc1, M, N, h.c, N, 1));
  if (r == TAKEN) r = gemm_fast_path(&h, fused, 1); /* the caller's C is untouched until this has launched */
  if (r == TAKEN && !c_in_place && !d->rq.q_only) /* with q_only the result went to the requantised copy alone */
    r = outcome(skl_hip_launch_pack(4, M, N, h.c, N, 1, d->m0, d->n0, d->c, d->rsc0, d->csc0, d->rsc1, d->csc1, 0)) == TAKEN ? TAKEN : FAILED;
  skl_hip_sequence_end();
  return r;
}

/* K-packed B with more rows of A than one call of the decode-batch kernel takes (128): chunks of 128 rows, one pass
 * over B each. Up to 256 rows that is cheaper than copying B into a layout the tile kernels read (a transpose of
 * 32-bit groups, about one pass over B each way). Every chunk is checked before the first is launched. */
static int k4_in_row_chunks(const skl_gemm_desc *d) {
  skl_gemm_canon g;
  int launch;
  if (d->ta != SKL_DT_I8 || d->k0 != 4 || d->m0 != 1 || d->m1 <= 128 || d->m1 > 256) return DECLINED;
  for (launch = 0; launch < 2; ++launch) {
    size_t i;
    /* A chunk that fails after others have run would leave C half updated: the one thing a chunk may lack, the
     * scratch of the single-row kernel, is reserved before the first is launched. */
    if (launch && d->m1 % 128 == 1 && skl_hip_gemv_reserve_scratch() != 0) return DECLINED;
    for (i = 0; i < d->m1; i += 128) {
      skl_gemm_desc part = *d;
      int rc = 0;
      part.m1 = d->m1 - i < 128 ? d->m1 - i : 128;
      part.a = (const char *)d->a + i * d->rsa1;
      part.c = (char *)d->c + 4 * i * d->rsc1;
      if (part.m1 == 1) {
        if (!canonicalize_k4(&part, &g, 0) || !skl_hip_gemv_supported(&g, 1)) return DECLINED;
        if (launch) rc = skl_hip_launch_gemv(&g, 1);
      } else {
        if (!canonicalize_k4(&part, &g, 1) || !skl_hip_gemv_mfma_rows_supported(&g, 1)) return DECLINED;
        if (launch) rc = skl_hip_launch_gemv_mfma_rows(&g, 1);
      }
      /* A first chunk that could not get scratch memory has launched nothing: the call goes on to the next kernel.
       * Any other error, or a later chunk's: recorded, C is not to be relied on. */
      if (rc != 0) return i == 0 ? outcome(rc) : FAILED;
    }
  }
  return TAKEN;
}

/* 0, or nonzero when no kernel could be launched (the error is recorded). */
static int gemm_on_device(const skl_gemm_desc *d) {
  skl_gemm_canon g;
  const int fused = d->bias != NULL || d->max != NULL || d->rq.act != 0 || d->rq.q != NULL;
  const int pending = skl_hip_pending_error(); /* what an earlier call left unread is not this call's to withdraw */
  int r = DECLINED;
  if (d->k0 * d->k1 != 0 && d->ta <= SKL_DT_F8E5M2) {
    if (canonicalize_k4(d, &g, 0) && skl_hip_gemv_supported(&g, 1)) { /* one row: the kernel applies fused steps itself */
      g.bias = d->bias, g.max = d->max, g.rq = d->rq;
      r = outcome(skl_hip_launch_gemv(&g, 1));
    }
    if (r == DECLINED && !fused && canonicalize_k4(d, &g, 1) && skl_hip_gemv_mfma_rows_supported(&g, 1))
      r = outcome(skl_hip_launch_gemv_mfma_rows(&g, 1));
    if (r == DECLINED && !fused) r = k4_in_row_chunks(d);
    if (r == DECLINED && fused) r = k4_then_epilogue(d);
    if (r == DECLINED) {
      if (canonicalize(d, &g)) {
        if (!fused) r = gemv_paths(&g, 1);
        /* these apply the fused steps themselves: B with K contiguous (1 to 4 rows, 5 to 96 rows), B row-major (1 row) */
        if (fused && skl_hip_gemv_kc_supported(&g)) r = outcome(skl_hip_launch_gemv_kc(&g));
        if (fused && r == DECLINED && skl_hip_gemv_kc_rows_supported(&g)) r = outcome(skl_hip_launch_gemv_kc_rows(&g));
        if (fused && r == DECLINED && g.m == 1 && skl_hip_gemv_supported(&g, 0)) r = outcome(skl_hip_launch_gemv(&g, 0));
        if (fused && r == DECLINED) r = gemv_then_epilogue(&g); /* uses the operand scratch itself: only here, on the caller's own operands */
        if (r == DECLINED) r = gemm_padded_to_tiles(&g);
        if (r == DECLINED) r = gemm_fast_path(&g, fused, 1);
        if (r == DECLINED) r = gemm_with_realigned_operands(&g, fused);
      } else {
        r = gemm_through_copies(d, fused);
      }
    }
  }
  if (r == DECLINED && d->k0 * d->k1 != 0 && !fused && canonicalize(d, &g) && skl_hip_gemm_tiled_supported(&g) &&
      g.m * g.n * g.k >= ((size_t)1 << 15))
    r = outcome(skl_hip_launch_gemm_tiled(&g));
  if (r == DECLINED) r = outcome(skl_hip_launch_gemm_generic(d)); /* needs no scratch memory */
  /* a kernel further down the list ran in place of one that could not get its scratch memory: the call succeeded */
  if (r == TAKEN && pending != SKL_HIP_ERR_WORKSPACE) skl_hip_withdraw_error(SKL_HIP_ERR_WORKSPACE);
  return r == TAKEN ? 0 : -1;
}

/* The kinds whose alpha and beta travel as a float (F16H: widened). */
static int scalars_are_float(int dt) { return dt != SKL_DT_I8 && dt != SKL_DT_F64; }


static void gemm_run(const skl_gemm_desc *in, const char *who) {
  skl_gemm_desc with_mode = *in;
  const skl_gemm_desc *d = &with_mode;
  const size_t M = d->m0 * d->m1, N = d->n0 * d->n1, K = d->k0 * d->k1;
  int where;
  if (M == 0 || N == 0) return; /* nothing is addressed */
  if (scalars_are_float(d->ta)) { /* beta carries the thread's choice of what beta == 0 means (skl_launch.h) */
    const float beta = in->beta.f;
    memset(&with_mode.beta, 0, sizeof with_mode.beta);
    with_mode.beta.fz.value = beta;
    with_mode.beta.fz.skip_c_read = skl_hip_get_beta_zero_mode() != SKL_HIP_BETA_ZERO_AS_REFERENCE;
    /* a call that writes only the 8-bit copy does not read C either when beta is zero: C need not be a matrix */
    if (with_mode.beta.fz.skip_c_read && beta == 0.0f && in->rq.q && in->rq.q_only) with_mode.beta.fz.skip_c_read = SKL_C_UNTOUCHED;
  }
  where = classify(K ? d->a : NULL, K ? d->b : NULL, d->c, who);
  if (where < 0) return;
  if (d->rq.act < SKL_GFX950_ACT_NONE || d->rq.act > (d->ta == SKL_DT_I8 ? SKL_GFX950_ACT_RELU : SKL_GFX950_ACT_GELU) ||
      (d->rq.q && (!d->rq.q_scale || d->rq.q_zero < -128 || d->rq.q_zero > 127 || d->rq.q_fmt < SKL_GFX950_Q_INT8 ||
                   d->rq.q_fmt > SKL_GFX950_Q_F8E5M2_SAT))) {
    skl_hip_record_error(SKL_HIP_ERR_BAD_ARGUMENT, who);
    return;
  }
  if (d->bias || d->max) { /* the fused operands must be of the same kind as C */
    const int extra = classify(d->bias, d->max, NULL, who);
    if (extra < 0) return;
    if (extra != where) {
      skl_hip_record_error(SKL_HIP_ERR_MIXED_POINTERS, who);
      return;
    }
  }
  if (d->rq.q) {
    const int extra = classify(d->rq.q, d->rq.q_scale, NULL, who);
    if (extra < 0) return;
    if (extra != where) {
      skl_hip_record_error(SKL_HIP_ERR_MIXED_POINTERS, who);
      return;
    }
  }
  if (where == 1) {
    (void)gemm_on_device(d);
    return;
  }
  {
    /* Ordinary host memory: stage the addressed spans. C's whole span travels
     * both ways, so elements in its stride gaps come back unchanged. */
    const size_t esa = elem_size(d->ta), esb = elem_size(d->tb);
    const size_t na = K ? span4(d->m1, d->rsa1, d->k1, d->csa1, d->m0, d->rsa0, d->k0, d->csa0) : 0;
    const size_t nb = K ? span4(d->k1, d->rsb1, d->n1, d->csb1, d->k0, d->rsb0, d->n0, d->csb0) : 0;
    const size_t nc = span4(d->m1, d->rsc1, d->n1, d->csc1, d->m0, d->rsc0, d->n0, d->csc0);
    skl_gemm_desc dd = *d;
    const size_t esc = c_elem_size(d->ta);
    const int untouched = c_untouched(d); /* then the caller's C need not exist: a stand-in that no kernel touches */
    void *da = stage_in(d->a, na * esa), *db = stage_in(d->b, nb * esb), *dc = untouched ? skl_hip_malloc(16) : stage_in(d->c, nc * esc);
    void *dbias = d->bias ? stage_in(d->bias, N * esc) : NULL, *dmax = d->max ? stage_in(d->max, esc) : NULL;
    /* the requantised copy: its whole span travels both ways, like C's */
    const size_t nq = d->rq.q ? (M - 1) * d->rq.rsq + (N - 1) * d->rq.csq + 1 : 0;
    void *dq = d->rq.q ? stage_in(d->rq.q, nq) : NULL;
    void *dqs = d->rq.q ? stage_in(d->rq.q_scale, (d->rq.q_per_column ? N : 1) * sizeof(float)) : NULL;
    if ((na && !da) || (nb && !db) || !dc || (d->bias && !dbias) || (d->max && !dmax) || (d->rq.q && (!dq || !dqs))) {
      skl_hip_free(da);
      skl_hip_free(db);
      skl_hip_free(dc);
      skl_hip_free(dbias);
      skl_hip_free(dmax);
      skl_hip_free(dq);
      skl_hip_free(dqs);
      return;
    }
    dd.a = da;
    dd.b = db;
    dd.c = dc;
    dd.bias = dbias;
    dd.max = dmax;
    dd.rq.q = dq;
    dd.rq.q_scale = dqs;
    if (gemm_on_device(&dd) == 0) { /* after a failure the caller's memory stays as it was */
      if (!untouched) skl_hip_memcpy_d2h(d->c, dc, nc * esc);
      if (dmax) skl_hip_memcpy_d2h(d->max, dmax, esc);
      if (dq) skl_hip_memcpy_d2h(d->rq.q, dq, nq);
    }
    skl_hip_free(dq);
    skl_hip_free(dqs);
    skl_hip_free(da);
    skl_hip_free(db);
    skl_hip_free(dc);
    skl_hip_free(dbias);
    skl_hip_free(dmax);
  }
}

#define SCALAR_i32(x) .i = (x)
#define SCALAR_f32(x) .f = (x)
#define SCALAR_f64(x) .d = (x)

/* strided (rc) form: one element per block */
#define DEFINE_GEMM_RC(NAME, TA_T, TC_T, DTA, DTB, SC)                                             \
  void NAME(size_t m, size_t n, size_t k, TC_T alpha, const TA_T *a, size_t rsa, size_t csa,       \
            const TA_T *b, size_t rsb, size_t csb, TC_T beta, TC_T *c, size_t rsc, size_t csc) {   \
    skl_gemm_desc d = {DTA, DTB, 1,   1,   1,   m,    n,    k,   a,    0, 0, rsa, csa,             \
                       b,   0,   0,   rsb, csb, c,    0,    0,   rsc,  csc, {SC(alpha)}, {SC(beta)}, \
                       NULL, NULL, {0}};                                                           \
    gemm_run(&d, #NAME);                                                                           \
  }

DEFINE_GEMM_RC(skl_gemm_i8rc_i8rc_i32rc_gfx950, int8_t, int32_t, SKL_DT_I8, SKL_DT_I8, SCALAR_i32)
DEFINE_GEMM_RC(skl_gemm_bf16rc_bf16rc_f32rc_gfx950, skl_bf16_t, float, SKL_DT_BF16, SKL_DT_BF16, SCALAR_f32)
DEFINE_GEMM_RC(skl_gemm_f16rc_f16rc_f32rc_gfx950, skl_f16_t, float, SKL_DT_F16, SKL_DT_F16, SCALAR_f32)
DEFINE_GEMM_RC(skl_gemm_f8e4m3rc_f8e4m3rc_f32rc_gfx950, uint8_t, float, SKL_DT_F8E4M3, SKL_DT_F8E4M3, SCALAR_f32)
DEFINE_GEMM_RC(skl_gemm_f8e5m2rc_f8e5m2rc_f32rc_gfx950, uint8_t, float, SKL_DT_F8E5M2, SKL_DT_F8E5M2, SCALAR_f32)
DEFINE_GEMM_RC(skl_gemm_f8e4m3rc_f8e5m2rc_f32rc_gfx950, uint8_t, float, SKL_DT_F8E4M3, SKL_DT_F8E5M2, SCALAR_f32)
DEFINE_GEMM_RC(skl_gemm_f32rc_f32rc_f32rc_gfx950, float, float, SKL_DT_F32, SKL_DT_F32, SCALAR_f32)
DEFINE_GEMM_RC(skl_gemm_f64rc_f64rc_f64rc_gfx950, double, double, SKL_DT_F64, SKL_DT_F64, SCALAR_f64)
/* _Float16 scalars widen exactly */
DEFINE_GEMM_RC(skl_gemm_f16rc_f16rc_f16rc_gfx950, skl_f16_t, skl_f16_t, SKL_DT_F16H, SKL_DT_F16H, SCALAR_f32)

/* blocked (rcprc) form */
#define DEFINE_GEMM_RCPRC(NAME, TA_T, TC_T, DT, SC)                                                \
  void NAME(size_t m0, size_t n0, size_t k0, size_t m1, size_t n1, size_t k1, TC_T alpha,          \
            const TA_T *a, size_t rsa0, size_t csa0, size_t rsa1, size_t csa1, const TA_T *b,      \
            size_t rsb0, size_t csb0, size_t rsb1, size_t csb1, TC_T beta, TC_T *c, size_t rsc0,   \
            size_t csc0, size_t rsc1, size_t csc1) {                                               \
    skl_gemm_desc d = {DT,   DT,   m0,   n0,   k0,   m1,   n1,   k1,   a,    rsa0, csa0, rsa1, csa1, \
                       b,    rsb0, csb0, rsb1, csb1, c,    rsc0, csc0, rsc1, csc1, {SC(alpha)},    \
                       {SC(beta)}, NULL, NULL, {0}};                                               \
    gemm_run(&d, #NAME);                                                                           \
  }

DEFINE_GEMM_RCPRC(skl_gemm_i8rcprc_i8rcprc_i32rcprc_gfx950, int8_t, int32_t, SKL_DT_I8, SCALAR_i32)
DEFINE_GEMM_RCPRC(skl_gemm_bf16rcprc_bf16rcprc_f32rcprc_gfx950, skl_bf16_t, float, SKL_DT_BF16, SCALAR_f32)
DEFINE_GEMM_RCPRC(skl_gemm_f16rcprc_f16rcprc_f32rcprc_gfx950, skl_f16_t, float, SKL_DT_F16, SCALAR_f32)
DEFINE_GEMM_RCPRC(skl_gemm_f8e4m3rcprc_f8e4m3rcprc_f32rcprc_gfx950, uint8_t, float, SKL_DT_F8E4M3, SCALAR_f32)
DEFINE_GEMM_RCPRC(skl_gemm_f8e5m2rcprc_f8e5m2rcprc_f32rcprc_gfx950, uint8_t, float, SKL_DT_F8E5M2, SCALAR_f32)
DEFINE_GEMM_RCPRC(skl_gemm_f32rcprc_f32rcprc_f32rcprc_gfx950, float, float, SKL_DT_F32, SCALAR_f32)
DEFINE_GEMM_RCPRC(skl_gemm_f64rcprc_f64rcprc_f64rcprc_gfx950, double, double, SKL_DT_F64, SCALAR_f64)
DEFINE_GEMM_RCPRC(skl_gemm_f16rcprc_f16rcprc_f16rcprc_gfx950, skl_f16_t, skl_f16_t, SKL_DT_F16H, SCALAR_f32)

static skl_requant requant_of(const skl_gfx950_epilogue_t *ep) {
  skl_requant rq = {ep->activation, ep->q_scale_per_column != 0, ep->q_only != 0 && ep->q != NULL, ep->q_zero, ep->q, ep->rsq, ep->csq, ep->q_scale,
                    ep->q_format};
  return rq;
}

/* The same two forms with the fused steps of `ep` behind the alpha/beta step; ep == NULL is the plain GEMM. */
#define DEFINE_GEMM_FUSED_RC(NAME, TA_T, TC_T, DT, SC)                                             \
  void NAME(size_t m, size_t n, size_t k, TC_T alpha, const TA_T *a, size_t rsa, size_t csa,       \
            const TA_T *b, size_t rsb, size_t csb, TC_T beta, TC_T *c, size_t rsc, size_t csc,     \
            const skl_gfx950_epilogue_t *ep) {                                                     \
    skl_gemm_desc d = {DT,  DT,  1,   1,   1,   m,    n,    k,   a,    0, 0, rsa, csa,             \
                       b,   0,   0,   rsb, csb, c,    0,    0,   rsc,  csc, {SC(alpha)}, {SC(beta)}, \
                       ep ? ep->bias : NULL, ep ? ep->max : NULL, {0}};                            \
    if (ep) d.rq = requant_of(ep);                                                                 \
    gemm_run(&d, #NAME);                                                                           \
  }
#define DEFINE_GEMM_FUSED_RCPRC(NAME, TA_T, TC_T, DT, SC)                                          \
  void NAME(size_t m0, size_t n0, size_t k0, size_t m1, size_t n1, size_t k1, TC_T alpha,          \
            const TA_T *a, size_t rsa0, size_t csa0, size_t rsa1, size_t csa1, const TA_T *b,      \
            size_t rsb0, size_t csb0, size_t rsb1, size_t csb1, TC_T beta, TC_T *c, size_t rsc0,   \
            size_t csc0, size_t rsc1, size_t csc1, const skl_gfx950_epilogue_t *ep) {              \
    skl_gemm_desc d = {DT,   DT,   m0,   n0,   k0,   m1,   n1,   k1,   a,    rsa0, csa0, rsa1, csa1, \
                       b,    rsb0, csb0, rsb1, csb1, c,    rsc0, csc0, rsc1, csc1, {SC(alpha)},    \
                       {SC(beta)}, ep ? ep->bias : NULL, ep ? ep->max : NULL, {0}};                \
    if (ep) d.rq = requant_of(ep);                                                                 \
    gemm_run(&d, #NAME);                                                                           \
  }
DEFINE_GEMM_FUSED_RC(skl_gemm_fused_i8rc_i8rc_i32rc_gfx950, int8_t, int32_t, SKL_DT_I8, SCALAR_i32)
DEFINE_GEMM_FUSED_RC(skl_gemm_fused_bf16rc_bf16rc_f32rc_gfx950, skl_bf16_t, float, SKL_DT_BF16, SCALAR_f32)
DEFINE_GEMM_FUSED_RC(skl_gemm_fused_f16rc_f16rc_f32rc_gfx950, skl_f16_t, float, SKL_DT_F16, SCALAR_f32)
DEFINE_GEMM_FUSED_RC(skl_gemm_fused_f8e4m3rc_f8e4m3rc_f32rc_gfx950, uint8_t, float, SKL_DT_F8E4M3, SCALAR_f32)
DEFINE_GEMM_FUSED_RC(skl_gemm_fused_f8e5m2rc_f8e5m2rc_f32rc_gfx950, uint8_t, float, SKL_DT_F8E5M2, SCALAR_f32)
DEFINE_GEMM_FUSED_RCPRC(skl_gemm_fused_i8rcprc_i8rcprc_i32rcprc_gfx950, int8_t, int32_t, SKL_DT_I8, SCALAR_i32)
DEFINE_GEMM_FUSED_RCPRC(skl_gemm_fused_bf16rcprc_bf16rcprc_f32rcprc_gfx950, skl_bf16_t, float, SKL_DT_BF16, SCALAR_f32)
DEFINE_GEMM_FUSED_RCPRC(skl_gemm_fused_f16rcprc_f16rcprc_f32rcprc_gfx950, skl_f16_t, float, SKL_DT_F16, SCALAR_f32)
DEFINE_GEMM_FUSED_RCPRC(skl_gemm_fused_f8e4m3rcprc_f8e4m3rcprc_f32rcprc_gfx950, uint8_t, float, SKL_DT_F8E4M3, SCALAR_f32)
DEFINE_GEMM_FUSED_RCPRC(skl_gemm_fused_f8e5m2rcprc_f8e5m2rcprc_f32rcprc_gfx950, uint8_t, float, SKL_DT_F8E5M2, SCALAR_f32)

/* row-major A, B, C: the rc form with csa = csb = csc = 1
 * (src/gemm/gemm_i8_i8_i32_zve32x.h:38-48) */
#define DEFINE_GEMM_ROWMAJOR(NAME, RC, TA_T, TC_T)                                                 \
  void NAME(size_t m, size_t n, size_t k, TC_T alpha, const TA_T *a, size_t rsa, const TA_T *b,    \
            size_t rsb, TC_T beta, TC_T *c, size_t rsc) {                                          \
    RC(m, n, k, alpha, a, rsa, 1, b, rsb, 1, beta, c, rsc, 1);                                     \
  }
DEFINE_GEMM_ROWMAJOR(skl_gemm_i8_i8_i32_gfx950, skl_gemm_i8rc_i8rc_i32rc_gfx950, int8_t, int32_t)
DEFINE_GEMM_ROWMAJOR(skl_gemm_bf16_bf16_f32_gfx950, skl_gemm_bf16rc_bf16rc_f32rc_gfx950, skl_bf16_t, float)
DEFINE_GEMM_ROWMAJOR(skl_gemm_f16_f16_f32_gfx950, skl_gemm_f16rc_f16rc_f32rc_gfx950, skl_f16_t, float)
DEFINE_GEMM_ROWMAJOR(skl_gemm_f32_f32_f32_gfx950, skl_gemm_f32rc_f32rc_f32rc_gfx950, float, float)
DEFINE_GEMM_ROWMAJOR(skl_gemm_f64_f64_f64_gfx950, skl_gemm_f64rc_f64rc_f64rc_gfx950, double, double)
DEFINE_GEMM_ROWMAJOR(skl_gemm_f16_f16_f16_gfx950, skl_gemm_f16rc_f16rc_f16rc_gfx950, skl_f16_t, skl_f16_t)

/* The row-major int8 GEMM for callers that cannot allocate: decode shapes only, device pointers only, nothing
 * allocated, queried or freed on the way (see include/skl-gfx950.h). */
void skl_gemm_i8_i8_i32_noalloc_gfx950(size_t m, size_t n, size_t k, int32_t alpha, const int8_t *a, size_t rsa,
                                       const int8_t *b, size_t rsb, int32_t beta, int32_t *c, size_t rsc) {
  skl_gemm_desc d = {SKL_DT_I8, SKL_DT_I8, 1, 1, 1, m, n, k, a, 0, 0, rsa, 1, b, 0, 0, rsb, 1,
                     c, 0, 0, rsc, 1, {.i = alpha}, {.i = beta}, NULL, NULL, {0}};
  skl_gemm_canon g;
  if (m == 0 || n == 0) return;
  if (!canonicalize(&d, &g)) {
    skl_hip_record_error(SKL_HIP_ERR_BAD_ARGUMENT, __func__);
    return;
  }
  skl_hip_launch_gemv_noalloc(&g);
}

/* E4M3 A times OFP4 (E2M1) B, columns of B contiguous in K, two values per byte (see include/skl-gfx950.h). The
 * result is defined as the reference's conversion of B to E4M3 followed by its fp8 GEMM with rsb = 1, csb = ldb.
 * Decode shapes stream the 4-bit weights through the kernel that multiplies them as they are; everything else
 * converts B once into scratch memory of the stream and runs the fp8 GEMM on that. */
static int f4_gemm_on_device(size_t m, size_t n, size_t k, float alpha, const uint8_t *a, size_t rsa, size_t csa,
                             const uint8_t *b, size_t ldb, const uint8_t *scales, size_t lds, skl_scalar beta, float *c, size_t rsc,
                             size_t csc) {
  const skl_scalar alpha_s = {.f = alpha};
  int rc;
  if (k != 0 && skl_hip_gemv_f4_supported(m, n, k, a, rsa, csa, b, ldb))
    return skl_hip_launch_gemv_f4(m, n, k, alpha_s, a, rsa, csa, b, ldb, scales, lds, beta, c, rsc, csc);
  {
    const size_t values = k ? (n - 1) * ldb + k : 0; /* 4-bit values from B's first to its last, gaps included */
    skl_gemm_desc d = {SKL_DT_F8E4M3, SKL_DT_F8E4M3, 1, 1, 1, m, n, k, a, 0, 0, rsa, csa, NULL, 0, 0, 1, ldb,
                       c, 0, 0, rsc, csc, {.f = alpha}, beta, NULL, NULL, {0}};
    /* The converted operands live in the stream's scratch block; a stream without one (the 33rd on its device) or a
     * refused allocation gets a buffer of its own for this call, released once the stream has drained - slower,
     * but the call completes. Only when that fails too is C left unwritten, and then the error says so (a hard
     * error in place of the advisory one the scratch request left). */
    const size_t span_a = (values && scales) ? (m - 1) * rsa + (k - 1) * csa + 1 : 0, bytes_a = (2 * span_a + 255) / 256 * 256;
    const size_t bytes = !values ? 0 : scales ? bytes_a + 2 * values : values;
    const int pending = skl_hip_pending_error();
    char *block = NULL, *own = NULL;
    skl_hip_sequence_begin(); /* the converted operands travel from one launch to the next through the stream's scratch */
    if (bytes) {
      block = (char *)skl_hip_converted_scratch(bytes);
      if (!block) block = own = (char *)skl_hip_malloc(bytes);
    }
    if (bytes && !block) {
      skl_hip_withdraw_error(SKL_HIP_ERR_STREAM_SLOTS);
      skl_hip_record_error(SKL_HIP_ERR_WORKSPACE, "4-bit-weight GEMM: no memory for the converted operands, C not written");
      rc = SKL_HIP_ERR_WORKSPACE;
    } else if (values && !scales) { /* B as E4M3: exact */
      rc = skl_hip_launch_cvt_f4_f8e4m3((uint8_t *)block, b, values);
      d.b = block;
    } else if (values) { /* scaled values leave E4M3's range: both operands as bf16 (exact), then the bf16 GEMM */
      rc = skl_hip_launch_cvt_f8_bf16(SKL_DT_F8E4M3, (uint16_t *)block, a, span_a);
      if (rc == 0) rc = skl_hip_launch_cvt_mxf4_bf16((uint16_t *)(block + bytes_a), b, scales, lds, n, k, ldb);
      d.ta = d.tb = SKL_DT_BF16;
      d.a = block;
      d.b = block + bytes_a;
    } else {
      rc = 0;
    }
    if (rc == 0) rc = gemm_on_device(&d);
    skl_hip_sequence_end();
    if (own) {
      skl_hip_synchronize(); /* the kernels that read the buffer have finished */
      skl_hip_free(own);
      if (rc == 0 && pending != SKL_HIP_ERR_WORKSPACE) skl_hip_withdraw_error(SKL_HIP_ERR_WORKSPACE); /* the scratch block's refusal was made good */
    }
    return rc;
  }
}

static void f4_gemm_run(size_t m, size_t n, size_t k, float alpha, const uint8_t *a, size_t rsa, size_t csa, const uint8_t *b, size_t ldb,
                        const uint8_t *scales, size_t lds, float beta, float *c, size_t rsc, size_t csc, const char *who) {
  skl_scalar beta_s;
  int where;
  if (m == 0 || n == 0) return; /* nothing is addressed */
  memset(&beta_s, 0, sizeof beta_s);
  beta_s.fz.value = beta;
  beta_s.fz.skip_c_read = skl_hip_get_beta_zero_mode() != SKL_HIP_BETA_ZERO_AS_REFERENCE;
  where = classify(k ? a : NULL, k ? b : NULL, c, who);
  if (where < 0) return;
  if (k && scales && classify(scales, NULL, NULL, who) != where) {
    skl_hip_record_error(SKL_HIP_ERR_MIXED_POINTERS, who);
    return;
  }
  if (where == 1) {
    (void)f4_gemm_on_device(m, n, k, alpha, a, rsa, csa, b, ldb, scales, lds, beta_s, c, rsc, csc);
    return;
  }
  {
    const size_t na = k ? (m - 1) * rsa + (k - 1) * csa + 1 : 0, nb = k ? ((n - 1) * ldb + k + 1) / 2 : 0;
    const size_t ns = (k && scales) ? (n - 1) * lds + (k + 31) / 32 : 0, nc = (m - 1) * rsc + (n - 1) * csc + 1;
    void *da = stage_in(a, na), *db = stage_in(b, nb), *ds = stage_in(scales, ns), *dc = stage_in(c, nc * sizeof(float));
    if ((!na || da) && (!nb || db) && (!ns || ds) && dc &&
        f4_gemm_on_device(m, n, k, alpha, (const uint8_t *)da, rsa, csa, (const uint8_t *)db, ldb, (const uint8_t *)ds, lds, beta_s,
                          (float *)dc, rsc, csc) == 0)
      skl_hip_memcpy_d2h(c, dc, nc * sizeof(float)); /* C's whole span: the elements in its stride gaps come back unchanged */
    skl_hip_free(da);
    skl_hip_free(db);
    skl_hip_free(ds);
    skl_hip_free(dc);
  }
}

void skl_gemm_f8e4m3rc_f4e2m1c_f32rc_gfx950(size_t m, size_t n, size_t k, float alpha, const uint8_t *a, size_t rsa, size_t csa,
                                           const uint8_t *b, size_t ldb, float beta, float *c, size_t rsc, size_t csc) {
  f4_gemm_run(m, n, k, alpha, a, rsa, csa, b, ldb, NULL, 0, beta, c, rsc, csc, __func__);
}

void skl_gemm_f8e4m3rc_mxf4e2m1c_f32rc_gfx950(size_t m, size_t n, size_t k, float alpha, const uint8_t *a, size_t rsa, size_t csa,
                                             const uint8_t *b, size_t ldb, const uint8_t *scales, size_t lds, float beta, float *c,
                                             size_t rsc, size_t csc) {
  f4_gemm_run(m, n, k, alpha, a, rsa, csa, b, ldb, scales, lds, beta, c, rsc, csc, __func__);
}

/* column-major A: the rc form with rsa = 1
 * (src/gemm/gemm_i8c_i8_i32_xsfmm32a8i.h:38-48) */
#define DEFINE_GEMM_COLMAJOR_A(NAME, RC, TA_T, TC_T)                                               \
  void NAME(size_t m, size_t n, size_t k, TC_T alpha, const TA_T *a, size_t csa, const TA_T *b,    \
            size_t rsb, TC_T beta, TC_T *c, size_t rsc) {                                          \
    RC(m, n, k, alpha, a, 1, csa, b, rsb, 1, beta, c, rsc, 1);                                     \
  }
DEFINE_GEMM_COLMAJOR_A(skl_gemm_i8c_i8_i32_gfx950, skl_gemm_i8rc_i8rc_i32rc_gfx950, int8_t, int32_t)
DEFINE_GEMM_COLMAJOR_A(skl_gemm_bf16c_bf16_f32_gfx950, skl_gemm_bf16rc_bf16rc_f32rc_gfx950, skl_bf16_t, float)
DEFINE_GEMM_COLMAJOR_A(skl_gemm_f16c_f16_f32_gfx950, skl_gemm_f16rc_f16rc_f32rc_gfx950, skl_f16_t, float)
DEFINE_GEMM_COLMAJOR_A(skl_gemm_f8e4m3c_f8e4m3_f32_gfx950, skl_gemm_f8e4m3rc_f8e4m3rc_f32rc_gfx950, uint8_t, float)
DEFINE_GEMM_COLMAJOR_A(skl_gemm_f8e5m2c_f8e5m2_f32_gfx950, skl_gemm_f8e5m2rc_f8e5m2rc_f32rc_gfx950, uint8_t, float)
DEFINE_GEMM_COLMAJOR_A(skl_gemm_f32c_f32_f32_gfx950, skl_gemm_f32rc_f32rc_f32rc_gfx950, float, float)

/* panel-packed: the rcprc form with (m0, n0, k0) = (TE, TE, 1), rsa0 = 1, csb0 = 1
 * (src/gemm/gemm_i8c_i8_i32_xsfmm32a8i.h:85-95) */
#define DEFINE_GEMM_PANEL(NAME, RCPRC, TA_T, TC_T)                                                 \
  void NAME(size_t m1, size_t n1, size_t k, TC_T alpha, const TA_T *a, size_t rsa1, size_t csa1,   \
            const TA_T *b, size_t rsb1, size_t csb1, TC_T beta, TC_T *c, size_t rsc0, size_t csc0, \
            size_t rsc1, size_t csc1) {                                                            \
    RCPRC(SKL_TE, SKL_TE, 1, m1, n1, k, alpha, a, 1, 0, rsa1, csa1, b, 0, 1, rsb1, csb1, beta, c,  \
          rsc0, csc0, rsc1, csc1);                                                                 \
  }
DEFINE_GEMM_PANEL(skl_gemm_i8rcptex1c_i8rcp1xte_i32rcptexterc_gfx950, skl_gemm_i8rcprc_i8rcprc_i32rcprc_gfx950, int8_t, int32_t)
DEFINE_GEMM_PANEL(skl_gemm_bf16rcptex1c_bf16rcp1xte_f32rcptexterc_gfx950, skl_gemm_bf16rcprc_bf16rcprc_f32rcprc_gfx950, skl_bf16_t, float)
DEFINE_GEMM_PANEL(skl_gemm_f16rcptex1c_f16rcp1xte_f32rcptexterc_gfx950, skl_gemm_f16rcprc_f16rcprc_f32rcprc_gfx950, skl_f16_t, float)
DEFINE_GEMM_PANEL(skl_gemm_f8e4m3rcptex1c_f8e4m3rcp1xte_f32rcptexterc_gfx950, skl_gemm_f8e4m3rcprc_f8e4m3rcprc_f32rcprc_gfx950, uint8_t, float)
DEFINE_GEMM_PANEL(skl_gemm_f8e5m2rcptex1c_f8e5m2rcp1xte_f32rcptexterc_gfx950, skl_gemm_f8e5m2rcprc_f8e5m2rcprc_f32rcprc_gfx950, uint8_t, float)
DEFINE_GEMM_PANEL(skl_gemm_f32rcptex1c_f32rcp1xte_f32rcptexterc_gfx950, skl_gemm_f32rcprc_f32rcprc_f32rcprc_gfx950, float, float)

/* K-packed int8: the rcprc form with (m0, n0, k0) = (1, 1, 4)
 * (src/gemm/gemm_i8rcp1x4_i8p4x1c_i32_xsfvqdotq.h:43-53) */
void skl_gemm_i8rcp1x4_i8p4x1c_i32_gfx950(size_t m, size_t n, size_t k1, int32_t alpha, const int8_t *a,
                                          size_t rsa1, size_t csa1, const int8_t *b, size_t rsb1,
                                          int32_t beta, int32_t *c, size_t rsc) {
  skl_gemm_i8rcprc_i8rcprc_i32rcprc_gfx950(1, 1, 4, m, n, k1, alpha, a, 0, 1, rsa1, csa1, b, 1, 0, rsb1, 4,
                                           beta, c, 0, 0, rsc, 1);
}

/* src/gemm/packed-gemm.md:270-298 */
void skl_gemm_a1b01_i8p4x8_i8p8x4_i32p4x4_gfx950(size_t m1, size_t n1, size_t k1, const int8_t *a, size_t rsa1,
                                                 const int8_t *b, size_t rsb1, int32_t *c, size_t rsc1,
                                                 bool accum) {
  skl_gemm_desc d = {SKL_DT_I8, SKL_DT_I8, 4, 4, 8, m1, n1, k1, a, 8, 1, rsa1, 32, b, 4, 1, rsb1, 32,
                     c, 4, 1, rsc1, 16, {.i = 1}, {.i = accum ? 1 : 0}, NULL, NULL, {0}};
  gemm_run(&d, __func__);
}

/* ------------------------------------------------------------------------ */
/* pack / unpack / transpose                                                 */
/* ------------------------------------------------------------------------ */

static void pack_run(int esize, size_t m, size_t n, const void *src, size_t rs, size_t cs, size_t m0,
                     size_t n0, void *dst, size_t rs0, size_t cs0, size_t rs1, size_t cs1, uint32_t pad,
                     const char *who) {
  int where;
  if (m == 0 || n == 0 || m0 == 0 || n0 == 0) return;
  where = classify(src, dst, NULL, who);
  if (where < 0) return;
  if (where == 1) {
    skl_hip_launch_pack(esize, m, n, src, rs, cs, m0, n0, dst, rs0, cs0, rs1, cs1, pad);
    return;
  }
  {
    const size_t m1 = (m + m0 - 1) / m0, n1 = (n + n0 - 1) / n0;
    const size_t ns = span4(m, rs, n, cs, 1, 0, 1, 0);
    const size_t nd = span4(m1, rs1, n1, cs1, m0, rs0, n0, cs0);
    void *ds = stage_in(src, ns * esize), *dd = stage_in(dst, nd * esize);
    if (ds && dd) {
      skl_hip_launch_pack(esize, m, n, ds, rs, cs, m0, n0, dd, rs0, cs0, rs1, cs1, pad);
      skl_hip_memcpy_d2h(dst, dd, nd * esize);
    }
    skl_hip_free(ds);
    skl_hip_free(dd);
  }
}

static void unpack_run(int esize, size_t m0, size_t n0, const void *src, size_t rs0, size_t cs0,
                       size_t rs1, size_t cs1, size_t m, size_t n, void *dst, size_t rs, size_t cs,
                       const char *who) {
  int where;
  if (m == 0 || n == 0 || m0 == 0 || n0 == 0) return;
  where = classify(src, dst, NULL, who);
  if (where < 0) return;
  if (where == 1) {
    skl_hip_launch_unpack(esize, m0, n0, src, rs0, cs0, rs1, cs1, m, n, dst, rs, cs);
    return;
  }
  {
    /* Only the in-range part of the blocks is read: the last block row/column
     * may be shorter than m0 / n0 in the caller's buffer. The address is a row
     * term plus a column term; the farthest element maximises each. */
    const size_t m1 = (m + m0 - 1) / m0, n1 = (n + n0 - 1) / n0;
    const size_t lm = m - (m1 - 1) * m0, ln = n - (n1 - 1) * n0; /* extent of the last block */
    size_t max_r = (m1 - 1) * rs1 + (lm - 1) * rs0, max_c = (n1 - 1) * cs1 + (ln - 1) * cs0;
    size_t ns;
    const size_t nd = span4(m, rs, n, cs, 1, 0, 1, 0);
    void *ds, *dd;
    if (m1 > 1 && (m1 - 2) * rs1 + (m0 - 1) * rs0 > max_r) max_r = (m1 - 2) * rs1 + (m0 - 1) * rs0;
    if (n1 > 1 && (n1 - 2) * cs1 + (n0 - 1) * cs0 > max_c) max_c = (n1 - 2) * cs1 + (n0 - 1) * cs0;
    ns = max_r + max_c + 1;
    ds = stage_in(src, ns * esize);
    dd = stage_in(dst, nd * esize);
    if (ds && dd) {
      skl_hip_launch_unpack(esize, m0, n0, ds, rs0, cs0, rs1, cs1, m, n, dd, rs, cs);
      skl_hip_memcpy_d2h(dst, dd, nd * esize);
    }
    skl_hip_free(ds);
    skl_hip_free(dd);
  }
}

#define DEFINE_PACK_FAMILY(W, T, ES)                                                                 \
  void skl_pack_e##W##rc_e##W##rcprc_gfx950(size_t m, size_t n, const T *src, size_t rs, size_t cs, \
                                            size_t m0, size_t n0, T *dst, size_t rs0, size_t cs0,   \
                                            size_t rs1, size_t cs1, T pad) {                        \
    pack_run(ES, m, n, src, rs, cs, m0, n0, dst, rs0, cs0, rs1, cs1, (uint32_t)pad, __func__);      \
  }                                                                                                  \
  void skl_unpack_e##W##rcprc_e##W##rc_gfx950(size_t m0, size_t n0, const T *src, size_t rs0,       \
                                              size_t cs0, size_t rs1, size_t cs1, size_t m,         \
                                              size_t n, T *dst, size_t rs, size_t cs) {             \
    unpack_run(ES, m0, n0, src, rs0, cs0, rs1, cs1, m, n, dst, rs, cs, __func__);                   \
  }                                                                                                  \
  /* One m x n block written with strides (1, rsat): src/transpose/README.md:3-9 */                 \
  void skl_transpose_e##W##_gfx950(size_t m, size_t n, const T *a, size_t rsa, T *at, size_t rsat) { \
    pack_run(ES, m, n, a, rsa, 1, m, n, at, 1, rsat, 0, 0, 0, __func__);                            \
  }                                                                                                  \
  /* src/pack/pack_e16_xsfmmbase.h:34-43 */                                                          \
  void skl_pack_e##W##_e##W##rcptex1c_gfx950(size_t m, size_t n, const T *src, size_t rs, T *dst,   \
                                             size_t rs1, size_t cs1, T pad) {                       \
    pack_run(ES, m, n, src, rs, 1, SKL_TE, 1, dst, 1, 0, rs1, cs1, (uint32_t)pad, __func__);        \
  }
DEFINE_PACK_FAMILY(8, uint8_t, 1)
DEFINE_PACK_FAMILY(16, uint16_t, 2)
DEFINE_PACK_FAMILY(32, uint32_t, 4)

/* Block layouts of the 4x8x4 block GEMM (src/gemm/packed-gemm.md:270-298, src/pack/README.md:172-178). */
void skl_pack_e8_e8p4x8_gfx950(size_t m, size_t n, const uint8_t *src, size_t rs, uint8_t *dst, size_t rs1,
                               uint8_t pad) {
  pack_run(1, m, n, src, rs, 1, 4, 8, dst, 8, 1, rs1, 32, pad, __func__);
}
void skl_pack_e8_e8p8x4_gfx950(size_t m, size_t n, const uint8_t *src, size_t rs, uint8_t *dst, size_t rs1,
                               uint8_t pad) {
  pack_run(1, m, n, src, rs, 1, 8, 4, dst, 4, 1, rs1, 32, pad, __func__);
}
void skl_pack_e32_e32p4x4_gfx950(size_t m, size_t n, const uint32_t *src, size_t rs, uint32_t *dst, size_t rs1,
                                 uint32_t pad) {
  pack_run(4, m, n, src, rs, 1, 4, 4, dst, 4, 1, rs1, 16, pad, __func__);
}
void skl_unpack_e32p4x4_e32_gfx950(size_t m, size_t n, const uint32_t *src, size_t rs1, uint32_t *dst, size_t rs) {
  unpack_run(4, 4, 4, src, 4, 1, rs1, 16, m, n, dst, rs, 1, __func__);
}

/* ------------------------------------------------------------------------ */
/* cvt                                                                       */
/* ------------------------------------------------------------------------ */

/* kind: 0 f32->f8, 1 bf16->f8, 2 f8->bf16, 3 f4->f8e4m3 */
static void cvt_run(int kind, int fmt, int sat, void *dst, const void *src, float scale, size_t n,
                    const char *who) {
  static const size_t src_num[4] = {4, 2, 1, 1}, dst_size[4] = {1, 1, 2, 1};
  int where;
  void *ds = NULL, *dd = NULL;
  void *d = dst;
  const void *s = src;
  size_t src_bytes, dst_bytes;
  if (n == 0) return;
  where = classify(src, dst, NULL, who);
  if (where < 0) return;
  src_bytes = kind == 3 ? (n + 1) / 2 : n * src_num[kind];
  dst_bytes = n * dst_size[kind];
  if (where == 0) {
    ds = stage_in(src, src_bytes);
    dd = skl_hip_malloc(dst_bytes);
    if (!ds || !dd) {
      skl_hip_free(ds);
      skl_hip_free(dd);
      return;
    }
    d = dd;
    s = ds;
  }
  switch (kind) {
    case 0: skl_hip_launch_cvt_f32_f8(fmt, sat, (uint8_t *)d, (const float *)s, scale, n); break;
    case 1: skl_hip_launch_cvt_bf16_f8(fmt, sat, (uint8_t *)d, (const uint16_t *)s, scale, n); break;
    case 2: skl_hip_launch_cvt_f8_bf16(fmt, (uint16_t *)d, (const uint8_t *)s, n); break;
    default: skl_hip_launch_cvt_f4_f8e4m3((uint8_t *)d, (const uint8_t *)s, n); break;
  }
  if (where == 0) {
    skl_hip_memcpy_d2h(dst, dd, dst_bytes);
    skl_hip_free(ds);
    skl_hip_free(dd);
  }
}

#define DEFINE_CVT_TO_F8(NAME, SRC_T, KIND, FMT, SAT)                               \
  void NAME(uint8_t *dst, const SRC_T *src, float scale, size_t n) {                \
    cvt_run(KIND, FMT, SAT, dst, src, scale, n, #NAME);                             \
  }
DEFINE_CVT_TO_F8(skl_cvt_f32_f8e4m3_gfx950, float, 0, SKL_DT_F8E4M3, 0)
DEFINE_CVT_TO_F8(skl_cvt_sat_f32_f8e4m3_gfx950, float, 0, SKL_DT_F8E4M3, 1)
DEFINE_CVT_TO_F8(skl_cvt_f32_f8e5m2_gfx950, float, 0, SKL_DT_F8E5M2, 0)
DEFINE_CVT_TO_F8(skl_cvt_sat_f32_f8e5m2_gfx950, float, 0, SKL_DT_F8E5M2, 1)
DEFINE_CVT_TO_F8(skl_cvt_bf16_f8e4m3_gfx950, skl_bf16_t, 1, SKL_DT_F8E4M3, 0)
DEFINE_CVT_TO_F8(skl_cvt_sat_bf16_f8e4m3_gfx950, skl_bf16_t, 1, SKL_DT_F8E4M3, 1)
DEFINE_CVT_TO_F8(skl_cvt_bf16_f8e5m2_gfx950, skl_bf16_t, 1, SKL_DT_F8E5M2, 0)
DEFINE_CVT_TO_F8(skl_cvt_sat_bf16_f8e5m2_gfx950, skl_bf16_t, 1, SKL_DT_F8E5M2, 1)

void skl_cvt_f8e4m3_bf16_gfx950(skl_bf16_t *dst, const uint8_t *src, size_t n) {
  cvt_run(2, SKL_DT_F8E4M3, 0, dst, src, 1.0f, n, __func__);
}
void skl_cvt_f8e5m2_bf16_gfx950(skl_bf16_t *dst, const uint8_t *src, size_t n) {
  cvt_run(2, SKL_DT_F8E5M2, 0, dst, src, 1.0f, n, __func__);
}
void skl_cvt_f4e2m1_f8e4m3_gfx950(uint8_t *dst, const uint8_t *src, size_t n) {
  cvt_run(3, SKL_DT_F8E4M3, 0, dst, src, 1.0f, n, __func__);
}
