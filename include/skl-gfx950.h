/*
 * skl-gfx950.h - kernel entry points of the MI355X (gfx950) implementation of
 * SKL's gemm / pack / cvt families.
 *
 * Every function keeps the parameter list of the SKL routine it stands in for
 * (cited as `path:line` below the reference checkout) and only changes the
 * ISA suffix of the name to `gfx950`: dimensions and strides are `size_t` in
 * ELEMENTS, alpha and beta have C's element type, all functions return void,
 * buffers are owned by the caller, `C = alpha*A*B + beta*C` (and `C = beta*C`
 * when k == 0; beta == 0 initialises a floating-point C without reading it
 * unless skl_hip_set_beta_zero_mode asks for the reference's evaluation, see
 * skl-hip.h), elements outside the addressed set are never written. Pointers may be all device-accessible (asynchronous launch on the
 * current stream) or all ordinary host memory (staged, synchronous); see
 * skl-hip.h. Errors are reported through skl_hip_last_error().
 *
 * 16-bit floating types are passed as 16-bit patterns; where the compiler
 * knows `__bf16` / `_Float16` the typedefs below are those types, so the
 * reference's callers compile unchanged.
 */
#ifndef SKL_GFX950_H
#define SKL_GFX950_H

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#include "skl-hip.h"

#if defined(__clang__) || (defined(__GNUC__) && __GNUC__ >= 13)
typedef __bf16 skl_bf16_t;
typedef _Float16 skl_f16_t;
#define SKL_GFX950_HAS_F16_SCALARS 1 /* `_Float16` can be passed by value: the f16 -> f16 GEMMs are declared */
#else
typedef uint16_t skl_bf16_t;
typedef uint16_t skl_f16_t;
#endif

#ifdef __cplusplus
extern "C" {
#endif

/* ======================================================================== */
/* GEMM - full-stride forms (the reference's defining routines)              */
/* ======================================================================== */

/* ref/gemm/gemm_i8rc_i8rc_i32rc.h:45 (skl_gemm_i8rc_i8rc_i32rc_ref) */
void skl_gemm_i8rc_i8rc_i32rc_gfx950(size_t m, size_t n, size_t k, int32_t alpha, const int8_t *a,
                                     size_t rsa, size_t csa, const int8_t *b, size_t rsb, size_t csb,
                                     int32_t beta, int32_t *c, size_t rsc, size_t csc);
/* ref/gemm/gemm_bf16rc_bf16rc_f32rc.h:44 */
void skl_gemm_bf16rc_bf16rc_f32rc_gfx950(size_t m, size_t n, size_t k, float alpha, const skl_bf16_t *a,
                                         size_t rsa, size_t csa, const skl_bf16_t *b, size_t rsb,
                                         size_t csb, float beta, float *c, size_t rsc, size_t csc);
/* ref/gemm/gemm_f16rc_f16rc_f32rc.h:44 */
void skl_gemm_f16rc_f16rc_f32rc_gfx950(size_t m, size_t n, size_t k, float alpha, const skl_f16_t *a,
                                       size_t rsa, size_t csa, const skl_f16_t *b, size_t rsb, size_t csb,
                                       float beta, float *c, size_t rsc, size_t csc);
/* ref/gemm/gemm_f8e4m3rc_f8e4m3rc_f32rc.h:48 */
void skl_gemm_f8e4m3rc_f8e4m3rc_f32rc_gfx950(size_t m, size_t n, size_t k, float alpha, const uint8_t *a,
                                             size_t rsa, size_t csa, const uint8_t *b, size_t rsb,
                                             size_t csb, float beta, float *c, size_t rsc, size_t csc);
/* ref/gemm/gemm_f8e5m2rc_f8e5m2rc_f32rc.h:48 */
void skl_gemm_f8e5m2rc_f8e5m2rc_f32rc_gfx950(size_t m, size_t n, size_t k, float alpha, const uint8_t *a,
                                             size_t rsa, size_t csa, const uint8_t *b, size_t rsb,
                                             size_t csb, float beta, float *c, size_t rsc, size_t csc);
/* Mixed formats: A is E4M3, B is E5M2. The reference has no such routine; the
 * argument list is that of ref/gemm/gemm_f8e4m3rc_f8e4m3rc_f32rc.h:48 and the
 * result is that of decoding both operands (ref/cvt/cvt_ofp8.c:18-95) and
 * calling ref/gemm/gemm_f32rc_f32rc_f32rc.h:44. */
void skl_gemm_f8e4m3rc_f8e5m2rc_f32rc_gfx950(size_t m, size_t n, size_t k, float alpha, const uint8_t *a,
                                             size_t rsa, size_t csa, const uint8_t *b, size_t rsb,
                                             size_t csb, float beta, float *c, size_t rsc, size_t csc);
/* OFP4 weights: A is E4M3 (any strides), B is E2M1 stored column by column - element (p, j) is 4-bit value number
 * j * ldb + p of `b`, value 2i in the low nibble of byte i and 2i + 1 in the high nibble, the packing
 * ref/cvt/cvt_ofp4.c:59-68 reads. The reference has no GEMM over 4-bit operands: it converts them first. The
 * result is that of skl_cvt_f4e2m1_f8e4m3 (ref/cvt/cvt_ofp4.c:59-68; exact - every E2M1 value is an E4M3 value) on
 * `b` followed by ref/gemm/gemm_f8e4m3rc_f8e4m3rc_f32rc.h:48 with rsb = 1, csb = ldb, inside that routine's
 * error bound. With 1 <= m <= 16 (up to 128 when B holds at least 2^20 values), csa = 1, k a
 * multiple of 32 and 16-byte aligned rows of A and columns of B (ldb a multiple of 32) the weights are multiplied
 * as they are - decoded by the matrix cores' FP4 operand format, or widened to bf16 in registers when k <= 2304
 * (exact products) - so they cross memory at half a byte per element; every other call converts B once into
 * scratch memory and runs the fp8 GEMM on the copy. */
void skl_gemm_f8e4m3rc_f4e2m1c_f32rc_gfx950(size_t m, size_t n, size_t k, float alpha, const uint8_t *a,
                                            size_t rsa, size_t csa, const uint8_t *b, size_t ldb, float beta,
                                            float *c, size_t rsc, size_t csc);
/* The same with OCP microscaling (MXFP4): every 32 consecutive k of a column share a scale 2^(s - 127), s = the
 * E8M0 byte scales[j * lds + p / 32] (1 <= s <= 254; s == 127 everywhere or scales == NULL is the call above; the
 * two codes outside that range - 0, E8M0's 2^-127, and 255, its NaN - are not part of this entry point's domain: the
 * device cannot refuse them, and what a block that carries one contributes is unspecified - zero or 2^-127 times its
 * values, infinity or NaN, depending on which kernel the shape selects). The
 * reference has no notion of block scales: the result is that of decoding both operands to fp32 - A by
 * ref/cvt/cvt_ofp8.c:18-52, B's E2M1 values times their scales, all exact - and calling
 * ref/gemm/gemm_f32rc_f32rc_f32rc.h:44 (sums in fp32), inside the error bound of the reference's fp8 GEMM test.
 * Decode shapes (as above) stream the weights and hand the scales to the matrix cores one per lane and instruction;
 * every other call converts both operands to bf16 (exact) into scratch memory and runs the bf16 GEMM. */
void skl_gemm_f8e4m3rc_mxf4e2m1c_f32rc_gfx950(size_t m, size_t n, size_t k, float alpha, const uint8_t *a,
                                              size_t rsa, size_t csa, const uint8_t *b, size_t ldb,
                                              const uint8_t *scales, size_t lds, float beta, float *c, size_t rsc,
                                              size_t csc);
/* ref/gemm/gemm_f32rc_f32rc_f32rc.h:44. Vector ALUs (the result is defined operation by operation): the
 * register-tiled kernel, or the any-stride kernel for tiny or oddly blocked problems. */
void skl_gemm_f32rc_f32rc_f32rc_gfx950(size_t m, size_t n, size_t k, float alpha, const float *a, size_t rsa,
                                       size_t csa, const float *b, size_t rsb, size_t csb, float beta,
                                       float *c, size_t rsc, size_t csc);
/* ref/gemm/gemm_f64rc_f64rc_f64rc.h:44. Register-tiled or any-stride kernel, like f32. */
void skl_gemm_f64rc_f64rc_f64rc_gfx950(size_t m, size_t n, size_t k, double alpha, const double *a,
                                       size_t rsa, size_t csa, const double *b, size_t rsb, size_t csb,
                                       double beta, double *c, size_t rsc, size_t csc);

/* Blocked ("rcprc") forms: element (I,i ; P,p) of A is at
 * a[I*rsa1 + P*csa1 + i*rsa0 + p*csa0], likewise B (rows k) and C. */
#define SKL_GFX950_DECLARE_RCPRC(NAME, TA, TC)                                                       \
  void NAME(size_t m0, size_t n0, size_t k0, size_t m1, size_t n1, size_t k1, TC alpha, const TA *a, \
            size_t rsa0, size_t csa0, size_t rsa1, size_t csa1, const TA *b, size_t rsb0,            \
            size_t csb0, size_t rsb1, size_t csb1, TC beta, TC *c, size_t rsc0, size_t csc0,         \
            size_t rsc1, size_t csc1)
/* ref/gemm/gemm_i8rcprc_i8rcprc_i32rcprc.h:50 */
SKL_GFX950_DECLARE_RCPRC(skl_gemm_i8rcprc_i8rcprc_i32rcprc_gfx950, int8_t, int32_t);
/* ref/gemm/gemm_bf16rcprc_bf16rcprc_f32rcprc.h:49 */
SKL_GFX950_DECLARE_RCPRC(skl_gemm_bf16rcprc_bf16rcprc_f32rcprc_gfx950, skl_bf16_t, float);
/* ref/gemm/gemm_f16rcprc_f16rcprc_f32rcprc.h:49 */
SKL_GFX950_DECLARE_RCPRC(skl_gemm_f16rcprc_f16rcprc_f32rcprc_gfx950, skl_f16_t, float);
/* ref/gemm/gemm_f8e4m3rcprc_f8e4m3rcprc_f32rcprc.h:53 */
SKL_GFX950_DECLARE_RCPRC(skl_gemm_f8e4m3rcprc_f8e4m3rcprc_f32rcprc_gfx950, uint8_t, float);
/* ref/gemm/gemm_f8e5m2rcprc_f8e5m2rcprc_f32rcprc.h:53 */
SKL_GFX950_DECLARE_RCPRC(skl_gemm_f8e5m2rcprc_f8e5m2rcprc_f32rcprc_gfx950, uint8_t, float);
/* ref/gemm/gemm_f32rcprc_f32rcprc_f32rcprc.h:49 */
SKL_GFX950_DECLARE_RCPRC(skl_gemm_f32rcprc_f32rcprc_f32rcprc_gfx950, float, float);
/* ref/gemm/gemm_f64rcprc_f64rcprc_f64rcprc.h:49 */
SKL_GFX950_DECLARE_RCPRC(skl_gemm_f64rcprc_f64rcprc_f64rcprc_gfx950, double, double);

#ifdef SKL_GFX950_HAS_F16_SCALARS
/* f16 operands, f16 accumulator, f16 C; alpha and beta are `_Float16` by value, as in the reference.
 * `_Float16` expressions are evaluated in float and rounded to half where they are assigned (what a C
 * compiler does for a target without half arithmetic, i.e. how the reference's scalar library computes
 * on a general-purpose host); hardware with native half arithmetic rounds the product as well and may
 * differ in the last place, inside the reference's own bound (test/gemm/gemm_f16rcprc_f16rcprc_f16rcprc.c:157).
 * Register-tiled or any-stride kernel, like f32.
 * ref/gemm/gemm_f16rc_f16rc_f16rc.h:44 */
void skl_gemm_f16rc_f16rc_f16rc_gfx950(size_t m, size_t n, size_t k, skl_f16_t alpha, const skl_f16_t *a,
                                       size_t rsa, size_t csa, const skl_f16_t *b, size_t rsb, size_t csb,
                                       skl_f16_t beta, skl_f16_t *c, size_t rsc, size_t csc);
/* ref/gemm/gemm_f16rcprc_f16rcprc_f16rcprc.h:49 */
SKL_GFX950_DECLARE_RCPRC(skl_gemm_f16rcprc_f16rcprc_f16rcprc_gfx950, skl_f16_t, skl_f16_t);
#endif

/* ======================================================================== */
/* GEMM with a fused epilogue                                                */
/* ======================================================================== */

/* What the reference's per-tile fused kernels compute on the matrix engine's tile state
 * (src/gemm/fused-kernel-API.md:85-216: alpha/beta scaling :104-125, adding a bias :159-178, a global
 * maximum :186-207), applied here to the accumulators in registers before C is written - the fusion
 * src/gemm/README.md:141-146 tells users to approximate by tiling the output. The reference keeps its
 * fused kernels private (SKL_FUNC_PRIVATE), so these entry points have no public prototype to mirror;
 * they take the argument list of the rc / rcprc form plus the descriptor.
 * For every addressed element (i, j), (i, j) the logical row and column:
 *     v = beta*C(i,j) + alpha*(A*B)(i,j)        as in the plain GEMM, beta == 0 included
 *     v = v + bias[j]                            if bias != NULL (one rounded addition; int32 wraps)
 *     v = v > 0 ? v : 0                          if activation == SKL_GFX950_ACT_RELU (a NaN becomes 0)
 *     v = v / (1 + exp(-v))                      if activation == SKL_GFX950_ACT_SILU, v * Phi(v) if SKL_GFX950_ACT_GELU:
 *                                                floating-point C only; the values of the reference's
 *                                                skl_silu_f32_ref (ref/sigmoid/sigmoid_f32.c:36-38) and skl_gelu_f32_ref
 *                                                (ref/gelu/gelu_f32.c:12-22) to within the error its own vector kernels
 *                                                are held to (test/sigmoid/sigmoid_f32_zve32f.c: 52 ulp;
 *                                                test/gelu/skl_gelu_f32_zve32f.c: 4 ulp for v >= 0, 5 in [-1, 0),
 *                                                62 in [-2, -1), unbounded below), a NaN stays a NaN
 *     C(i,j) = v                                 unless q_only
 *     Q(i,j) = clamp(rne((float)v * s_j) + q_zero, -128, 127)      if q != NULL: the requantised int8 copy,
 *                                                at q[i*rsq + j*csq]; s_j = q_scale[j] with q_scale_per_column, else
 *                                                q_scale[0]; (float)v rounds an int32 to nearest even, the product is
 *                                                one fp32 multiplication, rne() rounds it to the nearest integer, ties
 *                                                to even (a NaN counts as 0, values beyond int32 as its ends)
 *                                                with q_format one of the fp8 codes below the byte is instead the OCP fp8
 *                                                encoding of (float)v * s_j as skl_cvt_[sat_]f32_f8e4m3 / _f8e5m2
 *                                                (ref/cvt/cvt_ofp8.c:174-242) produces it, q_zero unused
 *                                                with q_only C is not written; and with beta == 0 it is not read either
 *                                                (the pointer need not address a matrix): where the product is an
 *                                                exact zero a floating-point result then takes the sign that an old
 *                                                C of +0 would give it
 *     *max = v  if v > *max                      if max != NULL (a NaN never replaces the maximum;
 *                                                the sign of a zero maximum is unspecified)
 * Bias and maximum are the steps of the reference's fused kernels; activation and requantisation are what
 * src/gemm/README.md:46-47 names as the operations callers would fuse next ("requantization and activation
 * functions") and leaves to them - the reference has no routine for either, the rules above define them here.
 * bias points to n = n1*n0 values of C's type, max to one, q_scale to n floats or one; all of them and q must be
 * memory of the same kind as C (device or host) and must not overlap C or each other; *max must not be NaN on
 * entry; q_zero lies in [-128, 127]. With q_only the call still reads C when beta is not zero (or when
 * skl_hip_set_beta_zero_mode asked for the reference's evaluation of beta * C). Members left zero (e.g. by a
 * designated initialiser that names only bias and max) switch their step off. ep == NULL: the plain GEMM. */
#define SKL_GFX950_ACT_NONE 0
#define SKL_GFX950_ACT_RELU 1
#define SKL_GFX950_ACT_SILU 2 /* floating-point C only */
#define SKL_GFX950_ACT_GELU 3 /* floating-point C only */
#define SKL_GFX950_Q_INT8 0       /* what a byte of q holds: int8 by the rule above (default) */
#define SKL_GFX950_Q_F8E4M3 1     /* OCP E4M3, overflow to the format's NaN like skl_cvt_f32_f8e4m3 */
#define SKL_GFX950_Q_F8E4M3_SAT 2 /* ... saturating like skl_cvt_sat_f32_f8e4m3 */
#define SKL_GFX950_Q_F8E5M2 3     /* OCP E5M2, overflow to infinity like skl_cvt_f32_f8e5m2 */
#define SKL_GFX950_Q_F8E5M2_SAT 4 /* ... saturating like skl_cvt_sat_f32_f8e5m2 */
/* Every step off: `skl_gfx950_epilogue_t ep = SKL_GFX950_EPILOGUE_NONE; ep.bias = ...;` is valid C and C++. */
#define SKL_GFX950_EPILOGUE_NONE {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0}
typedef struct skl_gfx950_epilogue {
  const void *bias;
  void *max;
  int activation;
  int q_scale_per_column;
  int q_only;
  int32_t q_zero;
  int8_t *q;
  size_t rsq, csq;
  const float *q_scale;
  int q_format; /* SKL_GFX950_Q_* */
} skl_gfx950_epilogue_t;

#define SKL_GFX950_DECLARE_FUSED_RC(NAME, TA, TC)                                                    \
  void NAME(size_t m, size_t n, size_t k, TC alpha, const TA *a, size_t rsa, size_t csa, const TA *b, \
            size_t rsb, size_t csb, TC beta, TC *c, size_t rsc, size_t csc, const skl_gfx950_epilogue_t *ep)
#define SKL_GFX950_DECLARE_FUSED_RCPRC(NAME, TA, TC)                                                 \
  void NAME(size_t m0, size_t n0, size_t k0, size_t m1, size_t n1, size_t k1, TC alpha, const TA *a, \
            size_t rsa0, size_t csa0, size_t rsa1, size_t csa1, const TA *b, size_t rsb0,            \
            size_t csb0, size_t rsb1, size_t csb1, TC beta, TC *c, size_t rsc0, size_t csc0,         \
            size_t rsc1, size_t csc1, const skl_gfx950_epilogue_t *ep)
SKL_GFX950_DECLARE_FUSED_RC(skl_gemm_fused_i8rc_i8rc_i32rc_gfx950, int8_t, int32_t);
SKL_GFX950_DECLARE_FUSED_RC(skl_gemm_fused_bf16rc_bf16rc_f32rc_gfx950, skl_bf16_t, float);
SKL_GFX950_DECLARE_FUSED_RC(skl_gemm_fused_f16rc_f16rc_f32rc_gfx950, skl_f16_t, float);
SKL_GFX950_DECLARE_FUSED_RC(skl_gemm_fused_f8e4m3rc_f8e4m3rc_f32rc_gfx950, uint8_t, float);
SKL_GFX950_DECLARE_FUSED_RC(skl_gemm_fused_f8e5m2rc_f8e5m2rc_f32rc_gfx950, uint8_t, float);
SKL_GFX950_DECLARE_FUSED_RCPRC(skl_gemm_fused_i8rcprc_i8rcprc_i32rcprc_gfx950, int8_t, int32_t);
SKL_GFX950_DECLARE_FUSED_RCPRC(skl_gemm_fused_bf16rcprc_bf16rcprc_f32rcprc_gfx950, skl_bf16_t, float);
SKL_GFX950_DECLARE_FUSED_RCPRC(skl_gemm_fused_f16rcprc_f16rcprc_f32rcprc_gfx950, skl_f16_t, float);
SKL_GFX950_DECLARE_FUSED_RCPRC(skl_gemm_fused_f8e4m3rcprc_f8e4m3rcprc_f32rcprc_gfx950, uint8_t, float);
SKL_GFX950_DECLARE_FUSED_RCPRC(skl_gemm_fused_f8e5m2rcprc_f8e5m2rcprc_f32rcprc_gfx950, uint8_t, float);

/* ======================================================================== */
/* GEMM - the optimized entry points of skl.h                                */
/* ======================================================================== */

/* Row-major A, B, C. M == 1 is served by the streaming (GEMV) kernels.
 * src/gemm/gemm_i8_i8_i32_zve32x.h:50, src/gemm/gemm_i8_i8_i32_zve32x_x390.h:50 */
void skl_gemm_i8_i8_i32_gfx950(size_t m, size_t n, size_t k, int32_t alpha, const int8_t *a, size_t rsa,
                               const int8_t *b, size_t rsb, int32_t beta, int32_t *c, size_t rsc);
/* skl_gemm_i8_i8_i32_gfx950 for callers that cannot allocate device memory: code under HIP graph capture, serving
 * loops and harnesses that forbid hipMalloc. It has no counterpart in the reference. Same arguments and the same
 * result, bit for bit, but only for decode calls - 1 <= m <= 8, all pointers device-accessible (they are not
 * queried), k > 0, n a multiple of 16, b and rsb multiples of 16 bytes, a 4-byte aligned with rsa a multiple of 4
 * when m > 1 - and only while m * n <= 65536: the sums that workgroups share live in a static 512 KiB array on
 * each GPU instead of a block the library allocates. Anything else records SKL_HIP_ERR_BAD_ARGUMENT and does
 * nothing. The call itself allocates, frees and queries nothing (skl_hip_init on the device beforehand also
 * keeps the one address lookup out of it). All such calls on one GPU share that array: calls that overlap on the
 * device - different streams, or the branches of one graph - race, and leave sums behind that every later call
 * would add to; skl_hip_noalloc_reset() (skl-hip.h) puts the array back to zero. */
void skl_gemm_i8_i8_i32_noalloc_gfx950(size_t m, size_t n, size_t k, int32_t alpha, const int8_t *a, size_t rsa,
                                       const int8_t *b, size_t rsb, int32_t beta, int32_t *c, size_t rsc);
/* src/gemm/gemm_bf16_bf16_f32_zvfbfwma.h:49, src/gemm/gemm_bf16_bf16_f32_zvfbfwma_x390.h:49 */
void skl_gemm_bf16_bf16_f32_gfx950(size_t m, size_t n, size_t k, float alpha, const skl_bf16_t *a,
                                   size_t rsa, const skl_bf16_t *b, size_t rsb, float beta, float *c,
                                   size_t rsc);
/* src/gemm/gemm_f16_f16_f32_zvfh.h:49, src/gemm/gemm_f16_f16_f32_zvfh_x390.h:49 */
void skl_gemm_f16_f16_f32_gfx950(size_t m, size_t n, size_t k, float alpha, const skl_f16_t *a, size_t rsa,
                                 const skl_f16_t *b, size_t rsb, float beta, float *c, size_t rsc);
/* src/gemm/gemm_f32_f32_f32_zve32f.h:48, src/gemm/gemm_f32_f32_f32_zve32f_x390.h */
void skl_gemm_f32_f32_f32_gfx950(size_t m, size_t n, size_t k, float alpha, const float *a, size_t rsa,
                                 const float *b, size_t rsb, float beta, float *c, size_t rsc);
/* src/gemm/gemm_f64_f64_f64_zve64d.h:48, src/gemm/gemm_f64_f64_f64_zve64d_x390.h */
void skl_gemm_f64_f64_f64_gfx950(size_t m, size_t n, size_t k, double alpha, const double *a, size_t rsa,
                                 const double *b, size_t rsb, double beta, double *c, size_t rsc);
#ifdef SKL_GFX950_HAS_F16_SCALARS
/* src/gemm/gemm_f16_f16_f16_zvfh.h:48, src/gemm/gemm_f16_f16_f16_zvfh_x390.h */
void skl_gemm_f16_f16_f16_gfx950(size_t m, size_t n, size_t k, skl_f16_t alpha, const skl_f16_t *a, size_t rsa,
                                 const skl_f16_t *b, size_t rsb, skl_f16_t beta, skl_f16_t *c, size_t rsc);
#endif

/* Column-major A (= A^T stored row-major with row stride csa), row-major B, C.
 * src/gemm/gemm_i8c_i8_i32_xsfmm32a8i.h:57 */
void skl_gemm_i8c_i8_i32_gfx950(size_t m, size_t n, size_t k, int32_t alpha, const int8_t *a, size_t csa,
                                const int8_t *b, size_t rsb, int32_t beta, int32_t *c, size_t rsc);
/* src/gemm/gemm_bf16c_bf16_f32_xsfmm32a16f.h:56 */
void skl_gemm_bf16c_bf16_f32_gfx950(size_t m, size_t n, size_t k, float alpha, const skl_bf16_t *a,
                                    size_t csa, const skl_bf16_t *b, size_t rsb, float beta, float *c,
                                    size_t rsc);
/* src/gemm/gemm_f16c_f16_f32_xsfmm32a16f.h:56 */
void skl_gemm_f16c_f16_f32_gfx950(size_t m, size_t n, size_t k, float alpha, const skl_f16_t *a, size_t csa,
                                  const skl_f16_t *b, size_t rsb, float beta, float *c, size_t rsc);
/* src/gemm/gemm_f8e4m3c_f8e4m3_f32_xsfmm32a8f.h:57 */
void skl_gemm_f8e4m3c_f8e4m3_f32_gfx950(size_t m, size_t n, size_t k, float alpha, const uint8_t *a,
                                        size_t csa, const uint8_t *b, size_t rsb, float beta, float *c,
                                        size_t rsc);
/* src/gemm/gemm_f8e5m2c_f8e5m2_f32_xsfmm32a8f.h:57 */
void skl_gemm_f8e5m2c_f8e5m2_f32_gfx950(size_t m, size_t n, size_t k, float alpha, const uint8_t *a,
                                        size_t csa, const uint8_t *b, size_t rsb, float beta, float *c,
                                        size_t rsc);
/* src/gemm/gemm_f32c_f32_f32_xsfmm32a32f.h:56 */
void skl_gemm_f32c_f32_f32_gfx950(size_t m, size_t n, size_t k, float alpha, const float *a, size_t csa,
                                  const float *b, size_t rsb, float beta, float *c, size_t rsc);

/* Panel-packed operands, TE = skl_hip_te() = 64: A in TE x 1 column panels
 * (m0 = TE, k0 = 1, rsa0 = 1), B in 1 x TE row panels (n0 = TE, csb0 = 1), C in
 * TE x TE blocks with free strides. m1 / n1 count blocks.
 * src/gemm/gemm_i8c_i8_i32_xsfmm32a8i.h:97 */
#define SKL_GFX950_DECLARE_PANEL(NAME, TA, TC)                                                        \
  void NAME(size_t m1, size_t n1, size_t k, TC alpha, const TA *a, size_t rsa1, size_t csa1,          \
            const TA *b, size_t rsb1, size_t csb1, TC beta, TC *c, size_t rsc0, size_t csc0,          \
            size_t rsc1, size_t csc1)
SKL_GFX950_DECLARE_PANEL(skl_gemm_i8rcptex1c_i8rcp1xte_i32rcptexterc_gfx950, int8_t, int32_t);
/* src/gemm/gemm_bf16c_bf16_f32_xsfmm32a16f.h:97 */
SKL_GFX950_DECLARE_PANEL(skl_gemm_bf16rcptex1c_bf16rcp1xte_f32rcptexterc_gfx950, skl_bf16_t, float);
/* src/gemm/gemm_f16c_f16_f32_xsfmm32a16f.h:97 */
SKL_GFX950_DECLARE_PANEL(skl_gemm_f16rcptex1c_f16rcp1xte_f32rcptexterc_gfx950, skl_f16_t, float);
/* src/gemm/gemm_f8e4m3c_f8e4m3_f32_xsfmm32a8f.h:98 */
SKL_GFX950_DECLARE_PANEL(skl_gemm_f8e4m3rcptex1c_f8e4m3rcp1xte_f32rcptexterc_gfx950, uint8_t, float);
/* src/gemm/gemm_f8e5m2c_f8e5m2_f32_xsfmm32a8f.h:98 */
SKL_GFX950_DECLARE_PANEL(skl_gemm_f8e5m2rcptex1c_f8e5m2rcp1xte_f32rcptexterc_gfx950, uint8_t, float);
/* src/gemm/gemm_f32c_f32_f32_xsfmm32a32f.h:96 */
SKL_GFX950_DECLARE_PANEL(skl_gemm_f32rcptex1c_f32rcp1xte_f32rcptexterc_gfx950, float, float);

/* K-packed int8 ("dot4") layout: A in 1 x 4 K-blocks (A(i, 4P+p) at i*rsa1 +
 * P*csa1 + p), B in 4 x 1 K-blocks (B(4P+p, j) at P*rsb1 + 4*j + p), C row-major.
 * src/gemm/gemm_i8rcp1x4_i8p4x1c_i32_xsfvqdotq.h:70 */
void skl_gemm_i8rcp1x4_i8p4x1c_i32_gfx950(size_t m, size_t n, size_t k1, int32_t alpha, const int8_t *a,
                                          size_t rsa1, size_t csa1, const int8_t *b, size_t rsb1,
                                          int32_t beta, int32_t *c, size_t rsc);

/* 4 x 8 by 8 x 4 block products ("fat dot product" layout): A in row-major 4 x 8 blocks, block (I, P) at
 * I*rsa1 + P*32; B in row-major 8 x 4 blocks, block (P, J) at P*rsb1 + J*32; C in row-major 4 x 4 blocks, block
 * (I, J) at I*rsc1 + J*16. C = A*B, or C += A*B with `accum`. The reference documents this entry point and its
 * layouts (src/gemm/packed-gemm.md:270-298) and ships no implementation of it; the arithmetic is that of
 * ref/gemm/gemm_i8rcprc_i8rcprc_i32rcprc.c:10-37 with m0 = n0 = 4, k0 = 8, alpha = 1 and beta = accum. */
void skl_gemm_a1b01_i8p4x8_i8p8x4_i32p4x4_gfx950(size_t m1, size_t n1, size_t k1, const int8_t *a, size_t rsa1,
                                                 const int8_t *b, size_t rsb1, int32_t *c, size_t rsc1,
                                                 bool accum);

/* ======================================================================== */
/* pack / unpack / transpose                                                 */
/* ======================================================================== */

#define SKL_GFX950_DECLARE_PACK(W, T)                                                                  \
  /* ref/pack/pack_e8rc_e8rcprc.h:44 (+ e16, e32); src/pack/pack_e8_zve32x.h:49 */                     \
  void skl_pack_e##W##rc_e##W##rcprc_gfx950(size_t m, size_t n, const T *src, size_t rs, size_t cs,    \
                                            size_t m0, size_t n0, T *dst, size_t rs0, size_t cs0,      \
                                            size_t rs1, size_t cs1, T pad);                            \
  /* ref/pack/unpack_e8rcprc_e8rc.h:48; src/pack/pack_e8_zve32x.h:88. The reference ships the */      \
  /* 8-bit width only; the wider ones apply the same rule to wider elements. */                       \
  void skl_unpack_e##W##rcprc_e##W##rc_gfx950(size_t m0, size_t n0, const T *src, size_t rs0,          \
                                              size_t cs0, size_t rs1, size_t cs1, size_t m, size_t n,  \
                                              T *dst, size_t rs, size_t cs);                           \
  /* ref/pack/transpose_e8.h:33 (+ e16, e32); src/pack/pack_e8_zve32x.h:112, */                        \
  /* src/pack/pack_e8_xsfmmbase.h:38 */                                                                \
  void skl_transpose_e##W##_gfx950(size_t m, size_t n, const T *a, size_t rsa, T *at, size_t rsat);    \
  /* TE x 1 column panels of a row-major matrix: src/pack/pack_e16_xsfmmbase.h:49, */                  \
  /* src/pack/pack_e32_xsfmmbase.h:49 (the reference has no 8-bit one). */                             \
  void skl_pack_e##W##_e##W##rcptex1c_gfx950(size_t m, size_t n, const T *src, size_t rs, T *dst,      \
                                             size_t rs1, size_t cs1, T pad);
SKL_GFX950_DECLARE_PACK(8, uint8_t)
SKL_GFX950_DECLARE_PACK(16, uint16_t)
SKL_GFX950_DECLARE_PACK(32, uint32_t)

/* Packers of the 4 x 8 / 8 x 4 / 4 x 4 block layouts above, from and to a row-major matrix with row stride
 * `rs`; blocks of one block row are contiguous, block rows `rs1` apart; partial blocks are filled with `pad`.
 * src/pack/README.md:172-178 names these four kernels as required for that GEMM and gives no prototypes; the
 * argument list follows skl_pack_e16_e16rcptex1c (src/pack/pack_e16_xsfmmbase.h:49), the element rule is that of
 * ref/pack/pack_e8rc_e8rcprc.c:10-35 / ref/pack/unpack_e8rcprc_e8rc.c:10-37. */
void skl_pack_e8_e8p4x8_gfx950(size_t m, size_t n, const uint8_t *src, size_t rs, uint8_t *dst, size_t rs1,
                               uint8_t pad);
void skl_pack_e8_e8p8x4_gfx950(size_t m, size_t n, const uint8_t *src, size_t rs, uint8_t *dst, size_t rs1,
                               uint8_t pad);
void skl_pack_e32_e32p4x4_gfx950(size_t m, size_t n, const uint32_t *src, size_t rs, uint32_t *dst, size_t rs1,
                                 uint32_t pad);
void skl_unpack_e32p4x4_e32_gfx950(size_t m, size_t n, const uint32_t *src, size_t rs1, uint32_t *dst, size_t rs);

/* ======================================================================== */
/* OFP8 / OFP4 conversions: (dst, src, scale, n)                             */
/* ======================================================================== */

/* src/cvt/cvt_f32_f8_zvfofp8min.h:61,78,94,111; ref/cvt/cvt_ofp8.h:59-95 */
void skl_cvt_f32_f8e4m3_gfx950(uint8_t *dst, const float *src, float scale, size_t n);
void skl_cvt_sat_f32_f8e4m3_gfx950(uint8_t *dst, const float *src, float scale, size_t n);
void skl_cvt_f32_f8e5m2_gfx950(uint8_t *dst, const float *src, float scale, size_t n);
void skl_cvt_sat_f32_f8e5m2_gfx950(uint8_t *dst, const float *src, float scale, size_t n);
/* src/cvt/cvt_bf16_f8_zvfofp8min_zvfbfmin.h:67,84,102,119; ref/cvt/cvt_ofp8.h:106-141 */
void skl_cvt_bf16_f8e4m3_gfx950(uint8_t *dst, const skl_bf16_t *src, float scale, size_t n);
void skl_cvt_sat_bf16_f8e4m3_gfx950(uint8_t *dst, const skl_bf16_t *src, float scale, size_t n);
void skl_cvt_bf16_f8e5m2_gfx950(uint8_t *dst, const skl_bf16_t *src, float scale, size_t n);
void skl_cvt_sat_bf16_f8e5m2_gfx950(uint8_t *dst, const skl_bf16_t *src, float scale, size_t n);
/* src/cvt/cvt_f8_bf16_zvfofp8min.h:39,52; ref/cvt/cvt_ofp8.h:150,158 */
void skl_cvt_f8e4m3_bf16_gfx950(skl_bf16_t *dst, const uint8_t *src, size_t n);
void skl_cvt_f8e5m2_bf16_gfx950(skl_bf16_t *dst, const uint8_t *src, size_t n);
/* src/cvt/cvt_f4_f8_zvfofp4min.h:54; ref/cvt/cvt_ofp4.h:30. Two E2M1 values per
 * source byte, low nibble first. */
void skl_cvt_f4e2m1_f8e4m3_gfx950(uint8_t *dst, const uint8_t *src, size_t n);

#ifdef __cplusplus
}
#endif
#endif /* SKL_GFX950_H */
