/*
 * skl_oracle.h - CPU restatement of the SKL scalar reference semantics for the
 * gemm, pack and cvt families.
 *
 * THIS IS TEST INFRASTRUCTURE. It is the checker the GPU library is compared
 * with; it is never linked into, called from, or used as a fallback by the
 * product library. Only tests, the smoke check and the CPU-baseline leg of the
 * benchmark may load it.
 *
 * Every function restates one routine of the reference (file:line cited at
 * each definition in skl_oracle.c). 16-bit floating types travel as raw
 * uint16_t bit patterns so that the file builds with plain gcc.
 *
 * Parity status: every function below is pinned by tests/test_oracle_*.py
 * (compiled reference where it builds, documentation worked examples,
 * closed forms, numpy integer matmul, exhaustive byte tables), with one
 * exception. The f16 -> f16 GEMM (skl_gemm_f16rc_f16rc_f16rc_oracle and its
 * blocked twin) is "parity unpinned" against the reference's real targets: it
 * is bit-identical to the reference as compiled for x86, where
 * `_Float16 acc += a * b` multiplies in float and rounds to half once per
 * step; hardware with half arithmetic rounds the product as well (or
 * contracts to a half FMA) and may differ in the last place. The tests
 * therefore also hold it to the reference test's own bound (P = 11,
 * test/gemm/gemm_f16rcprc_f16rcprc_f16rcprc.c:157). The activation /
 * requantisation steps (skl_oracle_act_requant_*) have no reference routine:
 * their rules are stated in include/skl-gfx950.h and pinned by worked values.
 */
#ifndef SKL_ORACLE_H
#define SKL_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- scalar conversions ------------------------------------------------ */
float skl_oracle_f8e4m3_to_f32(uint8_t code);
float skl_oracle_f8e5m2_to_f32(uint8_t code);
float skl_oracle_f4e2m1_to_f32(uint8_t nibble);
uint8_t skl_oracle_f32_to_f8e4m3(float x, int saturate);
uint8_t skl_oracle_f32_to_f8e5m2(float x, int saturate);
float skl_oracle_bf16_to_f32(uint16_t bits);
float skl_oracle_f16_to_f32(uint16_t bits);
uint16_t skl_oracle_f32_to_bf16(float x);
uint16_t skl_oracle_f32_to_f16(float x);

/* ---- array conversions (dst, src, scale, n) ----------------------------- */
void skl_cvt_f32_f8e4m3_oracle(uint8_t *dst, const float *src, float scale, size_t n);
void skl_cvt_sat_f32_f8e4m3_oracle(uint8_t *dst, const float *src, float scale, size_t n);
void skl_cvt_f32_f8e5m2_oracle(uint8_t *dst, const float *src, float scale, size_t n);
void skl_cvt_sat_f32_f8e5m2_oracle(uint8_t *dst, const float *src, float scale, size_t n);
void skl_cvt_bf16_f8e4m3_oracle(uint8_t *dst, const uint16_t *src, float scale, size_t n);
void skl_cvt_sat_bf16_f8e4m3_oracle(uint8_t *dst, const uint16_t *src, float scale, size_t n);
void skl_cvt_bf16_f8e5m2_oracle(uint8_t *dst, const uint16_t *src, float scale, size_t n);
void skl_cvt_sat_bf16_f8e5m2_oracle(uint8_t *dst, const uint16_t *src, float scale, size_t n);
void skl_cvt_f8e4m3_bf16_oracle(uint16_t *dst, const uint8_t *src, size_t n);
void skl_cvt_f8e5m2_bf16_oracle(uint16_t *dst, const uint8_t *src, size_t n);
void skl_cvt_f4e2m1_f8e4m3_oracle(uint8_t *dst, const uint8_t *src, size_t n);

/* ---- pack / unpack / transpose ------------------------------------------ */
#define SKL_ORACLE_PACK_DECL(W, T)                                                      \
  void skl_pack_e##W##rc_e##W##rcprc_oracle(size_t m, size_t n, const T *src,          \
                                            size_t rs, size_t cs, size_t m0, size_t n0, \
                                            T *dst, size_t rs0, size_t cs0, size_t rs1, \
                                            size_t cs1, T pad);                         \
  void skl_unpack_e##W##rcprc_e##W##rc_oracle(size_t m0, size_t n0, const T *src,      \
                                              size_t rs0, size_t cs0, size_t rs1,       \
                                              size_t cs1, size_t m, size_t n, T *dst,   \
                                              size_t rs, size_t cs);                    \
  void skl_transpose_e##W##_oracle(size_t m, size_t n, const T *a, size_t rsa, T *at,  \
                                   size_t rsat);
SKL_ORACLE_PACK_DECL(8, uint8_t)
SKL_ORACLE_PACK_DECL(16, uint16_t)
SKL_ORACLE_PACK_DECL(32, uint32_t)

/* ---- GEMM: C = alpha*A*B + beta*C ---------------------------------------- */
#define SKL_ORACLE_GEMM_DECL(NAME, TA, TB, TC)                                          \
  void skl_gemm_##NAME##_oracle(size_t m, size_t n, size_t k, TC alpha, const TA *a,   \
                                size_t rsa, size_t csa, const TB *b, size_t rsb,        \
                                size_t csb, TC beta, TC *c, size_t rsc, size_t csc);
#define SKL_ORACLE_PGEMM_DECL(NAME, TA, TB, TC)                                         \
  void skl_gemm_##NAME##_oracle(size_t m0, size_t n0, size_t k0, size_t m1, size_t n1, \
                                size_t k1, TC alpha, const TA *a, size_t rsa0,          \
                                size_t csa0, size_t rsa1, size_t csa1, const TB *b,     \
                                size_t rsb0, size_t csb0, size_t rsb1, size_t csb1,     \
                                TC beta, TC *c, size_t rsc0, size_t csc0, size_t rsc1,  \
                                size_t csc1);

SKL_ORACLE_GEMM_DECL(i8rc_i8rc_i32rc, int8_t, int8_t, int32_t)
SKL_ORACLE_GEMM_DECL(bf16rc_bf16rc_f32rc, uint16_t, uint16_t, float)
SKL_ORACLE_GEMM_DECL(f16rc_f16rc_f32rc, uint16_t, uint16_t, float)
SKL_ORACLE_GEMM_DECL(f8e4m3rc_f8e4m3rc_f32rc, uint8_t, uint8_t, float)
SKL_ORACLE_GEMM_DECL(f8e5m2rc_f8e5m2rc_f32rc, uint8_t, uint8_t, float)
SKL_ORACLE_GEMM_DECL(f8e4m3rc_f8e5m2rc_f32rc, uint8_t, uint8_t, float)
SKL_ORACLE_GEMM_DECL(f32rc_f32rc_f32rc, float, float, float)
SKL_ORACLE_GEMM_DECL(f64rc_f64rc_f64rc, double, double, double)

SKL_ORACLE_PGEMM_DECL(i8rcprc_i8rcprc_i32rcprc, int8_t, int8_t, int32_t)
SKL_ORACLE_PGEMM_DECL(bf16rcprc_bf16rcprc_f32rcprc, uint16_t, uint16_t, float)
SKL_ORACLE_PGEMM_DECL(f16rcprc_f16rcprc_f32rcprc, uint16_t, uint16_t, float)
SKL_ORACLE_PGEMM_DECL(f8e4m3rcprc_f8e4m3rcprc_f32rcprc, uint8_t, uint8_t, float)
SKL_ORACLE_PGEMM_DECL(f8e5m2rcprc_f8e5m2rcprc_f32rcprc, uint8_t, uint8_t, float)
SKL_ORACLE_PGEMM_DECL(f32rcprc_f32rcprc_f32rcprc, float, float, float)
SKL_ORACLE_PGEMM_DECL(f64rcprc_f64rcprc_f64rcprc, double, double, double)
/* f16 accumulator and C (ref/gemm/gemm_f16rc_f16rc_f16rc.c:9-24 and the rcprc twin); alpha, beta: floats
 * holding half values */
void skl_gemm_f16rc_f16rc_f16rc_oracle(size_t m, size_t n, size_t k, float alpha, const uint16_t *a, size_t rsa,
                                       size_t csa, const uint16_t *b, size_t rsb, size_t csb, float beta,
                                       uint16_t *c, size_t rsc, size_t csc);
void skl_gemm_f16rcprc_f16rcprc_f16rcprc_oracle(size_t m0, size_t n0, size_t k0, size_t m1, size_t n1, size_t k1,
                                                float alpha, const uint16_t *a, size_t rsa0, size_t csa0,
                                                size_t rsa1, size_t csa1, const uint16_t *b, size_t rsb0,
                                                size_t csb0, size_t rsb1, size_t csb1, float beta, uint16_t *c,
                                                size_t rsc0, size_t csc0, size_t rsc1, size_t csc1);

/* E4M3 A times OFP4 B stored column by column: the reference's conversion (ref/cvt/cvt_ofp4.c:59-68) followed by its
 * fp8 GEMM with rsb = 1, csb = ldb. */
void skl_gemm_f8e4m3rc_f4e2m1c_f32rc_oracle(size_t m, size_t n, size_t k, float alpha, const uint8_t *a, size_t rsa,
                                            size_t csa, const uint8_t *b, size_t ldb, float beta, float *c, size_t rsc,
                                            size_t csc);

/* ... with one E8M0 scale per 32 consecutive k of a column (OCP microscaling): the reference's fp32 GEMM on the decoded
 * operands. scales may be NULL. */
void skl_gemm_f8e4m3rc_mxf4e2m1c_f32rc_oracle(size_t m, size_t n, size_t k, float alpha, const uint8_t *a, size_t rsa,
                                              size_t csa, const uint8_t *b, size_t ldb, const uint8_t *scales, size_t lds,
                                              float beta, float *c, size_t rsc, size_t csc);

/* GEMM + fused bias / maximum steps (src/gemm/fused-kernel-API.md:159-207); bias and max may be NULL. */
#define SKL_ORACLE_FUSED_DECL(NAME, TA, TC)                                                        \
  void skl_gemm_fused_##NAME##_oracle(size_t m, size_t n, size_t k, TC alpha, const TA *a, size_t rsa, \
                                      size_t csa, const TA *b, size_t rsb, size_t csb, TC beta, TC *c, \
                                      size_t rsc, size_t csc, const TC *bias, TC *max);
#define SKL_ORACLE_PFUSED_DECL(NAME, TA, TC)                                                       \
  void skl_gemm_fused_##NAME##_oracle(size_t m0, size_t n0, size_t k0, size_t m1, size_t n1, size_t k1, \
                                      TC alpha, const TA *a, size_t rsa0, size_t csa0, size_t rsa1, \
                                      size_t csa1, const TA *b, size_t rsb0, size_t csb0, size_t rsb1, \
                                      size_t csb1, TC beta, TC *c, size_t rsc0, size_t csc0, size_t rsc1, \
                                      size_t csc1, const TC *bias, TC *max);
SKL_ORACLE_FUSED_DECL(i8rc_i8rc_i32rc, int8_t, int32_t)
SKL_ORACLE_FUSED_DECL(bf16rc_bf16rc_f32rc, uint16_t, float)
SKL_ORACLE_FUSED_DECL(f16rc_f16rc_f32rc, uint16_t, float)
SKL_ORACLE_FUSED_DECL(f8e4m3rc_f8e4m3rc_f32rc, uint8_t, float)
SKL_ORACLE_FUSED_DECL(f8e5m2rc_f8e5m2rc_f32rc, uint8_t, float)
SKL_ORACLE_PFUSED_DECL(i8rcprc_i8rcprc_i32rcprc, int8_t, int32_t)
SKL_ORACLE_PFUSED_DECL(bf16rcprc_bf16rcprc_f32rcprc, uint16_t, float)
SKL_ORACLE_PFUSED_DECL(f16rcprc_f16rcprc_f32rcprc, uint16_t, float)
SKL_ORACLE_PFUSED_DECL(f8e4m3rcprc_f8e4m3rcprc_f32rcprc, uint8_t, float)
SKL_ORACLE_PFUSED_DECL(f8e5m2rcprc_f8e5m2rcprc_f32rcprc, uint8_t, float)

/* Activation and requantised int8 copy over an m x n strided C that holds the alpha/beta (+ bias) result: the
 * steps between bias and maximum of skl_gfx950_epilogue_t (include/skl-gfx950.h). The reference has no routine
 * for them (src/gemm/README.md:46-47 leaves them to callers); tests/test_oracle_gemm.py pins these against
 * hand-worked values and an independent numpy formulation. q may be NULL. */
float skl_oracle_silu_f32(float x); /* ref/sigmoid/sigmoid_f32.c:36-38 for one value */
float skl_oracle_gelu_f32(float x); /* ref/gelu/gelu_f32.c:12-22 for one value */
void skl_oracle_act_requant_i32(size_t m, size_t n, int32_t *c, size_t rsc, size_t csc, int activation, int8_t *q,
                                size_t rsq, size_t csq, const float *q_scale, int per_column, int32_t q_zero);
void skl_oracle_act_requant_f32(size_t m, size_t n, float *c, size_t rsc, size_t csc, int activation, int8_t *q,
                                size_t rsq, size_t csq, const float *q_scale, int per_column, int32_t q_zero);

/* Widening helpers used to build fp64 comparison operands on the host. */
void skl_oracle_widen_bf16_f64(double *dst, const uint16_t *src, size_t n);
void skl_oracle_widen_f16_f64(double *dst, const uint16_t *src, size_t n);
void skl_oracle_widen_f8e4m3_f64(double *dst, const uint8_t *src, size_t n);
void skl_oracle_widen_f8e5m2_f64(double *dst, const uint8_t *src, size_t n);

#ifdef __cplusplus
}
#endif
#endif /* SKL_ORACLE_H */
