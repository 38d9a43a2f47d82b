/*
 * skl_launch.h - internal C-ABI between the C host layer (skl_api.c) and the
 * HIP translation units. The host layer validates arguments, stages host
 * buffers and decides which kernel family serves a call; the functions below
 * compute grids and enqueue kernels on the calling thread's current stream.
 * Every pointer handed to these functions is device-accessible.
 *
 * All launchers return 0 or an error code that has also been recorded for
 * skl_hip_last_error().
 */
#ifndef SKL_LAUNCH_H
#define SKL_LAUNCH_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Element kinds of GEMM operands. */
enum {
  SKL_DT_I8 = 0,
  SKL_DT_BF16 = 1,
  SKL_DT_F16 = 2,
  SKL_DT_F8E4M3 = 3,
  SKL_DT_F8E5M2 = 4,
  SKL_DT_F32 = 5, /* any-stride kernel only */
  SKL_DT_F64 = 6, /* any-stride kernel only */
  SKL_DT_F16H = 7 /* f16 operands with an f16 accumulator and an f16 C; any-stride kernel only */
};

/* alpha or beta in C's type. With a float in `f`, `skip_c_read` shares the 8 bytes: set on beta (by the host
 * layer, unless skl_hip_set_beta_zero_mode asked for the reference's evaluation) it lets a kernel leave C unread
 * when beta is zero - 1: except where alpha * acc is an exact zero, whose sign the old C decides; 2
 * (SKL_C_UNTOUCHED): not even there, the old C counts as +0 (calls that do not write C either - q_only -, so that
 * C need not exist). */
#define SKL_C_UNTOUCHED 2u
typedef union {
  int32_t i;
  float f;
  double d;
  struct {
    float value;
    uint32_t skip_c_read;
  } fz;
} skl_scalar;

/* Further fused steps behind bias (see skl_gfx950_epilogue_t in include/skl-gfx950.h): an activation and a
 * requantised 8-bit copy of the result. All zero / NULL: nothing. */
typedef struct {
  int act;             /* 0 none, 1 max(v, 0) */
  int q_per_column;    /* q_scale holds one factor per logical column, else one in all */
  int q_only;          /* the result goes to q alone, C is not written */
  int32_t q_zero;
  int8_t *q;           /* Q(i, j) at q[i*rsq + j*csq], (i, j) the logical row and column; NULL: no requantised output */
  size_t rsq, csq;
  const float *q_scale;
  int q_fmt;           /* what a byte of q holds: 0 int8 (rounded, zero point, clamped); 1 / 2 OCP E4M3 without / with
                          saturation, 3 / 4 E5M2 likewise (the fp32 -> fp8 conversion of the cvt family on v * scale) */
} skl_requant;

/* The fully general blocked GEMM of the reference (the `rcprc` form): element
 * (I,i ; P,p) of A is at a + I*rsa1 + P*csa1 + i*rsa0 + p*csa0, and likewise
 * for B (rows = k, columns = n) and C. Strides are in elements. */
typedef struct {
  int ta, tb; /* element kind of A and B; C is int32 for SKL_DT_I8, f64 for SKL_DT_F64, f16 for SKL_DT_F16H,
                 else f32. alpha and beta of SKL_DT_F16H travel widened in `.f` */
  size_t m0, n0, k0, m1, n1, k1;
  const void *a;
  size_t rsa0, csa0, rsa1, csa1;
  const void *b;
  size_t rsb0, csb0, rsb1, csb1;
  void *c;
  size_t rsc0, csc0, rsc1, csc1;
  skl_scalar alpha, beta;
  /* Fused epilogue (both may be NULL): bias[j] of C's type is added to every element of logical column j after
   * the alpha/beta step; *max of C's type is raised to the largest element written. */
  const void *bias;
  void *max;
  skl_requant rq;
} skl_gemm_desc;

/* Canonical form served by the matrix-core kernels: flat in K, blocked by 64
 * in M and N. A(i,p) = a[(i/64)*a_s1 + (i%64)*a_s0 + p*a_sk] with exactly one of
 * a_s0 / a_sk equal to 1; B(p,j) = b[(j/64)*b_s1 + (j%64)*b_s0 + p*b_sk]
 * likewise; C(i,j) = c[(i/R)*rsc1 + (i%R)*rsc0 + (j/S)*csc1 + (j%S)*csc0] with
 * R = 1 << c_row_shift, S = 1 << c_col_shift: 64 x 64 blocks (shift 6) unless C
 * comes in smaller power-of-two blocks (rows: at least 4), which only the
 * matrix-core kernels address. */
typedef struct {
  int ta, tb;
  size_t m, n, k;
  const void *a;
  size_t a_s1, a_s0, a_sk;
  const void *b;
  size_t b_s1, b_s0, b_sk;
  void *c;
  size_t rsc0, csc0, rsc1, csc1;
  unsigned c_row_shift, c_col_shift;
  skl_scalar alpha, beta;
  const void *bias; /* as in skl_gemm_desc */
  void *max;
  skl_requant rq;
} skl_gemm_canon;

int skl_hip_launch_gemm_generic(const skl_gemm_desc *d);
/* Register-tiled kernel for f32, f64 and f16 -> f16 (bit-identical to the any-stride kernel); any strides of the
 * canonical form, no fused steps. */
int skl_hip_gemm_tiled_supported(const skl_gemm_canon *g);
int skl_hip_launch_gemm_tiled(const skl_gemm_canon *g);
/* Returns 1 if the canonical problem meets the matrix-core kernels' alignment
 * rules (16-byte aligned bases and strides along the non-unit dimensions). */
int skl_hip_gemm_mfma_supported(const skl_gemm_canon *g);
int skl_hip_launch_gemm_mfma(const skl_gemm_canon *g);

/* The streaming kernel on copies of A and B padded to whole tiles (see skl_gemm_mfma.hip): the plan returns the tile
 * width (256 / 128) and the padded extents when that pays, else 0; the launch takes the canonical description of the
 * copies (K contiguous, rows *kp apart, k == *kp) with the true m, n and C. */
int skl_hip_gemm_mfma_padded_plan(const skl_gemm_canon *g, size_t *mp, size_t *np, size_t *kp);
/* C = beta*C + alpha*P and the fused steps of g, P a row-major m x n int32 matrix (int8 problems only). */
int skl_hip_launch_gemm_epilogue(const skl_gemm_canon *g, const void *product);
/* The same with the product in the current stream's block of sums (skl_hip_zeroed_sums): every element is put back
 * to zero once it has been read. */
int skl_hip_launch_gemm_epilogue_zeroing(const skl_gemm_canon *g, void *product);
/* The first `bytes` of the current stream's block of sums (zero between calls), or NULL when it is smaller or missing:
 * a matrix that a decode-batch kernel can add into with beta == 1, without a kernel in front that clears it. */
void *skl_hip_zeroed_sums(size_t bytes);
/* 1 when the streaming kernel would take this int8 problem where it lies and write its blocked C (4 to 16 columns
 * per block, contiguous rows) 16 bytes per lane - as cheaply as a row-major C. */
int skl_hip_gemm_mfma_streams_c_quads(const skl_gemm_canon *g);
int skl_hip_launch_gemm_mfma_padded(const skl_gemm_canon *g, int tile_cols);

/* M == 1 streaming kernels: y[j*csc] = beta*y + alpha * sum_p x[p*x_sk] * B(p,j).
 * `layout`: 0 = B row-major (b_s0 == 1 within 64-blocks), 1 = K4-interleaved
 * int8 (`p4x1c`: B(p,j) at (p/4)*b_sk + j*4 + p%4). The launcher applies g's fused steps (bias, max, rq), if any,
 * in the kernel's last stage. */
int skl_hip_gemv_supported(const skl_gemm_canon *g, int layout);
int skl_hip_launch_gemv(const skl_gemm_canon *g, int layout);
/* 2 <= M <= 8 rows against a row-major int8 B: the same stream over B with the transposes shared by the rows. */
int skl_hip_gemv_rows_supported(const skl_gemm_canon *g);
int skl_hip_launch_gemv_rows(const skl_gemm_canon *g);
/* 4 <= M <= 16 rows against a row-major int8 B, 2 <= M <= 16 against an fp8 / bf16 / f16 one: the same stream with
 * the multiply-adds on the matrix cores (floating point: with the fused steps, if any). `layout` as for the M == 1
 * kernels: 1 = K4-interleaved int8 B, 2 <= M <= 16. */
int skl_hip_gemv_mfma_rows_supported(const skl_gemm_canon *g, int layout);
int skl_hip_launch_gemv_mfma_rows(const skl_gemm_canon *g, int layout);
/* 1 <= M <= 4 against a B with K contiguous (b_sk == 1): one dot product over contiguous memory per output; the
 * launcher applies g's fused steps, if any, where the outputs are written. */
int skl_hip_gemv_kc_supported(const skl_gemm_canon *g);
int skl_hip_launch_gemv_kc(const skl_gemm_canon *g);
/* 5 to 96 rows of A against a B with K contiguous, int8 and the fp8 kinds: one workgroup per 64 columns takes 4096 k
 * (a longer K: a launch per 4096 k) on the matrix cores and applies the fused steps itself (skl_gemv_kcrows.hip). No scratch memory. */
int skl_hip_gemv_kc_rows_supported(const skl_gemm_canon *g);
int skl_hip_launch_gemv_kc_rows(const skl_gemm_canon *g);

/* int8 decode calls (1 <= M <= 8, row-major B) on the M == 1 / few-rows kernels with a static device array as the
 * shared sums: no allocation, at most skl_hip_noalloc_max_sums() elements of C. skl_hip_noalloc_setup() looks the
 * array's address on the current device up (once per device; the launch does it itself where it was not called). */
int skl_hip_noalloc_setup(void);
size_t skl_hip_noalloc_max_sums(void);
int skl_hip_launch_gemv_noalloc(const skl_gemm_canon *g);
/* E4M3 A (1 to 16 rows, K contiguous) times OFP4 B (columns contiguous in K, two values per byte, `ldb` elements
 * apart): skl_gemv_f4.hip. */
int skl_hip_gemv_f4_supported(size_t m, size_t n, size_t k, const void *a, size_t rsa, size_t csa, const void *b, size_t ldb);
int skl_hip_launch_gemv_f4(size_t m, size_t n, size_t k, skl_scalar alpha, const void *a, size_t rsa, size_t csa, const void *b,
                           size_t ldb, const uint8_t *scales, size_t lds, skl_scalar beta, float *c, size_t rsc, size_t csc);
/* dst[j * ldb + p] (bf16) = E2M1 value number j * ldb + p of src times 2^(scales[j * lds + p / 32] - 127), for p < k, j < n. */
int skl_hip_launch_cvt_mxf4_bf16(uint16_t *dst, const uint8_t *src, const uint8_t *scales, size_t lds, size_t n, size_t k, size_t ldb);
/* Makes sure the current stream has the sums-and-counters block of the single-row kernels; 0 or SKL_HIP_ERR_WORKSPACE. */
int skl_hip_gemv_reserve_scratch(void);

/* A block of scratch memory of the current stream and device for operands copied into another layout ahead of a
 * launch (grows on demand, NULL when the device has no room; apart from the workspace of the split reductions). */
void *skl_hip_operand_scratch(size_t bytes);
/* A third block, for an operand converted to another element type ahead of a GEMM that may copy operands itself
 * (into the block above). NULL, with the error recorded, when there is no room. */
void *skl_hip_converted_scratch(size_t bytes);
/* Brackets a sequence of launches that hands data from one kernel to the next through the stream's scratch memory
 * (operand copies, partial sums), so that sequences of different host threads do not interleave on a stream.
 * Recursive. */
void skl_hip_sequence_begin(void);
void skl_hip_sequence_end(void);
/* Copies a GEMM operand in the reference's blocked description (element (x, p), x along M or N and p along K, at
 * (x/x0)*s1 + (x%x0)*s0 + (p/k0)*sk1 + (p%k0)*sk0; `esize` 1 or 2 bytes) into rows contiguous in K:
 * dst[x*kp + p], zero-filled for k <= p < kp. */
int skl_hip_launch_realign(int esize, size_t x, size_t k, const void *src, size_t x0, size_t s0, size_t s1, size_t k0,
                           size_t sk0, size_t sk1, void *dst, size_t kp);

/* pack / unpack over elements of `esize` bytes (1, 2 or 4). */
int skl_hip_launch_pack(int esize, size_t m, size_t n, const void *src, size_t rs, size_t cs,
                        size_t m0, size_t n0, void *dst, size_t rs0, size_t cs0, size_t rs1,
                        size_t cs1, uint32_t pad);
int skl_hip_launch_unpack(int esize, size_t m0, size_t n0, const void *src, size_t rs0,
                          size_t cs0, size_t rs1, size_t cs1, size_t m, size_t n, void *dst,
                          size_t rs, size_t cs);

/* OFP8 / OFP4 conversions. `fmt`: SKL_DT_F8E4M3 or SKL_DT_F8E5M2. */
int skl_hip_launch_cvt_f32_f8(int fmt, int saturate, uint8_t *dst, const float *src, float scale,
                              size_t n);
int skl_hip_launch_cvt_bf16_f8(int fmt, int saturate, uint8_t *dst, const uint16_t *src,
                               float scale, size_t n);
int skl_hip_launch_cvt_f8_bf16(int fmt, uint16_t *dst, const uint8_t *src, size_t n);
int skl_hip_launch_cvt_f4_f8e4m3(uint8_t *dst, const uint8_t *src, size_t n);

/* Error recording shared by both layers. */
void skl_hip_record_error(int code, const char *what);
/* Forgets the calling thread's recorded error if it is `code` (a failure that a later step of the same call made good). */
void skl_hip_withdraw_error(int code);
/* The calling thread's recorded error, left in place (skl_hip_last_error() reads and clears it). */
int skl_hip_pending_error(void);

#ifdef __cplusplus
}
#endif
#endif /* SKL_LAUNCH_H */
