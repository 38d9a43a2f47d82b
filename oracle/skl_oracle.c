/*
 * skl_oracle.c - CPU restatement of the SKL scalar reference semantics
 * (gemm, pack, cvt). TEST INFRASTRUCTURE ONLY: see skl_oracle.h.
 *
 * Citations are paths below the reference checkout. Build with
 * -fwrapv -ffp-contract=off so integer wrap and the two-rounding epilogue are
 * the ones the reference's C source denotes.
 */
#include "skl_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ======================================================================== */
/* Scalar conversions                                                        */
/* ======================================================================== */

static float bits_to_f32(uint32_t u) {
  float f;
  memcpy(&f, &u, sizeof f);
  return f;
}

static uint32_t f32_to_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, sizeof u);
  return u;
}

#define QNAN_BITS 0x7FC00000u /* sign-less quiet NaN the reference returns */

/*
 * Generic "small float byte -> f32" decode for a format with `mbits` mantissa
 * bits and exponent bias `bias`. Value = (-1)^s * 2^(e-bias) * (1 + m/2^mbits)
 * for e > 0 and (-1)^s * 2^(1-bias) * m/2^mbits for e == 0; every such value is
 * exactly representable in f32, so ldexpf() is exact. Special codes are
 * resolved by the callers.
 */
static float decode_small(uint32_t sign, uint32_t e, uint32_t m, int mbits, int bias) {
  float mag;
  if (e == 0) {
    mag = ldexpf((float)m, 1 - bias - mbits);
  } else {
    mag = ldexpf((float)((1u << mbits) | m), (int)e - bias - mbits);
  }
  return sign ? -mag : mag;
}

/* ref/cvt/cvt_ofp8.c:18-52 - E4M3: bias 7, no infinities, S.1111.111 is NaN
 * and decodes to the sign-less quiet NaN. */
float skl_oracle_f8e4m3_to_f32(uint8_t code) {
  uint32_t s = code >> 7, e = (code >> 3) & 0xFu, m = code & 0x7u;
  if (e == 0xFu && m == 0x7u) return bits_to_f32(QNAN_BITS);
  return decode_small(s, e, m, 3, 7);
}

/* ref/cvt/cvt_ofp8.c:54-95 - E5M2: bias 15, exponent 31 is inf (m == 0, signed)
 * or NaN (sign-less quiet NaN). */
float skl_oracle_f8e5m2_to_f32(uint8_t code) {
  uint32_t s = code >> 7, e = (code >> 2) & 0x1Fu, m = code & 0x3u;
  if (e == 0x1Fu) {
    if (m == 0) return bits_to_f32((s << 31) | 0x7F800000u);
    return bits_to_f32(QNAN_BITS);
  }
  return decode_small(s, e, m, 2, 15);
}

/* ref/cvt/cvt_ofp4.c:18-48 - E2M1 nibble: bias 1, no specials. Only the low
 * four bits of the argument are meaningful. */
float skl_oracle_f4e2m1_to_f32(uint8_t nibble) {
  uint32_t s = (nibble >> 3) & 1u, e = (nibble >> 1) & 0x3u, m = nibble & 1u;
  return decode_small(s, e, m, 1, 1);
}

/*
 * f32 -> OFP8 encode, the procedure of ref/cvt/cvt_ofp8.c:97-134 (E4M3) and
 * :136-172 (E5M2):
 *   - infinities give the "overflow" byte, NaN gives 0x7F;
 *   - E = floor(log2 |x|);
 *   - E below the minimum normal exponent: the byte is sign | rne(|x| * 2^(mbits - emin));
 *   - E above the largest exponent: overflow byte;
 *   - otherwise q = rne((|x| * 2^-E - 1) * 2^mbits) is ADDED to (E + bias) << mbits,
 *     so a mantissa carry moves into the exponent field; a magnitude above
 *     the largest finite code is an overflow.
 * All scalings are by powers of two and therefore exact; rne() is
 * nearbyintf() in the default rounding mode, as in the reference.
 * frexpf() yields the exact floor(log2 |x|); zero (where the reference's
 * log2f gives -inf and ends in the subnormal branch) is routed there too.
 */
static uint8_t encode_small(float x, int mbits, int bias, int emin, int emax,
                            uint8_t max_code, uint8_t overflow_code) {
  uint32_t xb = f32_to_bits(x);
  uint8_t sign = (xb & 0x80000000u) ? 0x80 : 0x00;
  float ax = fabsf(x);
  int E;
  unsigned mag;
  if (isinf(x)) return overflow_code;
  if (isnan(x)) return 0x7F;
  if (ax == 0.0f) return sign;
  (void)frexpf(ax, &E);
  E -= 1; /* ax = f * 2^(E+1) with f in [0.5, 1)  =>  floor(log2 ax) = E */
  if (E < emin) {
    float q = nearbyintf(ldexpf(ax, mbits - emin));
    return (uint8_t)(sign | (uint8_t)q);
  }
  if (E > emax) return overflow_code;
  {
    float frac = ldexpf(ax, -E) - 1.0f;
    float q = nearbyintf(ldexpf(frac, mbits));
    mag = ((unsigned)(E + bias) << mbits) + (unsigned)q;
  }
  if (mag > max_code) return overflow_code;
  return (uint8_t)(sign | mag);
}

/* ref/cvt/cvt_ofp8.c:97-134. Overflow byte: saturating -> sign | 0x7E (448);
 * non-saturating -> 0x7F with the sign dropped. */
uint8_t skl_oracle_f32_to_f8e4m3(float x, int saturate) {
  uint8_t sign = (f32_to_bits(x) & 0x80000000u) ? 0x80 : 0x00;
  uint8_t ovf = saturate ? (uint8_t)(sign | 0x7E) : (uint8_t)0x7F;
  return encode_small(x, 3, 7, -6, 8, 0x7E, ovf);
}

/* ref/cvt/cvt_ofp8.c:136-172. Overflow byte: saturating -> sign | 0x7B (57344);
 * non-saturating -> sign | 0x7C (infinity). */
uint8_t skl_oracle_f32_to_f8e5m2(float x, int saturate) {
  uint8_t sign = (f32_to_bits(x) & 0x80000000u) ? 0x80 : 0x00;
  uint8_t ovf = (uint8_t)(sign | (saturate ? 0x7B : 0x7C));
  return encode_small(x, 2, 15, -14, 15, 0x7B, ovf);
}

/* bf16 is the upper half of an f32: widening is exact. */
float skl_oracle_bf16_to_f32(uint16_t bits) { return bits_to_f32((uint32_t)bits << 16); }

/* IEEE binary16 -> f32, exact. */
float skl_oracle_f16_to_f32(uint16_t h) {
  uint32_t s = (uint32_t)(h >> 15) << 31;
  uint32_t e = (h >> 10) & 0x1Fu, m = h & 0x3FFu;
  if (e == 0x1Fu) return bits_to_f32(s | 0x7F800000u | (m << 13));
  if (e == 0) {
    float mag = ldexpf((float)m, -24);
    return s ? -mag : mag;
  }
  return bits_to_f32(s | ((e + 112u) << 23) | (m << 13));
}

/* f32 -> f16, round to nearest even, as the conversion `(_Float16)x` rounds: overflow goes to infinity,
 * results below the smallest normal are subnormal halves, NaN keeps its sign and the top payload bits. */
uint16_t skl_oracle_f32_to_f16(float x) {
  const uint32_t u = f32_to_bits(x);
  const uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
  const uint32_t mag = u & 0x7FFFFFFFu;
  if (mag > 0x7F800000u) return (uint16_t)(sign | 0x7E00u | ((mag >> 13) & 0x3FFu)); /* NaN, made quiet */
  if (mag >= 0x47800000u) return (uint16_t)(sign | 0x7C00u);                         /* >= 65536, incl. infinity */
  if (mag < 0x33000000u) return sign;                                                /* < 2^-25: to zero */
  {
    const int32_t e = (int32_t)(mag >> 23) - 127; /* unbiased exponent, -25 .. 15 */
    const uint32_t sig = (mag & 0x7FFFFFu) | 0x800000u; /* 24-bit significand, value sig * 2^(e-23) */
    /* target unit: 2^(e-10) for a normal half (e >= -14), 2^-24 for a subnormal */
    const int shift = e >= -14 ? 13 : (-24) - (e - 23); /* bits dropped from sig */
    const uint32_t kept = sig >> shift, rest = sig & ((1u << shift) - 1u), half = 1u << (shift - 1);
    uint32_t q = kept + ((rest > half || (rest == half && (kept & 1u))) ? 1u : 0u);
    if (e >= -14) { /* q in [2^10, 2^11]; a carry to 2^11 bumps the exponent through the addition */
      const uint32_t h = ((uint32_t)(e + 15) << 10) + (q - 0x400u);
      return (uint16_t)(sign | (h >= 0x7C00u ? 0x7C00u : h));
    }
    return (uint16_t)(sign | q); /* q <= 2^10: 2^10 is the smallest normal, encoded by the same bits */
  }
}

/* f32 -> bf16, round to nearest even; NaN becomes the quiet NaN with the
 * payload truncated (the C cast `(__bf16)x` the reference uses at
 * ref/cvt/cvt_ofp8.c:233,240). */
uint16_t skl_oracle_f32_to_bf16(float x) {
  uint32_t u = f32_to_bits(x);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x0040u);
  u += 0x7FFFu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

/* ======================================================================== */
/* Array conversions                                                         */
/* ======================================================================== */

/* ref/cvt/cvt_ofp8.c:174-200 - one fp32 multiply by the scale, then encode. */
#define CVT_FROM_F32(NAME, ENC, SAT)                                                  \
  void NAME(uint8_t *dst, const float *src, float scale, size_t n) {                  \
    for (size_t i = 0; i < n; ++i) {                                                  \
      volatile float scaled = src[i] * scale;                                         \
      dst[i] = ENC(scaled, SAT);                                                      \
    }                                                                                 \
  }
CVT_FROM_F32(skl_cvt_f32_f8e4m3_oracle, skl_oracle_f32_to_f8e4m3, 0)
CVT_FROM_F32(skl_cvt_sat_f32_f8e4m3_oracle, skl_oracle_f32_to_f8e4m3, 1)
CVT_FROM_F32(skl_cvt_f32_f8e5m2_oracle, skl_oracle_f32_to_f8e5m2, 0)
CVT_FROM_F32(skl_cvt_sat_f32_f8e5m2_oracle, skl_oracle_f32_to_f8e5m2, 1)

/* ref/cvt/cvt_ofp8.c:202-228 - widen bf16 exactly, multiply in fp32, encode. */
#define CVT_FROM_BF16(NAME, ENC, SAT)                                                 \
  void NAME(uint8_t *dst, const uint16_t *src, float scale, size_t n) {               \
    for (size_t i = 0; i < n; ++i) {                                                  \
      volatile float scaled = skl_oracle_bf16_to_f32(src[i]) * scale;                 \
      dst[i] = ENC(scaled, SAT);                                                      \
    }                                                                                 \
  }
CVT_FROM_BF16(skl_cvt_bf16_f8e4m3_oracle, skl_oracle_f32_to_f8e4m3, 0)
CVT_FROM_BF16(skl_cvt_sat_bf16_f8e4m3_oracle, skl_oracle_f32_to_f8e4m3, 1)
CVT_FROM_BF16(skl_cvt_bf16_f8e5m2_oracle, skl_oracle_f32_to_f8e5m2, 0)
CVT_FROM_BF16(skl_cvt_sat_bf16_f8e5m2_oracle, skl_oracle_f32_to_f8e5m2, 1)

/* ref/cvt/cvt_ofp8.c:230-242 - decode then narrow to bf16 (always exact). */
void skl_cvt_f8e4m3_bf16_oracle(uint16_t *dst, const uint8_t *src, size_t n) {
  for (size_t i = 0; i < n; ++i) dst[i] = skl_oracle_f32_to_bf16(skl_oracle_f8e4m3_to_f32(src[i]));
}
void skl_cvt_f8e5m2_bf16_oracle(uint16_t *dst, const uint8_t *src, size_t n) {
  for (size_t i = 0; i < n; ++i) dst[i] = skl_oracle_f32_to_bf16(skl_oracle_f8e5m2_to_f32(src[i]));
}

/* ref/cvt/cvt_ofp4.c:50-68 - two E2M1 values per source byte, low nibble
 * first; each is widened to f32 and encoded to E4M3 without saturation. With
 * an odd count the last source byte contributes its low nibble only. */
void skl_cvt_f4e2m1_f8e4m3_oracle(uint8_t *dst, const uint8_t *src, size_t n) {
  for (size_t i = 0; i < n; ++i) {
    uint8_t byte = src[i >> 1];
    uint8_t nib = (i & 1u) ? (uint8_t)(byte >> 4) : (uint8_t)(byte & 0xFu);
    dst[i] = skl_oracle_f32_to_f8e4m3(skl_oracle_f4e2m1_to_f32(nib), 0);
  }
}

/* ======================================================================== */
/* Pack / unpack / transpose                                                 */
/* ======================================================================== */

/*
 * pack:   ref/pack/pack_e8rc_e8rcprc.c:10-35 (e16, e32 twins identical).
 *         Block (I,J) of size m0 x n0 goes to dst + I*rs1 + J*cs1; inside a
 *         block element (i,j) sits at i*rs0 + j*cs0. Positions whose source
 *         coordinate falls outside m x n receive `pad`.
 * unpack: ref/pack/unpack_e8rcprc_e8rc.c:10-37. Inverse gather; only in-range
 *         destination elements are written; m0 == 0 or n0 == 0 is a no-op.
 *         The reference ships the 8-bit width only; the wider widths apply the
 *         same rule to wider elements.
 * transpose: ref/pack/transpose_e8.c:11-19. at[j*rsat + i] = a[i*rsa + j].
 */
#define PACK_FAMILY(W, T)                                                               \
  void skl_pack_e##W##rc_e##W##rcprc_oracle(size_t m, size_t n, const T *src,          \
                                            size_t rs, size_t cs, size_t m0, size_t n0, \
                                            T *dst, size_t rs0, size_t cs0, size_t rs1, \
                                            size_t cs1, T pad) {                        \
    size_t nbr = (m + m0 - 1) / m0, nbc = (n + n0 - 1) / n0;                            \
    for (size_t I = 0; I < nbr; ++I)                                                    \
      for (size_t J = 0; J < nbc; ++J)                                                  \
        for (size_t i = 0; i < m0; ++i)                                                 \
          for (size_t j = 0; j < n0; ++j) {                                             \
            size_t r = I * m0 + i, c = J * n0 + j;                                      \
            T v = (r < m && c < n) ? src[r * rs + c * cs] : pad;                        \
            dst[I * rs1 + J * cs1 + i * rs0 + j * cs0] = v;                             \
          }                                                                             \
  }                                                                                     \
  void skl_unpack_e##W##rcprc_e##W##rc_oracle(size_t m0, size_t n0, const T *src,      \
                                              size_t rs0, size_t cs0, size_t rs1,       \
                                              size_t cs1, size_t m, size_t n, T *dst,   \
                                              size_t rs, size_t cs) {                   \
    if (m0 == 0 || n0 == 0) return;                                                     \
    for (size_t r = 0; r < m; ++r)                                                      \
      for (size_t c = 0; c < n; ++c) {                                                  \
        size_t I = r / m0, i = r % m0, J = c / n0, j = c % n0;                          \
        dst[r * rs + c * cs] = src[I * rs1 + J * cs1 + i * rs0 + j * cs0];              \
      }                                                                                 \
  }                                                                                     \
  void skl_transpose_e##W##_oracle(size_t m, size_t n, const T *a, size_t rsa, T *at,  \
                                   size_t rsat) {                                       \
    for (size_t j = 0; j < n; ++j)                                                      \
      for (size_t i = 0; i < m; ++i) at[j * rsat + i] = a[i * rsa + j];                 \
  }
PACK_FAMILY(8, uint8_t)
PACK_FAMILY(16, uint16_t)
PACK_FAMILY(32, uint32_t)

/* ======================================================================== */
/* GEMM                                                                      */
/* ======================================================================== */

#define LOAD_ID(x) (x)

/*
 * Strided GEMM. ref/gemm/gemm_i8rc_i8rc_i32rc.c:10-26 and its typed twins
 * (bf16 :9-24, f16 :9-24, f8e4m3 :11-25, f8e5m2 :11-25, f32 :9-24, f64 :9-24):
 * accumulator of C's type starts at zero, k ascending, each product formed from
 * the widened operands, then C = beta*C + alpha*acc with C always read.
 */
#define GEMM_RC(NAME, TA, TB, TC, WA, WB)                                              \
  void skl_gemm_##NAME##_oracle(size_t m, size_t n, size_t k, TC alpha, const TA *a,   \
                                size_t rsa, size_t csa, const TB *b, size_t rsb,        \
                                size_t csb, TC beta, TC *c, size_t rsc, size_t csc) {   \
    for (size_t i = 0; i < m; ++i)                                                      \
      for (size_t j = 0; j < n; ++j) {                                                  \
        TC acc = 0;                                                                     \
        for (size_t p = 0; p < k; ++p)                                                  \
          acc += (TC)WA(a[i * rsa + p * csa]) * (TC)WB(b[p * rsb + j * csb]);           \
        TC *out = c + i * rsc + j * csc;                                                \
        *out = beta * *out + alpha * acc;                                               \
      }                                                                                 \
  }

/*
 * Blocked ("packed") GEMM. ref/gemm/gemm_i8rcprc_i8rcprc_i32rcprc.c:10-37 and
 * twins: element (I,i ; P,p) of A is at I*rsa1 + P*csa1 + i*rsa0 + p*csa0
 * (likewise B and C); for each C element the sum runs over P outer, p inner.
 */
#define GEMM_RCPRC(NAME, TA, TB, TC, WA, WB)                                           \
  void skl_gemm_##NAME##_oracle(size_t m0, size_t n0, size_t k0, size_t m1, size_t n1, \
                                size_t k1, TC alpha, const TA *a, size_t rsa0,          \
                                size_t csa0, size_t rsa1, size_t csa1, const TB *b,     \
                                size_t rsb0, size_t csb0, size_t rsb1, size_t csb1,     \
                                TC beta, TC *c, size_t rsc0, size_t csc0, size_t rsc1,  \
                                size_t csc1) {                                          \
    for (size_t I = 0; I < m1; ++I)                                                     \
      for (size_t J = 0; J < n1; ++J)                                                   \
        for (size_t i = 0; i < m0; ++i)                                                 \
          for (size_t j = 0; j < n0; ++j) {                                             \
            TC acc = 0;                                                                 \
            for (size_t P = 0; P < k1; ++P)                                             \
              for (size_t p = 0; p < k0; ++p) {                                         \
                TA av = a[I * rsa1 + P * csa1 + i * rsa0 + p * csa0];                   \
                TB bv = b[P * rsb1 + J * csb1 + p * rsb0 + j * csb0];                   \
                acc += (TC)WA(av) * (TC)WB(bv);                                         \
              }                                                                         \
            TC *out = c + I * rsc1 + J * csc1 + i * rsc0 + j * csc0;                    \
            *out = beta * *out + alpha * acc;                                           \
          }                                                                             \
  }

GEMM_RC(i8rc_i8rc_i32rc, int8_t, int8_t, int32_t, LOAD_ID, LOAD_ID)
GEMM_RC(bf16rc_bf16rc_f32rc, uint16_t, uint16_t, float, skl_oracle_bf16_to_f32,
        skl_oracle_bf16_to_f32)
GEMM_RC(f16rc_f16rc_f32rc, uint16_t, uint16_t, float, skl_oracle_f16_to_f32,
        skl_oracle_f16_to_f32)
GEMM_RC(f8e4m3rc_f8e4m3rc_f32rc, uint8_t, uint8_t, float, skl_oracle_f8e4m3_to_f32,
        skl_oracle_f8e4m3_to_f32)
GEMM_RC(f8e5m2rc_f8e5m2rc_f32rc, uint8_t, uint8_t, float, skl_oracle_f8e5m2_to_f32,
        skl_oracle_f8e5m2_to_f32)
/* No mixed-format routine exists in the reference. This one applies the E4M3
 * decode to A and the E5M2 decode to B inside the same loop nest, which is the
 * arithmetic of decoding both and calling ref/gemm/gemm_f32rc_f32rc_f32rc.c:9-24. */
GEMM_RC(f8e4m3rc_f8e5m2rc_f32rc, uint8_t, uint8_t, float, skl_oracle_f8e4m3_to_f32,
        skl_oracle_f8e5m2_to_f32)
GEMM_RC(f32rc_f32rc_f32rc, float, float, float, LOAD_ID, LOAD_ID)
GEMM_RC(f64rc_f64rc_f64rc, double, double, double, LOAD_ID, LOAD_ID)

GEMM_RCPRC(i8rcprc_i8rcprc_i32rcprc, int8_t, int8_t, int32_t, LOAD_ID, LOAD_ID)
GEMM_RCPRC(bf16rcprc_bf16rcprc_f32rcprc, uint16_t, uint16_t, float, skl_oracle_bf16_to_f32,
           skl_oracle_bf16_to_f32)
GEMM_RCPRC(f16rcprc_f16rcprc_f32rcprc, uint16_t, uint16_t, float, skl_oracle_f16_to_f32,
           skl_oracle_f16_to_f32)
/* No GEMM over 4-bit operands exists in the reference: its users convert OFP4 weights with skl_cvt_f4e2m1_f8e4m3
 * (ref/cvt/cvt_ofp4.c:59-68) and call the fp8 GEMM (ref/gemm/gemm_f8e4m3rc_f8e4m3rc_f32rc.c). This is that
 * composition, for a B stored column by column: 4-bit value number j * ldb + p of `b` is B(p, j). */
void skl_gemm_f8e4m3rc_f4e2m1c_f32rc_oracle(size_t m, size_t n, size_t k, float alpha, const uint8_t *a, size_t rsa,
                                            size_t csa, const uint8_t *b, size_t ldb, float beta, float *c, size_t rsc,
                                            size_t csc) {
  const size_t values = (n && k) ? (n - 1) * ldb + k : 0;
  uint8_t *b8 = (uint8_t *)malloc(values ? values : 1);
  skl_cvt_f4e2m1_f8e4m3_oracle(b8, b, values);
  skl_gemm_f8e4m3rc_f8e4m3rc_f32rc_oracle(m, n, k, alpha, a, rsa, csa, b8, 1, ldb, beta, c, rsc, csc);
  free(b8);
}

/* OCP microscaling on top: every 32 consecutive k of a column share the scale 2^(s - 127), s = scales[j * lds + p / 32].
 * Nothing in the reference knows block scales; the definition is the reference's fp32 GEMM
 * (ref/gemm/gemm_f32rc_f32rc_f32rc.c:9-24: acc += a * b in float, k ascending, then beta * c + alpha * acc) on the
 * decoded operands - A by ref/cvt/cvt_ofp8.c:18-52, B's E2M1 values (ref/cvt/cvt_ofp4.c:18-48) times their scales,
 * exact in float. scales == NULL: every scale is 1. */
void skl_gemm_f8e4m3rc_mxf4e2m1c_f32rc_oracle(size_t m, size_t n, size_t k, float alpha, const uint8_t *a, size_t rsa,
                                              size_t csa, const uint8_t *b, size_t ldb, const uint8_t *scales, size_t lds,
                                              float beta, float *c, size_t rsc, size_t csc) {
  for (size_t i = 0; i < m; ++i)
    for (size_t j = 0; j < n; ++j) {
      float acc = 0.0f;
      for (size_t p = 0; p < k; ++p) {
        const size_t at = j * ldb + p;
        const uint8_t nib = (at & 1u) ? (uint8_t)(b[at >> 1] >> 4) : (uint8_t)(b[at >> 1] & 0xFu);
        const float w = skl_oracle_f4e2m1_to_f32(nib) * (scales ? ldexpf(1.0f, (int)scales[j * lds + p / 32] - 127) : 1.0f);
        acc += skl_oracle_f8e4m3_to_f32(a[i * rsa + p * csa]) * w;
      }
      c[i * rsc + j * csc] = beta * c[i * rsc + j * csc] + alpha * acc;
    }
}

GEMM_RCPRC(f8e4m3rcprc_f8e4m3rcprc_f32rcprc, uint8_t, uint8_t, float,
           skl_oracle_f8e4m3_to_f32, skl_oracle_f8e4m3_to_f32)
GEMM_RCPRC(f8e5m2rcprc_f8e5m2rcprc_f32rcprc, uint8_t, uint8_t, float,
           skl_oracle_f8e5m2_to_f32, skl_oracle_f8e5m2_to_f32)
/* ref/gemm/gemm_f32rcprc_f32rcprc_f32rcprc.c:9-36 */
GEMM_RCPRC(f32rcprc_f32rcprc_f32rcprc, float, float, float, LOAD_ID, LOAD_ID)
GEMM_RCPRC(f64rcprc_f64rcprc_f64rcprc, double, double, double, LOAD_ID, LOAD_ID)

/*
 * f16 operands, f16 accumulator, f16 C: ref/gemm/gemm_f16rc_f16rc_f16rc.c:9-24 and
 * ref/gemm/gemm_f16rcprc_f16rcprc_f16rcprc.c. The reference writes `_Float16 acc; acc += a * b;` and
 * `c = beta * c + alpha * acc`. A C compiler for a target without half arithmetic evaluates `_Float16`
 * expressions in float and rounds to half where the value is assigned, so
 *   acc = half(float(acc) + a*b)            the product of two halves is exact in float
 *   c   = half(float(beta*c + alpha*acc))   both products exact, the sum rounded to float, then to half.
 * alpha and beta arrive as floats holding half values.
 */
static uint16_t f16h_step(uint16_t acc, uint16_t a, uint16_t b) {
  volatile float prod = skl_oracle_f16_to_f32(a) * skl_oracle_f16_to_f32(b);
  volatile float sum = skl_oracle_f16_to_f32(acc) + prod;
  return skl_oracle_f32_to_f16(sum);
}
static uint16_t f16h_finish(uint16_t acc, uint16_t c, float alpha, float beta) {
  volatile float bc = beta * skl_oracle_f16_to_f32(c), aa = alpha * skl_oracle_f16_to_f32(acc);
  volatile float sum = bc + aa;
  return skl_oracle_f32_to_f16(sum);
}
void skl_gemm_f16rc_f16rc_f16rc_oracle(size_t m, size_t n, size_t k, float alpha, const uint16_t *a, size_t rsa,
                                       size_t csa, const uint16_t *b, size_t rsb, size_t csb, float beta,
                                       uint16_t *c, size_t rsc, size_t csc) {
  for (size_t i = 0; i < m; ++i)
    for (size_t j = 0; j < n; ++j) {
      uint16_t acc = 0;
      for (size_t p = 0; p < k; ++p) acc = f16h_step(acc, a[i * rsa + p * csa], b[p * rsb + j * csb]);
      uint16_t *out = c + i * rsc + j * csc;
      *out = f16h_finish(acc, *out, alpha, beta);
    }
}
void skl_gemm_f16rcprc_f16rcprc_f16rcprc_oracle(size_t m0, size_t n0, size_t k0, size_t m1, size_t n1, size_t k1,
                                                float alpha, const uint16_t *a, size_t rsa0, size_t csa0,
                                                size_t rsa1, size_t csa1, const uint16_t *b, size_t rsb0,
                                                size_t csb0, size_t rsb1, size_t csb1, float beta, uint16_t *c,
                                                size_t rsc0, size_t csc0, size_t rsc1, size_t csc1) {
  for (size_t I = 0; I < m1; ++I)
    for (size_t J = 0; J < n1; ++J)
      for (size_t i = 0; i < m0; ++i)
        for (size_t j = 0; j < n0; ++j) {
          uint16_t acc = 0;
          for (size_t P = 0; P < k1; ++P)
            for (size_t p = 0; p < k0; ++p)
              acc = f16h_step(acc, a[I * rsa1 + P * csa1 + i * rsa0 + p * csa0],
                              b[P * rsb1 + J * csb1 + p * rsb0 + j * csb0]);
          uint16_t *out = c + I * rsc1 + J * csc1 + i * rsc0 + j * csc0;
          *out = f16h_finish(acc, *out, alpha, beta);
        }
}

/*
 * GEMM with the fused steps of the reference's per-tile fused kernels behind the alpha/beta step
 * (src/gemm/fused-kernel-API.md:159-178, "adding a bias": c_block[i,j] = tile[i,j] + bias_block[j], the bias
 * indexed by the logical column; :186-207, "computing a global maximum": if (tile[i,j] > *max) *max = tile[i,j],
 * the tile value being what is written to C). Every element is independent, so running the plain GEMM first
 * and the two steps over C afterwards computes what a fused kernel computes.
 */
#define FUSED_RC(NAME, TA, TC)                                                                     \
  void skl_gemm_fused_##NAME##_oracle(size_t m, size_t n, size_t k, TC alpha, const TA *a, size_t rsa, \
                                      size_t csa, const TA *b, size_t rsb, size_t csb, TC beta, TC *c, \
                                      size_t rsc, size_t csc, const TC *bias, TC *max) {            \
    skl_gemm_##NAME##_oracle(m, n, k, alpha, a, rsa, csa, b, rsb, csb, beta, c, rsc, csc);          \
    for (size_t i = 0; i < m; ++i)                                                                  \
      for (size_t j = 0; j < n; ++j) {                                                              \
        TC *out = c + i * rsc + j * csc;                                                            \
        TC v = *out;                                                                                \
        if (bias) v = v + bias[j];                                                                  \
        *out = v;                                                                                   \
        if (max && v > *max) *max = v;                                                              \
      }                                                                                             \
  }
#define FUSED_RCPRC(NAME, TA, TC)                                                                  \
  void skl_gemm_fused_##NAME##_oracle(size_t m0, size_t n0, size_t k0, size_t m1, size_t n1, size_t k1, \
                                      TC alpha, const TA *a, size_t rsa0, size_t csa0, size_t rsa1, \
                                      size_t csa1, const TA *b, size_t rsb0, size_t csb0, size_t rsb1, \
                                      size_t csb1, TC beta, TC *c, size_t rsc0, size_t csc0, size_t rsc1, \
                                      size_t csc1, const TC *bias, TC *max) {                       \
    skl_gemm_##NAME##_oracle(m0, n0, k0, m1, n1, k1, alpha, a, rsa0, csa0, rsa1, csa1, b, rsb0, csb0, rsb1, \
                             csb1, beta, c, rsc0, csc0, rsc1, csc1);                                \
    for (size_t I = 0; I < m1; ++I)                                                                 \
      for (size_t J = 0; J < n1; ++J)                                                               \
        for (size_t i = 0; i < m0; ++i)                                                             \
          for (size_t j = 0; j < n0; ++j) {                                                         \
            TC *out = c + I * rsc1 + J * csc1 + i * rsc0 + j * csc0;                                \
            TC v = *out;                                                                            \
            if (bias) v = v + bias[J * n0 + j];                                                     \
            *out = v;                                                                               \
            if (max && v > *max) *max = v;                                                          \
          }                                                                                         \
  }
FUSED_RC(i8rc_i8rc_i32rc, int8_t, int32_t)
FUSED_RC(bf16rc_bf16rc_f32rc, uint16_t, float)
FUSED_RC(f16rc_f16rc_f32rc, uint16_t, float)
FUSED_RC(f8e4m3rc_f8e4m3rc_f32rc, uint8_t, float)
FUSED_RC(f8e5m2rc_f8e5m2rc_f32rc, uint8_t, float)
FUSED_RCPRC(i8rcprc_i8rcprc_i32rcprc, int8_t, int32_t)
FUSED_RCPRC(bf16rcprc_bf16rcprc_f32rcprc, uint16_t, float)
FUSED_RCPRC(f16rcprc_f16rcprc_f32rcprc, uint16_t, float)
FUSED_RCPRC(f8e4m3rcprc_f8e4m3rcprc_f32rcprc, uint8_t, float)
FUSED_RCPRC(f8e5m2rcprc_f8e5m2rcprc_f32rcprc, uint8_t, float)

/*
 * The two steps src/gemm/README.md:46-47 names as what callers fuse behind a GEMM ("requantization and activation
 * functions") and for which the reference has no routine: the rules are the ones include/skl-gfx950.h states for
 * skl_gfx950_epilogue_t, restated here over a C that already holds the alpha/beta (and bias) result. They sit
 * between the bias and the maximum, so a test composes: plain GEMM, bias, these, maximum.
 *   activation 1:  v = v > 0 ? v : 0     (a NaN becomes 0), written back to C
 *   activation 2:  SiLU as ref/sigmoid/sigmoid_f32.c:10-28 evaluates skl_silu_f32_ref (beta = 1, y = x, no gate): the
 *                  logistic in double, times x, rounded to float once          (floating point only)
 *   activation 3:  GELU as ref/gelu/gelu_f32.c:12-22: fma(-|x|/2, erfc(|x|/sqrt 2), relu(x)) in double, rounded to
 *                  float once                                                   (floating point only)
 *   q != NULL:     Q(i,j) = clamp(rne((float)v * s_j) + zero, -128, 127), one fp32 product, rne to the nearest
 *                  integer with ties to even; a NaN counts as 0, values beyond int32 as its ends
 */
static int8_t requantised(float v, float scale, int32_t zero) {
  const float r = nearbyintf(v * scale); /* the default rounding mode: to nearest, ties to even */
  int64_t t = isnan(r) ? 0 : r >= 2147483648.0f ? INT32_MAX : r <= -2147483648.0f ? INT32_MIN : (int64_t)r;
  t += zero;
  return (int8_t)(t < -128 ? -128 : t > 127 ? 127 : t);
}
float skl_oracle_silu_f32(float x) {
  const double a = x;
  double o = 1. / (1. + exp(-1.f * a)); /* beta = 1.f, as skl_silu_f32_ref passes it */
  o *= x;
  return (float)o;
}
float skl_oracle_gelu_f32(float x) {
  const double sqrt2 = 0x1.6a09e667f3bcdp0;
  const float b = (x > 0) ? x : -0.f;
  const float h = -0.5f * fabsf(x);
  const double e = erfc(-sqrt2 * h);
  return (float)fma(h, e, b);
}
static int32_t activated_i32(int32_t v, int activation) { return activation == 1 ? (v > 0 ? v : 0) : v; }
static float activated_f32(float v, int activation) {
  return activation == 1 ? (v > 0 ? v : 0) : activation == 2 ? skl_oracle_silu_f32(v) : activation == 3 ? skl_oracle_gelu_f32(v) : v;
}
#define ACT_REQUANT(SUFFIX, TC)                                                                     \
  void skl_oracle_act_requant_##SUFFIX(size_t m, size_t n, TC *c, size_t rsc, size_t csc, int activation, \
                                       int8_t *q, size_t rsq, size_t csq, const float *q_scale,     \
                                       int per_column, int32_t q_zero) {                            \
    for (size_t i = 0; i < m; ++i)                                                                  \
      for (size_t j = 0; j < n; ++j) {                                                              \
        TC v = c[i * rsc + j * csc];                                                                \
        v = activated_##SUFFIX(v, activation);                                                      \
        c[i * rsc + j * csc] = v;                                                                   \
        if (q) q[i * rsq + j * csq] = requantised((float)v, q_scale[per_column ? j : 0], q_zero);   \
      }                                                                                             \
  }
ACT_REQUANT(i32, int32_t)
ACT_REQUANT(f32, float)

/* ======================================================================== */
/* Widening helpers                                                          */
/* ======================================================================== */

void skl_oracle_widen_bf16_f64(double *dst, const uint16_t *src, size_t n) {
  for (size_t i = 0; i < n; ++i) dst[i] = (double)skl_oracle_bf16_to_f32(src[i]);
}
void skl_oracle_widen_f16_f64(double *dst, const uint16_t *src, size_t n) {
  for (size_t i = 0; i < n; ++i) dst[i] = (double)skl_oracle_f16_to_f32(src[i]);
}
void skl_oracle_widen_f8e4m3_f64(double *dst, const uint8_t *src, size_t n) {
  for (size_t i = 0; i < n; ++i) dst[i] = (double)skl_oracle_f8e4m3_to_f32(src[i]);
}
void skl_oracle_widen_f8e5m2_f64(double *dst, const uint8_t *src, size_t n) {
  for (size_t i = 0; i < n; ++i) dst[i] = (double)skl_oracle_f8e5m2_to_f32(src[i]);
}
