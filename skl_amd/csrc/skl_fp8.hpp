// skl_fp8.hpp - OFP8 (E4M3 / E5M2) encode and decode on fp32 bit patterns,
// shared by the conversion kernels and the scalar-path GEMM.
//
// Encode follows ref/cvt/cvt_ofp8.c:97-172 (round to nearest even, gradual
// underflow, NaN -> 0x7F, overflow -> the format's overflow byte); decode
// follows ref/cvt/cvt_ofp8.c:18-95 (NaN codes give the sign-less quiet NaN).
#pragma once

#include <hip/hip_runtime.h>

namespace skl_fp8 {

struct E4M3 {
  static constexpr int kMant = 3, kBias = 7, kEmin = -6;
  static constexpr unsigned kMax = 0x7E;
  __device__ static unsigned overflow(unsigned sign, bool sat) { return sat ? (sign | 0x7Eu) : 0x7Fu; }
};
struct E5M2 {
  static constexpr int kMant = 2, kBias = 15, kEmin = -14;
  static constexpr unsigned kMax = 0x7B;
  __device__ static unsigned overflow(unsigned sign, bool sat) { return sign | (sat ? 0x7Bu : 0x7Cu); }
};

// fp32 bit pattern -> OFP8 byte, round to nearest even.
template <class F>
__device__ __forceinline__ unsigned encode_ofp8(unsigned bits, bool sat) {
  const unsigned sign = (bits >> 24) & 0x80u;
  const unsigned mag32 = bits & 0x7FFFFFFFu;
  if (mag32 > 0x7F800000u) return 0x7Fu;                  // NaN
  if (mag32 == 0x7F800000u) return F::overflow(sign, sat);  // +-inf
  int e = (int)(mag32 >> 23) - 127;
  unsigned sig = (mag32 & 0x7FFFFFu) | 0x800000u;
  if ((mag32 >> 23) == 0) {  // fp32 subnormal: no hidden bit
    e = -126;
    sig = mag32;
  }
  const int te = e > F::kEmin ? e : F::kEmin;  // exponent of the target's quantum
  int shift = (te - F::kMant) - (e - 23);      // low bits of sig that are dropped (> 0)
  if (shift > 31) shift = 31;                  // sig < 2^24: everything rounds to 0
  unsigned q = sig >> shift;
  const unsigned rem = sig & ((1u << shift) - 1u);
  const unsigned half = 1u << (shift - 1);
  if (rem > half || (rem == half && (q & 1u))) ++q;
  // Adding q (which carries the hidden bit for normals) to the exponent field
  // lets a mantissa carry bump the exponent and a subnormal round up to the
  // smallest normal.
  const unsigned mag = (e < F::kEmin) ? q : ((unsigned)(te + F::kBias - 1) << F::kMant) + q;
  if (mag > F::kMax) return F::overflow(sign, sat);
  return sign | mag;
}

// The same byte through the hardware's conversion, for epilogues that convert their accumulators in place (the
// integer route above costs about 30 operations per element, which shows next to the matrix cores; in the
// conversion kernels, which wait for memory, it does not). v_cvt_pk_fp8_f32 / v_cvt_pk_bf8_f32 round to nearest even
// into the OCP codes, gradual underflow included, and never saturate: a value beyond the largest becomes the
// format's NaN (E4M3) or infinity (E5M2) with its sign. That is the rule of ref/cvt/cvt_ofp8.c:97-172 except where
// the rule leaves IEEE habits - every NaN is the sign-less 0x7F, E4M3's overflow without saturation drops the sign,
// saturation ends at the largest finite code - and two selects restore those (compared with the integer route on the
// hardware for every fp32 bit pattern and all four formats: no difference; the GEMM tests hold the copies to the
// checker's conversion). The format comes as values, uniform across the wave, so one code path serves both.
// `fmt`: 1 / 2 E4M3 without / with saturation, 3 / 4 E5M2 likewise.
struct Ofp8Format {
  bool e5m2;
  unsigned max, overflow_sign, overflow_code;
  __host__ __device__ explicit Ofp8Format(int fmt) {
    const bool sat = fmt == 2 || fmt == 4;
    e5m2 = fmt >= 3;
    max = e5m2 ? 0x7Bu : 0x7Eu;
    overflow_sign = (sat || e5m2) ? 0x80u : 0u;            // E4M3's overflow without saturation is the sign-less NaN
    overflow_code = sat ? max : e5m2 ? 0x7Cu : 0x7Fu;
  }
};
__device__ __forceinline__ unsigned encode_ofp8_hw(float x, const Ofp8Format &f) {
  const unsigned e4 = (unsigned)__builtin_amdgcn_cvt_pk_fp8_f32(x, x, 0, false), e5 = (unsigned)__builtin_amdgcn_cvt_pk_bf8_f32(x, x, 0, false);
  const unsigned hw = (f.e5m2 ? e5 : e4) & 0xFFu;
  const unsigned out = (hw & 0x7Fu) > f.max ? ((hw & f.overflow_sign) | f.overflow_code) : hw;   // beyond the largest: overflow, infinity or NaN
  return x != x ? 0x7Fu : out;
}

// OFP8 byte -> fp32 bit pattern. NaN codes give the sign-less quiet NaN.
template <class F>
__device__ __forceinline__ unsigned decode_ofp8_bits(unsigned code) {
  const unsigned sign = (code & 0x80u) << 24;
  const unsigned e = (code & 0x7Fu) >> F::kMant;
  const unsigned m = code & ((1u << F::kMant) - 1u);
  constexpr unsigned emax = (1u << (7 - F::kMant)) - 1u;
  if (F::kMant == 3) {
    if ((code & 0x7Fu) == 0x7Fu) return 0x7FC00000u;
  } else if (e == emax) {
    return m ? 0x7FC00000u : (sign | 0x7F800000u);
  }
  if (e == 0) {
    // m * 2^(emin - mant): exact in fp32
    float v = (float)m * __uint_as_float((unsigned)(127 + F::kEmin - F::kMant) << 23);
    return sign | __float_as_uint(v);
  }
  return sign | ((e + 127u - (unsigned)F::kBias) << 23) | (m << (23 - F::kMant));
}

// Eight OFP8 bytes (two dwords, ascending) as eight f16 values. Exact: every E4M3 and E5M2 value is an f16 value
// (E5M2 is f16 cut to its top byte, E4M3 has fewer exponent and significand bits than f16), subnormal codes included.
template <bool IS_E5M2>
__device__ __forceinline__ auto widen8_to_f16(unsigned lo, unsigned hi) {
  typedef _Float16 v2h __attribute__((ext_vector_type(2)));
  typedef _Float16 v8h __attribute__((ext_vector_type(8)));
  v2h p[4];
  if constexpr (IS_E5M2) {
    p[0] = __builtin_amdgcn_cvt_scalef32_pk_f16_bf8(lo, 1.0f, false);
    p[1] = __builtin_amdgcn_cvt_scalef32_pk_f16_bf8(lo, 1.0f, true);
    p[2] = __builtin_amdgcn_cvt_scalef32_pk_f16_bf8(hi, 1.0f, false);
    p[3] = __builtin_amdgcn_cvt_scalef32_pk_f16_bf8(hi, 1.0f, true);
  } else {
    p[0] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(lo, 1.0f, false);
    p[1] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(lo, 1.0f, true);
    p[2] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(hi, 1.0f, false);
    p[3] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(hi, 1.0f, true);
  }
  return v8h{p[0].x, p[0].y, p[1].x, p[1].y, p[2].x, p[2].y, p[3].x, p[3].y};
}

}  // namespace skl_fp8
