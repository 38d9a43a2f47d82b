// skl_cvt.hip - OFP8 (E4M3 / E5M2) and OFP4 (E2M1) conversions for gfx950.
//
// Semantics are those of the reference's scalar routines
// (ref/cvt/cvt_ofp8.c:18-242, ref/cvt/cvt_ofp4.c:18-68): one fp32 multiply by
// the scale, then round-to-nearest-even to the 8-bit format with gradual
// underflow; NaN -> 0x7F; overflow and infinities -> the format's "overflow
// byte" (saturating: signed max finite; non-saturating: 0x7F without sign for
// E4M3, signed infinity for E5M2). The reference expresses the rounding with
// libm calls; here it is integer arithmetic on the fp32 bit pattern, which gives
// the same byte for every input. The kernels are pure streaming: each thread
// moves 8 (or 16) elements with 128-bit/64-bit accesses.
#include <hip/hip_runtime.h>

#include "skl_device.hpp"
#include "skl_fp8.hpp"

namespace {

using namespace skl_fp8;

__device__ __forceinline__ unsigned scaled_bits(float x, float scale) {
  // One IEEE fp32 multiply; fp32 subnormals are kept (no flush).
  return __float_as_uint(__fmul_rn(x, scale));
}

// A workgroup converts 4096 consecutive elements: four rounds in which the 256 threads read 256
// consecutive float4 (every load instruction of a wave covers one contiguous KiB) and write 256
// consecutive dwords; the four loads of a thread are all requested before the first is used.
constexpr int kCvtRounds = 4;
template <class F>
__global__ void __launch_bounds__(256) cvt_f32_f8_kernel(uint8_t *__restrict__ dst, const float *__restrict__ src,
                                                         float scale, size_t n, bool sat, bool vec) {
  const size_t block0 = (size_t)blockIdx.x * (256 * 4 * kCvtRounds);
  if (vec && block0 + 256 * 4 * kCvtRounds <= n) {
    typedef float f4v __attribute__((ext_vector_type(4)));
    f4v x[kCvtRounds];
#pragma unroll
    for (int j = 0; j < kCvtRounds; ++j)
      x[j] = __builtin_nontemporal_load(reinterpret_cast<const f4v *>(src + block0) + j * 256 + threadIdx.x);
#pragma unroll
    for (int j = 0; j < kCvtRounds; ++j) {
      const unsigned out = encode_ofp8<F>(scaled_bits(x[j].x, scale), sat) | (encode_ofp8<F>(scaled_bits(x[j].y, scale), sat) << 8) |
                           (encode_ofp8<F>(scaled_bits(x[j].z, scale), sat) << 16) |
                           (encode_ofp8<F>(scaled_bits(x[j].w, scale), sat) << 24);
      __builtin_nontemporal_store(out, reinterpret_cast<unsigned *>(dst + block0) + j * 256 + threadIdx.x);
    }
  } else {
    for (int j = 0; j < kCvtRounds; ++j) {
      const size_t base = block0 + ((size_t)j * 256 + threadIdx.x) * 4;
      for (size_t i = base; i < base + 4 && i < n; ++i) dst[i] = (uint8_t)encode_ofp8<F>(scaled_bits(src[i], scale), sat);
    }
  }
}

template <class F>
__global__ void __launch_bounds__(256) cvt_bf16_f8_kernel(uint8_t *__restrict__ dst, const uint16_t *__restrict__ src,
                                                          float scale, size_t n, bool sat, bool vec) {
  const size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t base = t * 8;
  if (base >= n) return;
  if (vec && base + 8 <= n) {
    const uint4 x = *reinterpret_cast<const uint4 *>(src + base);
    const unsigned w[4] = {x.x, x.y, x.z, x.w};
    unsigned o[2] = {0u, 0u};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const unsigned lo = encode_ofp8<F>(scaled_bits(__uint_as_float(w[i] << 16), scale), sat);
      const unsigned hi = encode_ofp8<F>(scaled_bits(__uint_as_float(w[i] & 0xFFFF0000u), scale), sat);
      o[i >> 1] |= (lo | (hi << 8)) << ((i & 1) * 16);
    }
    *reinterpret_cast<uint2 *>(dst + base) = make_uint2(o[0], o[1]);
  } else {
    const size_t end = base + 8 < n ? base + 8 : n;
    for (size_t i = base; i < end; ++i)
      dst[i] = (uint8_t)encode_ofp8<F>(scaled_bits(__uint_as_float((unsigned)src[i] << 16), scale), sat);
  }
}

template <class F>
__global__ void __launch_bounds__(256) cvt_f8_bf16_kernel(uint16_t *__restrict__ dst, const uint8_t *__restrict__ src,
                                                          size_t n, bool vec) {
  const size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t base = t * 8;
  if (base >= n) return;
  if (vec && base + 8 <= n) {
    const uint2 x = *reinterpret_cast<const uint2 *>(src + base);
    const unsigned w[2] = {x.x, x.y};
    unsigned o[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const unsigned pair = w[i >> 1] >> ((i & 1) * 16);
      // Every OFP8 value (and the quiet NaN) has zero low 16 bits in fp32.
      o[i] = (decode_ofp8_bits<F>(pair & 0xFFu) >> 16) | (decode_ofp8_bits<F>((pair >> 8) & 0xFFu) & 0xFFFF0000u);
    }
    *reinterpret_cast<uint4 *>(dst + base) = make_uint4(o[0], o[1], o[2], o[3]);
  } else {
    const size_t end = base + 8 < n ? base + 8 : n;
    for (size_t i = base; i < end; ++i) dst[i] = (uint16_t)(decode_ofp8_bits<F>(src[i]) >> 16);
  }
}

// E2M1 nibble -> E4M3 byte. Every E2M1 value is exactly representable in E4M3.
__device__ __forceinline__ unsigned f4_to_e4m3(unsigned nib) {
  const unsigned sign = (nib & 0x8u) << 4;
  const unsigned e = (nib >> 1) & 0x3u, m = nib & 0x1u;
  if (e == 0) return sign | (m ? 0x30u : 0x00u);  // 0.5 = 2^-1 -> exponent field 6
  return sign | ((e + 6u) << 3) | (m << 2);
}

__global__ void __launch_bounds__(256) cvt_f4_f8e4m3_kernel(uint8_t *__restrict__ dst, const uint8_t *__restrict__ src,
                                                            size_t n, bool vec) {
  const size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t base = t * 16;  // 16 outputs from 8 source bytes
  if (base >= n) return;
  if (vec && base + 16 <= n) {
    const uint2 x = *reinterpret_cast<const uint2 *>(src + base / 2);
    const unsigned w[2] = {x.x, x.y};
    unsigned o[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const unsigned half = (w[i >> 1] >> ((i & 1) * 16)) & 0xFFFFu;  // 2 bytes = 4 nibbles, low first
      o[i] = f4_to_e4m3(half & 0xFu) | (f4_to_e4m3((half >> 4) & 0xFu) << 8) |
             (f4_to_e4m3((half >> 8) & 0xFu) << 16) | (f4_to_e4m3((half >> 12) & 0xFu) << 24);
    }
    *reinterpret_cast<uint4 *>(dst + base) = make_uint4(o[0], o[1], o[2], o[3]);
  } else {
    const size_t end = base + 16 < n ? base + 16 : n;
    for (size_t i = base; i < end; ++i) {
      const unsigned byte = src[i >> 1];
      dst[i] = (uint8_t)f4_to_e4m3((i & 1) ? (byte >> 4) : (byte & 0xFu));
    }
  }
}

// One thread per block of 32 k of a column: E2M1 values times the block's scale 2^(s - 127), as bf16 (exact: one
// or two significant bits). Columns may start inside a byte (odd ldb): nibbles are addressed one by one.
__global__ void __launch_bounds__(256) cvt_mxf4_bf16_kernel(uint16_t *__restrict__ dst, const uint8_t *__restrict__ src,
                                                            const uint8_t *__restrict__ scales, size_t lds, size_t n, size_t k,
                                                            size_t ldb) {
  const size_t blocks_per_col = (k + 31) / 32;
  const size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= n * blocks_per_col) return;
  const size_t j = t / blocks_per_col, p0 = (t % blocks_per_col) * 32;
  const float scale = __uint_as_float((unsigned)scales[j * lds + p0 / 32] << 23);
  const size_t end = p0 + 32 < k ? p0 + 32 : k;
  for (size_t p = p0; p < end; ++p) {
    const size_t i = j * ldb + p;
    const unsigned byte = src[i >> 1], nib = (i & 1) ? (byte >> 4) : (byte & 0xFu);
    const unsigned e = (nib >> 1) & 3u, m = nib & 1u;
    const float mag = e == 0 ? (m ? 0.5f : 0.0f) : __uint_as_float(((e + 126u) << 23) | (m << 22));
    const float v = __fmul_rn((nib & 8u) ? -mag : mag, scale);
    dst[i] = (uint16_t)(__float_as_uint(v) >> 16);
  }
}

inline bool aligned(const void *p, size_t a) { return ((uintptr_t)p & (a - 1)) == 0; }

}  // namespace

extern "C" {

int skl_hip_launch_cvt_f32_f8(int fmt, int saturate, uint8_t *dst, const float *src, float scale, size_t n) {
  if (n == 0) return 0;
  const bool vec = aligned(src, 16) && aligned(dst, 4);
  const unsigned blocks = skl_div_up(n, 256 * 4 * kCvtRounds);
  hipStream_t s = skl_current_stream();
  if (fmt == SKL_DT_F8E4M3)
    cvt_f32_f8_kernel<E4M3><<<blocks, 256, 0, s>>>(dst, src, scale, n, saturate != 0, vec);
  else
    cvt_f32_f8_kernel<E5M2><<<blocks, 256, 0, s>>>(dst, src, scale, n, saturate != 0, vec);
  return skl_check_launch("cvt_f32_f8");
}

int skl_hip_launch_cvt_bf16_f8(int fmt, int saturate, uint8_t *dst, const uint16_t *src, float scale, size_t n) {
  if (n == 0) return 0;
  const bool vec = aligned(src, 16) && aligned(dst, 8);
  const unsigned blocks = skl_div_up(skl_div_up(n, 8), 256);
  hipStream_t s = skl_current_stream();
  if (fmt == SKL_DT_F8E4M3)
    cvt_bf16_f8_kernel<E4M3><<<blocks, 256, 0, s>>>(dst, src, scale, n, saturate != 0, vec);
  else
    cvt_bf16_f8_kernel<E5M2><<<blocks, 256, 0, s>>>(dst, src, scale, n, saturate != 0, vec);
  return skl_check_launch("cvt_bf16_f8");
}

int skl_hip_launch_cvt_f8_bf16(int fmt, uint16_t *dst, const uint8_t *src, size_t n) {
  if (n == 0) return 0;
  const bool vec = aligned(src, 8) && aligned(dst, 16);
  const unsigned blocks = skl_div_up(skl_div_up(n, 8), 256);
  hipStream_t s = skl_current_stream();
  if (fmt == SKL_DT_F8E4M3)
    cvt_f8_bf16_kernel<E4M3><<<blocks, 256, 0, s>>>(dst, src, n, vec);
  else
    cvt_f8_bf16_kernel<E5M2><<<blocks, 256, 0, s>>>(dst, src, n, vec);
  return skl_check_launch("cvt_f8_bf16");
}

int skl_hip_launch_cvt_mxf4_bf16(uint16_t *dst, const uint8_t *src, const uint8_t *scales, size_t lds, size_t n, size_t k, size_t ldb) {
  if (n == 0 || k == 0) return 0;
  const size_t threads = n * ((k + 31) / 32), blocks = (threads + 255) / 256;
  if (blocks > 0x7FFFFFFFu) {
    skl_hip_record_error(-2, "cvt_mxf4_bf16: too large");
    return -2;
  }
  cvt_mxf4_bf16_kernel<<<(unsigned)blocks, 256, 0, skl_current_stream()>>>(dst, src, scales, lds, n, k, ldb);
  return skl_check_launch("cvt_mxf4_bf16");
}

int skl_hip_launch_cvt_f4_f8e4m3(uint8_t *dst, const uint8_t *src, size_t n) {
  if (n == 0) return 0;
  const bool vec = aligned(src, 8) && aligned(dst, 16);
  const unsigned blocks = skl_div_up(skl_div_up(n, 16), 256);
  cvt_f4_f8e4m3_kernel<<<blocks, 256, 0, skl_current_stream()>>>(dst, src, n, vec);
  return skl_check_launch("cvt_f4_f8e4m3");
}

}  // extern "C"
