// skl_probe.hip - the two ceilings a report prices the kernels against, measured on the device itself rather than
// taken from a data sheet: how fast memory can be read at all, and how fast the matrix cores multiply when nothing
// but they is busy. Declared in include/skl-hip.h next to the timing helpers; not part of any kernel's path.
#include <hip/hip_runtime.h>

#include "../../include/skl-hip.h"
#include "skl_device.hpp"

namespace {

typedef unsigned u4v __attribute__((ext_vector_type(4)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));

constexpr int kReadUnroll = 8, kReadThreads = 256;

// Every thread asks for kReadUnroll 16-byte pieces, a whole grid apart, before it looks at the first: consecutive
// lanes read consecutive pieces, so a wave's load covers one contiguous KiB.
__global__ void __launch_bounds__(kReadThreads) probe_read_kernel(const u4v *src, size_t pieces, unsigned *sink) {
  const size_t threads = (size_t)gridDim.x * kReadThreads, first = (size_t)blockIdx.x * kReadThreads + threadIdx.x;
  u4v v[kReadUnroll];
#pragma unroll
  for (int u = 0; u < kReadUnroll; ++u) {
    const size_t i = first + (size_t)u * threads;
    v[u] = i < pieces ? __builtin_nontemporal_load(src + i) : u4v{0, 0, 0, 0};
  }
  unsigned s = 0;
#pragma unroll
  for (int u = 0; u < kReadUnroll; ++u) s += v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  if (s == 0x9E3779B9u && sink) *sink = s;  // keeps the loads alive; practically never taken, and harmless if it is
}

constexpr int kMfmaChains = 8;  // independent accumulators per wave: 128 accumulator registers, two waves per SIMD

// KIND 0: v_mfma_i32_32x32x32_i8, 1: v_mfma_f32_32x32x16_bf16, 2: v_mfma_f32_32x32x64_f8f6f4 (E4M3 x E4M3).
template <int KIND>
__global__ void __launch_bounds__(256) probe_mfma_kernel(int iters, int random_operands, unsigned *sink) {
  unsigned h = (threadIdx.x + blockIdx.x * 977u + 1u) * 2654435761u;
  // Operand words. Random: int8 any byte; bf16 with either sign, any significand and an exponent of 2^-7 .. 2^0;
  // E4M3 with either sign, any significand and an exponent of 2^-4 .. 2^3 - operands as a GEMM on random data
  // sees them, and sums that stay finite. Otherwise one value everywhere.
  auto word = [&]() -> int {
    if (!random_operands) return KIND == 0 ? 0x03030303 : KIND == 1 ? 0x3F803F80 : 0x38383838;
    unsigned w = 0;
    if (KIND == 1) {
      for (int e = 0; e < 2; ++e) {
        h ^= h << 13, h ^= h >> 17, h ^= h << 5;
        w |= (((h & 0x807Fu) | ((120u + ((h >> 8) & 7u)) << 7)) & 0xFFFFu) << (16 * e);
      }
    } else {
      for (int e = 0; e < 4; ++e) {
        h ^= h << 13, h ^= h >> 17, h ^= h << 5;
        const unsigned byte = KIND == 0 ? (h & 0xFFu) : ((h & 0x87u) | ((3u + ((h >> 8) & 7u)) << 3));
        w |= byte << (8 * e);
      }
    }
    return (int)w;
  };
  v8i a[kMfmaChains / 2], b[kMfmaChains / 2];  // four operand pairs, taken in turn
#pragma unroll
  for (int q = 0; q < kMfmaChains / 2; ++q)
#pragma unroll
    for (int r = 0; r < 8; ++r) a[q][r] = word(), b[q][r] = word();
  v16i ci[kMfmaChains];
  v16f cf[kMfmaChains];
#pragma unroll
  for (int j = 0; j < kMfmaChains; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) ci[j][r] = 0, cf[j][r] = 0.0f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int j = 0; j < kMfmaChains; ++j) {
      const v8i x = a[j % (kMfmaChains / 2)], y = b[j % (kMfmaChains / 2)];
      const v4i x4 = {x[0], x[1], x[2], x[3]}, y4 = {y[0], y[1], y[2], y[3]};
      if constexpr (KIND == 0)
        ci[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(x4, y4, ci[j], 0, 0, 0);
      else if constexpr (KIND == 1)
        cf[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, x4), __builtin_bit_cast(v8bf, y4), cf[j], 0, 0, 0);
      else
        cf[j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(x, y, cf[j], 0, 0, 0, 0, 0, 0);
    }
  }
  unsigned s = 0;
#pragma unroll
  for (int j = 0; j < kMfmaChains; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) s += (unsigned)ci[j][r] + __float_as_uint(cf[j][r]);
  if (s == 0x9E3779B9u && sink) *sink = s;
}

}  // namespace

extern "C" int skl_hip_probe_hbm_read(const void *src, size_t bytes) {
  if (!src || bytes < 16 || (bytes & 15) != 0 || ((uintptr_t)src & 15) != 0) {
    skl_hip_record_error(SKL_HIP_ERR_BAD_ARGUMENT, "skl_hip_probe_hbm_read: 16-byte aligned, a multiple of 16 bytes");
    return SKL_HIP_ERR_BAD_ARGUMENT;
  }
  const size_t pieces = bytes / 16, per_block = (size_t)kReadThreads * kReadUnroll;
  const size_t blocks = (pieces + per_block - 1) / per_block;
  if (blocks > 0x7FFFFFFFu) {
    skl_hip_record_error(SKL_HIP_ERR_BAD_ARGUMENT, "skl_hip_probe_hbm_read: too large");
    return SKL_HIP_ERR_BAD_ARGUMENT;
  }
  probe_read_kernel<<<(unsigned)blocks, kReadThreads, 0, skl_current_stream()>>>((const u4v *)src, pieces, nullptr);
  return skl_check_launch("skl_hip_probe_hbm_read");
}

extern "C" double skl_hip_probe_mfma(int kind, int random_operands, int iters) {
  int dev = 0;
  hipDeviceProp_t prop;
  if (kind < 0 || kind > 2 || iters <= 0 || skl_check_hip(hipGetDevice(&dev), "hipGetDevice") != 0 ||
      skl_check_hip(hipGetDeviceProperties(&prop, dev), "hipGetDeviceProperties") != 0) {
    skl_hip_record_error(SKL_HIP_ERR_BAD_ARGUMENT, "skl_hip_probe_mfma");
    return 0.0;
  }
  const unsigned grid = 2u * (unsigned)prop.multiProcessorCount;  // two workgroups of four waves per compute unit
  static const double ops_per_instruction[3] = {2.0 * 32 * 32 * 32, 2.0 * 32 * 32 * 16, 2.0 * 32 * 32 * 64};
  if (kind == 0)
    probe_mfma_kernel<0><<<grid, 256, 0, skl_current_stream()>>>(iters, random_operands, nullptr);
  else if (kind == 1)
    probe_mfma_kernel<1><<<grid, 256, 0, skl_current_stream()>>>(iters, random_operands, nullptr);
  else
    probe_mfma_kernel<2><<<grid, 256, 0, skl_current_stream()>>>(iters, random_operands, nullptr);
  if (skl_check_launch("skl_hip_probe_mfma") != 0) return 0.0;
  return (double)grid * 4.0 * (double)iters * kMfmaChains * ops_per_instruction[kind];
}
