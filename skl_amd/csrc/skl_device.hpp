// skl_device.hpp - helpers shared by the HIP translation units (not installed).
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "skl_fp8.hpp"
#include "skl_launch.h"

// Stream the calling thread launches on (set through skl_hip_set_stream).
hipStream_t skl_current_stream();

// Scratch of the current stream (on the current device) used by split reductions. Grows on
// demand; contents are only meaningful inside one launch sequence.
void *skl_workspace(size_t bytes);

// A block of the current stream (on the current device) that is zero when a kernel starts and
// that every kernel leaves zero again: sums and counters shared by the workgroups of a launch.
// Allocated and cleared at the first call; every caller asks for the same size.
void *skl_zeroed_scratch(size_t bytes);

// Records a HIP failure for skl_hip_last_error() and returns its code.
int skl_check_hip(hipError_t e, const char *what);

// Checks the launch that was just enqueued.
static inline int skl_check_launch(const char *what) { return skl_check_hip(hipGetLastError(), what); }

static inline unsigned skl_div_up(size_t a, size_t b) { return (unsigned)((a + b - 1) / b); }

// ---------------------------------------------------------------------------
// C = beta*C + alpha*acc for one element, as the reference's C computes it: two
// products and a sum, each rounded on its own (the translation units are built
// with -ffp-contract=off); int32 wraps.
//
// beta == 0 initialises C (src/gemm/README.md:43 of the reference: "accumulation (beta=1) and initialization
// (beta=0)"): there beta*C is a zero whose sign is all the old value contributes, and the sign matters only when
// alpha*acc is itself a zero - the old value is read for exactly those elements, and only its sign bit is used.
// The result has the reference's bits for every finite C; an Inf or NaN in C, which
// ref/gemm/gemm_bf16rc_bf16rc_f32rc.c:21 (beta*c evaluated whatever beta is) turns into NaN, is overwritten
// everywhere (so C may be uninitialised memory). A caller that wants the reference's result there too asks
// for it (skl_hip_set_beta_zero_mode(SKL_HIP_BETA_ZERO_AS_REFERENCE)): beta then arrives without
// fz.skip_c_read and C is read and combined whatever beta is. int32: 0 * c is 0 for every c, so C is never read
// with beta == 0. f64 has no room for the switch next to the value: always read. A call that leaves C unwritten
// (q_only) with beta == 0 does not touch C at all: the old C counts as +0 (skip_c_read == SKL_C_UNTOUCHED).
// ---------------------------------------------------------------------------
template <typename T>
__device__ __forceinline__ bool skl_beta_is_zero(skl_scalar beta);  // "C need not be read"
template <>
__device__ __forceinline__ bool skl_beta_is_zero<int>(skl_scalar beta) { return beta.i == 0; }
template <>
__device__ __forceinline__ bool skl_beta_is_zero<float>(skl_scalar beta) { return beta.fz.skip_c_read != 0 && beta.f == 0.0f; }
template <>
__device__ __forceinline__ bool skl_beta_is_zero<double>(skl_scalar) { return false; }  // no room for the switch: always read

__device__ __forceinline__ int skl_combine(int acc, int old, skl_scalar alpha, skl_scalar beta) {
  return (int)((unsigned)beta.i * (unsigned)old + (unsigned)alpha.i * (unsigned)acc);
}
__device__ __forceinline__ float skl_combine(float acc, float old, skl_scalar alpha, skl_scalar beta) {
  return __fadd_rn(__fmul_rn(beta.f, old), __fmul_rn(alpha.f, acc));
}
__device__ __forceinline__ double skl_combine(double acc, double old, skl_scalar alpha, skl_scalar beta) {
  return __dadd_rn(__dmul_rn(beta.d, old), __dmul_rn(alpha.d, acc));
}

// The beta == 0 case; `c` is dereferenced only where alpha*acc is a zero, and only for its sign: beta*c is the zero
// whose sign is the product of the two signs (what 0 * c is for every finite c).
__device__ __forceinline__ int skl_initialise(int acc, const int *, skl_scalar alpha, skl_scalar) {
  return (int)((unsigned)alpha.i * (unsigned)acc);
}
__device__ __forceinline__ float skl_initialise(float acc, const float *c, skl_scalar alpha, skl_scalar beta) {
  const float x = __fmul_rn(alpha.f, acc);
  const bool read_c = x == 0.0f && beta.fz.skip_c_read != SKL_C_UNTOUCHED;  // a call that does not write C does not read it either
  const unsigned old = read_c ? __float_as_uint(*c) : 0u;
  return x == 0.0f ? __fadd_rn(__uint_as_float((old ^ __float_as_uint(beta.f)) & 0x80000000u), x) : x;
}
__device__ __forceinline__ double skl_initialise(double acc, const double *c, skl_scalar alpha, skl_scalar beta) {
  const double x = __dmul_rn(alpha.d, acc);
  if (x != 0.0) return x;
  const unsigned long long sign = (unsigned long long)(__double_as_longlong(*c) ^ __double_as_longlong(beta.d)) & 0x8000000000000000ull;
  return __dadd_rn(__longlong_as_double((long long)sign), x);
}

// The same in two steps, for kernels in which a lane writes many elements: a load that sits between two stores -
// taken or not - makes the second store wait for the first to complete (one memory round trip per element). Such a
// kernel first asks, for a batch of elements, whether any of them needs its old C at all, requests those values
// together if so (a rare, wave-uniform branch), and then writes the batch. The old value matters only where
// alpha*acc is the negative zero: (+0) + (+-0) is +0 whatever the sign of beta*c.
__device__ __forceinline__ bool skl_initialise_needs_c(int, skl_scalar, skl_scalar) { return false; }
__device__ __forceinline__ bool skl_initialise_needs_c(float acc, skl_scalar alpha, skl_scalar beta) {
  return __float_as_uint(__fmul_rn(alpha.f, acc)) == 0x80000000u && beta.fz.skip_c_read != SKL_C_UNTOUCHED;
}
__device__ __forceinline__ int skl_initialise_with(int acc, int, skl_scalar alpha, skl_scalar) {
  return (int)((unsigned)alpha.i * (unsigned)acc);
}
// `old`: the old C where skl_initialise_needs_c() said so, anything finite (+0) elsewhere.
__device__ __forceinline__ float skl_initialise_with(float acc, float old, skl_scalar alpha, skl_scalar beta) {
  const float x = __fmul_rn(alpha.f, acc);
  return x == 0.0f ? __fadd_rn(__uint_as_float((__float_as_uint(old) ^ __float_as_uint(beta.f)) & 0x80000000u), x) : x;
}

// skl_initialise_with() for an element that does not need its old C (skl_initialise_needs_c() false: the product is
// not the negative zero, or C counts as +0): a product that is a zero takes the sign (+0) + (+-0) has, which adding
// the zero of beta's sign yields; every other value is unchanged by that sum.
__device__ __forceinline__ int skl_initialise_plain(int acc, skl_scalar alpha, skl_scalar) {
  return (int)((unsigned)alpha.i * (unsigned)acc);
}
__device__ __forceinline__ float skl_initialise_plain(float acc, skl_scalar alpha, skl_scalar beta) {
  return __fadd_rn(__uint_as_float(__float_as_uint(beta.f) & 0x80000000u), __fmul_rn(alpha.f, acc));
}

template <typename T>
__device__ __forceinline__ void skl_update(T acc, T *c, skl_scalar alpha, skl_scalar beta) {
  *c = skl_beta_is_zero<T>(beta) ? skl_initialise(acc, c, alpha, beta) : skl_combine(acc, *c, alpha, beta);
}

// ---------------------------------------------------------------------------
// Fused epilogue steps after the alpha/beta step (the GPU form of the reference's per-tile fused
// kernels, src/gemm/fused-kernel-API.md:159-178 "adding a bias", :186-207 "computing a global maximum").
// ---------------------------------------------------------------------------
__device__ __forceinline__ int skl_add_bias(int v, int b) { return (int)((unsigned)v + (unsigned)b); }
__device__ __forceinline__ float skl_add_bias(float v, float b) { return __fadd_rn(v, b); }

// The activation step: 0 none, 1 max(v, 0) (a NaN becomes 0, like `v > 0 ? v : 0`); integers have no other.
__device__ __forceinline__ int skl_activate(int v, int act) {
  const int floor = act == 1 ? 0 : (int)0x80000000;  // uniform: one max per element
  return v < floor ? floor : v;
}
// SiLU, x * logistic(x). ref/sigmoid/sigmoid_f32.c:10-28 evaluates 1 / (1 + exp(-x)) * x in double and rounds once;
// here in fp32, arranged so that nothing cancels and nothing leaves the normal range before the last product:
// below -17, 1 + e^x is 1 to beyond fp32 and the value is x e^x; below -80, where e^x is a denormal and would
// carry only a few bits, e^(x + 64) is multiplied in first and e^-64 last. Within a few ulp of the reference's
// value (its own vector kernels are tested to 52 ulp, test/sigmoid/sigmoid_f32_zve32f.c).
__device__ __forceinline__ float skl_silu(float x) {
  if (x < -17.0f) {
    const bool deep = x < -80.0f;
    const float r = x * expf(deep ? x + 64.0f : x);
    return deep ? r * 1.6038108905486378e-28f : r;  // e^-64
  }
  return x / (1.0f + expf(-x));
}
// GELU, x Phi(x), in the reference's arrangement (ref/gelu/gelu_f32.c:12-22): an offset from the ReLU,
// fma(-|x| / 2, erfc(|x| / sqrt 2), relu(x)) - nothing cancels on either side of zero. The reference evaluates erfc
// and the fma in double; here fp32 (its own vector kernels are tested to 4 to 62 ulp by range,
// test/gelu/skl_gelu_f32_zve32f.c).
__device__ __forceinline__ float skl_gelu(float x) {
  const float h = -0.5f * __builtin_fabsf(x);
  const float e = erfcf(-1.41421356237309504880f * h);
  return __builtin_fmaf(h, e, x > 0.0f ? x : -0.0f);
}
// 0 none, 1 ReLU, 2 SiLU, 3 GELU (floating point only).
__device__ __forceinline__ float skl_activate(float v, int act) {
  if (act == 0) return v;
  if (act == 1) return v > 0.0f ? v : 0.0f;
  return act == 2 ? skl_silu(v) : skl_gelu(v);
}

// The requantised int8 value of v: round-to-nearest-even of (float)v * scale as an integer (a NaN counts as 0, values
// beyond int32 as its ends), plus the zero point, clamped to [-128, 127].
__device__ __forceinline__ int skl_requantise_int(float v, float scale, int zero) {
  const float r = __builtin_rintf(__fmul_rn(v, scale));
  int t;
  // the hardware's conversion is the rule itself: a NaN gives 0, values beyond int32 its ends (the C cast leaves
  // both undefined)
  asm("v_cvt_i32_f32 %0, %1" : "=v"(t) : "v"(r));
  // The zero point lies in [-128, 127], so anything beyond +-512 ends at the same end of int8 as the int32 ends would.
  t = (t < -512 ? -512 : t > 512 ? 512 : t) + zero;
  return t < -128 ? -128 : t > 127 ? 127 : t;
}
__device__ __forceinline__ int8_t skl_requantise(float v, float scale, int zero) { return (int8_t)skl_requantise_int(v, scale, zero); }
// The byte of the 8-bit copy for value v: int8 by the rule above, or the OCP fp8 encoding of v * scale exactly as the
// conversion kernels produce it (ref/cvt/cvt_ofp8.c:174-242: one fp32 product, round to nearest even, saturating or
// not) - a fused skl_cvt_[sat_]f32_f8e*.
__device__ __forceinline__ int8_t skl_quantise(float v, float scale, int zero, int fmt) {
  if (fmt == 0) return skl_requantise(v, scale, zero);
  return (int8_t)skl_fp8::encode_ofp8_hw(__fmul_rn(v, scale), skl_fp8::Ofp8Format(fmt));
}
// Element (row, col) of the requantised output, if there is one.
template <typename T>
__device__ __forceinline__ void skl_emit_requantised(const skl_requant &rq, T v, size_t row, size_t col) {
  if (rq.q) rq.q[row * rq.rsq + col * rq.csq] = skl_quantise((float)v, rq.q_scale[rq.q_per_column ? col : 0], rq.q_zero, rq.q_fmt);
}

template <typename T>
__device__ __forceinline__ T skl_lowest();
template <>
__device__ __forceinline__ int skl_lowest<int>() { return (int)0x80000000; }
template <>
__device__ __forceinline__ float skl_lowest<float>() { return -__builtin_inff(); }

// Largest value over the 64 lanes of a wave (all lanes must take part); NaN never wins, as in `if (x > max)`.
template <typename T>
__device__ __forceinline__ T skl_wave_max(T v) {
#pragma unroll
  for (int step = 32; step > 0; step >>= 1) {
    const T other = __shfl_xor(v, step, 64);
    if (other > v) v = other;
  }
  return v;
}

// *p = max(*p, v) for a v that is not NaN. Floats order like sign-magnitude integers: non-negative ones
// ascend as signed ints, negative ones descend as unsigned ints, so one integer atomic does it.
__device__ __forceinline__ void skl_atomic_max(int *p, int v) { atomicMax(p, v); }
__device__ __forceinline__ void skl_atomic_max(float *p, float v) {
  if (!(v < 0.0f) && !__builtin_signbit(v))
    atomicMax(reinterpret_cast<int *>(p), __float_as_int(v));
  else
    atomicMin(reinterpret_cast<unsigned *>(p), __float_as_uint(v));
}
