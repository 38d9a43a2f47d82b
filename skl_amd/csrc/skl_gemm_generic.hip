// skl_gemm_generic.hip - the any-stride GEMM of the library: serves every call
// the matrix-core and streaming kernels decline (odd strides, misaligned bases,
// blocked layouts with k0 > 1, tiny shapes).
//
// It evaluates exactly the loop nest of the reference's blocked routine
// (ref/gemm/gemm_i8rcprc_i8rcprc_i32rcprc.c:10-37 and its typed twins): one
// thread per element of C, accumulator of C's type starting at zero, k1 outer
// and k0 inner, products of the widened operands, then C = beta*C + alpha*acc
// with C always read. Because every bf16/f16/fp8 product is exact in fp32 the
// fused multiply-add used for the accumulation rounds exactly like the
// reference's separate multiply and add, and the epilogue is kept as two
// roundings, so for finite data the fp results are bit-identical to the
// reference's, not merely within tolerance. The f32 and f64 contractions
// (ref/gemm/gemm_f32rc_f32rc_f32rc.c:9-24, gemm_f64rc_f64rc_f64rc.c:9-24 and
// the blocked twins) run here only; their products are not exact, so they are
// accumulated with a separately rounded multiply and add, as the reference's C
// source spells it.
#include <hip/hip_runtime.h>

#include <type_traits>

#include "skl_device.hpp"
#include "skl_fp8.hpp"

namespace {

template <int DT>
struct Elem;
template <>
struct Elem<SKL_DT_I8> {
  using type = int8_t;
  using acc = int32_t;
  __device__ static acc widen(type v) { return (acc)v; }
};
template <>
struct Elem<SKL_DT_BF16> {
  using type = uint16_t;
  using acc = float;
  __device__ static acc widen(type v) { return __uint_as_float((unsigned)v << 16); }
};
template <>
struct Elem<SKL_DT_F16> {
  using type = _Float16;
  using acc = float;
  __device__ static acc widen(type v) { return (float)v; }
};
template <>
struct Elem<SKL_DT_F8E4M3> {
  using type = uint8_t;
  using acc = float;
  __device__ static acc widen(type v) { return __uint_as_float(skl_fp8::decode_ofp8_bits<skl_fp8::E4M3>(v)); }
};
template <>
struct Elem<SKL_DT_F8E5M2> {
  using type = uint8_t;
  using acc = float;
  __device__ static acc widen(type v) { return __uint_as_float(skl_fp8::decode_ofp8_bits<skl_fp8::E5M2>(v)); }
};

template <>
struct Elem<SKL_DT_F32> {
  using type = float;
  using acc = float;
  __device__ static acc widen(type v) { return v; }
};
// f16 operands with an f16 accumulator (ref/gemm/gemm_f16rc_f16rc_f16rc.c:9-24). `_Float16` arithmetic is
// evaluated the way a C compiler evaluates it for a target without half-precision arithmetic, which is
// how the reference's scalar library comes out when it is built for a general-purpose host: operands are
// promoted to float, an expression is evaluated in float, and the value is rounded to half where it is
// assigned. So acc = half(float(acc) + a*b) per step (the product of two halves is exact in float) and
// C = half(beta*C + alpha*acc) with exact products, one float rounding of the sum and one to half.
template <>
struct Elem<SKL_DT_F16H> {
  using type = _Float16;
  using acc = _Float16;
  __device__ static float widen(type v) { return (float)v; }
};
template <>
struct Elem<SKL_DT_F64> {
  using type = double;
  using acc = double;
  __device__ static acc widen(type v) { return v; }
};

template <int TA, int TB>
__global__ void __launch_bounds__(256) gemm_generic_kernel(skl_gemm_desc d, unsigned tiles_n) {
  using EA = Elem<TA>;
  using EB = Elem<TB>;
  using Acc = typename EA::acc;
  const size_t M = d.m1 * d.m0, N = d.n1 * d.n0;
  const size_t tile_i = blockIdx.x / tiles_n, tile_j = blockIdx.x % tiles_n;
  const size_t i = tile_i * 16 + threadIdx.x / 16, j = tile_j * 16 + threadIdx.x % 16;
  if (i >= M || j >= N) return;
  const size_t I = i / d.m0, i0 = i % d.m0, J = j / d.n0, j0 = j % d.n0;
  const typename EA::type *a = (const typename EA::type *)d.a + I * d.rsa1 + i0 * d.rsa0;
  const typename EB::type *b = (const typename EB::type *)d.b + J * d.csb1 + j0 * d.csb0;
  Acc acc = 0;
  for (size_t P = 0; P < d.k1; ++P) {
    const typename EA::type *ap = a + P * d.csa1;
    const typename EB::type *bp = b + P * d.rsb1;
    for (size_t p = 0; p < d.k0; ++p) {
      const auto av = EA::widen(ap[p * d.csa0]);
      const auto bv = EB::widen(bp[p * d.rsb0]);
      if constexpr (TA == SKL_DT_F16H)
        acc = (_Float16)__fadd_rn((float)acc, __fmul_rn(av, bv));
      else if constexpr (TA == SKL_DT_I8)
        acc = (Acc)((uint32_t)acc + (uint32_t)av * (uint32_t)bv);
      else if constexpr (TA == SKL_DT_F32)  // products are not exact here: multiply, then add, as the reference's C does
        acc = __fadd_rn(acc, __fmul_rn(av, bv));
      else if constexpr (TA == SKL_DT_F64)
        acc = __dadd_rn(acc, __dmul_rn(av, bv));
      else
        acc = __fmaf_rn(av, bv, acc);
    }
  }
  Acc *c = (Acc *)d.c + I * d.rsc1 + J * d.csc1 + i0 * d.rsc0 + j0 * d.csc0;
  if constexpr (TA == SKL_DT_F16H) {
    float wide = (float)*c;
    float *alias = &wide;
    skl_update((float)acc, alias, d.alpha, d.beta);
    *c = (_Float16)wide;
  } else {
    if constexpr (std::is_same<Acc, int32_t>::value || std::is_same<Acc, float>::value) {
      // the alpha/beta step, then the fused steps: bias, activation, C, requantised copy, maximum
      Acc v = skl_beta_is_zero<Acc>(d.beta) ? skl_initialise(acc, c, d.alpha, d.beta) : skl_combine(acc, *c, d.alpha, d.beta);
      if (d.bias) v = skl_add_bias(v, reinterpret_cast<const Acc *>(d.bias)[j]);
      v = skl_activate(v, d.rq.act);
      if (!d.rq.q_only) *c = v;
      skl_emit_requantised(d.rq, v, i, j);
      if (d.max && v > skl_lowest<Acc>()) skl_atomic_max(reinterpret_cast<Acc *>(d.max), v);
    } else {
      skl_update(acc, c, d.alpha, d.beta);
    }
  }
}

template <int TA, int TB>
int launch(const skl_gemm_desc &d) {
  const size_t M = d.m1 * d.m0, N = d.n1 * d.n0;
  const size_t tm = (M + 15) / 16, tn = (N + 15) / 16;
  if (tm * tn > 0x7FFFFFFFu) {
    skl_hip_record_error(-2, "gemm: too many tiles for one launch");
    return -2;
  }
  gemm_generic_kernel<TA, TB><<<(unsigned)(tm * tn), 256, 0, skl_current_stream()>>>(d, (unsigned)tn);
  return skl_check_launch("gemm_generic");
}

}  // namespace

extern "C" int skl_hip_launch_gemm_generic(const skl_gemm_desc *d) {
  if (d->m0 * d->m1 == 0 || d->n0 * d->n1 == 0) return 0;
  const int key = d->ta * 8 + d->tb;
  switch (key) {
    case SKL_DT_I8 * 8 + SKL_DT_I8: return launch<SKL_DT_I8, SKL_DT_I8>(*d);
    case SKL_DT_BF16 * 8 + SKL_DT_BF16: return launch<SKL_DT_BF16, SKL_DT_BF16>(*d);
    case SKL_DT_F16 * 8 + SKL_DT_F16: return launch<SKL_DT_F16, SKL_DT_F16>(*d);
    case SKL_DT_F8E4M3 * 8 + SKL_DT_F8E4M3: return launch<SKL_DT_F8E4M3, SKL_DT_F8E4M3>(*d);
    case SKL_DT_F8E5M2 * 8 + SKL_DT_F8E5M2: return launch<SKL_DT_F8E5M2, SKL_DT_F8E5M2>(*d);
    case SKL_DT_F8E4M3 * 8 + SKL_DT_F8E5M2: return launch<SKL_DT_F8E4M3, SKL_DT_F8E5M2>(*d);
    case SKL_DT_F8E5M2 * 8 + SKL_DT_F8E4M3: return launch<SKL_DT_F8E5M2, SKL_DT_F8E4M3>(*d);
    case SKL_DT_F32 * 8 + SKL_DT_F32: return launch<SKL_DT_F32, SKL_DT_F32>(*d);
    case SKL_DT_F64 * 8 + SKL_DT_F64: return launch<SKL_DT_F64, SKL_DT_F64>(*d);
    case SKL_DT_F16H * 8 + SKL_DT_F16H: return launch<SKL_DT_F16H, SKL_DT_F16H>(*d);
    default:
      skl_hip_record_error(-2, "gemm: operand type pair");
      return -2;
  }
}
