// skl_gemm_tiled.hip - register-tiled GEMM for the contractions that have no matrix-core path here because
// their results are defined operation by operation: f32 x f32 -> f32 (ref/gemm/gemm_f32rc_f32rc_f32rc.c:9-24),
// f64 x f64 -> f64 (ref/gemm/gemm_f64rc_f64rc_f64rc.c:9-24), f16 x f16 -> f16 with an f16 accumulator
// (ref/gemm/gemm_f16rc_f16rc_f16rc.c:9-24) and their blocked twins in the canonical layouts.
//
// Every element of C is accumulated exactly as the reference's loop does it - k ascending, a separately rounded
// multiply and add per step (f16: the sum rounded to half per step) - so results equal the reference's bit for
// bit for finite data, like the any-stride kernel's; what changes is where the operands come from: a workgroup
// of 256 threads keeps a 128 x 128 (or 64 x 64) tile of C in registers, 8 x 8 (4 x 4) per thread, and walks K in
// slabs of 16 staged through LDS (two stages, the next slab's global loads issued before the current slab's
// arithmetic). A thread's rows and columns are two runs of TM/2, half a tile apart, so that the lanes of a wave
// read consecutive 16-byte pieces of the LDS rows. The last slab is zero-filled past K: adding the product
// (+0)*(+0) leaves an accumulator unchanged, and an accumulator that started at +0 is never -0.
#include <hip/hip_runtime.h>

#include "skl_device.hpp"

namespace {

constexpr int kThreads = 256;

template <int DT>
struct Kind;
template <>
struct Kind<SKL_DT_F32> {
  using In = float;     // element type in memory
  using Stage = float;  // element type in LDS
  using Acc = float;
  using C = float;
  __device__ static Stage stage(In v) { return v; }
  __device__ static Acc step(Acc acc, Stage a, Stage b) { return __fadd_rn(acc, __fmul_rn(a, b)); }
};
template <>
struct Kind<SKL_DT_F64> {
  using In = double;
  using Stage = double;
  using Acc = double;
  using C = double;
  __device__ static Stage stage(In v) { return v; }
  __device__ static Acc step(Acc acc, Stage a, Stage b) { return __dadd_rn(acc, __dmul_rn(a, b)); }
};
// `_Float16` arithmetic as a C compiler evaluates it without half-precision instructions: operands promoted to
// float (the product of two halves is exact there), the sum rounded to float and then to half on assignment.
template <>
struct Kind<SKL_DT_F16H> {
  using In = _Float16;
  using Stage = float;
  using Acc = _Float16;
  using C = _Float16;
  __device__ static Stage stage(In v) { return (float)v; }
  __device__ static Acc step(Acc acc, Stage a, Stage b) { return (_Float16)__fadd_rn((float)acc, __fmul_rn(a, b)); }
};

struct TiledArgs {
  const void *a, *b;
  void *c;
  size_t m, n, k;
  size_t a_s1, a_s0, a_sk, b_s1, b_s0, b_sk;
  size_t rsc0, csc0, rsc1, csc1;
  skl_scalar alpha, beta;
  unsigned tiles_n;
  int a_along_k, b_along_k;  // lanes run along K when fetching (the operand's unit stride is along K)
};

// One operand's share of a slab: BT rows/columns x kSlab k (16, or 8 for the 128 x 128 tile of doubles, whose
// two stages would not fit the 64 KiB of static LDS otherwise), kPer elements per thread. Element e of the thread is
// (x, p) = (e*kThreads + tid) split along K first (`along_k`) or along x first.
template <int DT, int BT, int kSlab>
struct Fetch {
  static constexpr int kPer = BT * kSlab / kThreads;
  using In = typename Kind<DT>::In;
  using Stage = typename Kind<DT>::Stage;

  __device__ static void coords(int e, int tid, int along_k, int &x, int &p) {
    const int idx = e * kThreads + tid;
    if (along_k) {
      p = idx % kSlab;
      x = idx / kSlab;
    } else {
      x = idx % BT;
      p = idx / BT;
    }
  }

  __device__ static void load(Stage (&r)[kPer], const In *base, size_t s1, size_t s0, size_t sk, size_t x0, size_t xn,
                              size_t p0, size_t k, int tid, int along_k) {
#pragma unroll
    for (int e = 0; e < kPer; ++e) {
      int x, p;
      coords(e, tid, along_k, x, p);
      const size_t xx = x0 + x, pp = p0 + p;
      r[e] = (xx < xn && pp < k) ? Kind<DT>::stage(base[(xx / 64) * s1 + (xx % 64) * s0 + pp * sk]) : Stage(0);
    }
  }

  __device__ static void store(const Stage (&r)[kPer], Stage (*tile)[BT + 4], int tid, int along_k) {
#pragma unroll
    for (int e = 0; e < kPer; ++e) {
      int x, p;
      coords(e, tid, along_k, x, p);
      tile[p][x] = r[e];
    }
  }
};

template <int DT, int TM>
__global__ void __launch_bounds__(kThreads) gemm_tiled_kernel(TiledArgs g) {
  using K = Kind<DT>;
  using Stage = typename K::Stage;
  using Acc = typename K::Acc;
  constexpr int BT = 16 * TM;  // tile edge
  constexpr int H = TM / 2;    // a thread's rows (columns): H at ty*H and H at BT/2 + ty*H
  constexpr int kSlab = (sizeof(Stage) == 8 && TM == 8) ? 8 : 16;
  constexpr int kUnrollK = TM == 8 ? 2 : 4;
  using F = Fetch<DT, BT, kSlab>;
  __shared__ Stage As[2][kSlab][BT + 4];
  __shared__ Stage Bs[2][kSlab][BT + 4];

  const int tid = threadIdx.x, ty = tid / 16, tx = tid % 16;
  const size_t row0 = (size_t)(blockIdx.x / g.tiles_n) * BT, col0 = (size_t)(blockIdx.x % g.tiles_n) * BT;
  const typename K::In *a = (const typename K::In *)g.a, *b = (const typename K::In *)g.b;

  Acc acc[TM][TM];
#pragma unroll
  for (int r = 0; r < TM; ++r)
#pragma unroll
    for (int c = 0; c < TM; ++c) acc[r][c] = Acc(0);

  Stage ra[F::kPer], rb[F::kPer];
  const size_t slabs = (g.k + kSlab - 1) / kSlab;
  F::load(ra, a, g.a_s1, g.a_s0, g.a_sk, row0, g.m, 0, g.k, tid, g.a_along_k);
  F::load(rb, b, g.b_s1, g.b_s0, g.b_sk, col0, g.n, 0, g.k, tid, g.b_along_k);
  F::store(ra, As[0], tid, g.a_along_k);
  F::store(rb, Bs[0], tid, g.b_along_k);
  __syncthreads();
  for (size_t s = 0; s < slabs; ++s) {
    const int cur = (int)(s & 1);
    if (s + 1 < slabs) {
      F::load(ra, a, g.a_s1, g.a_s0, g.a_sk, row0, g.m, (s + 1) * kSlab, g.k, tid, g.a_along_k);
      F::load(rb, b, g.b_s1, g.b_s0, g.b_sk, col0, g.n, (s + 1) * kSlab, g.k, tid, g.b_along_k);
    }
#pragma unroll kUnrollK  // a full unroll makes the compiler fetch a whole slab into registers (256 + AGPRs)
    for (int kk = 0; kk < kSlab; ++kk) {
      Stage av[TM], bv[TM];
#pragma unroll
      for (int r = 0; r < H; ++r) {
        av[r] = As[cur][kk][ty * H + r];
        av[H + r] = As[cur][kk][BT / 2 + ty * H + r];
        bv[r] = Bs[cur][kk][tx * H + r];
        bv[H + r] = Bs[cur][kk][BT / 2 + tx * H + r];
      }
#pragma unroll
      for (int r = 0; r < TM; ++r)
#pragma unroll
        for (int c = 0; c < TM; ++c) acc[r][c] = K::step(acc[r][c], av[r], bv[c]);
    }
    if (s + 1 < slabs) {
      F::store(ra, As[cur ^ 1], tid, g.a_along_k);
      F::store(rb, Bs[cur ^ 1], tid, g.b_along_k);
    }
    __syncthreads();
  }

  typename K::C *cbase = (typename K::C *)g.c;
#pragma unroll
  for (int r = 0; r < TM; ++r) {
    const size_t i = row0 + (r < H ? ty * H + r : BT / 2 + ty * H + (r - H));
    if (i >= g.m) continue;
#pragma unroll
    for (int c = 0; c < TM; ++c) {
      const size_t j = col0 + (c < H ? tx * H + c : BT / 2 + tx * H + (c - H));
      if (j >= g.n) continue;
      typename K::C *cp = cbase + (i / 64) * g.rsc1 + (i % 64) * g.rsc0 + (j / 64) * g.csc1 + (j % 64) * g.csc0;
      if constexpr (DT == SKL_DT_F16H) {
        float wide = (float)*cp;
        float *alias = &wide;
        skl_update((float)acc[r][c], alias, g.alpha, g.beta);
        *cp = (_Float16)wide;
      } else {
        skl_update(acc[r][c], cp, g.alpha, g.beta);
      }
    }
  }
}

template <int DT, int TM>
int launch(const skl_gemm_canon *g) {
  constexpr int BT = 16 * TM;
  TiledArgs p;
  p.a = g->a, p.b = g->b, p.c = g->c;
  p.m = g->m, p.n = g->n, p.k = g->k;
  p.a_s1 = g->a_s1, p.a_s0 = g->a_s0, p.a_sk = g->a_sk;
  p.b_s1 = g->b_s1, p.b_s0 = g->b_s0, p.b_sk = g->b_sk;
  p.rsc0 = g->rsc0, p.csc0 = g->csc0, p.rsc1 = g->rsc1, p.csc1 = g->csc1;
  p.alpha = g->alpha, p.beta = g->beta;
  p.a_along_k = g->a_sk <= g->a_s0;
  p.b_along_k = g->b_sk <= g->b_s0;
  const size_t tm = (g->m + BT - 1) / BT, tn = (g->n + BT - 1) / BT;
  if (tm * tn > 0x7FFFFFFFu) {
    skl_hip_record_error(-2, "gemm_tiled: too many tiles for one launch");
    return -2;
  }
  p.tiles_n = (unsigned)tn;
  gemm_tiled_kernel<DT, TM><<<(unsigned)(tm * tn), kThreads, 0, skl_current_stream()>>>(p);
  return skl_check_launch("gemm_tiled");
}

template <int DT>
int launch_sized(const skl_gemm_canon *g) {
  // 128 x 128 tiles once they fill the chip twice over, 64 x 64 below that
  const size_t big = ((g->m + 127) / 128) * ((g->n + 127) / 128);
  return big >= 512 ? launch<DT, 8>(g) : launch<DT, 4>(g);
}

}  // namespace

extern "C" int skl_hip_gemm_tiled_supported(const skl_gemm_canon *g) {
  if (g->ta != g->tb || g->bias || g->max || g->rq.act || g->rq.q || g->c_row_shift != 6 || g->c_col_shift != 6) return 0;
  if (g->ta != SKL_DT_F32 && g->ta != SKL_DT_F64 && g->ta != SKL_DT_F16H) return 0;
  return g->m != 0 && g->n != 0 && g->k != 0;
}

extern "C" int skl_hip_launch_gemm_tiled(const skl_gemm_canon *g) {
  if (!skl_hip_gemm_tiled_supported(g)) {
    skl_hip_record_error(-2, "gemm_tiled: unsupported problem");
    return -2;
  }
  switch (g->ta) {
    case SKL_DT_F32: return launch_sized<SKL_DT_F32>(g);
    case SKL_DT_F64: return launch_sized<SKL_DT_F64>(g);
    default: return launch_sized<SKL_DT_F16H>(g);
  }
}
