// skl_gemv_kcrows.hip - decode batches against weights stored column by column: 5 to 96 rows of A (K contiguous)
// times a B whose columns are contiguous in K - a linear layer's [out][in] weight -, int8 and the OCP fp8 kinds
// (4096 k per launch; a longer K takes a launch per 4096 k, the later ones adding to C). The reference's generic kernels take any strides (ref/gemm/gemm_i8rc_i8rc_i32rc.c:9-24,
// ref/gemm/gemm_f8rc_f8rc_f32rc.c); up to four rows skl_gemv.hip's gemv_kc_kernel streams such a B with dot
// products, and without this file everything above went to the tile kernels (16 x 4096 x 11008: 27 us for 45 MB).
//
// With K contiguous in both operands a 16-byte load IS a matrix-core operand: 16 consecutive k of one column of B,
// or of one row of A. A workgroup of eight waves owns 64 columns (four groups of 16) and ALL of K, 512 k per wave,
// so the sums of a column tile never leave the workgroup: they meet in LDS in wave order - the same bits on every
// run -, C is written once with the alpha / beta step (and the fused steps of a fused call) applied in place, and no
// scratch memory is involved. All of
// B is in flight from the start (32 loads per lane) and stays in registers while up to six groups of 16 rows of A
// take their turns; a group's pieces of A (from L2: every workgroup reads all of A) are requested two groups ahead.
// Instruction t of a 256-k chunk takes k = chunk + 64 t + 16 g + (0..15) from the lanes of k group g: the four
// groups read 64 consecutive bytes of a column per load. Which k meet in which instruction is free as long as
// A's and B's lanes hold the same ones.
// int8: v_mfma_i32_16x16x64_i8. fp8: every E4M3 / E5M2 value is an f16 value, so the bytes are widened in registers
// and multiplied by v_mfma_f32_16x16x32_f16 - exact products, fp32 sums, inside the reference's bound for any K (the
// fp8 instructions align the products of an instruction and drop low bits, which short K would show).
// Loads are clamped into the operands instead of guarded (a guard is a branch, and the compiler waits for the loads in
// flight at a branch it cannot prove uniform): k beyond K meets zeros of A, rows beyond M and columns beyond N are
// computed and not written.
#include <hip/hip_runtime.h>

#include <atomic>
#include <type_traits>

#include "skl_device.hpp"
#include "skl_fp8.hpp"

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kWaves = 8;  // a workgroup owns 16, 32 or 64 columns
constexpr int kChunk = 256, kChunks = 2;                           // k per wave: 512
constexpr int kMaxRowGroups = 6, kMinRows = 5;  // 96 rows: beyond, the tile kernels are level (64 rows 21.5 against 23.5 us,
                                                // a row group more costs 2.3 us, the tile kernels take 28-29 us for 128 rows)
constexpr size_t kMaxK = (size_t)kWaves * kChunks * kChunk;        // 4096
enum { kI8 = 0, kE4M3 = 1, kE5M2 = 2, kMixed = 3 };  // kMixed: E4M3 A with E5M2 B

struct KcRowsArgs {
  const char *a;  // row i at a + i * a_row (bytes), K contiguous
  size_t a_row;
  const char *b;  // column j at b + j * b_col (bytes), K contiguous
  size_t b_col;
  void *c;        // element (i, j) is written at i * c_row + j * c_col (elements) ...
  size_t c_row, c_col;
  const void *cin;  // ... and its old value read at i * cin_row + j * cin_col of cin (the same place, except in the
  size_t cin_row, cin_col;  // passes of a long K whose call does not write C: those meet in a matrix of their own)
  size_t m, n, k;
  skl_scalar alpha, beta;
  const void *bias;  // fused steps behind alpha / beta (bias and maximum of C's type, or null) ...
  void *max;
  skl_requant rq;    // ... activation and 8-bit copy
};

__device__ __forceinline__ v4i load16(const char *p) { return __builtin_nontemporal_load(reinterpret_cast<const v4i *>(p)); }

// CG groups of 16 columns per workgroup: four where that still leaves at least 128 workgroups (a wave's pieces of A
// then serve four instructions each), fewer for a narrow B - 4096 columns are 64 workgroups of 64 columns, which
// cannot pull the weights fast enough.
template <int KIND, int RG, int CG>
__global__ void __launch_bounds__(kWaves * 64) gemv_kc_rows_kernel(KcRowsArgs p) {
  constexpr int kColGroups = CG, kCols = 16 * CG, kPitch = kCols + 1;
  constexpr bool kInt = KIND == kI8;
  using Acc = typename std::conditional<kInt, int, float>::type;
  typedef Acc v4acc __attribute__((ext_vector_type(4)));
  extern __shared__ __attribute__((aligned(16))) int kc_red_raw[];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int jl = lane & 15, g = lane >> 4;
  const size_t kwave = (size_t)wave * (kChunks * kChunk) + (size_t)g * 16;  // the lane's first k
  const v4i zero = {0, 0, 0, 0};
  // piece (u, t) of a lane: 16 k from kwave + 256 u + 64 t
  auto fragment_of = [&](int rg, v4i(&xa)[kChunks][4]) {
    const size_t row = (size_t)rg * 16 + jl;
    const bool row_ok = row < p.m;
    const char *ap = p.a + (row_ok ? row : p.m - 1) * p.a_row;
#pragma unroll
    for (int u = 0; u < kChunks; ++u)
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const size_t k0 = kwave + (size_t)u * kChunk + (size_t)t * 64;  // k is a multiple of 16: inside or outside
        const v4i v = *reinterpret_cast<const v4i *>(ap + (k0 < p.k ? k0 : 0));
        xa[u][t] = k0 < p.k && row_ok ? v : zero;
      }
  };
  v4i xa[2][kChunks][4];
  fragment_of(0, xa[0]);  // ahead of B: loads come back in the order of their requests
  v4i b[kColGroups][kChunks][4];
#pragma unroll
  for (int cg = 0; cg < kColGroups; ++cg) {
    const size_t col = (size_t)blockIdx.x * kCols + (size_t)cg * 16 + jl;
    const char *bp = p.b + (col < p.n ? col : p.n - 1) * p.b_col;
#pragma unroll
    for (int u = 0; u < kChunks; ++u)
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const size_t k0 = kwave + (size_t)u * kChunk + (size_t)t * 64;
        b[cg][u][t] = load16(bp + (k0 < p.k ? k0 : 0));
      }
  }
  if constexpr (RG > 1) fragment_of(1, xa[1]);
  __builtin_amdgcn_sched_barrier(0);  // every request is out before the first use
  constexpr int kRowsAtATime = kWaves * 64 / kCols, kPasses = 16 / kRowsAtATime;  // 512 threads: 8, 16 or 32 -> 16 rows x kCols columns at a time
  static_assert(kRowsAtATime <= 16 || CG == 1, "one group of 16 columns: half of the threads have nothing to write");
  const int row = threadIdx.x / kCols, tc = threadIdx.x % kCols;
  const size_t j = (size_t)blockIdx.x * kCols + tc;
  Acc *cbase = reinterpret_cast<Acc *>(p.c);
  const Acc *cin_base = reinterpret_cast<const Acc *>(p.cin);
  const bool fused = p.bias || p.max || p.rq.act || p.rq.q;  // the same for every thread
  Acc largest = skl_lowest<Acc>();                           // what this thread wrote, for the maximum
#pragma unroll
  for (int rg = 0; rg < RG; ++rg) {
    if ((size_t)rg * 16 >= p.m) break;  // the same for every thread of the workgroup
    v4acc acc[kColGroups];
#pragma unroll
    for (int cg = 0; cg < kColGroups; ++cg) acc[cg] = v4acc{0, 0, 0, 0};
#pragma unroll
    for (int u = 0; u < kChunks; ++u)
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const v4i av = xa[rg & 1][u][t];
        if constexpr (kInt) {
#pragma unroll
          for (int cg = 0; cg < kColGroups; ++cg) acc[cg] = __builtin_amdgcn_mfma_i32_16x16x64_i8(av, b[cg][u][t], acc[cg], 0, 0, 0);
        } else {
          constexpr bool a_e5m2 = KIND == kE5M2, b_e5m2 = KIND != kE4M3;
          const auto a0 = skl_fp8::widen8_to_f16<a_e5m2>((unsigned)av.x, (unsigned)av.y);
          const auto a1 = skl_fp8::widen8_to_f16<a_e5m2>((unsigned)av.z, (unsigned)av.w);
#pragma unroll
          for (int cg = 0; cg < kColGroups; ++cg) {
            // an opaque copy: the widened form of B (twice the registers) must not be kept from one row group to
            // the next
            v4i bv = b[cg][u][t];
            asm volatile("" : "+v"(bv));
            acc[cg] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0, skl_fp8::widen8_to_f16<b_e5m2>((unsigned)bv.x, (unsigned)bv.y), acc[cg], 0, 0, 0);
            acc[cg] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1, skl_fp8::widen8_to_f16<b_e5m2>((unsigned)bv.z, (unsigned)bv.w), acc[cg], 0, 0, 0);
          }
        }
      }
    if (rg + 2 < RG) fragment_of(rg + 2, xa[rg & 1]);
    // acc[cg][r] is row 16 rg + 4 g + r of C, column 16 cg + jl of the workgroup's. Two blocks of sums take turns:
    // the next group's barrier stands between this group's readers and the writers of the group after it.
    Acc(*red)[16][kPitch] = reinterpret_cast<Acc(*)[16][kPitch]>(kc_red_raw + (rg & 1) * kWaves * 16 * kPitch);
#pragma unroll
    for (int cg = 0; cg < kColGroups; ++cg)
#pragma unroll
      for (int r = 0; r < 4; ++r) red[wave][4 * g + r][cg * 16 + jl] = acc[cg][r];
    __syncthreads();
    constexpr int kSums = kPasses > 0 ? kPasses : 1;
    Acc sums[kSums];
#pragma unroll
    for (int q = 0; q < kSums; ++q) {
      const int il = (row + kRowsAtATime * q) & 15;
      Acc sum = red[0][il][tc];
#pragma unroll
      for (int w = 1; w < kWaves; ++w) {
        if constexpr (kInt) sum = (int)((unsigned)sum + (unsigned)red[w][il][tc]);
        else sum = __fadd_rn(sum, red[w][il][tc]);
      }
      sums[q] = sum;
    }
#pragma unroll
    for (int q = 0; q < kSums; ++q) {
      const size_t i = (size_t)rg * 16 + row + kRowsAtATime * q;
      if (row + kRowsAtATime * q >= 16 || i >= p.m || j >= p.n) continue;
      Acc *c = cbase + i * p.c_row + j * p.c_col;
      const Acc *old = cin_base + i * p.cin_row + j * p.cin_col;
      if (!fused) {
        *c = skl_beta_is_zero<Acc>(p.beta) ? skl_initialise(sums[q], old, p.alpha, p.beta) : skl_combine(sums[q], *old, p.alpha, p.beta);
      } else {  // the steps of include/skl-gfx950.h's fused calls on the same sums: a fused call gives the plain call's bits plus the steps
        Acc v = skl_beta_is_zero<Acc>(p.beta) ? skl_initialise(sums[q], old, p.alpha, p.beta) : skl_combine(sums[q], *old, p.alpha, p.beta);
        if (p.bias) v = skl_add_bias(v, reinterpret_cast<const Acc *>(p.bias)[j]);
        v = skl_activate(v, p.rq.act);
        if (!p.rq.q_only) *c = v;
        skl_emit_requantised(p.rq, v, i, j);
        if (v > largest) largest = v;
      }
    }
  }
  if (fused && p.max) {  // one atomic per wave that wrote something
    const Acc best = skl_wave_max(largest);
    if ((threadIdx.x & 63) == 0 && best > skl_lowest<Acc>()) skl_atomic_max(reinterpret_cast<Acc *>(p.max), best);
  }
}

constexpr size_t lds_bytes(int cg) { return (size_t)2 * kWaves * 16 * (16 * cg + 1) * 4; }  // 66 560 bytes with four groups

template <int KIND, int RG, int CG>
int launch_groups(const KcRowsArgs &p, unsigned grid, hipStream_t st) {
  constexpr size_t kLds = lds_bytes(CG);
  static std::atomic<bool> configured{false};  // per instantiation; racing threads set the same value
  if (!configured.load(std::memory_order_acquire)) {
    int rc = skl_check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(gemv_kc_rows_kernel<KIND, RG, CG>),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLds), "gemv_kc_rows: LDS size");
    if (rc != 0) return rc;
    configured.store(true, std::memory_order_release);
  }
  gemv_kc_rows_kernel<KIND, RG, CG><<<grid, kWaves * 64, kLds, st>>>(p);
  return skl_check_launch("gemv_kc_rows");
}

template <int KIND, int CG>
int launch_width(const KcRowsArgs &p, unsigned grid, hipStream_t st) {
  switch ((p.m + 15) / 16) {
    case 1: return launch_groups<KIND, 1, CG>(p, grid, st);
    case 2: return launch_groups<KIND, 2, CG>(p, grid, st);
    case 3: return launch_groups<KIND, 3, CG>(p, grid, st);
    case 4: return launch_groups<KIND, 4, CG>(p, grid, st);
    case 5: return launch_groups<KIND, 5, CG>(p, grid, st);
    default: return launch_groups<KIND, 6, CG>(p, grid, st);
  }
}

// Columns per workgroup: 64 where that leaves at least 128 workgroups, else 32, else 16.
inline int col_groups_for(size_t n) { return n >= 128 * 64 ? 4 : 1; }

template <int KIND>
int launch_kind(const KcRowsArgs &p) {
  hipStream_t st = skl_current_stream();
  const int cg = col_groups_for(p.n);
  const unsigned grid = (unsigned)((p.n + 16 * (size_t)cg - 1) / (16 * (size_t)cg));
  switch (cg) {
    case 4: return launch_width<KIND, 4>(p, grid, st);
    case 2: return launch_width<KIND, 2>(p, grid, st);
    default: return launch_width<KIND, 1>(p, grid, st);
  }
}

int kind_of(const skl_gemm_canon *g) {
  if (g->ta == SKL_DT_I8 && g->tb == SKL_DT_I8) return kI8;
  if (g->ta == SKL_DT_F8E4M3 && g->tb == SKL_DT_F8E4M3) return kE4M3;
  if (g->ta == SKL_DT_F8E5M2 && g->tb == SKL_DT_F8E5M2) return kE5M2;
  if (g->ta == SKL_DT_F8E4M3 && g->tb == SKL_DT_F8E5M2) return kMixed;
  return -1;
}

inline bool aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }

}  // namespace

// 5 to 96 rows of A and a B of at least 1 MiB, both with K contiguous (16-byte aligned rows and columns a fixed
// distance apart, K a multiple of 16), C flat or in blocks of 64; fused steps in the last stage.
extern "C" int skl_hip_gemv_kc_rows_supported(const skl_gemm_canon *g) {
  if (kind_of(g) < 0) return 0;
  if (g->c_row_shift != 6 || g->c_col_shift != 6) return 0;
  if (g->m < (size_t)kMinRows || g->m > (size_t)(16 * kMaxRowGroups) || g->n == 0 || g->k == 0) return 0;
  // a longer K goes in passes of 4096 k, which pays only while a pass fills the chip (16 x 11008 x 4096: three
  // passes of 256 narrow workgroups 22.8 us, the tile kernels with shared K 19.1 us)
  if (g->k > kMaxK && col_groups_for(g->n) != 4) return 0;
  if ((g->k % 16) != 0 || g->k * g->n < (size_t(1) << 20)) return 0;
  if (g->a_sk != 1 || g->b_sk != 1) return 0;
  if (!aligned16(g->a) || (g->a_s0 % 16) != 0 || (g->m > 64 && g->a_s1 != 64 * g->a_s0)) return 0;
  if (!aligned16(g->b) || (g->b_s0 % 16) != 0 || (g->n > 64 && g->b_s1 != 64 * g->b_s0)) return 0;
  if ((g->m > 64 && g->rsc1 != 64 * g->rsc0) || (g->n > 64 && g->csc1 != 64 * g->csc0)) return 0;
  return 1;
}

extern "C" int skl_hip_launch_gemv_kc_rows(const skl_gemm_canon *g) {
  if (!skl_hip_gemv_kc_rows_supported(g)) {
    skl_hip_record_error(-2, "gemv_kc_rows: unsupported problem");
    return -2;
  }
  const size_t grid = (g->n + 15) / 16;  // at most: one group of 16 columns per workgroup
  if (grid > 0x7FFFFFFFu) {
    skl_hip_record_error(-2, "gemv_kc_rows: grid too large");
    return -2;
  }
  // A K beyond what the registers hold goes in passes of 4096 k: the first applies the caller's beta, the others add
  // to what it wrote (beta = 1), the last one carries the fused steps - launches on one stream, in order; the same
  // bits on every run, and a fused call still gives the plain call's bits plus the steps. The passes meet in C -
  // except for a call that does not write C (the 8-bit copy alone): its passes meet in a row-major matrix in the
  // stream's workspace, and only the last one's copy leaves the kernel.
  const int kind = kind_of(g);
  const bool many = g->k > kMaxK, aside = many && g->rq.q && g->rq.q_only;
  struct Sequence {  // the workspace travels from pass to pass: other host threads on this stream must not get in between
    const bool held;
    explicit Sequence(bool hold) : held(hold) { if (held) skl_hip_sequence_begin(); }
    ~Sequence() { if (held) skl_hip_sequence_end(); }
  } sequence(aside);
  void *meet = g->c;
  size_t meet_row = g->rsc0, meet_col = g->csc0;
  if (aside) {
    meet = skl_workspace(g->m * g->n * 4);
    if (!meet) return -4;
    meet_row = g->n, meet_col = 1;
  }
  for (size_t k0 = 0; k0 < g->k; k0 += kMaxK) {
    const size_t kk = g->k - k0 < kMaxK ? g->k - k0 : kMaxK;
    const bool first = k0 == 0, last = k0 + kk == g->k;
    skl_scalar beta = g->beta;
    if (!first) {
      if (kind == kI8) beta.i = 1;
      else beta.fz.value = 1.0f, beta.fz.skip_c_read = 0;
    }
    KcRowsArgs p = {(const char *)g->a + k0, g->a_s0, (const char *)g->b + k0, g->b_s0,
                    last ? g->c : meet, last ? g->rsc0 : meet_row, last ? g->csc0 : meet_col,  // written (the last pass of a call that does not write C writes nothing)
                    first ? g->c : meet, first ? g->rsc0 : meet_row, first ? g->csc0 : meet_col,  // read
                    g->m, g->n, kk, g->alpha, beta, last ? g->bias : nullptr, last ? g->max : nullptr, g->rq};
    if (!last) p.rq.act = 0, p.rq.q = nullptr, p.rq.q_only = 0;
    int rc;
    switch (kind) {
      case kI8: rc = launch_kind<kI8>(p); break;
      case kE4M3: rc = launch_kind<kE4M3>(p); break;
      case kE5M2: rc = launch_kind<kE5M2>(p); break;
      default: rc = launch_kind<kMixed>(p); break;
    }
    if (rc != 0) return rc;
  }
  return 0;
}
