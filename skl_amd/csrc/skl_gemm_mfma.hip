// skl_gemm_mfma.hip - the dense contractions on the gfx950 matrix cores:
// int8 x int8 -> int32 (v_mfma_i32_32x32x32_i8), bf16 / f16 -> f32
// (v_mfma_f32_32x32x16_{bf16,f16}) and OCP fp8 E4M3 / E5M2, in any pairing,
// -> f32 (v_mfma_f32_32x32x64_f8f6f4).
//
// Semantics: C = alpha*A*B + beta*C of ref/gemm/gemm_i8rcprc_i8rcprc_i32rcprc.c:10-37
// and its typed twins, for the layouts the optimized SKL entry points use
// (src/gemm/gemm_i8_i8_i32_zve32x.h:38-48 row-major, src/gemm/gemm_i8c_i8_i32_xsfmm32a8i.h:38-48
// column-major A, :85-95 TE x 1 / 1 x TE panels with TE x TE blocks of C). The
// integer result is exact; the fp result accumulates exact products in fp32
// in an order that differs from the reference's k-ascending loop.
//
// One kernel template serves every layout pair. Each operand is either
// "K-contiguous" (row-major A, column-major B) or "MN-contiguous" (column-major
// A, row-major B, and both panel formats); blocks of 64 along M / N may sit
// anywhere (block stride), which is what the panel formats need. A workgroup
// owns a BM x BN tile of C (256 x 256 on four waves of 128 x 128 each - the
// largest accumulator block a wave's 512 registers hold, which minimises LDS
// reads per MFMA - or 128 x 128 on eight waves for small or ragged problems); per 128-byte slice of K it copies the
// A and B tiles global -> registers -> LDS in their native orientation with
// 128-bit accesses (double-buffered: the next slice is in flight while the
// current one is multiplied) and the waves read MFMA operands straight from
// LDS: ds_read_b128 for a K-contiguous tile (row pitch padded to 144 bytes),
// ds_read_b64_tr_b8 / _tr_b16 - the LDS transpose loads - for an
// MN-contiguous one (row pitch padded so the eight/four rows of one transpose
// land in distinct banks). No data is transposed by VALU work. The k order
// inside an MFMA is the same for both operands whichever way they were read, so
// any layout pair multiplies matching k. alpha / beta are applied per wave on
// the accumulator registers in the epilogue.
#include <hip/hip_runtime.h>

#include <cstdlib>
#include <utility>

#include "skl_device.hpp"

namespace {

typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef short v4s __attribute__((ext_vector_type(4)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

#define LDS_PTR(T, p) ((__attribute__((address_space(3))) T *)(p))

constexpr int kSliceBytes = 128;    // bytes of K per LDS stage and operand row
constexpr int kPitchKC = 144;       // LDS row pitch of a K-contiguous tile

struct MfmaArgs {
  const char *a;
  const char *b;
  char *c;
  size_t m, n, k;
  size_t a_s1, a_s0, a_sk;  // elements
  size_t b_s1, b_s0, b_sk;
  size_t rsc0, csc0, rsc1, csc1;
  skl_scalar alpha, beta;
  unsigned tiles_m, tiles_n;
};

// Operand kinds of the MFMA: element size, accumulator type, k per instruction.
template <int DT>
struct Kind;
template <>
struct Kind<SKL_DT_I8> {
  static constexpr int ES = 1, KB = 32;  // KB: bytes of K consumed per MFMA per operand row
  using Acc = v16i;
};
template <>
struct Kind<SKL_DT_BF16> {
  static constexpr int ES = 2, KB = 32;
  using Acc = v16f;
};
template <>
struct Kind<SKL_DT_F16> {
  static constexpr int ES = 2, KB = 32;
  using Acc = v16f;
};
template <>
struct Kind<SKL_DT_F8E4M3> {
  static constexpr int ES = 1, KB = 64;
  using Acc = v16f;
};
template <>
struct Kind<SKL_DT_F8E5M2> {
  static constexpr int ES = 1, KB = 64;
  using Acc = v16f;
};

// One MFMA: FR = bytes per lane / 4 registers of each operand fragment.
template <int TA, int TB>
struct Mma;
template <>
struct Mma<SKL_DT_I8, SKL_DT_I8> {
  using Frag = v4i;
  __device__ static v16i run(v4i a, v4i b, v16i c) { return __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0); }
};
template <>
struct Mma<SKL_DT_BF16, SKL_DT_BF16> {
  using Frag = v4i;
  __device__ static v16f run(v4i a, v4i b, v16f c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, b), c, 0, 0, 0);
  }
};
template <>
struct Mma<SKL_DT_F16, SKL_DT_F16> {
  using Frag = v4i;
  __device__ static v16f run(v4i a, v4i b, v16f c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, a), __builtin_bit_cast(v8h, b), c, 0, 0, 0);
  }
};
// f8f6f4 format codes: 0 = E4M3, 1 = E5M2. Scales 0/0 select the unscaled instruction.
#define SKL_F8_MMA(TA_, TB_, FA_, FB_)                                                                   \
  template <>                                                                                            \
  struct Mma<TA_, TB_> {                                                                                 \
    using Frag = v8i;                                                                                    \
    __device__ static v16f run(v8i a, v8i b, v16f c) {                                                   \
      return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, FA_, FB_, 0, 0, 0, 0);             \
    }                                                                                                    \
  };
SKL_F8_MMA(SKL_DT_F8E4M3, SKL_DT_F8E4M3, 0, 0)
SKL_F8_MMA(SKL_DT_F8E5M2, SKL_DT_F8E5M2, 1, 1)
SKL_F8_MMA(SKL_DT_F8E4M3, SKL_DT_F8E5M2, 0, 1)
SKL_F8_MMA(SKL_DT_F8E5M2, SKL_DT_F8E4M3, 1, 0)

// ---------------------------------------------------------------------------
// LDS tile geometry of one operand: ROWS along M or N, 128 bytes of K.
// ---------------------------------------------------------------------------
template <int ES, int ROWS, bool KC, int NT>
struct Tile {
  static constexpr int CE = 16 / ES;                 // elements per 16-byte chunk
  static constexpr int KE = kSliceBytes / ES;        // k elements per slice
  // MN-contiguous tile: KE rows of ROWS*ES bytes. A transpose load is served 32
  // lanes at a time: 8 rows x 32 B (8-bit) or 4 rows x 64 B (16-bit). Skewing
  // consecutive rows by that width spreads them over all 64 banks (measured:
  // zero bank conflicts with 32 / 64 bytes of padding, conflicts with 16 / 32).
  static constexpr int kPitchMC = ROWS * ES + (ES == 1 ? 32 : 64);
  static constexpr int kBytes = KC ? ROWS * kPitchKC : KE * kPitchMC;
  static constexpr int kChunks = ROWS * 8;           // 16-byte chunks per slice
  static constexpr int kPerThread = kChunks / NT;    // chunks each of the NT threads moves
  static constexpr int kMnChunks = ROWS * ES / 16;   // chunks along MN of an MN-contiguous row
};

// 16 bytes from global memory with `valid` (<= CE) leading elements in range.
template <int ES>
__device__ __forceinline__ v4i load_chunk(const char *p, long valid) {
  constexpr int CE = 16 / ES;
  if (valid >= CE) return *reinterpret_cast<const v4i *>(p);
  v4i v = {0, 0, 0, 0};
  if (valid > 0) {
    unsigned w[4] = {0, 0, 0, 0};
    for (int e = 0; e < CE; ++e) {
      if (e < valid) {
        unsigned x = ES == 1 ? (unsigned)*reinterpret_cast<const uint8_t *>(p + e)
                             : (unsigned)*reinterpret_cast<const uint16_t *>(p + 2 * e);
        w[(e * ES) / 4] |= x << (8 * ((e * ES) % 4));
      }
    }
    v = v4i{(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
  }
  return v;
}

// Per-thread source bookkeeping for one operand. A chunk's address is a
// workgroup-uniform 64-bit tile base (advanced by one slice per iteration) plus
// a 32-bit per-thread offset, so the loop carries one scalar pointer instead of
// a vector pointer per chunk.
template <int ES, int ROWS, bool KC, int NT>
struct Loader {
  using T = Tile<ES, ROWS, KC, NT>;
  const char *tile_base;         // uniform: first byte of the tile's first 64-block at k = 0
  size_t k_step;                 // bytes between consecutive slices
  unsigned off[T::kPerThread];   // byte offset of each chunk from tile_base
  unsigned lds_off[T::kPerThread];
  long mn_valid[T::kPerThread];  // guarded path - KC: row in range (1/0); MC: elements in range along MN
  int k_off[T::kPerThread];      // guarded path - KC: k element offset of the chunk; MC: k row

  __device__ void init(const char *base, size_t mn0, size_t mn_dim, size_t s1, size_t s0, size_t sk) {
    const int t = threadIdx.x;
    tile_base = base + (mn0 >> 6) * s1 * ES;  // mn0 is a multiple of 64
#pragma unroll
    for (int i = 0; i < T::kPerThread; ++i) {
      const int q = t + NT * i;
      if (KC) {
        const int row = q >> 3, c = q & 7;
        off[i] = (unsigned)(((size_t)(row >> 6) * s1 + (size_t)(row & 63) * s0 + (size_t)c * T::CE) * ES);
        mn_valid[i] = mn0 + row < mn_dim ? 1 : 0;
        k_off[i] = c * T::CE;
        lds_off[i] = row * kPitchKC + c * 16;
      } else {
        const int mc = q % T::kMnChunks, kr = q / T::kMnChunks;
        const int r = mc * T::CE;
        off[i] = (unsigned)(((size_t)(r >> 6) * s1 + (size_t)(r & 63) + (size_t)kr * sk) * ES);
        mn_valid[i] = (long)mn_dim - (long)(mn0 + r);
        k_off[i] = kr;
        lds_off[i] = kr * T::kPitchMC + mc * 16;
      }
    }
    k_step = KC ? (size_t)kSliceBytes : (size_t)T::KE * sk * ES;
  }

  // Interior tiles of problems whose extents are multiples of the tile: every chunk is whole.
  __device__ __forceinline__ void fetch_whole(v4i (&regs)[T::kPerThread], size_t slice) const {
    const char *b = tile_base + slice * k_step;
#pragma unroll
    for (int i = 0; i < T::kPerThread; ++i) regs[i] = *reinterpret_cast<const v4i *>(b + off[i]);
  }

  // Any extents: chunks that stick out of the matrix are zero-filled (zeros along
  // K add nothing; rows/columns beyond M/N are never stored).
  __device__ __forceinline__ void fetch_guarded(v4i (&regs)[T::kPerThread], size_t slice, size_t k_dim) const {
    const long k0 = (long)(slice * T::KE);
    const char *b = tile_base + slice * k_step;
#pragma unroll
    for (int i = 0; i < T::kPerThread; ++i) {
      long valid;
      if (KC)
        valid = mn_valid[i] ? (long)k_dim - (k0 + k_off[i]) : 0;
      else
        valid = (k0 + k_off[i] < (long)k_dim) ? mn_valid[i] : 0;
      regs[i] = load_chunk<ES>(b + off[i], valid);
    }
  }

  template <bool GUARDED>
  __device__ __forceinline__ void fetch(v4i (&regs)[T::kPerThread], size_t slice, size_t k_dim) const {
    if constexpr (GUARDED)
      fetch_guarded(regs, slice, k_dim);
    else
      fetch_whole(regs, slice);
  }

  __device__ __forceinline__ void stash(char *tile, const v4i (&regs)[T::kPerThread]) const {
#pragma unroll
    for (int i = 0; i < T::kPerThread; ++i) *reinterpret_cast<v4i *>(tile + lds_off[i]) = regs[i];
  }
};

// Reads the MFMA operand fragment of 32 rows starting at `row0` for the k-step
// that starts `kb` bytes into the slice. FRB = bytes per lane (16 or 32).
template <int ES, int ROWS, bool KC, int FRB>
__device__ __forceinline__ auto read_frag(const char *tile, int row0, int kb) {
  using T = Tile<ES, ROWS, KC, 64>;
  const int lane = threadIdx.x & 63;
  const int h = lane >> 5;  // which half of the k-step this lane feeds
  if constexpr (KC) {
    const char *p = tile + (row0 + (lane & 31)) * kPitchKC + kb + h * FRB;
    if constexpr (FRB == 16) {
      return *reinterpret_cast<const v4i *>(p);
    } else {
      const v4i lo = *reinterpret_cast<const v4i *>(p), hi = *reinterpret_cast<const v4i *>(p + 16);
      return v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    }
  } else if constexpr (ES == 1) {
    // ds_read_b64_tr_b8: 16 lanes read an 8 (k) x 16 (mn) byte block; lane j receives column j.
    const int g16 = (lane >> 4) & 1, j = lane & 15;
    const int kfirst = kb + h * FRB + (j >> 1);
    const char *p = tile + kfirst * T::kPitchMC + row0 + g16 * 16 + (j & 1) * 8;
    v2i r[FRB / 8];
#pragma unroll
    for (int s = 0; s < FRB / 8; ++s) r[s] = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_PTR(v2i, p + s * 8 * T::kPitchMC));
    if constexpr (FRB == 16) {
      return v4i{r[0].x, r[0].y, r[1].x, r[1].y};
    } else {
      return v8i{r[0].x, r[0].y, r[1].x, r[1].y, r[2].x, r[2].y, r[3].x, r[3].y};
    }
  } else {
    // ds_read_b64_tr_b16: 16 lanes read a 4 (k) x 16 (mn) block of 16-bit elements.
    static_assert(FRB == 16, "16-bit fragments are 16 bytes");
    const int g16 = (lane >> 4) & 1, j = lane & 15;
    const int kfirst = kb / 2 + h * 8 + (j >> 2);
    const char *p = tile + kfirst * T::kPitchMC + (row0 + g16 * 16 + (j & 3) * 4) * 2;
    const v4s r0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(v4s, p));
    const v4s r1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(v4s, p + 4 * T::kPitchMC));
    const v2i a = __builtin_bit_cast(v2i, r0), b = __builtin_bit_cast(v2i, r1);
    return v4i{a.x, a.y, b.x, b.y};
  }
}

__device__ __forceinline__ int epilogue(int acc, int c, skl_scalar alpha, skl_scalar beta) {
  return (int)((unsigned)beta.i * (unsigned)c + (unsigned)alpha.i * (unsigned)acc);
}
__device__ __forceinline__ float epilogue(float acc, float c, skl_scalar alpha, skl_scalar beta) {
  return __fadd_rn(__fmul_rn(beta.f, c), __fmul_rn(alpha.f, acc));
}

// Tile index of a workgroup. Consecutive workgroup ids go to different XCDs
// (eight of them, each with its own L2), so ids are first regrouped per XCD into
// contiguous ranges, then walked in column-major groups of kGroupM tile rows so
// that the tiles resident on one XCD at a time share A and B panels.
__device__ __forceinline__ void tile_of_block(unsigned bid, unsigned tiles_m, unsigned tiles_n, unsigned &tm,
                                              unsigned &tn) {
  constexpr unsigned kXcd = 8, kGroupM = 8;
  const unsigned total = tiles_m * tiles_n;
  unsigned t = bid;
  if (total % kXcd == 0) t = (bid % kXcd) * (total / kXcd) + bid / kXcd;
  const unsigned per_group = kGroupM * tiles_n;
  const unsigned group = t / per_group, first_m = group * kGroupM;
  const unsigned rows = tiles_m - first_m < kGroupM ? tiles_m - first_m : kGroupM;
  const unsigned in_group = t % per_group;
  tm = first_m + in_group % rows;
  tn = in_group / rows;
}

template <int TA, int TB, bool A_KC, bool B_KC, int BM, int BN, int WAVES_M, int WAVES_N, bool GUARDED>
__global__ void __launch_bounds__(WAVES_M *WAVES_N * 64) gemm_mfma_kernel(MfmaArgs p) {
  constexpr int NT = WAVES_M * WAVES_N * 64;
  using KA = Kind<TA>;
  using M = Mma<TA, TB>;
  using Acc = typename KA::Acc;
  using AccElem = decltype(Acc{}.x);
  constexpr int ES = KA::ES;
  constexpr int KB = KA::KB;                    // bytes of K per MFMA
  constexpr int FRB = KB / 2;                   // fragment bytes per lane
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;  // wave tile
  constexpr int MI = WM / 32, NI = WN / 32;     // MFMA blocks per wave
  using TileA = Tile<ES, BM, A_KC, NT>;
  using TileB = Tile<ES, BN, B_KC, NT>;
  constexpr int kStage = TileA::kBytes + TileB::kBytes;

  extern __shared__ __attribute__((aligned(16))) char smem[];

  unsigned tm, tn;
  tile_of_block(blockIdx.x, p.tiles_m, p.tiles_n, tm, tn);
  const size_t m0 = (size_t)tm * BM, n0 = (size_t)tn * BN;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int wm = (wave / WAVES_N) * WM, wn = (wave % WAVES_N) * WN;

  Loader<ES, BM, A_KC, NT> la;
  Loader<ES, BN, B_KC, NT> lb;
  la.init(p.a, m0, p.m, p.a_s1, p.a_s0, p.a_sk);
  lb.init(p.b, n0, p.n, p.b_s1, p.b_s0, p.b_sk);

  Acc acc[MI][NI];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NI; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

  const size_t slices = (p.k * ES + kSliceBytes - 1) / kSliceBytes;
  v4i ra[TileA::kPerThread], rb[TileB::kPerThread];
  la.template fetch<GUARDED>(ra, 0, p.k);
  lb.template fetch<GUARDED>(rb, 0, p.k);
  la.stash(smem, ra);
  lb.stash(smem + TileA::kBytes, rb);
  __syncthreads();

  constexpr int kSteps = kSliceBytes / KB;  // MFMA k-steps per slice
  typename M::Frag fa[2][MI], fb[2][NI];    // operand fragments, double-buffered across k-steps
#pragma unroll
  for (int i = 0; i < MI; ++i) fa[0][i] = read_frag<ES, BM, A_KC, FRB>(smem, wm + i * 32, 0);
#pragma unroll
  for (int j = 0; j < NI; ++j) fb[0][j] = read_frag<ES, BN, B_KC, FRB>(smem + TileA::kBytes, wn + j * 32, 0);

  for (size_t s = 0; s < slices; ++s) {
    const char *ta = smem + (s & 1) * kStage;
    const char *tb = ta + TileA::kBytes;
    char *na = smem + ((s + 1) & 1) * kStage;
    // Next slice: global -> registers while this one is multiplied. The last
    // iteration fetches its own slice again (in range, never consumed) so that
    // the loop body has no branch around the loads.
    const size_t nxt = s + 1 < slices ? s + 1 : s;
    la.template fetch<GUARDED>(ra, nxt, p.k);
    lb.template fetch<GUARDED>(rb, nxt, p.k);
    // Keep the loads up here: left alone, the scheduler sinks them to just before
    // the LDS stores below and the whole memory latency lands on every slice.
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int ks = 0; ks < kSteps; ++ks) {
      const int cur = ks & 1, nx = cur ^ 1;
      if (ks + 1 < kSteps) {  // fragments of the next k-step are requested before this step's MFMAs
#pragma unroll
        for (int i = 0; i < MI; ++i) fa[nx][i] = read_frag<ES, BM, A_KC, FRB>(ta, wm + i * 32, (ks + 1) * KB);
#pragma unroll
        for (int j = 0; j < NI; ++j) fb[nx][j] = read_frag<ES, BN, B_KC, FRB>(tb, wn + j * 32, (ks + 1) * KB);
      }
      // The LDS reads above are all issued before the first MFMA below and are
      // not needed until the next k-step: the scheduler must not pull them
      // down next to their uses (with one wave per SIMD nothing else would
      // hide their latency).
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j) acc[i][j] = M::run(fa[cur][i], fb[cur][j], acc[i][j]);
      __builtin_amdgcn_sched_barrier(0);
    }
    la.stash(na, ra);
    lb.stash(na + TileA::kBytes, rb);
    __syncthreads();
    // First fragments of the next slice (kSteps is even, so they land in buffer 0 again).
#pragma unroll
    for (int i = 0; i < MI; ++i) fa[0][i] = read_frag<ES, BM, A_KC, FRB>(na, wm + i * 32, 0);
#pragma unroll
    for (int j = 0; j < NI; ++j) fb[0][j] = read_frag<ES, BN, B_KC, FRB>(na + TileA::kBytes, wn + j * 32, 0);
  }

  // Epilogue: lane l of a 32x32 block holds column l%32 and rows 8*(r/4) + 4*(l/32) + r%4.
  AccElem *c = reinterpret_cast<AccElem *>(p.c);
  const bool read_c = !(TA == SKL_DT_I8 && p.beta.i == 0);  // 0*c == 0 only for integers
#pragma unroll
  for (int j = 0; j < NI; ++j) {
    const size_t col = n0 + wn + j * 32 + (lane & 31);
    if (GUARDED && col >= p.n) continue;
    const size_t col_off = (col >> 6) * p.csc1 + (col & 63) * p.csc0;
#pragma unroll
    for (int i = 0; i < MI; ++i) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const size_t row = m0 + wm + i * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
        if (!GUARDED || row < p.m) {
          AccElem *out = c + (row >> 6) * p.rsc1 + (row & 63) * p.rsc0 + col_off;
          const AccElem old = read_c ? *out : (AccElem)0;
          *out = epilogue(acc[i][j][r], old, p.alpha, p.beta);
        }
      }
    }
  }
}

// ===========================================================================
// Streaming variant for whole 256 x 256 tiles: global -> LDS without passing
// through registers (global_load_lds_dwordx4). Each wave-level load deposits
// 64 x 16 bytes as one contiguous KiB of LDS, so the tiles are stored without
// padding and bank conflicts are avoided by an XOR swizzle of the 16-byte
// chunk index instead; the swizzle is applied on the global side (which chunk
// a lane fetches) and again by the fragment reads. Four waves, one per SIMD,
// each own a 128 x 128 block of C (256 accumulator registers): half the LDS
// bytes per MFMA of a 128 x 64 block, and the registers and LDS-store
// instructions of the staged copy are gone, which matters because a wave's
// instruction stream is serial - every load or LDS store it issues is a slot
// in which it issues no MFMA.
// ===========================================================================
template <int ES, bool KC>
struct STile {
  static constexpr int kBytes = 256 * kSliceBytes;  // 256 rows x 128 bytes of K, 32 KiB
  // Byte offset of 16-byte chunk `c` of line `r`. A line is an M/N row holding
  // 128 bytes of K (KC), or a k-row holding 256 elements along M/N (MC).
  __device__ static __forceinline__ int chunk(int r, int c) {
    if constexpr (KC)
      return r * 128 + ((c ^ ((r >> 1) & 7)) << 4);   // 8 chunks; b128 reads take 16 consecutive rows
    else if constexpr (ES == 1)
      return r * 256 + ((c ^ ((r & 7) << 1)) << 4);   // 16 chunks; tr8 reads take 8 k-rows x 32 B
    else
      return r * 512 + ((c ^ ((r & 3) << 2)) << 4);   // 32 chunks; tr16 reads take 4 k-rows x 64 B
  }
};

template <int ES, bool KC, int WAVES>
struct SLoader {
  static constexpr int kBlocks = 32 / WAVES;  // KiB blocks per wave, operand and slice
  const char *tile_base;
  size_t k_step;
  unsigned off[kBlocks];
  unsigned lds_block;  // byte offset of this wave's first block inside the operand tile

  __device__ void init(const char *base, size_t mn0, size_t s1, size_t s0, size_t sk) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    tile_base = base + (mn0 >> 6) * s1 * ES;
    lds_block = wave * kBlocks * 1024;
#pragma unroll
    for (int i = 0; i < kBlocks; ++i) {
      const int b = wave * kBlocks + i;
      if constexpr (KC) {
        const int row = 8 * b + (lane >> 3), pos = lane & 7;
        const int c = pos ^ ((row >> 1) & 7);
        off[i] = (unsigned)(((size_t)(row >> 6) * s1 + (size_t)(row & 63) * s0 + (size_t)c * (16 / ES)) * ES);
      } else if constexpr (ES == 1) {
        const int kr = 4 * b + (lane >> 4), pos = lane & 15;
        const int mn = (pos ^ ((kr & 7) << 1)) * 16;
        off[i] = (unsigned)((size_t)(mn >> 6) * s1 + (size_t)(mn & 63) + (size_t)kr * sk);
      } else {
        const int kr = 2 * b + (lane >> 5), pos = lane & 31;
        const int mn = (pos ^ ((kr & 3) << 2)) * 8;
        off[i] = (unsigned)(((size_t)(mn >> 6) * s1 + (size_t)(mn & 63) + (size_t)kr * sk) * 2);
      }
    }
    k_step = KC ? (size_t)kSliceBytes : (size_t)(kSliceBytes / ES) * sk * ES;
  }

  // Requests block `i` of this wave's share of `slice`; the data lands in `tile` (LDS).
  __device__ __forceinline__ void issue_one(char *tile, size_t slice, int i) const {
    const char *g = tile_base + slice * k_step;
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(g + off[i]),
                                     (__attribute__((address_space(3))) void *)(tile + lds_block + i * 1024), 16, 0, 0);
  }
  __device__ __forceinline__ void issue(char *tile, size_t slice) const {
#pragma unroll
    for (int i = 0; i < kBlocks; ++i) issue_one(tile, slice, i);
  }
};

template <int ES, bool KC, int FRB>
__device__ __forceinline__ auto read_frag_s(const char *tile, int row0, int kb) {
  using T = STile<ES, KC>;
  const int lane = threadIdx.x & 63;
  const int h = lane >> 5;
  if constexpr (KC) {
    const int row = row0 + (lane & 31), c0 = (kb + h * FRB) >> 4;
    if constexpr (FRB == 16) {
      return *reinterpret_cast<const v4i *>(tile + T::chunk(row, c0));
    } else {
      const v4i lo = *reinterpret_cast<const v4i *>(tile + T::chunk(row, c0));
      const v4i hi = *reinterpret_cast<const v4i *>(tile + T::chunk(row, c0 + 1));
      return v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    }
  } else if constexpr (ES == 1) {
    const int g16 = (lane >> 4) & 1, j = lane & 15;
    const int kfirst = kb + h * FRB + (j >> 1), c = (row0 >> 4) + g16, sub = (j & 1) * 8;
    v2i r[FRB / 8];
#pragma unroll
    for (int s = 0; s < FRB / 8; ++s)
      r[s] = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_PTR(v2i, tile + T::chunk(kfirst + 8 * s, c) + sub));
    if constexpr (FRB == 16) {
      return v4i{r[0].x, r[0].y, r[1].x, r[1].y};
    } else {
      return v8i{r[0].x, r[0].y, r[1].x, r[1].y, r[2].x, r[2].y, r[3].x, r[3].y};
    }
  } else {
    static_assert(FRB == 16, "16-bit fragments are 16 bytes");
    const int g16 = (lane >> 4) & 1, j = lane & 15;
    const int kfirst = kb / 2 + h * 8 + (j >> 2);
    const int c = (row0 >> 3) + g16 * 2 + ((j & 3) >> 1), sub = (j & 1) * 8;
    const v4s r0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(v4s, tile + T::chunk(kfirst, c) + sub));
    const v4s r1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(v4s, tile + T::chunk(kfirst + 4, c) + sub));
    const v2i a = __builtin_bit_cast(v2i, r0), b = __builtin_bit_cast(v2i, r1);
    return v4i{a.x, a.y, b.x, b.y};
  }
}

// Scheduling recipe for one k-step of the streaming kernel: after each of the
// MFMAs place this step's share of LDS reads (ND in total) and of global
// loads (NV in total), evenly spread. A wave issues in order, so a burst of 16
// loads or 12 LDS reads in front of the MFMAs is a stretch in which the matrix
// pipe of its SIMD has nothing to do; one memory instruction in the shadow of
// each MFMA costs nothing.
template <int NM, int ND, int NV, int M>
__device__ __forceinline__ void sched_slot() {
  constexpr int d = (M + 1) * ND / NM - M * ND / NM;
  constexpr int v = (M + 1) * NV / NM - M * NV / NM;
  __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                   // one MFMA
  if constexpr (d > 0) __builtin_amdgcn_sched_group_barrier(0x100, d, 0);  // LDS reads
  if constexpr (v > 0) __builtin_amdgcn_sched_group_barrier(0x020, v, 0);  // global loads
}
template <int ND, int NV, int... Ms>
__device__ __forceinline__ void sched_kstep(std::integer_sequence<int, Ms...>) {
  (sched_slot<(int)sizeof...(Ms), ND, NV, Ms>(), ...);
}

template <int TA, int TB, bool A_KC, bool B_KC, int WAVES_N>
__global__ void __launch_bounds__(128 * WAVES_N) gemm_mfma_stream_kernel(MfmaArgs p) {
  using KA = Kind<TA>;
  using M = Mma<TA, TB>;
  using Acc = typename KA::Acc;
  using AccElem = decltype(Acc{}.x);
  constexpr int ES = KA::ES, KB = KA::KB, FRB = KB / 2;
  constexpr int BM = 256, BN = 256, WM = 128, WN = BN / WAVES_N, MI = 4, NI = WN / 32, WAVES = 2 * WAVES_N;
  constexpr int kTile = STile<ES, true>::kBytes, kStage = 2 * kTile;
  constexpr int kSteps = kSliceBytes / KB;
  constexpr int kMfmas = MI * NI;

  extern __shared__ __attribute__((aligned(16))) char smem[];

  unsigned tm, tn;
  tile_of_block(blockIdx.x, p.tiles_m, p.tiles_n, tm, tn);
  const size_t m0 = (size_t)tm * BM, n0 = (size_t)tn * BN;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int wm = (wave / WAVES_N) * WM, wn = (wave % WAVES_N) * WN;

  SLoader<ES, A_KC, WAVES> la;
  SLoader<ES, B_KC, WAVES> lb;
  la.init(p.a, m0, p.a_s1, p.a_s0, p.a_sk);
  lb.init(p.b, n0, p.b_s1, p.b_s0, p.b_sk);

  Acc acc[MI][NI];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NI; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

  const size_t slices = p.k * ES / kSliceBytes;
  la.issue(smem, 0);
  lb.issue(smem + kTile, 0);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  typename M::Frag fa[2][MI], fb[2][NI];
#pragma unroll
  for (int i = 0; i < MI; ++i) fa[0][i] = read_frag_s<ES, A_KC, FRB>(smem, wm + i * 32, 0);
#pragma unroll
  for (int j = 0; j < NI; ++j) fb[0][j] = read_frag_s<ES, B_KC, FRB>(smem + kTile, wn + j * 32, 0);

  for (size_t s = 0; s < slices; ++s) {
    const char *ta = smem + (s & 1) * kStage;
    const char *tb = ta + kTile;
    char *na = smem + ((s + 1) & 1) * kStage;
    // The other stage was last read before the barrier that ended the previous
    // iteration: the next slice streams into it while this one is multiplied.
    // (The last iteration requests its own slice again: in range, never read.)
    const size_t nxt = s + 1 < slices ? s + 1 : s;
    // A wave issues in order and the compute unit has one load path, so the
    // loads of the next slice are dealt out between the MFMAs (one load per
    // kGap MFMAs) instead of being issued in a burst, and the LDS reads of the
    // next k-step go out ahead of this step's MFMAs. The scheduling fences pin
    // that order: left alone the compiler bunches loads and sinks reads.
    // The last k-step of the slice is multiplied AFTER the barrier, from
    // fragments already in registers, so that its MFMAs cover the latency of the
    // first fragment reads of the next slice.
    constexpr int kLoads = 2 * (32 / WAVES);        // this wave's loads per slice (A then B)
    constexpr int kItems = kLoads;
    constexpr int kSlots = (kSteps - 1) * kMfmas;   // MFMAs before the barrier
    static_assert(kSteps % 2 == 0, "fragment buffers alternate per k-step");
    int issued = 0;
    auto deal = [&](int item) {
      if (item < kLoads / 2) {
        la.issue_one(na, nxt, item);
      } else {
        lb.issue_one(na + kTile, nxt, item - kLoads / 2);
      }
    };
#pragma unroll
    for (int ks = 0; ks < kSteps - 1; ++ks) {
      const int cur = ks & 1, nx = cur ^ 1;
#pragma unroll
      for (int i = 0; i < MI; ++i) fa[nx][i] = read_frag_s<ES, A_KC, FRB>(ta, wm + i * 32, (ks + 1) * KB);
#pragma unroll
      for (int j = 0; j < NI; ++j) fb[nx][j] = read_frag_s<ES, B_KC, FRB>(tb, wn + j * 32, (ks + 1) * KB);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int q = 0; q < kMfmas; ++q) {
        const int slot = ks * kMfmas + q;
#pragma unroll
        for (int it = 0; it < kItems; ++it)  // items due by this slot (spread evenly over the slots)
          if (it == issued && it * kSlots <= slot * kItems) {
            deal(it);
            ++issued;
          }
        const int i = q / NI, j = q % NI;
        acc[i][j] = M::run(fa[cur][i], fb[cur][j], acc[i][j]);
        if ((q & 1) == 1) __builtin_amdgcn_sched_barrier(0);
      }
    }
#pragma unroll
    for (int it = 0; it < kItems; ++it)
      if (it >= issued) deal(it);
    // Every LDS read of this stage has been issued; wait for them and for the
    // next slice's data, then let the other waves overwrite this stage.
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
#pragma unroll
    for (int i = 0; i < MI; ++i) fa[0][i] = read_frag_s<ES, A_KC, FRB>(na, wm + i * 32, 0);
#pragma unroll
    for (int j = 0; j < NI; ++j) fb[0][j] = read_frag_s<ES, B_KC, FRB>(na + kTile, wn + j * 32, 0);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
      for (int j = 0; j < NI; ++j) acc[i][j] = M::run(fa[1][i], fb[1][j], acc[i][j]);
    __builtin_amdgcn_sched_barrier(0);
  }

  AccElem *c = reinterpret_cast<AccElem *>(p.c);
  const bool read_c = !(TA == SKL_DT_I8 && p.beta.i == 0);
#pragma unroll
  for (int j = 0; j < NI; ++j) {
    const size_t col = n0 + wn + j * 32 + (lane & 31);
    const size_t col_off = (col >> 6) * p.csc1 + (col & 63) * p.csc0;
#pragma unroll
    for (int i = 0; i < MI; ++i) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const size_t row = m0 + wm + i * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
        AccElem *out = c + (row >> 6) * p.rsc1 + (row & 63) * p.rsc0 + col_off;
        const AccElem old = read_c ? *out : (AccElem)0;
        *out = epilogue(acc[i][j][r], old, p.alpha, p.beta);
      }
    }
  }
}

template <int TA, int TB, bool A_KC, bool B_KC, int WAVES_N>
int launch_stream(const MfmaArgs &args) {
  constexpr int lds = 4 * STile<1, true>::kBytes;  // two stages of two 32 KiB tiles
  auto kernel = gemm_mfma_stream_kernel<TA, TB, A_KC, B_KC, WAVES_N>;
  static bool configured = false;
  if (!configured) {
    int rc = skl_check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, lds),
                           "gemm_mfma_stream: LDS size");
    if (rc != 0) return rc;
    configured = true;
  }
  MfmaArgs p = args;
  p.tiles_m = (unsigned)(p.m / 256);
  p.tiles_n = (unsigned)(p.n / 256);
  const size_t grid = (size_t)p.tiles_m * p.tiles_n;
  if (grid > 0x7FFFFFFFu) {
    skl_hip_record_error(-2, "gemm_mfma: grid too large");
    return -2;
  }
  kernel<<<(unsigned)grid, 128 * WAVES_N, lds, skl_current_stream()>>>(p);
  return skl_check_launch("gemm_mfma_stream");
}

template <int TA, int TB, bool A_KC, bool B_KC, int BM, int BN, int WAVES_M, int WAVES_N, bool GUARDED>
int launch_one(const MfmaArgs &args) {
  constexpr int ES = Kind<TA>::ES;
  constexpr int NT = WAVES_M * WAVES_N * 64;
  constexpr int lds = 2 * (Tile<ES, BM, A_KC, NT>::kBytes + Tile<ES, BN, B_KC, NT>::kBytes);
  auto kernel = gemm_mfma_kernel<TA, TB, A_KC, B_KC, BM, BN, WAVES_M, WAVES_N, GUARDED>;
  static bool configured = false;  // per instantiation; racing threads would set the same value
  if (!configured) {
    int rc = skl_check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, lds),
                           "gemm_mfma: LDS size");
    if (rc != 0) return rc;
    configured = true;
  }
  MfmaArgs p = args;
  p.tiles_m = skl_div_up(p.m, BM);
  p.tiles_n = skl_div_up(p.n, BN);
  const size_t grid = (size_t)p.tiles_m * p.tiles_n;
  if (grid > 0x7FFFFFFFu) {
    skl_hip_record_error(-2, "gemm_mfma: grid too large");
    return -2;
  }
  kernel<<<(unsigned)grid, NT, lds, skl_current_stream()>>>(p);
  return skl_check_launch("gemm_mfma");
}

template <int TA, int TB, bool A_KC, bool B_KC>
int launch_tile(const MfmaArgs &p) {
  constexpr int ES = Kind<TA>::ES;
  // The large tile takes problems that it divides evenly and that can fill the
  // 256 compute units with it; everything else runs on the small, bounds-checked one.
  const bool whole = p.m % 256 == 0 && p.n % 256 == 0 && (p.k * ES) % kSliceBytes == 0;
  const size_t big_tiles = (p.m / 256) * (p.n / 256);
  if (whole && big_tiles >= 200) {
    static const int waves_n = getenv("SKL_STREAM_WAVES_N") ? atoi(getenv("SKL_STREAM_WAVES_N")) : 4;
    if (waves_n == 2) return launch_stream<TA, TB, A_KC, B_KC, 2>(p);
    return launch_stream<TA, TB, A_KC, B_KC, 4>(p);
  }
  return launch_one<TA, TB, A_KC, B_KC, 128, 128, 2, 4, true>(p);
}

template <int TA, int TB>
int launch_layout(const MfmaArgs &p) {
  const bool a_kc = p.a_sk == 1, b_kc = p.b_sk == 1;
  if (a_kc && b_kc) return launch_tile<TA, TB, true, true>(p);
  if (a_kc) return launch_tile<TA, TB, true, false>(p);
  if (b_kc) return launch_tile<TA, TB, false, true>(p);
  return launch_tile<TA, TB, false, false>(p);
}

inline bool mult16(size_t bytes) { return (bytes & 15) == 0; }

// One operand: exactly one unit stride; the other strides and the base 16-byte aligned.
bool operand_ok(const void *base, size_t es, size_t s1, size_t s0, size_t sk, size_t mn, size_t k) {
  if (((uintptr_t)base & 15) != 0) return false;
  // Offsets inside one tile (up to four 64-blocks, 64 rows, 128 k-rows) are kept in 32 bits.
  const size_t limit = size_t(1) << 31;
  if (sk == 1) {  // K-contiguous: rows anywhere on 16-byte boundaries
    if (s1 * es * 4 >= limit || s0 * es * 64 >= limit) return false;
    return (mn <= 1 || mult16(s0 * es)) && (mn <= 64 || mult16(s1 * es));
  }
  if (s0 == 1) {  // MN-contiguous in runs of 64 elements
    if (s1 * es * 4 >= limit || sk * es * 128 >= limit) return false;
    return (k <= 1 || mult16(sk * es)) && (mn <= 64 || mult16(s1 * es));
  }
  return false;
}

}  // namespace

extern "C" int skl_hip_gemm_mfma_supported(const skl_gemm_canon *g) {
  if (g->m == 0 || g->n == 0 || g->k == 0) return 0;
  const bool fp8a = g->ta == SKL_DT_F8E4M3 || g->ta == SKL_DT_F8E5M2;
  const bool fp8b = g->tb == SKL_DT_F8E4M3 || g->tb == SKL_DT_F8E5M2;
  if (!(g->ta == g->tb || (fp8a && fp8b))) return 0;
  const size_t es = (g->ta == SKL_DT_BF16 || g->ta == SKL_DT_F16) ? 2 : 1;
  if (!operand_ok(g->a, es, g->a_s1, g->a_s0, g->a_sk, g->m, g->k)) return 0;
  if (!operand_ok(g->b, es, g->b_s1, g->b_s0, g->b_sk, g->n, g->k)) return 0;
  if (((uintptr_t)g->c & 3) != 0) return 0;
  return 1;
}

extern "C" int skl_hip_launch_gemm_mfma(const skl_gemm_canon *g) {
  if (!skl_hip_gemm_mfma_supported(g)) {
    skl_hip_record_error(-2, "gemm_mfma: unsupported problem");
    return -2;
  }
  MfmaArgs p;
  p.a = (const char *)g->a;
  p.b = (const char *)g->b;
  p.c = (char *)g->c;
  p.m = g->m, p.n = g->n, p.k = g->k;
  p.a_s1 = g->a_s1, p.a_s0 = g->a_s0, p.a_sk = g->a_sk;
  p.b_s1 = g->b_s1, p.b_s0 = g->b_s0, p.b_sk = g->b_sk;
  p.rsc0 = g->rsc0, p.csc0 = g->csc0, p.rsc1 = g->rsc1, p.csc1 = g->csc1;
  p.alpha = g->alpha, p.beta = g->beta;
  p.tiles_m = p.tiles_n = 0;
  switch (g->ta * 8 + g->tb) {
    case SKL_DT_I8 * 8 + SKL_DT_I8: return launch_layout<SKL_DT_I8, SKL_DT_I8>(p);
#ifndef SKL_MFMA_INT8_ONLY  // kernel-development builds compile one operand kind only
    case SKL_DT_BF16 * 8 + SKL_DT_BF16: return launch_layout<SKL_DT_BF16, SKL_DT_BF16>(p);
    case SKL_DT_F16 * 8 + SKL_DT_F16: return launch_layout<SKL_DT_F16, SKL_DT_F16>(p);
    case SKL_DT_F8E4M3 * 8 + SKL_DT_F8E4M3: return launch_layout<SKL_DT_F8E4M3, SKL_DT_F8E4M3>(p);
    case SKL_DT_F8E5M2 * 8 + SKL_DT_F8E5M2: return launch_layout<SKL_DT_F8E5M2, SKL_DT_F8E5M2>(p);
    case SKL_DT_F8E4M3 * 8 + SKL_DT_F8E5M2: return launch_layout<SKL_DT_F8E4M3, SKL_DT_F8E5M2>(p);
    case SKL_DT_F8E5M2 * 8 + SKL_DT_F8E4M3: return launch_layout<SKL_DT_F8E5M2, SKL_DT_F8E4M3>(p);
#endif
    default:
      skl_hip_record_error(-2, "gemm_mfma: operand type pair");
      return -2;
  }
}
