// skl_gemm_mfma_impl.hpp - the dense contractions on the gfx950 matrix cores (kernel templates and their
// launchers; included by one translation unit per operand kind, skl_gemm_mfma_<kind>.hip, and by the dispatch in
// skl_gemm_mfma.hip):
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
#pragma once
#include <hip/hip_runtime.h>

#include <atomic>

#include <cstdlib>
#include <utility>

#include "skl_device.hpp"
#include "skl_fp8.hpp"

// The arguments of a launch, shared by the translation units of the operand kinds and the dispatch.
struct MfmaArgs {
  const char *a;
  const char *b;
  char *c;
  size_t m, n, k;
  size_t a_s1, a_s0, a_sk;  // elements
  size_t b_s1, b_s0, b_sk;
  size_t rsc0, csc0, rsc1, csc1;
  unsigned crs, ccs;  // log2 of C's block rows / columns (6 unless C comes in smaller power-of-two blocks; crs >= 2)
  skl_scalar alpha, beta;
  const char *bias;  // fused epilogue: per-column addend and running maximum of C's type, or null
  char *max;
  skl_requant rq;    // ... activation and requantised int8 copy
  unsigned tiles_m, tiles_n;
  // Split along K (bounds-checked kernel only): workgroup b works on tile b % (tiles_m * tiles_n) and on the
  // slices [split * slices_per_split, ...) with split = b / (tiles_m * tiles_n); splits > 1 stores the raw
  // sums to partial[split][m][n] (row-major, 4-byte elements) for gemm_split_reduce_kernel.
  unsigned splits, slices_per_split;
  char *partial;
};

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


// The fused steps behind the alpha/beta step, for one lane: bias of the lane's column, activation, running maximum,
// requantised copy.
// EXTRA: with the activation and the requantised copy (kernels are instantiated with and without: the two steps cost
// code in every one of a lane's 128 stores, which calls without them should not carry). 1: any descriptor, decided
// element by element at run time. 2 and 3: for kernels that hand every lane's elements to rows4() with all lanes
// active - a row-major copy on 4-byte boundaries, written as dwords, without (2, q_only) or with (3) C; no
// branches inside the epilogue, which with 128 accumulators live is what keeps the registers from spilling (the
// run-time form in the streaming kernel: 240 spilled registers, an 8192^3 call 45 % longer).
template <typename T, int EXTRA = 0>
struct FusedSteps {
  const T *bias;
  T *max;
  const skl_requant rq;
  T bias_j, running;
  size_t col;
  float q_scale_j;  // EXTRA: the current column's scale
  const skl_fp8::Ofp8Format f8;  // modes 2 and 3: the constants of an fp8 copy (uniform; unused for an int8 copy)
  __device__ explicit FusedSteps(const MfmaArgs &p)
      : bias(reinterpret_cast<const T *>(p.bias)), max(reinterpret_cast<T *>(p.max)), rq(p.rq), bias_j(0), running(skl_lowest<T>()), col(0),
        q_scale_j(0.0f), f8(p.rq.q_fmt) {}
  // What a descriptor must look like for modes 2 and 3: a row-major copy on 4-byte boundaries, no activation beyond
  // ReLU (the others cost too much code in each of a lane's 128 elements), and the copy's format the one these
  // modes are built with for C's type - int8 behind an int32 C, OCP fp8 behind a floating-point C (an int8 product
  // feeding an int8 layer, an fp8 product an fp8 layer; other pairings run on the bounds-checked kernels).
  static constexpr bool kCopyIsFp8 = !std::is_same<T, int>::value;
  __host__ __device__ static bool dword_copy(const skl_requant &r) {
    return r.q && r.act <= 1 && (r.q_fmt != 0) == kCopyIsFp8 && r.csq == 1 && (r.rsq & 3) == 0 && ((uintptr_t)r.q & 3) == 0;
  }
  // What the steps need to know about column c, fetched ahead of the stores (a load issued behind a store has to
  // wait for that store's acknowledgement before its value can be used) ...
  struct Column {
    T bias;
    float q_scale;
  };
  __device__ __forceinline__ Column fetch(size_t c) const {
    Column k{T(0), 0.0f};
    if (bias) k.bias = bias[c];
    if constexpr (EXTRA >= 2) k.q_scale = rq.q_scale[rq.q_per_column ? c : 0];
    if constexpr (EXTRA == 1) {
      if (rq.q) k.q_scale = rq.q_scale[rq.q_per_column ? c : 0];
    }
    return k;
  }
  // ... and made current.
  __device__ __forceinline__ void column(size_t c, const Column &k) {
    col = c;
    bias_j = k.bias;
    q_scale_j = k.q_scale;
  }
  __device__ __forceinline__ void column(size_t c) { column(c, fetch(c)); }
  __device__ __forceinline__ T apply(T v) {
    if (bias) v = skl_add_bias(v, bias_j);
    if constexpr (EXTRA == 1) v = skl_activate(v, rq.act);
    if constexpr (EXTRA >= 2) v = skl_activate(v, rq.act != 0);  // none or ReLU
    if (max && v > running) running = v;
    return v;
  }
  // The element of logical row `row` in the current column: the steps, then C (written once and not read again: a
  // non-temporal store keeps it out of the operands' caches) and, in mode 1, the requantised copy. Returns what
  // was written.
  __device__ __forceinline__ T put(T v, T *dst, size_t row) {
    v = apply(v);
    if constexpr (EXTRA == 1) {
      if (!rq.q_only) __builtin_nontemporal_store(v, dst);
      if (rq.q) rq.q[row * rq.rsq + col * rq.csq] = skl_quantise((float)v, q_scale_j, rq.q_zero, rq.q_fmt);
    } else {
      (void)row;
      if constexpr (EXTRA != 2) __builtin_nontemporal_store(v, dst);
    }
    return v;
  }
  // Modes 2 and 3: the requantised copy of rows row0 .. row0 + 3 of the current column, v as put() returned them.
  // A lane's four values are one column of a 4 x 4 block of bytes whose other columns its quad's lanes hold (four
  // neighbouring columns, the first a multiple of four); the block is transposed across the quad (four broadcasts
  // and three byte permutes per lane), and lane q stores row row0 + q of it as one dword - a quarter of the store
  // instructions and address arithmetic of single bytes.
  __device__ __forceinline__ void rows4(const T (&v)[4], size_t row0) {
    if constexpr (EXTRA >= 2) {
      unsigned packed = 0;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if constexpr (kCopyIsFp8)
          packed |= skl_fp8::encode_ofp8_hw(__fmul_rn((float)v[i], q_scale_j), f8) << (8 * i);
        else
          packed |= ((unsigned)skl_requantise_int((float)v[i], q_scale_j, rq.q_zero) & 0xFFu) << (8 * i);
      }
      const unsigned p0 = (unsigned)__builtin_amdgcn_update_dpp(0, (int)packed, 0x00, 0xF, 0xF, true);  // quad_perm: lane 0 of the quad
      const unsigned p1 = (unsigned)__builtin_amdgcn_update_dpp(0, (int)packed, 0x55, 0xF, 0xF, true);
      const unsigned p2 = (unsigned)__builtin_amdgcn_update_dpp(0, (int)packed, 0xAA, 0xF, 0xF, true);
      const unsigned p3 = (unsigned)__builtin_amdgcn_update_dpp(0, (int)packed, 0xFF, 0xF, 0xF, true);
      const unsigned q = threadIdx.x & 3u;
      const unsigned sel = 0x0C0C0400u + q * 0x0101u;  // byte q of the second operand, byte q of the first, zeros
      const unsigned lo = __builtin_amdgcn_perm(p1, p0, sel), hi = __builtin_amdgcn_perm(p3, p2, sel);
      const unsigned out = __builtin_amdgcn_perm(hi, lo, 0x05040100u);
      *reinterpret_cast<unsigned *>(rq.q + (row0 + q) * rq.rsq + (col - q)) = out;
    } else {
      (void)v, (void)row0;
    }
  }
  // Every lane of the wave calls this once, after its last element.
  __device__ __forceinline__ void finish() {
    if (!max) return;
    const T best = skl_wave_max(running);
    if ((threadIdx.x & 63) == 0 && best > skl_lowest<T>()) skl_atomic_max(max, best);
  }
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

// OCP fp8 operands multiplied exactly: the bytes are widened to f16 in registers (every E4M3 / E5M2 value is an
// f16 value) and two f16 instructions take 32 bytes of K - exact products, fp32 sums, which is what the reference's
// error bound assumes. The fp8 instructions above align the products of one instruction to a common exponent and
// keep about 12 bits below the largest; that is inside the bound only once K is a few thousand (the bound grows
// with K, the instruction's error does not), so short K runs here, at the f16 rate.
template <int TA, int TB>
struct MmaF8Exact {
  static constexpr int KB = 32;  // bytes of K per step: a 16-byte fragment per lane, like int8
  using Frag = v4i;
  struct Ready {
    v8h lo, hi;
  };
  template <int DT>
  __device__ static Ready widen(v4i f) {
    constexpr bool e5m2 = DT == SKL_DT_F8E5M2;
    return Ready{skl_fp8::widen8_to_f16<e5m2>((unsigned)f.x, (unsigned)f.y), skl_fp8::widen8_to_f16<e5m2>((unsigned)f.z, (unsigned)f.w)};
  }
  __device__ static Ready prep_a(v4i f) { return widen<TA>(f); }
  __device__ static Ready prep_b(v4i f) { return widen<TB>(f); }
  __device__ static v16f run(const Ready &a, const Ready &b, v16f c) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_f16(a.lo, b.lo, c, 0, 0, 0);
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a.hi, b.hi, c, 0, 0, 0);
  }
};
// K up to which the fp8 kinds run on MmaF8Exact: the reference's bound 2((1 + 2^-24)^(K+2) - 1) passes the fp8
// instructions' 2^-11.9 at K = 2193.
constexpr size_t kF8ExactMaxK = 2304;

// A fragment as the multiply wants it: widened where the operand kind asks for that, else as it was read.
template <typename M, typename F>
__device__ __forceinline__ auto prep_a(F f) {
  if constexpr (requires { M::prep_a(f); }) return M::prep_a(f); else return f;
}
template <typename M, typename F>
__device__ __forceinline__ auto prep_b(F f) {
  if constexpr (requires { M::prep_b(f); }) return M::prep_b(f); else return f;
}

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

// ---------------------------------------------------------------------------
// The epilogue of both kernels: one wave writes its MI x NI blocks of 32 x 32, lane l of a block holding column
// l % 32 and rows 8 * (r / 4) + 4 * (l / 32) + r % 4 in register r, as C = beta*C + alpha*acc followed by the fused
// steps. C is written once and not read again: non-temporal stores keep it out of the operands' caches.
//
// What decides the time is how the wave's loads and stores follow each other. On this target one counter covers
// both, in issue order, so the value of a load cannot be used before every store issued in front of it has been
// acknowledged - and under the write burst of a whole chip ending its tiles together that takes microseconds.
// Hence: (1) when C is not read (beta == 0, and no element is the one case below) the 16 * MI * NI stores of a
// lane go out with no load between them - the columns' bias values and scales are fetched first; (2) when C is
// read, the old values of block b + kAhead are requested before block b is stored, so a wait only ever covers
// loads that were issued in front of the stores still in flight.
// beta == 0 in floating point reads C only where alpha*acc is the negative zero (skl_initialise_needs_c); whether
// any element of the wave's tile is one is decided once, for the whole wave, before the first store.
// CHECK: rows / columns beyond p.m / p.n are left alone.
// ---------------------------------------------------------------------------
template <int MI, int NI, bool CHECK, int EXTRA, typename Acc>
__device__ __forceinline__ void write_wave_tile(const MfmaArgs &p, const Acc (&acc)[MI][NI], size_t row0, size_t col0) {
  using AccElem = decltype(Acc{}.x);
  using Steps = FusedSteps<AccElem, EXTRA>;
  constexpr int kBlocks = MI * NI;            // block b: j = b / MI, i = b % MI (a column strip at a time)
  constexpr int kAhead = (kBlocks < 2 || CHECK) ? 1 : 2;  // the bounds-checked kernels run four waves per SIMD: 128 registers
  // The lane index from the execution mask rather than from threadIdx: nothing the epilogue needs is then computed
  // in front of the main loop and held in a vector register across it (the loop uses every one of them).
  const int lane = (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
  AccElem *c = reinterpret_cast<AccElem *>(p.c);
  const size_t rmask = (size_t(1) << p.crs) - 1, cmask = (size_t(1) << p.ccs) - 1;
  const bool init = skl_beta_is_zero<AccElem>(p.beta);  // C is initialised, not updated
  bool read_c = !init;
  if constexpr (!std::is_same<AccElem, int>::value) {
    if (init) {
      // alpha through a copy the compiler cannot identify with p.alpha: the products of this test are then not
      // kept (all 16 * MI * NI of them, spilled) for the stores below, which multiply again.
      skl_scalar alpha = p.alpha;
      asm volatile("" : "+s"(alpha.i));
      bool need = false;
#pragma unroll
      for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j)
#pragma unroll
          for (int r = 0; r < 16; ++r) need |= skl_initialise_needs_c(acc[i][j][r], alpha, p.beta);
      read_c = __builtin_amdgcn_ballot_w64(need) != 0;
    }
  }
  auto col_of = [&](int j) { return col0 + (size_t)j * 32 + (lane & 31); };
  // first of the four consecutive rows of register group g (all in one block of C: blocks have a multiple of 4 rows)
  auto first_row = [&](int i, int g) { return row0 + (size_t)i * 32 + g * 8 + (lane >> 5) * 4; };
  auto inside = [&](int j, int i, int r) { return !CHECK || (col_of(j) < p.n && first_row(i, r >> 2) + (r & 3) < p.m); };
  // The four row groups of block (i, j): where the first row of each starts.
  struct Where {
    AccElem *out[4];
  };
  auto where = [&](int j, int i) {
    // A zero the compiler cannot see through, new at every use: the addresses of a block are then computed where
    // the block is written and not, all 16 * MI * NI of them, ahead of the first block (which spills half of them).
    unsigned opaque = 0;
    asm volatile("" : "+s"(opaque));
    const size_t col = col_of(j) + opaque, col_off = (col >> p.ccs) * p.csc1 + (col & cmask) * p.csc0;
    Where w;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const size_t row = first_row(i, g);
      w.out[g] = c + (row >> p.crs) * p.rsc1 + (row & rmask) * p.rsc0 + col_off;
    }
    return w;
  };
  Steps fused(p);
  typename Steps::Column columns[NI];
#pragma unroll
  for (int j = 0; j < NI; ++j) columns[j] = (!CHECK || col_of(j) < p.n) ? fused.fetch(col_of(j)) : typename Steps::Column{AccElem(0), 0.0f};

  // Block B. MODE 0: C is not read; 1: with the old values `old` (C is updated, or beta == 0 and they decide the sign of
  // zeros); 2: C is not read and there is no fused step (no bias, no maximum, no copy).
  // (Block numbers are compile-time constants throughout, so that the buffers of old values stay in registers.)
  auto write_block = [&](auto mode, auto bc, const AccElem (&old)[16]) {
    constexpr int MODE = decltype(mode)::value, B = decltype(bc)::value;
    constexpr int j = B / MI, i = B % MI;
    fused.column(col_of(j), columns[j]);
    const Where w = where(j, i);
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      AccElem four[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int r = 4 * g + q;
        four[q] = AccElem(0);
        if (inside(j, i, r)) {
          AccElem v;
          if constexpr (MODE == 0 || MODE == 2) v = skl_initialise_plain(acc[i][j][r], p.alpha, p.beta);
          if constexpr (MODE == 1) {  // one path for both ways of using the old value: a select per element
            const AccElem vi = skl_initialise_with(acc[i][j][r], old[r], p.alpha, p.beta), vc = skl_combine(acc[i][j][r], old[r], p.alpha, p.beta);
            v = init ? vi : vc;
          }
          if constexpr (MODE == 2) {  // no fused step at all: the value as it is
            __builtin_nontemporal_store(v, w.out[g] + q * p.rsc0);
            four[q] = v;
          } else {
            four[q] = fused.put(v, w.out[g] + q * p.rsc0, first_row(i, g) + q);
          }
        }
      }
      fused.rows4(four, first_row(i, g));
    }
    __builtin_amdgcn_sched_barrier(0);  // a block at a time: the addresses of later blocks are not computed (and held) early
  };
  // The blocks in order, block B + kAhead requested before block B is written.
  auto update_blocks = [&](auto mode) {
    AccElem old[kAhead + 1][16];
    auto request = [&](auto bc) {
      constexpr int B = decltype(bc)::value;
      if constexpr (B < kBlocks) {
        constexpr int j = B / MI, i = B % MI;
        const Where w = where(j, i);
#pragma unroll
        for (int r = 0; r < 16; ++r) old[B % (kAhead + 1)][r] = inside(j, i, r) ? w.out[r >> 2][(r & 3) * p.rsc0] : AccElem(0);
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    [&]<int... Bs>(std::integer_sequence<int, Bs...>) { (request(std::integral_constant<int, Bs>{}), ...); }(std::make_integer_sequence<int, kAhead>{});
    [&]<int... Bs>(std::integer_sequence<int, Bs...>) {
      ((request(std::integral_constant<int, Bs + kAhead>{}), write_block(mode, std::integral_constant<int, Bs>{}, old[Bs % (kAhead + 1)])), ...);
    }(std::make_integer_sequence<int, kBlocks>{});
  };
  if (!read_c) {
    const AccElem none[16] = {};
    if (EXTRA == 0 && !p.bias && !p.max) {  // the plain product: two or three instructions and a store per element
      [&]<int... Bs>(std::integer_sequence<int, Bs...>) {
        (write_block(std::integral_constant<int, 2>{}, std::integral_constant<int, Bs>{}, none), ...);
      }(std::make_integer_sequence<int, kBlocks>{});
    } else {
      [&]<int... Bs>(std::integer_sequence<int, Bs...>) {
        (write_block(std::integral_constant<int, 0>{}, std::integral_constant<int, Bs>{}, none), ...);
      }(std::make_integer_sequence<int, kBlocks>{});
    }
  } else {
    update_blocks(std::integral_constant<int, 1>{});
  }
  fused.finish();
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

template <int TA, int TB, bool A_KC, bool B_KC, int BM, int BN, int WAVES_M, int WAVES_N, bool GUARDED, bool EXACT = false, bool EXTRA = false>
__global__ void __launch_bounds__(WAVES_M *WAVES_N * 64, (BM == 128 ? 4 : 6)) gemm_mfma_kernel(MfmaArgs p) {
  constexpr int NT = WAVES_M * WAVES_N * 64;
  using KA = Kind<TA>;
  using M = typename std::conditional<EXACT, MmaF8Exact<TA, TB>, Mma<TA, TB>>::type;
  using Acc = typename KA::Acc;
  using AccElem = decltype(Acc{}.x);
  constexpr int ES = KA::ES;
  constexpr int KB = EXACT ? 32 : KA::KB;       // bytes of K per MFMA step
  constexpr int FRB = KB / 2;                   // fragment bytes per lane
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;  // wave tile
  constexpr int MI = WM / 32, NI = WN / 32;     // MFMA blocks per wave
  using TileA = Tile<ES, BM, A_KC, NT>;
  using TileB = Tile<ES, BN, B_KC, NT>;
  constexpr int kStage = TileA::kBytes + TileB::kBytes;

  extern __shared__ __attribute__((aligned(16))) char smem[];

  unsigned tm, tn;
  const unsigned tiles = p.tiles_m * p.tiles_n, split = blockIdx.x / tiles;
  tile_of_block(blockIdx.x % tiles, p.tiles_m, p.tiles_n, tm, tn);
  const size_t m0 = (size_t)tm * BM, n0 = (size_t)tn * BN;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;  // the wave index as a scalar: nothing derived from it occupies a vector register across the main loop
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

  const size_t all_slices = (p.k * ES + kSliceBytes - 1) / kSliceBytes;
  const size_t s_begin = (size_t)split * p.slices_per_split;  // the host makes every split non-empty
  const size_t slices = all_slices - s_begin < p.slices_per_split ? all_slices : s_begin + p.slices_per_split;
  v4i ra[TileA::kPerThread], rb[TileB::kPerThread];
  la.template fetch<GUARDED>(ra, s_begin, p.k);
  lb.template fetch<GUARDED>(rb, s_begin, p.k);
  la.stash(smem, ra);
  lb.stash(smem + TileA::kBytes, rb);
  __syncthreads();

  constexpr int kSteps = kSliceBytes / KB;  // MFMA k-steps per slice
  typename M::Frag fa[2][MI], fb[2][NI];    // operand fragments, double-buffered across k-steps
#pragma unroll
  for (int i = 0; i < MI; ++i) fa[0][i] = read_frag<ES, BM, A_KC, FRB>(smem, wm + i * 32, 0);
#pragma unroll
  for (int j = 0; j < NI; ++j) fb[0][j] = read_frag<ES, BN, B_KC, FRB>(smem + TileA::kBytes, wn + j * 32, 0);

  for (size_t s = s_begin; s < slices; ++s) {
    const char *ta = smem + ((s - s_begin) & 1) * kStage;
    const char *tb = ta + TileA::kBytes;
    char *na = smem + ((s - s_begin + 1) & 1) * kStage;
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
      {
        decltype(prep_a<M>(fa[cur][0])) wa[MI];
        decltype(prep_b<M>(fb[cur][0])) wb[NI];
#pragma unroll
        for (int i = 0; i < MI; ++i) wa[i] = prep_a<M>(fa[cur][i]);
#pragma unroll
        for (int j = 0; j < NI; ++j) wb[j] = prep_b<M>(fb[cur][j]);
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
          for (int j = 0; j < NI; ++j) acc[i][j] = M::run(wa[i], wb[j], acc[i][j]);
      }
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

  // Lane l of a 32x32 block holds column l%32 and rows 8*(r/4) + 4*(l/32) + r%4.
  if (p.splits > 1) {  // a share of K: the raw sums go to this split's M x N plane
    AccElem *plane = reinterpret_cast<AccElem *>(p.partial) + (size_t)split * p.m * p.n;
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      const size_t col = n0 + wn + j * 32 + (lane & 31);
      if (col >= p.n) continue;
#pragma unroll
      for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const size_t row = m0 + wm + i * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
          if (row < p.m) plane[row * p.n + col] = acc[i][j][r];
        }
    }
    return;
  }
  write_wave_tile<MI, NI, GUARDED, EXTRA ? 1 : 0>(p, acc, m0 + wm, n0 + wn);
}

// ===========================================================================
// Streaming kernel for whole tiles (256 x 256 or 256 x 128): global -> LDS
// without passing through registers (global_load_lds_dwordx4), K in slices of
// 64 bytes held in a ring of four LDS stages. Each wave-level load deposits
// 64 x 16 bytes as one contiguous KiB of LDS, so tiles are stored without
// padding and bank conflicts are avoided by an XOR swizzle of the 16-byte
// chunk index instead; the swizzle is applied on the global side (which chunk
// a lane fetches) and again by the fragment reads. Eight waves, two per SIMD.
//
// An MN-contiguous operand (k-rows of ROWS elements) is loaded a slice at a
// time: a load covers whole k-rows, i.e. whole 128-byte lines. A K-contiguous
// operand is different: a 64-byte slice is HALF a line of each row, and loads
// made of half lines run at less than half the rate of loads made of whole
// ones. So its loads cover 8 rows x 128 bytes - two slices at once - and the
// four stages of such an operand are interleaved in LDS at 512-byte granularity
// (8 rows x 64 bytes of stage 0, then of stage 1, ...), which puts the two
// halves of such a load next to each other: one KiB, as the load writes it.
// ===========================================================================
constexpr int kRingSlice = 64;   // bytes of K per stage
constexpr int kRingStages = 4;
// Stages of the ring for tiles of BN columns. The kernel's load schedule is written for any even number of stages;
// four it is for both tile widths: six stages for the 256 x 128 tile (144 KiB; its slices take half the time, so
// the same number of slices ahead is half the time ahead) measured no faster - bf16 2048 x 4096 x 4096 without its
// epilogue 75 us against 71-74 us - i.e. that kernel does not wait for its loads.
constexpr int ring_stages(int /*bn*/) { return kRingStages; }

template <int ES, bool KC, int ROWS, int NS = kRingStages>
struct STile {
  static constexpr int kStages = NS;
  static constexpr int kBytes = ROWS * kRingSlice;            // one stage
  static constexpr int kRegion = kBytes * NS;                 // all stages of the operand
  static constexpr int kRowBytes = ROWS * ES;                 // a k-row of an MN-contiguous tile
  static constexpr int kStageStep = KC ? 512 : kBytes;        // from one stage to the next
  static constexpr int kGroup = NS * 512;                     // K-contiguous: from 8 rows to the next 8
  // Byte offset (inside stage 0) of 16-byte chunk `c` of line `r`. A line is an M/N row
  // holding 64 bytes of K (KC), or a k-row holding ROWS elements along M/N (MC).
  __device__ static __forceinline__ int chunk(int r, int c) {
    if constexpr (KC)  // 4 chunks: rows r and r+4 share banks, the XOR parts them; 16 rows fill the banks once
      return (r >> 3) * kGroup + (r & 7) * 64 + ((c ^ ((r >> 2) & 3)) << 4);
    else if constexpr (ES == 1 && kRowBytes == 256)
      return r * 256 + ((c ^ ((r & 7) << 1)) << 4);   // 16 chunks; tr8 reads take 8 k-rows x 32 B
    else if constexpr (ES == 1)
      return r * 128 + ((c ^ (((r >> 1) & 3) << 1)) << 4);  // 8 chunks: two k-rows fill the banks once
    else
      return r * kRowBytes + ((c ^ ((r & 3) << 2)) << 4);   // 32 or 16 chunks; tr16 reads take 4 k-rows x 64 B
  }
};

// Global -> LDS loads of one operand, this wave's share. `unit` below is a slice
// for an MN-contiguous operand and a pair of slices for a K-contiguous one.
template <int ES, bool KC, int WAVES, int ROWS, int NS>
struct SLoader {
  using T = STile<ES, KC, ROWS, NS>;
  static constexpr int kUnitBytes = KC ? 2 * T::kBytes : T::kBytes;
  static constexpr int kBlocks = kUnitBytes / 1024 / WAVES;  // KiB blocks per wave and unit
  static_assert(kBlocks >= 1, "every wave loads at least one block per unit");
  const char *tile_base;
  size_t k_step;           // bytes from one unit to the next
  unsigned off[kBlocks];   // global byte offsets of this lane
  unsigned lds[kBlocks];   // LDS byte offsets (inside the operand's region, stage 0) of the blocks

  __device__ void init(const char *base, size_t mn0, size_t s1, size_t s0, size_t sk) {
    // The wave index as a scalar: the LDS address of a block (which goes into M0) is then scalar arithmetic, not a
    // vector add and a v_readfirstlane per load, and lds[] lives in scalar registers.
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    tile_base = base + (mn0 >> 6) * s1 * ES;
#pragma unroll
    for (int i = 0; i < kBlocks; ++i) {
      const int b = wave * kBlocks + i;
      if constexpr (KC) {  // block = 8 rows x (64 bytes of the even slice, then 64 bytes of the odd one)
        const int half = lane >> 5, row = 8 * b + ((lane & 31) >> 2), pos = lane & 3;
        const int c = pos ^ ((row >> 2) & 3);
        off[i] = (unsigned)(((size_t)(row >> 6) * s1 + (size_t)(row & 63) * s0) * ES + half * 64 + c * 16);
        lds[i] = b * T::kGroup;
      } else {
        constexpr int kLanesPerRow = T::kRowBytes / 16, kRowsPerBlock = 1024 / T::kRowBytes;
        const int kr = kRowsPerBlock * b + lane / kLanesPerRow, pos = lane % kLanesPerRow;
        const int mn = ((T::chunk(kr, pos) - kr * T::kRowBytes) >> 4) * (16 / ES);  // the chunk stored at position `pos`
        off[i] = (unsigned)(((size_t)(mn >> 6) * s1 + (size_t)(mn & 63) + (size_t)kr * sk) * ES);
        lds[i] = b * 1024;
      }
    }
    // (spelled out as a scalar: as a member next to per-lane offsets it otherwise ends up in a vector register, and
    // every load of an MN-contiguous operand pays a 64-bit vector multiply-add for its address)
    const size_t step = KC ? (size_t)(2 * kRingSlice) : (size_t)(kRingSlice / ES) * sk * ES;
    k_step = ((size_t)(unsigned)__builtin_amdgcn_readfirstlane((int)(step >> 32)) << 32) | (unsigned)__builtin_amdgcn_readfirstlane((int)step);
  }

  // Requests block `i` of `unit`; it lands in stage `stage` (the even one of the pair for KC) of `region`.
  __device__ __forceinline__ void issue_one(char *region, int stage, size_t unit, int i) const {
    const char *g = tile_base + unit * k_step;
    // The lane's offset through a copy the compiler cannot follow: it otherwise widens every offset to 64 bits ahead
    // of the loop (two registers each) and adds the scalar base with a 64-bit vector add per load; this way the load
    // takes the scalar base and the 32-bit offset as they are.
    unsigned o = off[i];
    asm volatile("" : "+v"(o));
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(g + o),
                                     (__attribute__((address_space(3))) void *)(region + stage * T::kStageStep + lds[i]),
                                     16, 0, 0);
  }
  __device__ __forceinline__ void issue(char *region, int stage, size_t unit) const {
#pragma unroll
    for (int i = 0; i < kBlocks; ++i) issue_one(region, stage, unit, i);
  }
};

// ---------------------------------------------------------------------------
// The software pipeline is written out by hand:
//   * Fragment reads are inline assembly. The compiler cannot tell an LDS read
//     from the LDS writes of outstanding global->LDS loads apart and makes every
//     ds_read_tr wait for ALL loads in flight (vmcnt(0)), and it waits for reads
//     it has only just issued (lgkmcnt(0) in front of every k-step) - either
//     one exposes a memory latency per k-step. Here the kernel does its own
//     counting: one lgkmcnt(0) at the top of a k-step, when the only reads in
//     flight are the ones issued during the previous k-step; one vmcnt(n) per
//     slice in front of the barrier.
//   * Reads and loads are dealt out one at a time behind the MFMAs instead of
//     going out in bursts: a wave issues in order, and a burst that finds the
//     LDS or the load path busy is a stretch in which it issues no MFMA. The
//     reads sit behind the first half of a k-step's MFMAs, which leaves the
//     second half for them to land.
// ---------------------------------------------------------------------------
template <int N>
__device__ __forceinline__ void wait_loads_upto() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

template <int OFF>
__device__ __forceinline__ v4i lds_read_b128(unsigned addr) {
  v4i r;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFF) : "memory");
  return r;
}
template <int OFF>
__device__ __forceinline__ v2i lds_read_tr8(unsigned addr) {
  v2i r;
  asm volatile("ds_read_b64_tr_b8 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFF) : "memory");
  return r;
}
template <int OFF>
__device__ __forceinline__ v2i lds_read_tr16(unsigned addr) {
  v2i r;
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFF) : "memory");
  return r;
}

// The fragments of one operand for one wave: NFRAG blocks of 32 rows, read from a stage in pieces of one
// LDS instruction each. Offsets inside the stage are per lane and computed once; what changes from k-step to
// k-step and from fragment to fragment is, wherever the swizzle allows, an immediate offset.
template <int ES, bool KC, int FRB, int KB, int ROWS, int NS, int NFRAG>
struct FragReader {
  using T = STile<ES, KC, ROWS, NS>;
  using Piece = typename std::conditional<KC, v4i, v2i>::type;
  static constexpr int RB = T::kRowBytes;
  static constexpr int kPieceBytes = KC ? 16 : 8;
  static constexpr int kPieces = FRB / kPieceBytes;  // LDS instructions per fragment
  static constexpr int kSteps = kRingSlice / KB;
  static constexpr int kBases = KC ? kSteps * kPieces : NFRAG;
  unsigned base[kBases];

  __device__ void init(int row0) {
    const int lane = threadIdx.x & 63, h = lane >> 5;
    if constexpr (KC) {
#pragma unroll
      for (int ks = 0; ks < kSteps; ++ks)
#pragma unroll
        for (int pc = 0; pc < kPieces; ++pc)
          base[ks * kPieces + pc] = (unsigned)T::chunk(row0 + (lane & 31), ((ks * KB + h * FRB) >> 4) + pc);
    } else if constexpr (ES == 1) {
      const int g16 = (lane >> 4) & 1, j = lane & 15;
#pragma unroll
      for (int f = 0; f < NFRAG; ++f)
        base[f] = (unsigned)(T::chunk(h * FRB + (j >> 1), ((row0 + 32 * f) >> 4) + g16) + (j & 1) * 8);
    } else {
      const int g16 = (lane >> 4) & 1, j = lane & 15;
#pragma unroll
      for (int f = 0; f < NFRAG; ++f)
        base[f] = (unsigned)(T::chunk(h * 8 + (j >> 2), ((row0 + 32 * f) >> 3) + g16 * 2 + ((j & 3) >> 1)) + (j & 1) * 8);
    }
  }
  // Piece PC of fragment F for k-step KS of the stage at LDS address `stage`.
  template <int F, int KS, int PC>
  __device__ __forceinline__ Piece read(unsigned stage) const {
    if constexpr (KC)
      return lds_read_b128<F * 4 * T::kGroup>(stage + base[KS * kPieces + PC]);  // 32 rows = four groups of 8
    else if constexpr (ES == 1)
      return lds_read_tr8<KS * KB * RB + PC * 8 * RB>(stage + base[F]);
    else
      return lds_read_tr16<KS * (KB / 2) * RB + PC * 4 * RB>(stage + base[F]);
  }
};

template <typename Frag, typename Piece, int N>
__device__ __forceinline__ Frag join_pieces(const Piece (&pc)[N]) {
  if constexpr (sizeof(Piece) == sizeof(Frag)) {
    return pc[0];
  } else if constexpr (sizeof(Piece) == 16) {  // two 128-bit pieces
    return Frag{pc[0].x, pc[0].y, pc[0].z, pc[0].w, pc[1].x, pc[1].y, pc[1].z, pc[1].w};
  } else if constexpr (N == 2) {
    return Frag{pc[0].x, pc[0].y, pc[1].x, pc[1].y};
  } else {
    return Frag{pc[0].x, pc[0].y, pc[1].x, pc[1].y, pc[2].x, pc[2].y, pc[3].x, pc[3].y};
  }
}

constexpr int ceil_div(int a, int b) { return (a + b - 1) / b; }

// EDGE: the operands are copies padded to whole tiles, C is not - its last tile rows / columns end at p.m / p.n and
// the epilogue touches nothing beyond them.
// CQUADS: an int32 C in small blocks with contiguous rows (the 4 x 4 blocks of src/gemm/packed-gemm.md:270-298, up to
// 16 columns), no fused steps - see the epilogue.
// SCAN (floating-point row-major C, beta == 0 evaluated like the reference's loops, whole tiles, K of at least 64
// slices on the wide tile and 32 on the narrow one): whether 0 * c is a zero for every old c of the tile - i.e. no NaN,
// no infinity - is found out while the tile is multiplied. Every even slice each wave requests 1 KiB of the tile's
// old C (a row of the wide tile, two rows of the narrow one; wave w takes every eighth) into one of four slots of LDS
// behind the operand stages; three and four slices later it reads them back, 8 bytes per lane and slice (its own
// loads, its own counter: no barrier), and tests the exponents. After the loop the waves put their findings together.
// A tile without such a value is then written as an initialised one (the sign of exact zeros is still taken from the
// old c, see write_wave_tile); a tile with one takes the path that reads all of C. Either way the bits are those of
// 0 * c + alpha * acc.
// (Measured on fp8 8192^3, old C in memory: a first version - every wave its own block, lane addresses for any
// layout of C, 64-bit block arithmetic per load - cost 62-70 us of 415 whether it loaded 4 bytes per lane every slice
// or 16 every other one, 25-43 us of that with the rows already in cache: the instructions between two MFMAs, not the
// loads. Hence contiguous rows, whose address is a scalar product and a shift of the lane index.)
template <int TA, int TB, bool A_KC, bool B_KC, int BN, bool EDGE = false, int EXTRA = 0, bool CQUADS = false, bool SCAN = false>
__global__ void __launch_bounds__(512) gemm_mfma_ring_kernel(MfmaArgs p) {
  using KA = Kind<TA>;
  using M = Mma<TA, TB>;
  using Frag = typename M::Frag;
  using Acc = typename KA::Acc;
  using AccElem = decltype(Acc{}.x);
  constexpr int SB = kRingSlice, STAGES = ring_stages(BN);
  static_assert(STAGES % 2 == 0, "pair loads fill two neighbouring stages");
  constexpr int ES = KA::ES, KB = KA::KB, FRB = KB / 2;
  // Eight waves: 2 x 4 blocks of 128 x 64 on a 256 x 256 tile, 4 x 2 blocks of 64 x 64 on a 256 x 128 one.
  constexpr int BM = 256, WAVES = 8, WAVES_N = BN == 256 ? 4 : 2, WAVES_M = WAVES / WAVES_N;
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N, MI = WM / 32, NI = WN / 32;
  constexpr int kEpilogueBatch = 2;              // blocks whose old C values are requested together
  constexpr int kSteps = SB / KB;
  constexpr int kMfmas = MI * NI;
  constexpr int kSlots = kSteps * kMfmas;        // MFMA slots per slice
  constexpr int kPre = (kSteps - 1) * kMfmas;    // slots before the slice's barrier
  // Four stages per operand. A slice's fragments are read from LDS while the k-step before them is
  // multiplied; with one k-step per slice (64 bytes of K per MFMA) that is the slice before, and the
  // stage of the slice being multiplied is free from its barrier on. So loads run kExtra = 1 slice
  // further ahead there: every-slice loads fill the issuing slice's own stage with slice s+4, pair loads
  // go out on odd slices for slices s+3 and s+4. Otherwise: slice s+3, and pairs on even slices for
  // s+2 and s+3. (Six stages for a K-contiguous operand fit the 160 KiB of LDS next to an MN-contiguous
  // partner, and measured slower.)
  constexpr int NSA = STAGES, NSB = STAGES;
  constexpr int kExtra = kSteps == 1 ? 1 : 0;
  constexpr int kEachAhead = STAGES - 1 + kExtra, kPairAhead = STAGES - 2 + kExtra;
  constexpr int kPairU = kPairAhead & 1;             // parity of the slices that issue pair loads
  constexpr int kPairsPrologue = (kPairU + kPairAhead) / 2;
  using LA = SLoader<ES, A_KC, WAVES, BM, NSA>;
  using LB = SLoader<ES, B_KC, WAVES, BN, NSB>;
  using TileA = STile<ES, A_KC, BM, NSA>;
  using TileB = STile<ES, B_KC, BN, NSB>;
  // Load `it` of a slice's kLoads goes out behind MFMA slot it * kSlots / kLoads, pair loads first.
  constexpr int kPairA = A_KC ? LA::kBlocks : 0, kPairB = B_KC ? LB::kBlocks : 0;
  constexpr int kEachA = A_KC ? 0 : LA::kBlocks, kEachB = B_KC ? 0 : LB::kBlocks;
  constexpr int kEach = kEachA + kEachB, kPairs = kPairA + kPairB;
  constexpr int kLoadsOfU[2] = {(kPairU == 0 ? kPairs : 0) + kEach, (kPairU == 1 ? kPairs : 0) + kEach};
  // SCAN: one more load in every even slice, the first thing that slice requests (behind its first MFMA, in front
  // of its pair loads): older than every load of its slice, so it has landed whenever the slice's own loads are
  // waited for. It counts as younger wherever a whole slice counted below is an even one, and in front of the
  // barrier of its own slice when that barrier is not in the slice's first k-step.
  constexpr int kScanSlots = 4, kScanSlot = WAVES * 1024;
  static_assert(!SCAN || (std::is_same<AccElem, float>::value && !EDGE && EXTRA == 0 && !CQUADS), "a plain floating-point product on whole tiles");
  static_assert(kPairAhead <= 3, "the rows requested in slice 2q are read back in slices 2q + 3 and 2q + 4");
  constexpr int kPreOfU[2] = {ceil_div(kPre * kLoadsOfU[0], kSlots), ceil_div(kPre * kLoadsOfU[1], kSlots)};
  constexpr auto younger = [](int u, const int (&loads)[2], int each, int pair_ahead, bool scan, int pre_slots) {
    int n = u == 0 ? 0 : each;
    // the whole slices counted: t - pair_ahead + u + d for d = 1 .. pair_ahead - 1 - u, t (of parity u) being this slice
    for (int d = 1; d <= pair_ahead - 1 - u; ++d) {
      n += loads[(u + d) % 2];
      if (scan && (pair_ahead + d) % 2 == 0) n += 1;
    }
    if (scan && u == 0 && pre_slots > 0) n += 1;  // this slice's own, requested in its first k-step
    return n;
  };
  constexpr int kInFlightOfU[2] = {younger(0, kLoadsOfU, kEach, kPairAhead, SCAN, kPre) + kPreOfU[0],
                                   younger(1, kLoadsOfU, kEach, kPairAhead, SCAN, kPre) + kPreOfU[1]};
  static_assert(STAGES != 4 || SCAN || (kInFlightOfU[0] == (kExtra ? 2 * kEach + kPairs : kEach) + kPreOfU[0] &&
                                        kInFlightOfU[1] == (kExtra ? 2 * kEach : kEach) + kPreOfU[1]),
                "the four-stage counts, as derived by hand above");
  static_assert(kInFlightOfU[0] < 64 && kInFlightOfU[1] < 64, "vmcnt is a 6-bit counter");

  using RA = FragReader<ES, A_KC, FRB, KB, BM, NSA, MI>;
  using RB = FragReader<ES, B_KC, FRB, KB, BN, NSB, NI>;
  constexpr int PA = RA::kPieces, PB = RB::kPieces;
  constexpr int kReads = MI * PA + NI * PB;      // LDS instructions per k-step
  constexpr int kReadSlots = kMfmas / 2;         // ... issued behind the first half of its MFMAs, the rest is time to land (all of them behind the first of four MFMAs on the narrow tile: 73.5-74.0 against 72.7-73.0 us)

  extern __shared__ __attribute__((aligned(16))) char smem[];
  char *region_a = smem, *region_b = smem + TileA::kRegion;
  const unsigned addr_a = (unsigned)(size_t)LDS_PTR(char, smem), addr_b = addr_a + TileA::kRegion;

  // K may be shared between `splits` workgroups per tile: p.k is then one share (whole slice pairs), split s
  // starts s shares into K and leaves its raw sums in plane s of the workspace.
  unsigned tm, tn;
  const unsigned tiles = p.tiles_m * p.tiles_n, split = blockIdx.x / tiles;
  tile_of_block(blockIdx.x % tiles, p.tiles_m, p.tiles_n, tm, tn);
  const size_t m0 = (size_t)tm * BM, n0 = (size_t)tn * BN;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;  // the wave index as a scalar: nothing derived from it occupies a vector register across the main loop
  const int wm = (wave / WAVES_N) * WM, wn = (wave % WAVES_N) * WN;

  LA la;
  LB lb;
  la.init(p.a + (size_t)split * p.k * p.a_sk * ES, m0, p.a_s1, p.a_s0, p.a_sk);
  lb.init(p.b + (size_t)split * p.k * p.b_sk * ES, n0, p.b_s1, p.b_s0, p.b_sk);
  RA ra;
  RB rb;
  ra.init(wm);
  rb.init(wn);

  Acc acc[MI][NI];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NI; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

  // K is a whole number of slice pairs. Units beyond the end are requested as the last unit
  // again: in range, and the stage they land in is never read, which keeps the load counts static.
  // (32-bit counters - the host refuses a K of 2^31 slices or more: a 64-bit "less than" of two scalars is a vector
  // compare and two vector registers)
  const unsigned slices = (unsigned)(p.k * ES / SB), pairs = slices / 2;

  // SCAN: the tile's old C, 1 KiB per wave and two slices (the host has checked that K has the slices for it and
  // that C is row-major with 16-byte aligned rows).
  unsigned long long scan_bad = 0;   // lanes that have seen a NaN or an infinity
  v2i scan_pend = {0, 0};            // the 8 bytes read back during the k-step before
  char *const scan_region = smem + TileA::kRegion + TileB::kRegion + wave * 1024;
  const unsigned scan_addr = addr_b + TileB::kRegion + wave * 1024;
  // (row of this wave's first load, and the bytes from one load's rows to the next: scalars, 64 x rsc0 fits 32 bits)
  constexpr unsigned kScanRowsPerLoad = BN == 256 ? 1 : 2, kScanLoadsPerWave = BM / (WAVES * kScanRowsPerLoad);
  // C in panels of 64 x 64 contiguous values (rsc0 == 64): 1 KiB is four rows of a panel; the tile's panels row by
  // row, 16 such pieces each, piece 8 q + w is wave w's load q.
  const bool scan_panels = p.rsc0 == 64 && p.rsc1 != 64 * 64;
  const char *const scan_rows = scan_panels ? reinterpret_cast<const char *>(p.c) + ((m0 >> 6) * p.rsc1 + (n0 >> 6) * p.csc1) * 4
                                            : reinterpret_cast<const char *>(p.c) + ((m0 + (size_t)wave * kScanRowsPerLoad) * p.rsc0 + n0) * 4;
  const unsigned scan_step = (unsigned)p.rsc0 * (WAVES * kScanRowsPerLoad * 4u);
  [[maybe_unused]] auto scan_issue = [&](size_t s) {  // s even: load s / 2 of this wave (the last one again beyond the tile)
    const unsigned q = (unsigned)(s >> 1) < kScanLoadsPerWave ? (unsigned)(s >> 1) : kScanLoadsPerWave - 1;  // uniform
    const char *rows = scan_rows + (size_t)q * scan_step;
    if (scan_panels) {
      const unsigned piece = q * WAVES + wave, panel = piece >> 4, pi = panel / (BN / 64), pj = panel % (BN / 64);
      rows = scan_rows + ((size_t)pi * p.rsc1 + (size_t)pj * p.csc1) * 4 + (piece & 15u) * 1024u;
    }
    // The lane's own part of the address is computed anew for every load, from a lane index the compiler cannot
    // follow: held across the loop it would be a register that the loop does not have.
    unsigned l = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
    asm volatile("" : "+v"(l));
    unsigned mine;
    if constexpr (BN == 256)
      mine = l * 16u;                                                                // 64 lanes x 16 bytes: one row of 256 columns
    else
      mine = (l & 31u) * 16u + ((unsigned)((int)(l << 26) >> 31) & (scan_panels ? 512u : (unsigned)p.rsc0 * 4u));  // lanes 32-63: the row below (panels: the next 512 bytes)
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(rows + mine),
                                     (__attribute__((address_space(3))) void *)(scan_region + (unsigned)((s >> 1) % kScanSlots) * kScanSlot), 16, 0, 0);
  };
  [[maybe_unused]] auto scan_read = [&](unsigned slot, unsigned half) {  // 512 of this wave's 1024 bytes in `slot`; the value counts from the next lgkmcnt(0) on
    unsigned l = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
    asm volatile("" : "+v"(l));
    const unsigned addr = scan_addr + slot * kScanSlot + half * 512 + l * 8;
    asm volatile("ds_read_b64 %0, %1" : "=v"(scan_pend) : "v"(addr) : "memory");
  };
  [[maybe_unused]] auto scan_check = [&]() {  // behind an lgkmcnt(0): NaN or infinity, either sign, in either dword
    asm volatile("" : "+v"(scan_pend));
    unsigned long long x, y;
    asm volatile("v_cmp_class_f32_e64 %0, %1, %2" : "=s"(x) : "v"(scan_pend.x), "s"(0x207));
    asm volatile("v_cmp_class_f32_e64 %0, %1, %2" : "=s"(y) : "v"(scan_pend.y), "s"(0x207));
    scan_bad |= x | y;
  };

  if constexpr (A_KC) {
#pragma unroll
    for (int i = 0; i < kPairsPrologue; ++i) la.issue(region_a, 2 * i, (unsigned)i < pairs ? (unsigned)i : pairs - 1);
  } else {
#pragma unroll
    for (int i = 0; i < kEachAhead; ++i) la.issue(region_a, i, (unsigned)i < slices ? (unsigned)i : slices - 1);
  }
  if constexpr (B_KC) {
#pragma unroll
    for (int i = 0; i < kPairsPrologue; ++i) lb.issue(region_b, 2 * i, (unsigned)i < pairs ? (unsigned)i : pairs - 1);
  } else {
#pragma unroll
    for (int i = 0; i < kEachAhead; ++i) lb.issue(region_b, i, (unsigned)i < slices ? (unsigned)i : slices - 1);
  }
  if constexpr (SCAN) {  // the slots start as zeros: the first slices read slots that no load has filled yet
#pragma unroll
    for (int slot = 0; slot < kScanSlots; ++slot)
#pragma unroll
      for (int quarter = 0; quarter < 4; ++quarter)
        *reinterpret_cast<float *>(scan_region + slot * kScanSlot + quarter * 256 + (threadIdx.x & 63) * 4) = 0.0f;
  }
  wait_loads_upto<0>();
  __syncthreads();

  typename RA::Piece pa[2][MI][PA];
  typename RB::Piece pb[2][NI][PB];

  // Read item R of a k-step: fragment by fragment, A and B alternating, so that
  // what the next k-step's first MFMAs need is requested first.
  auto read_item = [&](auto rc, auto ksc, int buf, unsigned stage_a, unsigned stage_b) {
    constexpr int R = decltype(rc)::value, KS = decltype(ksc)::value;
    constexpr int kPair = PA + PB, kBoth = (MI < NI ? MI : NI) * kPair;
    if constexpr (R < kBoth) {
      constexpr int F = R / kPair, W = R % kPair;
      if constexpr (W < PA)
        pa[buf][F][W] = ra.template read<F, KS, W>(stage_a);
      else
        pb[buf][F][W - PA] = rb.template read<F, KS, W - PA>(stage_b);
    } else if constexpr (MI > NI) {
      constexpr int X = R - kBoth, F = NI + X / PA, W = X % PA;
      pa[buf][F][W] = ra.template read<F, KS, W>(stage_a);
    } else {
      constexpr int X = R - kBoth, F = MI + X / PB, W = X % PB;
      pb[buf][F][W] = rb.template read<F, KS, W>(stage_b);
    }
  };
  // All reads in flight have landed; from here on the compiler may use buffer `buf`.
  auto landed = [&](int buf) {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
      for (int w = 0; w < PA; ++w) asm volatile("" : "+v"(pa[buf][i][w]));
#pragma unroll
    for (int j = 0; j < NI; ++j)
#pragma unroll
      for (int w = 0; w < PB; ++w) asm volatile("" : "+v"(pb[buf][j][w]));
  };

  [&]<int... Rs>(std::integer_sequence<int, Rs...>) {
    (read_item(std::integral_constant<int, Rs>{}, std::integral_constant<int, 0>{}, 0, addr_a, addr_b), ...);
  }(std::make_integer_sequence<int, kReads>{});

  // Two slices per trip: the parity of the slice decides which loads it issues, and (for the
  // operand kinds with one k-step per slice) which fragment buffer a k-step uses.
  for (unsigned s0 = 0; s0 < slices; s0 += 2) {
    [&]<int... Us>(std::integer_sequence<int, Us...>) {
      (
          [&](auto uc) {
            constexpr int U = decltype(uc)::value;
            constexpr int kLoads = kLoadsOfU[U];
            const unsigned s = s0 + U;
            const unsigned fill_slice = s + kEachAhead < slices ? s + kEachAhead : slices - 1;  // every-slice operands
            const unsigned fill_pair = (s + kPairAhead) / 2 < pairs ? (s + kPairAhead) / 2 : pairs - 1;  // pair operands (s of parity kPairU)
            const unsigned s32 = s;
            const int cur_a = (int)(s32 % NSA), nxt_a = (int)((s32 + 1) % NSA), cur_b = (int)(s32 % NSB), nxt_b = (int)((s32 + 1) % NSB);
            const int fill_a = (int)((s32 + (A_KC ? kPairAhead : kEachAhead)) % NSA), fill_b = (int)((s32 + (B_KC ? kPairAhead : kEachAhead)) % NSB);
            [&]<int... KSs>(std::integer_sequence<int, KSs...>) {
              (
                  [&](auto ksc) {
                    constexpr int KS = decltype(ksc)::value;
                    constexpr bool kLast = KS == kSteps - 1;
                    constexpr int KSN = kLast ? 0 : KS + 1;  // k-step whose fragments are read during this one
                    constexpr int cur = (U * kSteps + KS) & 1, nx = cur ^ 1;
                    if constexpr (kLast) {
                      // The reads below cross into the next slice: its data must have landed for every wave.
                      // Own reads first, so that nobody's read of the stage refilled next is still in flight.
                      wait_loads_upto<kInFlightOfU[U]>();
                      landed(cur);
                      __builtin_amdgcn_s_barrier();
                    } else {
                      landed(cur);
                    }
                    Frag fa[MI], fb[NI];
#pragma unroll
                    for (int i = 0; i < MI; ++i) fa[i] = join_pieces<Frag>(pa[cur][i]);
#pragma unroll
                    for (int j = 0; j < NI; ++j) fb[j] = join_pieces<Frag>(pb[cur][j]);
                    const unsigned sa = addr_a + (kLast ? nxt_a : cur_a) * TileA::kStageStep;
                    const unsigned sb = addr_b + (kLast ? nxt_b : cur_b) * TileB::kStageStep;
                    __builtin_amdgcn_sched_barrier(0);
                    [&]<int... Qs>(std::integer_sequence<int, Qs...>) {
                      (
                          [&](auto qc) {
                            constexpr int Q = decltype(qc)::value, kSlot = KS * kMfmas + Q;
                            constexpr int i = Q / NI, j = Q % NI;
                            acc[i][j] = M::run(fa[i], fb[j], acc[i][j]);
                            // The MFMA first, what belongs to its slot in its shadow. Left to itself the compiler moves a slot's address
                            // arithmetic, reads and loads in front of the MFMA - and behind a barrier, which the waves leave together,
                            // instructions in front of the first MFMA are a gap in every SIMD's matrix core at once (measured, same job,
                            // alternating libraries: int8 8192^3 -1.5 %, fp8 with column-major A -3 %, bf16 config 3 -2.3 %; for the
                            // extra instructions of SCAN the difference between +43 and +14 us).
                            __builtin_amdgcn_sched_barrier(0);
                            if constexpr (SCAN && U == 0 && kSlot == 0) scan_issue(s);
                            if constexpr (SCAN && kSlot == 1) scan_check();  // what the last slot of the k-step before has read, behind this k-step's lgkmcnt(0)
                            // Behind the barrier of slice 2q + 3 the rows requested in slice 2q have landed: half of them is
                            // read back in that slice, half in the next (the first slices find zeros).
                            if constexpr (SCAN && kSlot == kSlots - 1) scan_read(((s32 >> 1) + kScanSlots - (U == 1 ? 1 : 2)) % kScanSlots, U == 1 ? 0 : 1);
                            // this slot's share of the next k-step's reads
                            [&]<int... Rs>(std::integer_sequence<int, Rs...>) {
                              (
                                  [&](auto rc) {
                                    constexpr int R = decltype(rc)::value;
                                    if constexpr (R * kReadSlots / kReads == Q)
                                      read_item(rc, std::integral_constant<int, KSN>{}, nx, sa, sb);
                                  }(std::integral_constant<int, Rs>{}),
                                  ...);
                            }(std::make_integer_sequence<int, kReads>{});
                            // and this slot's share of the slice's loads
                            [&]<int... Ls>(std::integer_sequence<int, Ls...>) {
                              (
                                  [&](auto lc) {
                                    constexpr int L = decltype(lc)::value;
                                    if constexpr (L * kSlots / kLoads == kSlot) {
                                      constexpr int kPairsNow = U == kPairU ? kPairs : 0;
                                      if constexpr (L < kPairsNow) {
                                        if constexpr (L < kPairA)
                                          la.issue_one(region_a, fill_a, fill_pair, L);
                                        else
                                          lb.issue_one(region_b, fill_b, fill_pair, L - kPairA);
                                      } else if constexpr (L - kPairsNow < kEachA) {
                                        la.issue_one(region_a, fill_a, fill_slice, L - kPairsNow);
                                      } else {
                                        lb.issue_one(region_b, fill_b, fill_slice, L - kPairsNow - kEachA);
                                      }
                                    }
                                  }(std::integral_constant<int, Ls>{}),
                                  ...);
                            }(std::make_integer_sequence<int, kLoads>{});
                            __builtin_amdgcn_sched_barrier(0);
                          }(std::integral_constant<int, Qs>{}),
                          ...);
                    }(std::make_integer_sequence<int, kMfmas>{});
                  }(std::integral_constant<int, KSs>{}),
                  ...);
            }(std::make_integer_sequence<int, kSteps>{});
          }(std::integral_constant<int, Us>{}),
          ...);
    }(std::make_integer_sequence<int, 2>{});
  }
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
  if constexpr (SCAN) {
    // The last rows requested have not been read back or in part only, and the last 8 bytes read have not been
    // tested: all slots once more (a row tested twice changes nothing).
    scan_check();
#pragma unroll
    for (int slot = 0; slot < kScanSlots; ++slot)
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        scan_read(slot, half);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        scan_check();
      }
  }

  if (p.splits > 1) {  // a share of K: the raw sums go to this split's M x N plane
    AccElem *plane = reinterpret_cast<AccElem *>(p.partial) + (size_t)split * p.m * p.n;
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      const size_t col = n0 + wn + j * 32 + (lane & 31);
      if (EDGE && col >= p.n) continue;
#pragma unroll
      for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const size_t row = m0 + wm + i * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
          if (!EDGE || row < p.m) plane[row * p.n + col] = acc[i][j][r];
        }
    }
    return;
  }
  if constexpr (CQUADS) {
    // A lane holds four consecutive rows of one column, and with blocks of four columns a row of a block is 16
    // bytes: stored as they are, a wave's stores are 16-byte runs 64 bytes apart (8192^3: 100 us more than a
    // row-major C). The four lanes of a quad hold the four columns of those rows, so the 4 x 4 values are exchanged
    // inside the quad - lane q ends up with row q's four columns - and every lane moves 16 bytes per instruction: a
    // quad covers 64 contiguous bytes, lanes 0-31 eight neighbouring blocks.
    static_assert(std::is_same<AccElem, int>::value && !EDGE && EXTRA == 0, "int32 C, whole tiles, no fused steps");
    int *c = reinterpret_cast<int *>(p.c);
    const bool init = p.beta.i == 0;
    const int qd = lane & 3;
    const size_t cmask = (size_t(1) << p.ccs) - 1, rmask = (size_t(1) << p.crs) - 1;
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      const size_t col4 = n0 + wn + j * 32 + (lane & 28);   // the quad's first column, a multiple of four
      const size_t col_off = (col4 >> p.ccs) * p.csc1 + (col4 & cmask);
#pragma unroll
      for (int i0 = 0; i0 < MI; i0 += kEpilogueBatch) {
        v4i *out[kEpilogueBatch][4];
        v4i old[kEpilogueBatch][4];
#pragma unroll
        for (int i = 0; i < kEpilogueBatch; ++i)
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const size_t row = m0 + wm + (i0 + i) * 32 + g * 8 + (lane >> 5) * 4 + qd;
            out[i][g] = reinterpret_cast<v4i *>(c + (row >> p.crs) * p.rsc1 + (row & rmask) * p.rsc0 + col_off);
          }
        if (!init) {
#pragma unroll
          for (int i = 0; i < kEpilogueBatch; ++i)
#pragma unroll
            for (int g = 0; g < 4; ++g) old[i][g] = *out[i][g];
        }
#pragma unroll
        for (int i = 0; i < kEpilogueBatch; ++i)
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const Acc &t = acc[i0 + i][j];
            v4i r;
#define SKL_ROW_OF_QUAD(CC, CTRL)                                                                                    \
  {                                                                                                                   \
    const int b0 = __builtin_amdgcn_update_dpp(0, t[4 * g + 0], CTRL, 0xF, 0xF, true), b1 = __builtin_amdgcn_update_dpp(0, t[4 * g + 1], CTRL, 0xF, 0xF, true); \
    const int b2 = __builtin_amdgcn_update_dpp(0, t[4 * g + 2], CTRL, 0xF, 0xF, true), b3 = __builtin_amdgcn_update_dpp(0, t[4 * g + 3], CTRL, 0xF, 0xF, true); \
    r[CC] = qd == 0 ? b0 : qd == 1 ? b1 : qd == 2 ? b2 : b3;                                                          \
  }
            SKL_ROW_OF_QUAD(0, 0x00)   // quad_perm: every lane reads the quad's lane 0 - column 0 of the four rows
            SKL_ROW_OF_QUAD(1, 0x55)
            SKL_ROW_OF_QUAD(2, 0xAA)
            SKL_ROW_OF_QUAD(3, 0xFF)
#undef SKL_ROW_OF_QUAD
            v4i v;
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = init ? skl_initialise(r[e], (const int *)nullptr, p.alpha, p.beta) : skl_combine(r[e], old[i][g][e], p.alpha, p.beta);
            __builtin_nontemporal_store(v, out[i][g]);
          }
      }
    }
    return;
  }
  if constexpr (SCAN) {
    // What the eight waves have found, put together: each wave's word where its first slot began (its own reads of
    // the slots are over), a barrier, and everybody reads all eight.
    unsigned *const found = reinterpret_cast<unsigned *>(smem + TileA::kRegion + TileB::kRegion);
    found[wave * 256] = scan_bad != 0;
    __syncthreads();
    unsigned any = 0;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) any |= found[w * 256];
    MfmaArgs q = p;
    if (any == 0) q.beta.fz.skip_c_read = 1;  // 0 * c is a zero everywhere in this tile
    write_wave_tile<MI, NI, EDGE, EXTRA>(q, acc, m0 + wm, n0 + wn);
  } else {
    write_wave_tile<MI, NI, EDGE, EXTRA>(p, acc, m0 + wm, n0 + wn);
  }
}

// C = beta*C + alpha * (sum of the splits' planes, in split order), then the fused steps: the second
// half of a GEMM whose K range was shared out between workgroups.
template <typename T>
__global__ void __launch_bounds__(256) gemm_split_reduce_kernel(MfmaArgs p) {
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= p.m * p.n) return;
  const size_t row = idx / p.n, col = idx % p.n;
  // Eight planes are requested before the first is used (one memory round trip per eight, not per plane); the
  // sum still runs over the planes in order, starting from plane 0 itself.
  const T *plane = reinterpret_cast<const T *>(p.partial) + idx;
  const size_t mn = p.m * p.n;
  T sum = plane[0];
  for (unsigned q0 = 1; q0 < p.splits; q0 += 8) {
    T v[8];
#pragma unroll
    for (unsigned u = 0; u < 8; ++u) v[u] = q0 + u < p.splits ? plane[(size_t)(q0 + u) * mn] : T(0);
#pragma unroll
    for (unsigned u = 0; u < 8; ++u) {
      if (q0 + u >= p.splits) continue;
      if constexpr (std::is_same<T, int>::value)
        sum = (int)((unsigned)sum + (unsigned)v[u]);
      else
        sum = __fadd_rn(sum, v[u]);
    }
  }
  T *c = reinterpret_cast<T *>(p.c) + (row >> p.crs) * p.rsc1 + (row & ((size_t(1) << p.crs) - 1)) * p.rsc0 +
         (col >> p.ccs) * p.csc1 + (col & ((size_t(1) << p.ccs) - 1)) * p.csc0;
  T v = skl_beta_is_zero<T>(p.beta) ? skl_initialise(sum, c, p.alpha, p.beta) : skl_combine(sum, *c, p.alpha, p.beta);
  if (p.bias) v = skl_add_bias(v, reinterpret_cast<const T *>(p.bias)[col]);
  v = skl_activate(v, p.rq.act);
  if (!p.rq.q_only) *c = v;
  skl_emit_requantised(p.rq, v, row, col);
  if (p.max && v > skl_lowest<T>()) skl_atomic_max(reinterpret_cast<T *>(p.max), v);
}

struct SequenceGuard {
  const bool held;
  explicit SequenceGuard(bool hold) : held(hold) { if (held) skl_hip_sequence_begin(); }
  ~SequenceGuard() { if (held) skl_hip_sequence_end(); }
};

constexpr size_t kRingMinSlicesPerSplit = 64;  // below 8 KiB of K per row the pass over the planes costs what the split saves

// The streaming kernels for whole tiles also exist with the activation (none or ReLU) and requantisation steps, for a
// copy that can be written as dwords (a quantised layer's 8-bit output at a quarter of C's bytes: int8 behind an
// int32 C, fp8 behind an fp32 C); every other call with those steps goes to the bounds-checked kernels.
template <int TA, int TB>
constexpr bool kRingCarriesExtraSteps = TA == TB;   // every kind but the mixed fp8 pairings

// An int32 C the streaming kernel writes 16 bytes per lane: blocks of 4 to 16 columns with contiguous rows, a
// multiple of four rows per block, everything on 16-byte boundaries, no fused steps.
inline bool c_in_row_quads(const MfmaArgs &p) {
  return !p.bias && !p.max && !p.rq.act && !p.rq.q && p.csc0 == 1 && p.ccs >= 2 && p.ccs <= 4 && p.crs >= 2 &&
         (((uintptr_t)p.c | (p.rsc0 * 4) | (p.rsc1 * 4) | (p.csc1 * 4)) & 15) == 0;
}

template <int TA, int TB, bool A_KC, bool B_KC, int BN, bool EDGE = false, int EXTRA = 0, bool CQUADS = false, bool SCAN = false>
int launch_ring(const MfmaArgs &args) {
  if constexpr (EXTRA == 0 && kRingCarriesExtraSteps<TA, TB> && !EDGE) {
    if (args.rq.q) return args.rq.q_only ? launch_ring<TA, TB, A_KC, B_KC, BN, EDGE, 2>(args) : launch_ring<TA, TB, A_KC, B_KC, BN, EDGE, 3>(args);
  }
  if constexpr (TA == SKL_DT_I8 && TB == SKL_DT_I8 && A_KC && B_KC && !EDGE && EXTRA == 0 && !CQUADS) {  // what copies of blocked operands look like
    if (c_in_row_quads(args)) return launch_ring<TA, TB, A_KC, B_KC, BN, EDGE, 0, true>(args);
  }
  constexpr int ES = Kind<TA>::ES;
  using AccElem = decltype(typename Kind<TA>::Acc{}.x);
  if constexpr (std::is_same<AccElem, float>::value && !EDGE && EXTRA == 0 && !CQUADS && !SCAN) {
    // beta == 0 evaluated as the reference's loops do (0 * c: a NaN or an infinity in C stays a NaN): the old C is
    // looked through while the tile is multiplied, 8 KiB of it per two slices - needs 64 slices on the wide tile, 32
    // on the narrow one, a tile to itself (no shared K) and a row-major C.
    const size_t scan_slices = args.k * ES / kRingSlice, scan_tiles = (args.m / 256) * (args.n / BN);
    const bool shared_k = scan_tiles <= 128 && scan_slices % 4 == 0 && scan_slices / 2 >= kRingMinSlicesPerSplit;
    // C row-major: rows and columns at one stride each across the blocks, rows of 16-byte aligned starts ...
    const bool row_major = args.csc0 == 1 && args.csc1 == (size_t(1) << args.ccs) && args.rsc1 == (args.rsc0 << args.crs) &&
                           (((uintptr_t)args.c | (args.rsc0 * 4)) & 15) == 0 && args.rsc0 < (size_t(1) << 26) &&
                           !(args.rsc0 == 64 && args.rsc1 != 64 * 64);
    // ... or in panels of 64 x 64 contiguous values on 16-byte boundaries
    const bool panels = args.csc0 == 1 && args.rsc0 == 64 && args.crs == 6 && args.ccs == 6 && args.rsc1 != 64 * 64 &&
                        (((uintptr_t)args.c | (args.rsc1 * 4) | (args.csc1 * 4)) & 15) == 0;
    if (args.beta.f == 0.0f && args.beta.fz.skip_c_read == 0 && !shared_k && (row_major || panels) && scan_slices >= (BN == 256 ? 64 : 32))
      return launch_ring<TA, TB, A_KC, B_KC, BN, EDGE, EXTRA, CQUADS, true>(args);
  }
  constexpr int lds = ring_stages(BN) * (256 + BN) * kRingSlice + (SCAN ? 4 * 8 * 1024 : 0);
  auto kernel = gemm_mfma_ring_kernel<TA, TB, A_KC, B_KC, BN, EDGE, EXTRA, CQUADS, SCAN>;
  static std::atomic<bool> configured{false};  // per instantiation; racing threads set the same value
  if (!configured.load(std::memory_order_acquire)) {
    int rc = skl_check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, lds),
                           "gemm_mfma_ring: LDS size");
    if (rc != 0) return rc;
    configured.store(true, std::memory_order_release);
  }
  MfmaArgs p = args;
  p.tiles_m = (unsigned)((p.m + (EDGE ? 255 : 0)) / 256);
  p.tiles_n = (unsigned)((p.n + (EDGE ? BN - 1 : 0)) / BN);
  const size_t tiles = (size_t)p.tiles_m * p.tiles_n;
  // Tiles for at most half of the 256 compute units: K is shared between two workgroups per tile (each at least
  // kRingMinSlicesPerSplit slices long) and a second pass adds the two planes and applies alpha / beta.
  const size_t slices = p.k * ES / kRingSlice;
  if (slices >= (size_t(1) << 31)) {
    skl_hip_record_error(-2, "gemm_mfma: K too long");
    return -2;
  }
  p.splits = (tiles <= 128 && slices % 4 == 0 && slices / 2 >= kRingMinSlicesPerSplit) ? 2 : 1;
  SequenceGuard sequence(p.splits > 1);
  if (p.splits > 1) {
    p.partial = (char *)skl_workspace((size_t)p.splits * p.m * p.n * 4);
    if (!p.partial) return -4;
    p.k /= p.splits;  // one share; whole slice pairs
  }
  const size_t grid = tiles * p.splits;
  if (grid > 0x7FFFFFFFu) {
    skl_hip_record_error(-2, "gemm_mfma: grid too large");
    return -2;
  }
  kernel<<<(unsigned)grid, 512, lds, skl_current_stream()>>>(p);
  int rc = skl_check_launch("gemm_mfma_ring");
  if (rc != 0 || p.splits == 1) return rc;
  const size_t blocks = (p.m * p.n + 255) / 256;
  if (blocks > 0x7FFFFFFFu) {
    skl_hip_record_error(-2, "gemm_mfma: grid too large");
    return -2;
  }
  gemm_split_reduce_kernel<AccElem><<<(unsigned)blocks, 256, 0, skl_current_stream()>>>(p);
  return skl_check_launch("gemm_split_reduce");
}

// How many ways K is shared out when a problem has too few tiles for the chip: enough to put about two
// workgroups on every compute unit, each share at least kMinSlicesPerSplit slices long, planes within 64 MiB.
// (Four slices: the reference's benchmark shapes of one 128 x 128 tile - 8192 k of int8, 4096 k of bf16 - 10.2 -> 8.9 us
// and 10.0 -> 9.0 us against shares of eight; two slices measure the same.)
constexpr size_t kMinSlicesPerSplit = 4, kSplitFromSlices = 32, kSplitPlaneLimit = size_t(64) << 20;
inline unsigned splits_for(size_t tiles, size_t slices, size_t m, size_t n) {
  if (tiles >= 256 || slices < kSplitFromSlices) return 1;
  size_t want = (512 + tiles - 1) / tiles;
  if (want > slices / kMinSlicesPerSplit) want = slices / kMinSlicesPerSplit;
  while (want > 1 && want * m * n * 4 > kSplitPlaneLimit) --want;
  return (unsigned)(want < 1 ? 1 : want);
}

template <int TA, int TB, bool A_KC, bool B_KC, int BM, int BN, int WAVES_M, int WAVES_N, bool GUARDED, bool EXACT = false, bool EXTRA = false>
int launch_one(const MfmaArgs &args) {
  if constexpr (!EXTRA) {  // calls with an activation or a requantised copy take the kernels that carry those steps
    if (args.rq.act || args.rq.q) return launch_one<TA, TB, A_KC, B_KC, BM, BN, WAVES_M, WAVES_N, GUARDED, EXACT, true>(args);
  }
  constexpr int ES = Kind<TA>::ES;
  constexpr int NT = WAVES_M * WAVES_N * 64;
  constexpr int lds = 2 * (Tile<ES, BM, A_KC, NT>::kBytes + Tile<ES, BN, B_KC, NT>::kBytes);
  auto kernel = gemm_mfma_kernel<TA, TB, A_KC, B_KC, BM, BN, WAVES_M, WAVES_N, GUARDED, EXACT, EXTRA>;
  static std::atomic<bool> configured{false};  // per instantiation; racing threads set the same value
  if (!configured.load(std::memory_order_acquire)) {
    int rc = skl_check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, lds),
                           "gemm_mfma: LDS size");
    if (rc != 0) return rc;
    configured.store(true, std::memory_order_release);
  }
  MfmaArgs p = args;
  p.tiles_m = skl_div_up(p.m, BM);
  p.tiles_n = skl_div_up(p.n, BN);
  const size_t tiles = (size_t)p.tiles_m * p.tiles_n;
  const size_t slices = (p.k * ES + kSliceBytes - 1) / kSliceBytes;
  p.splits = splits_for(tiles, slices, p.m, p.n);
  p.slices_per_split = (unsigned)((slices + p.splits - 1) / p.splits);
  p.splits = (unsigned)((slices + p.slices_per_split - 1) / p.slices_per_split);  // no empty share
  SequenceGuard sequence(p.splits > 1);  // the partial sums travel from this kernel to the next through the workspace
  if (p.splits > 1) {
    p.partial = (char *)skl_workspace((size_t)p.splits * p.m * p.n * 4);
    if (!p.partial) return -4;
  }
  const size_t grid = tiles * p.splits;
  if (grid > 0x7FFFFFFFu) {
    skl_hip_record_error(-2, "gemm_mfma: grid too large");
    return -2;
  }
  kernel<<<(unsigned)grid, NT, lds, skl_current_stream()>>>(p);
  int rc = skl_check_launch("gemm_mfma");
  if (rc != 0 || p.splits == 1) return rc;
  using AccElem = decltype(typename Kind<TA>::Acc{}.x);
  const size_t blocks = (p.m * p.n + 255) / 256;
  if (blocks > 0x7FFFFFFFu) {
    skl_hip_record_error(-2, "gemm_mfma: grid too large");
    return -2;
  }
  gemm_split_reduce_kernel<AccElem><<<(unsigned)blocks, 256, 0, skl_current_stream()>>>(p);
  return skl_check_launch("gemm_split_reduce");
}

template <int TA, int TB, bool A_KC, bool B_KC>
int launch_tile(const MfmaArgs &p) {
  constexpr int ES = Kind<TA>::ES;
  constexpr size_t kRing128FromTiles = 96;
  constexpr bool kFp8 = TA == SKL_DT_F8E4M3 || TA == SKL_DT_F8E5M2;
  if constexpr (kFp8) {
    // short K: exact products (see MmaF8Exact), on the bounds-checked kernel whatever the shape
    if (p.k <= kF8ExactMaxK) {
      if (skl_div_up(p.m, 128) * (size_t)skl_div_up(p.n, 128) < 64)
        return launch_one<TA, TB, A_KC, B_KC, 64, 64, 2, 2, true, true>(p);
      return launch_one<TA, TB, A_KC, B_KC, 128, 128, 2, 4, true, true>(p);
    }
  }
  // The streaming kernel takes problems that its tiles divide evenly: 256 x 256 tiles when those
  // can fill the 256 compute units, 256 x 128 tiles for the sizes below that; everything else runs
  // on the small, bounds-checked kernel.
  // activation / requantised copy: on the streaming kernel only int8 with a copy that goes out as dwords
  using AccElem = decltype(typename Kind<TA>::Acc{}.x);
  const bool extra_steps = (p.rq.act || p.rq.q) && !(kRingCarriesExtraSteps<TA, TB> && FusedSteps<AccElem, 2>::dword_copy(p.rq));
  if (!extra_steps && p.m % 256 == 0 && (p.k * ES) % 128 == 0) {
    const size_t tiles_m = p.m / 256;
    if (p.n % 256 == 0 && tiles_m * (p.n / 256) >= 200) {
      // A last round that would fill at most half of the 256 compute units is run as 256 x 128 tiles
      // instead (a second launch on the trailing columns): twice the workgroups at half the length.
      const size_t tiles = tiles_m * (p.n / 256), rest = tiles % 256;
      if (rest != 0 && rest <= 128 && rest % tiles_m == 0) {
        const size_t tail_cols = rest / tiles_m * 256, head_cols = p.n - tail_cols;
        MfmaArgs head = p, tail = p;
        head.n = head_cols;
        tail.n = tail_cols;
        tail.b = p.b + (head_cols / 64) * p.b_s1 * ES;
        tail.c = p.c + (head_cols >> p.ccs) * p.csc1 * sizeof(float);  // whole blocks; C elements are 4 bytes for every kind
        if (p.bias) tail.bias = p.bias + head_cols * sizeof(float);
        if (p.rq.q) tail.rq.q = p.rq.q + head_cols * p.rq.csq;
        if (p.rq.q && p.rq.q_per_column) tail.rq.q_scale = p.rq.q_scale + head_cols;
        const int rc = launch_ring<TA, TB, A_KC, B_KC, 256>(head);
        return rc != 0 ? rc : launch_ring<TA, TB, A_KC, B_KC, 128>(tail);
      }
      return launch_ring<TA, TB, A_KC, B_KC, 256>(p);
    }
    // ... from 96 tiles on, or from 64 when K is long enough to be shared between two workgroups per tile
    const size_t tiles128 = p.n % 128 == 0 ? tiles_m * (p.n / 128) : 0, slices = p.k * ES / kRingSlice;
    if (tiles128 >= kRing128FromTiles || (tiles128 >= 64 && slices % 4 == 0 && slices / 2 >= kRingMinSlicesPerSplit))
      return launch_ring<TA, TB, A_KC, B_KC, 128>(p);
  }
  // Small problems: 64 x 64 tiles put four times as many workgroups on the chip.
  // ... and for the 16-bit kinds up to 64 rows of A: a 128-row tile would fetch and multiply rows that do not exist
  // (bf16 64 x 11008 x 4096: 36 -> 28 us; the 8-bit kinds are faster on the larger tile, 23 against 25 us).
  if ((ES == 2 && p.m <= 64) || skl_div_up(p.m, 128) * (size_t)skl_div_up(p.n, 128) < 64)
    return launch_one<TA, TB, A_KC, B_KC, 64, 64, 2, 2, true>(p);
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
inline bool operand_ok(const void *base, size_t es, size_t s1, size_t s0, size_t sk, size_t mn, size_t k) {
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

template <int TA, int TB>
int launch_padded(const MfmaArgs &p, size_t tile_cols) {
  return tile_cols == 256 ? launch_ring<TA, TB, true, true, 256, true>(p) : launch_ring<TA, TB, true, true, 128, true>(p);
}

}  // namespace

// One translation unit per operand kind defines these two (SKL_MFMA_DEFINE_KIND below); the dispatch calls them.
#define SKL_MFMA_DECLARE_KIND(NAME)                 \
  int skl_mfma_launch_##NAME(const MfmaArgs &p);    \
  int skl_mfma_launch_padded_##NAME(const MfmaArgs &p, size_t tile_cols);
#define SKL_MFMA_DEFINE_KIND(NAME, TA, TB)                                                                   \
  int skl_mfma_launch_##NAME(const MfmaArgs &p) { return launch_layout<TA, TB>(p); }                         \
  int skl_mfma_launch_padded_##NAME(const MfmaArgs &p, size_t tile_cols) { return launch_padded<TA, TB>(p, tile_cols); }
