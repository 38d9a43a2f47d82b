/* A C caller of the library with ordinary malloc'ed buffers - the literal drop-in use: the calls an SKL
 * program makes, under SKL's own function names (skl-gfx950-compat.h maps them), plus this library's fused form. Checks int8 GEMM (strided, alpha / beta), the fused bias +
 * maximum epilogue, a 16-bit panel pack / unpack round trip and the saturating fp32 -> E4M3 conversion
 * against plain loops written from the definitions. Prints "dropin ok" and returns 0 on success. */
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "skl-gfx950-compat.h"

static uint64_t rng_state = 0x9E3779B97F4A7C15ull;
static uint32_t next_u32(void) {
  rng_state ^= rng_state << 13;
  rng_state ^= rng_state >> 7;
  rng_state ^= rng_state << 17;
  return (uint32_t)(rng_state >> 32);
}

static int check_error(const char *what) {
  if (skl_hip_last_error()) {
    fprintf(stderr, "%s: %s\n", what, skl_hip_last_error_string());
    return 1;
  }
  return 0;
}

int main(void) {
  enum { M = 70, N = 96, K = 130, LDA = 132, LDB = 100, LDC = 97 };
  int8_t *a = malloc(M * LDA), *b = malloc(K * LDB);
  int32_t *c = malloc(sizeof(int32_t) * M * LDC), *want = malloc(sizeof(int32_t) * M * LDC), bias[N], top = INT32_MIN;
  int bad = 0;
  if (skl_hip_init(0) != 0) {
    fprintf(stderr, "skl_hip_init: %s\n", skl_hip_last_error_string());
    return 2;
  }
  for (int i = 0; i < M * LDA; ++i) a[i] = (int8_t)next_u32();
  for (int i = 0; i < K * LDB; ++i) b[i] = (int8_t)next_u32();
  for (int i = 0; i < M * LDC; ++i) c[i] = want[i] = (int32_t)(next_u32() % 2001) - 1000;
  for (int j = 0; j < N; ++j) bias[j] = (int32_t)(next_u32() % 101) - 50;

  /* C = 3*A*B - 2*C, then + bias[j], running maximum */
  int32_t want_top = INT32_MIN;
  for (int i = 0; i < M; ++i)
    for (int j = 0; j < N; ++j) {
      int32_t acc = 0;
      for (int p = 0; p < K; ++p) acc += (int32_t)a[i * LDA + p] * (int32_t)b[p * LDB + j];
      want[i * LDC + j] = -2 * want[i * LDC + j] + 3 * acc + bias[j];
      if (want[i * LDC + j] > want_top) want_top = want[i * LDC + j];
    }
  skl_gfx950_epilogue_t ep = SKL_GFX950_EPILOGUE_NONE;
  ep.bias = bias;
  ep.max = &top;
  skl_gemm_fused_i8rc_i8rc_i32rc_gfx950(M, N, K, 3, a, LDA, 1, b, LDB, 1, -2, c, LDC, 1, &ep);
  bad |= check_error("fused int8 GEMM");
  if (memcmp(c, want, sizeof(int32_t) * M * LDC) != 0 || top != want_top) {
    fprintf(stderr, "int8 GEMM with fused epilogue differs (max %d, expected %d)\n", top, want_top);
    bad = 1;
  }

  /* the same product through SKL's row-major entry point: C = A*B */
  skl_gemm_i8_i8_i32_zve32x_x390(M, N, K, 1, a, LDA, b, LDB, 0, c, LDC);
  bad |= check_error("int8 GEMM");
  for (int i = 0; i < M && !bad; ++i)
    for (int j = 0; j < N; ++j) {
      int32_t acc = 0;
      for (int p = 0; p < K; ++p) acc += (int32_t)a[i * LDA + p] * (int32_t)b[p * LDB + j];
      if (c[i * LDC + j] != acc) {
        fprintf(stderr, "int8 GEMM differs at (%d, %d)\n", i, j);
        bad = 1;
        break;
      }
    }

  /* 16-bit panels: pack 70 x 96 into TE x 1 column panels and unpack again */
  {
    const size_t te = skl_get_ete_xsfmmbase(), m1 = (M + te - 1) / te;
    uint16_t *src = malloc(2 * M * N), *panels = malloc(2 * m1 * N * te), *back = calloc(M * N, 2);
    for (int i = 0; i < M * N; ++i) src[i] = (uint16_t)next_u32();
    skl_pack_e16_e16rcptex1c_xsfmmbase(M, N, src, N, panels, N * te, te, 0);
    for (int i = 0; i < M && !bad; ++i)
      for (int j = 0; j < N; ++j)
        if (panels[(i / te) * N * te + j * te + i % te] != src[i * N + j]) {
          fprintf(stderr, "panel pack differs at (%d, %d)\n", i, j);
          bad = 1;
          break;
        }
    skl_unpack_e16rcprc_e16rc_gfx950(te, 1, panels, 1, te, N * te, te, M, N, back, N, 1);
    bad |= check_error("pack / unpack");
    if (memcmp(back, src, 2 * M * N) != 0) {
      fprintf(stderr, "unpack(pack(x)) != x\n");
      bad = 1;
    }
    free(src), free(panels), free(back);
  }

  /* fp32 -> E4M3, saturating: known answers of the format (1.0 -> 0x38, 448 -> 0x7E, 1e6 -> 0x7E, -0.0 -> 0x80) */
  {
    const float x[4] = {1.0f, 448.0f, 1e6f, -0.0f};
    const uint8_t expect[4] = {0x38, 0x7E, 0x7E, 0x80};
    uint8_t q[4] = {0, 0, 0, 0};
    skl_cvt_sat_f32_f8e4m3_zvfofp8min(q, x, 1.0f, 4);
    bad |= check_error("cvt");
    if (memcmp(q, expect, 4) != 0) {
      fprintf(stderr, "cvt differs: %02x %02x %02x %02x\n", q[0], q[1], q[2], q[3]);
      bad = 1;
    }
  }
  free(a), free(b), free(c), free(want);
  skl_hip_shutdown();
  if (!bad) printf("dropin ok\n");
  return bad;
}
