/*
 * skl-gfx950-compat.h - the names of SKL's own entry points mapped onto the gfx950 library.
 *
 * A C caller of SKL's optimized kernels (the ISA-suffixed functions of src/gemm, src/pack, src/transpose, src/cvt)
 * or of its scalar routines (the `_ref` functions of ref/) includes this header instead of SKL's, links
 * libskl_gfx950 and is otherwise unchanged: every target has the argument list of the prototype cited beside it.
 * Pointers may be ordinary host memory (the library stages them) or device memory from skl_hip_malloc().
 */
#ifndef SKL_GFX950_COMPAT_H
#define SKL_GFX950_COMPAT_H

#include "skl-gfx950.h"

/* test/gemm/skl_test_gemm.h:27-31: the tile edge the panel layouts are built on */
#define skl_get_ete_xsfmmbase() skl_hip_te()

#define skl_gemm_bf16_bf16_f32_zvfbfwma                                 skl_gemm_bf16_bf16_f32_gfx950 /* src/gemm/gemm_bf16_bf16_f32_zvfbfwma.h:49 */
#define skl_gemm_bf16_bf16_f32_zvfbfwma_x390                            skl_gemm_bf16_bf16_f32_gfx950 /* src/gemm/gemm_bf16_bf16_f32_zvfbfwma_x390.h:49 */
#define skl_gemm_bf16c_bf16_f32_xsfmm32a16f                             skl_gemm_bf16c_bf16_f32_gfx950 /* src/gemm/gemm_bf16c_bf16_f32_xsfmm32a16f.h:56 */
#define skl_gemm_bf16rcptex1c_bf16rcp1xte_f32rcptexterc_xsfmm32a16f     skl_gemm_bf16rcptex1c_bf16rcp1xte_f32rcptexterc_gfx950 /* src/gemm/gemm_bf16c_bf16_f32_xsfmm32a16f.h:97 */
#define skl_gemm_f16_f16_f16_zvfh                                       skl_gemm_f16_f16_f16_gfx950 /* src/gemm/gemm_f16_f16_f16_zvfh.h:48 */
#define skl_gemm_f16_f16_f16_zvfh_x390                                  skl_gemm_f16_f16_f16_gfx950 /* src/gemm/gemm_f16_f16_f16_zvfh_x390.h:48 */
#define skl_gemm_f16_f16_f32_zvfh                                       skl_gemm_f16_f16_f32_gfx950 /* src/gemm/gemm_f16_f16_f32_zvfh.h:49 */
#define skl_gemm_f16_f16_f32_zvfh_x390                                  skl_gemm_f16_f16_f32_gfx950 /* src/gemm/gemm_f16_f16_f32_zvfh_x390.h:49 */
#define skl_gemm_f16c_f16_f32_xsfmm32a16f                               skl_gemm_f16c_f16_f32_gfx950 /* src/gemm/gemm_f16c_f16_f32_xsfmm32a16f.h:56 */
#define skl_gemm_f16rcptex1c_f16rcp1xte_f32rcptexterc_xsfmm32a16f       skl_gemm_f16rcptex1c_f16rcp1xte_f32rcptexterc_gfx950 /* src/gemm/gemm_f16c_f16_f32_xsfmm32a16f.h:97 */
#define skl_gemm_f32_f32_f32_zve32f                                     skl_gemm_f32_f32_f32_gfx950 /* src/gemm/gemm_f32_f32_f32_zve32f.h:48 */
#define skl_gemm_f32_f32_f32_zve32f_x390                                skl_gemm_f32_f32_f32_gfx950 /* src/gemm/gemm_f32_f32_f32_zve32f_x390.h:48 */
#define skl_gemm_f32c_f32_f32_xsfmm32a32f                               skl_gemm_f32c_f32_f32_gfx950 /* src/gemm/gemm_f32c_f32_f32_xsfmm32a32f.h:56 */
#define skl_gemm_f32rcptex1c_f32rcp1xte_f32rcptexterc_xsfmm32a32f       skl_gemm_f32rcptex1c_f32rcp1xte_f32rcptexterc_gfx950 /* src/gemm/gemm_f32c_f32_f32_xsfmm32a32f.h:96 */
#define skl_gemm_f64_f64_f64_zve64d                                     skl_gemm_f64_f64_f64_gfx950 /* src/gemm/gemm_f64_f64_f64_zve64d.h:48 */
#define skl_gemm_f64_f64_f64_zve64d_x390                                skl_gemm_f64_f64_f64_gfx950 /* src/gemm/gemm_f64_f64_f64_zve64d_x390.h:48 */
#define skl_gemm_f8e4m3c_f8e4m3_f32_xsfmm32a8f                          skl_gemm_f8e4m3c_f8e4m3_f32_gfx950 /* src/gemm/gemm_f8e4m3c_f8e4m3_f32_xsfmm32a8f.h:57 */
#define skl_gemm_f8e4m3rcptex1c_f8e4m3rcp1xte_f32rcptexterc_xsfmm32a8f  skl_gemm_f8e4m3rcptex1c_f8e4m3rcp1xte_f32rcptexterc_gfx950 /* src/gemm/gemm_f8e4m3c_f8e4m3_f32_xsfmm32a8f.h:98 */
#define skl_gemm_f8e5m2c_f8e5m2_f32_xsfmm32a8f                          skl_gemm_f8e5m2c_f8e5m2_f32_gfx950 /* src/gemm/gemm_f8e5m2c_f8e5m2_f32_xsfmm32a8f.h:57 */
#define skl_gemm_f8e5m2rcptex1c_f8e5m2rcp1xte_f32rcptexterc_xsfmm32a8f  skl_gemm_f8e5m2rcptex1c_f8e5m2rcp1xte_f32rcptexterc_gfx950 /* src/gemm/gemm_f8e5m2c_f8e5m2_f32_xsfmm32a8f.h:98 */
#define skl_gemm_i8_i8_i32_zve32x                                       skl_gemm_i8_i8_i32_gfx950 /* src/gemm/gemm_i8_i8_i32_zve32x.h:50 */
#define skl_gemm_i8_i8_i32_zve32x_x390                                  skl_gemm_i8_i8_i32_gfx950 /* src/gemm/gemm_i8_i8_i32_zve32x_x390.h:50 */
#define skl_gemm_i8c_i8_i32_xsfmm32a8i                                  skl_gemm_i8c_i8_i32_gfx950 /* src/gemm/gemm_i8c_i8_i32_xsfmm32a8i.h:57 */
#define skl_gemm_i8rcptex1c_i8rcp1xte_i32rcptexterc_xsfmm32a8i          skl_gemm_i8rcptex1c_i8rcp1xte_i32rcptexterc_gfx950 /* src/gemm/gemm_i8c_i8_i32_xsfmm32a8i.h:97 */
#define skl_gemm_i8rcp1x4_i8p4x1c_i32_xsfvqdotq                         skl_gemm_i8rcp1x4_i8p4x1c_i32_gfx950 /* src/gemm/gemm_i8rcp1x4_i8p4x1c_i32_xsfvqdotq.h:70 */
#define skl_pack_e16_e16rcptex1c_xsfmmbase                              skl_pack_e16_e16rcptex1c_gfx950 /* src/pack/pack_e16_xsfmmbase.h:49 */
#define skl_transpose_e16_xsfmmbase                                     skl_transpose_e16_gfx950 /* src/pack/pack_e16_xsfmmbase.h:70 */
#define skl_pack_e16rc_e16rcprc_zve32x                                  skl_pack_e16rc_e16rcprc_gfx950 /* src/pack/pack_e16_zve32x.h:49 */
#define skl_transpose_e16_zve32x                                        skl_transpose_e16_gfx950 /* src/pack/pack_e16_zve32x.h:73 */
#define skl_pack_e32_e32rcptex1c_xsfmmbase                              skl_pack_e32_e32rcptex1c_gfx950 /* src/pack/pack_e32_xsfmmbase.h:49 */
#define skl_transpose_e32_xsfmmbase                                     skl_transpose_e32_gfx950 /* src/pack/pack_e32_xsfmmbase.h:70 */
#define skl_pack_e32rc_e32rcprc_zve32x                                  skl_pack_e32rc_e32rcprc_gfx950 /* src/pack/pack_e32_zve32x.h:49 */
#define skl_transpose_e32_zve32x                                        skl_transpose_e32_gfx950 /* src/pack/pack_e32_zve32x.h:73 */
#define skl_transpose_e8_xsfmmbase                                      skl_transpose_e8_gfx950 /* src/pack/pack_e8_xsfmmbase.h:38 */
#define skl_pack_e8rc_e8rcprc_zve32x                                    skl_pack_e8rc_e8rcprc_gfx950 /* src/pack/pack_e8_zve32x.h:49 */
#define skl_unpack_e8rcprc_e8rc_zve32x                                  skl_unpack_e8rcprc_e8rc_gfx950 /* src/pack/pack_e8_zve32x.h:88 */
#define skl_transpose_e8_zve32x                                         skl_transpose_e8_gfx950 /* src/pack/pack_e8_zve32x.h:112 */
#define skl_cvt_bf16_f8e4m3_zvfofp8min_zvfbfmin                         skl_cvt_bf16_f8e4m3_gfx950 /* src/cvt/cvt_bf16_f8_zvfofp8min_zvfbfmin.h:67 */
#define skl_cvt_sat_bf16_f8e4m3_zvfofp8min_zvfbfmin                     skl_cvt_sat_bf16_f8e4m3_gfx950 /* src/cvt/cvt_bf16_f8_zvfofp8min_zvfbfmin.h:84 */
#define skl_cvt_bf16_f8e5m2_zvfofp8min_zvfbfmin                         skl_cvt_bf16_f8e5m2_gfx950 /* src/cvt/cvt_bf16_f8_zvfofp8min_zvfbfmin.h:102 */
#define skl_cvt_sat_bf16_f8e5m2_zvfofp8min_zvfbfmin                     skl_cvt_sat_bf16_f8e5m2_gfx950 /* src/cvt/cvt_bf16_f8_zvfofp8min_zvfbfmin.h:119 */
#define skl_cvt_f32_f8e4m3_zvfofp8min                                   skl_cvt_f32_f8e4m3_gfx950 /* src/cvt/cvt_f32_f8_zvfofp8min.h:61 */
#define skl_cvt_sat_f32_f8e4m3_zvfofp8min                               skl_cvt_sat_f32_f8e4m3_gfx950 /* src/cvt/cvt_f32_f8_zvfofp8min.h:78 */
#define skl_cvt_f32_f8e5m2_zvfofp8min                                   skl_cvt_f32_f8e5m2_gfx950 /* src/cvt/cvt_f32_f8_zvfofp8min.h:94 */
#define skl_cvt_sat_f32_f8e5m2_zvfofp8min                               skl_cvt_sat_f32_f8e5m2_gfx950 /* src/cvt/cvt_f32_f8_zvfofp8min.h:111 */
#define skl_cvt_f4e2m1_f8e4m3_zvfofp4min                                skl_cvt_f4e2m1_f8e4m3_gfx950 /* src/cvt/cvt_f4_f8_zvfofp4min.h:54 */
#define skl_cvt_f8e4m3_bf16_zvfofp8min                                  skl_cvt_f8e4m3_bf16_gfx950 /* src/cvt/cvt_f8_bf16_zvfofp8min.h:39 */
#define skl_cvt_f8e5m2_bf16_zvfofp8min                                  skl_cvt_f8e5m2_bf16_gfx950 /* src/cvt/cvt_f8_bf16_zvfofp8min.h:52 */
#define skl_gemm_bf16rc_bf16rc_f32rc_ref                                skl_gemm_bf16rc_bf16rc_f32rc_gfx950 /* ref/gemm/gemm_bf16rc_bf16rc_f32rc.h:44 */
#define skl_gemm_bf16rcprc_bf16rcprc_f32rcprc_ref                       skl_gemm_bf16rcprc_bf16rcprc_f32rcprc_gfx950 /* ref/gemm/gemm_bf16rcprc_bf16rcprc_f32rcprc.h:49 */
#define skl_gemm_f16rc_f16rc_f16rc_ref                                  skl_gemm_f16rc_f16rc_f16rc_gfx950 /* ref/gemm/gemm_f16rc_f16rc_f16rc.h:44 */
#define skl_gemm_f16rc_f16rc_f32rc_ref                                  skl_gemm_f16rc_f16rc_f32rc_gfx950 /* ref/gemm/gemm_f16rc_f16rc_f32rc.h:44 */
#define skl_gemm_f16rcprc_f16rcprc_f16rcprc_ref                         skl_gemm_f16rcprc_f16rcprc_f16rcprc_gfx950 /* ref/gemm/gemm_f16rcprc_f16rcprc_f16rcprc.h:49 */
#define skl_gemm_f16rcprc_f16rcprc_f32rcprc_ref                         skl_gemm_f16rcprc_f16rcprc_f32rcprc_gfx950 /* ref/gemm/gemm_f16rcprc_f16rcprc_f32rcprc.h:49 */
#define skl_gemm_f32rc_f32rc_f32rc_ref                                  skl_gemm_f32rc_f32rc_f32rc_gfx950 /* ref/gemm/gemm_f32rc_f32rc_f32rc.h:44 */
#define skl_gemm_f32rcprc_f32rcprc_f32rcprc_ref                         skl_gemm_f32rcprc_f32rcprc_f32rcprc_gfx950 /* ref/gemm/gemm_f32rcprc_f32rcprc_f32rcprc.h:49 */
#define skl_gemm_f64rc_f64rc_f64rc_ref                                  skl_gemm_f64rc_f64rc_f64rc_gfx950 /* ref/gemm/gemm_f64rc_f64rc_f64rc.h:44 */
#define skl_gemm_f64rcprc_f64rcprc_f64rcprc_ref                         skl_gemm_f64rcprc_f64rcprc_f64rcprc_gfx950 /* ref/gemm/gemm_f64rcprc_f64rcprc_f64rcprc.h:49 */
#define skl_gemm_f8e4m3rc_f8e4m3rc_f32rc_ref                            skl_gemm_f8e4m3rc_f8e4m3rc_f32rc_gfx950 /* ref/gemm/gemm_f8e4m3rc_f8e4m3rc_f32rc.h:48 */
#define skl_gemm_f8e4m3rcprc_f8e4m3rcprc_f32rcprc_ref                   skl_gemm_f8e4m3rcprc_f8e4m3rcprc_f32rcprc_gfx950 /* ref/gemm/gemm_f8e4m3rcprc_f8e4m3rcprc_f32rcprc.h:53 */
#define skl_gemm_f8e5m2rc_f8e5m2rc_f32rc_ref                            skl_gemm_f8e5m2rc_f8e5m2rc_f32rc_gfx950 /* ref/gemm/gemm_f8e5m2rc_f8e5m2rc_f32rc.h:48 */
#define skl_gemm_f8e5m2rcprc_f8e5m2rcprc_f32rcprc_ref                   skl_gemm_f8e5m2rcprc_f8e5m2rcprc_f32rcprc_gfx950 /* ref/gemm/gemm_f8e5m2rcprc_f8e5m2rcprc_f32rcprc.h:53 */
#define skl_gemm_i8rc_i8rc_i32rc_ref                                    skl_gemm_i8rc_i8rc_i32rc_gfx950 /* ref/gemm/gemm_i8rc_i8rc_i32rc.h:45 */
#define skl_gemm_i8rcprc_i8rcprc_i32rcprc_ref                           skl_gemm_i8rcprc_i8rcprc_i32rcprc_gfx950 /* ref/gemm/gemm_i8rcprc_i8rcprc_i32rcprc.h:50 */
#define skl_pack_e16rc_e16rcprc_ref                                     skl_pack_e16rc_e16rcprc_gfx950 /* ref/pack/pack_e16rc_e16rcprc.h:44 */
#define skl_pack_e32rc_e32rcprc_ref                                     skl_pack_e32rc_e32rcprc_gfx950 /* ref/pack/pack_e32rc_e32rcprc.h:44 */
#define skl_pack_e8rc_e8rcprc_ref                                       skl_pack_e8rc_e8rcprc_gfx950 /* ref/pack/pack_e8rc_e8rcprc.h:44 */
#define skl_transpose_e16_ref                                           skl_transpose_e16_gfx950 /* ref/pack/transpose_e16.h:33 */
#define skl_transpose_e32_ref                                           skl_transpose_e32_gfx950 /* ref/pack/transpose_e32.h:33 */
#define skl_transpose_e8_ref                                            skl_transpose_e8_gfx950 /* ref/pack/transpose_e8.h:33 */
#define skl_unpack_e8rcprc_e8rc_ref                                     skl_unpack_e8rcprc_e8rc_gfx950 /* ref/pack/unpack_e8rcprc_e8rc.h:48 */
#define skl_cvt_f4e2m1_f8e4m3_ref                                       skl_cvt_f4e2m1_f8e4m3_gfx950 /* ref/cvt/cvt_ofp4.h:30 */
#define skl_cvt_f32_f8e4m3_ref                                          skl_cvt_f32_f8e4m3_gfx950 /* ref/cvt/cvt_ofp8.h:59 */
#define skl_cvt_sat_f32_f8e4m3_ref                                      skl_cvt_sat_f32_f8e4m3_gfx950 /* ref/cvt/cvt_ofp8.h:71 */
#define skl_cvt_f32_f8e5m2_ref                                          skl_cvt_f32_f8e5m2_gfx950 /* ref/cvt/cvt_ofp8.h:83 */
#define skl_cvt_sat_f32_f8e5m2_ref                                      skl_cvt_sat_f32_f8e5m2_gfx950 /* ref/cvt/cvt_ofp8.h:95 */
#define skl_cvt_bf16_f8e4m3_ref                                         skl_cvt_bf16_f8e4m3_gfx950 /* ref/cvt/cvt_ofp8.h:106 */
#define skl_cvt_sat_bf16_f8e4m3_ref                                     skl_cvt_sat_bf16_f8e4m3_gfx950 /* ref/cvt/cvt_ofp8.h:118 */
#define skl_cvt_bf16_f8e5m2_ref                                         skl_cvt_bf16_f8e5m2_gfx950 /* ref/cvt/cvt_ofp8.h:129 */
#define skl_cvt_sat_bf16_f8e5m2_ref                                     skl_cvt_sat_bf16_f8e5m2_gfx950 /* ref/cvt/cvt_ofp8.h:141 */
#define skl_cvt_f8e4m3_bf16_ref                                         skl_cvt_f8e4m3_bf16_gfx950 /* ref/cvt/cvt_ofp8.h:150 */
#define skl_cvt_f8e5m2_bf16_ref                                         skl_cvt_f8e5m2_bf16_gfx950 /* ref/cvt/cvt_ofp8.h:158 */

#endif /* SKL_GFX950_COMPAT_H */
