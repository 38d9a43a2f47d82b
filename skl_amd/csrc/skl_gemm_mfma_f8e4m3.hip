// skl_gemm_mfma_f8e4m3.hip - the matrix-core GEMM kernels of one operand kind (skl_gemm_mfma_impl.hpp), compiled on their own.
#include "skl_gemm_mfma_impl.hpp"

SKL_MFMA_DEFINE_KIND(f8e4m3, SKL_DT_F8E4M3, SKL_DT_F8E4M3)
