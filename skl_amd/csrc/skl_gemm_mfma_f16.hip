// skl_gemm_mfma_f16.hip - the matrix-core GEMM kernels of one operand kind (skl_gemm_mfma_impl.hpp), compiled on their own.
#include "skl_gemm_mfma_impl.hpp"

SKL_MFMA_DEFINE_KIND(f16, SKL_DT_F16, SKL_DT_F16)
