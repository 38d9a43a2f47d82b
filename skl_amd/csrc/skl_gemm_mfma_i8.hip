// skl_gemm_mfma_i8.hip - the matrix-core GEMM kernels of one operand kind (skl_gemm_mfma_impl.hpp), compiled on their own.
#include "skl_gemm_mfma_impl.hpp"

SKL_MFMA_DEFINE_KIND(i8, SKL_DT_I8, SKL_DT_I8)
