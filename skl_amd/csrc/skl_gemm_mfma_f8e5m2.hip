// skl_gemm_mfma_f8e5m2.hip - the matrix-core GEMM kernels of one operand kind (skl_gemm_mfma_impl.hpp), compiled on their own.
#include "skl_gemm_mfma_impl.hpp"

SKL_MFMA_DEFINE_KIND(f8e5m2, SKL_DT_F8E5M2, SKL_DT_F8E5M2)
