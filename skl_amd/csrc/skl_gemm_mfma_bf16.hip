// skl_gemm_mfma_bf16.hip - the matrix-core GEMM kernels of one operand kind (skl_gemm_mfma_impl.hpp), compiled on their own.
#include "skl_gemm_mfma_impl.hpp"

SKL_MFMA_DEFINE_KIND(bf16, SKL_DT_BF16, SKL_DT_BF16)
