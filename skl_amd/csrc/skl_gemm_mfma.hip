// placeholder until the matrix-core kernels land
#include "skl_device.hpp"
extern "C" int skl_hip_gemm_mfma_supported(const skl_gemm_canon *) { return 0; }
extern "C" int skl_hip_launch_gemm_mfma(const skl_gemm_canon *) { return -2; }
