// placeholder until the streaming kernels land
#include "skl_device.hpp"
extern "C" int skl_hip_gemv_supported(const skl_gemm_canon *, int) { return 0; }
extern "C" int skl_hip_launch_gemv(const skl_gemm_canon *, int) { return -2; }
