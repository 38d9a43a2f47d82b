// skl_device.hpp - helpers shared by the HIP translation units (not installed).
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "skl_launch.h"

// Stream the calling thread launches on (set through skl_hip_set_stream).
hipStream_t skl_current_stream();

// Per-device scratch used by split reductions. Grows on demand; contents are
// only meaningful inside one launch sequence on one stream.
void *skl_workspace(size_t bytes);

// Records a HIP failure for skl_hip_last_error() and returns its code.
int skl_check_hip(hipError_t e, const char *what);

// Checks the launch that was just enqueued.
static inline int skl_check_launch(const char *what) { return skl_check_hip(hipGetLastError(), what); }

static inline unsigned skl_div_up(size_t a, size_t b) { return (unsigned)((a + b - 1) / b); }
