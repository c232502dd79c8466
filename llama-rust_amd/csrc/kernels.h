// Host-callable launchers of the gfx950 kernels (kernels.hip).
#pragma once
#include <hip/hip_runtime.h>

#include "matview.h"

namespace nh {

// CU count and the largest dynamic LDS a workgroup may ask for on this device.
void set_device_limits(int cu_count, size_t lds_per_block);

// Scatter the GGUF bytes at src_device (device memory) into the planes of m.
hipError_t launch_repack(hipStream_t stream, const MatView &m, const void *src_device);

// y[t, r] = sum_c W[r, c] x[t, c]; x and y are device pointers, token-major.
hipError_t launch_gemm(hipStream_t stream, const MatView &m, uint32_t tokens, const float *x, float *y);

}  // namespace nh
