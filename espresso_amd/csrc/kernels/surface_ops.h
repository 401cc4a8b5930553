#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace esp {
hipError_t launch_gather_columns(const uint16_t *surface, int channels, int spatial, int lanes, uint16_t *out16, float *out32, hipStream_t s);
hipError_t launch_scatter_columns(const float *in, int channels, int spatial, int lanes, uint16_t *surface, hipStream_t s);
hipError_t launch_row_max(const float *in, int channels, int spatial, int lanes, uint16_t *surface, hipStream_t s);
}  // namespace esp
