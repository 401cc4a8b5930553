// Moves decode tokens between channel-first fp16 surfaces [channels, spatial] and the contiguous
// per-token vectors the GEMV kernels take.  A token occupies one spatial column
// (Sources/Espresso/DecodeForwardPass.swift:1563-1575).
#include "../common.h"
#include "surface_ops.h"

namespace esp {
namespace {

__device__ __forceinline__ float h2f(uint16_t b) { return (float)__builtin_bit_cast(_Float16, b); }
__device__ __forceinline__ uint16_t f2h(float v) { return __builtin_bit_cast(uint16_t, (_Float16)v); }

// out16[l][c] / out32[l][c] = surface[c * spatial + l] for l < lanes
__global__ void gather_columns_kernel(const uint16_t *surface, int channels, int spatial, int lanes, uint16_t *out16, float *out32) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x, l = blockIdx.y;
    if (c >= channels || l >= lanes) return;
    const uint16_t v = surface[(size_t)c * spatial + l];
    if (out16) out16[(size_t)l * channels + c] = v;
    if (out32) out32[(size_t)l * channels + c] = h2f(v);
}

// surface[c * spatial + l] = fp16(in[l][c])
__global__ void scatter_columns_kernel(const float *in, int channels, int spatial, int lanes, uint16_t *surface) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x, l = blockIdx.y;
    if (c >= channels || l >= lanes) return;
    surface[(size_t)c * spatial + l] = f2h(in[(size_t)l * channels + c]);
}

// surface[l] = fp16(max_c in[l][c]) — the reduce_max output of the classifier kernel
__global__ __launch_bounds__(256) void row_max_kernel(const float *in, int channels, int spatial, uint16_t *surface) {
    __shared__ float red[256];
    const int l = blockIdx.x;
    float m = -INFINITY;
    for (int c = threadIdx.x; c < channels; c += 256) m = fmaxf(m, in[(size_t)l * channels + c]);
    red[threadIdx.x] = m;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) {
        if (threadIdx.x < s) red[threadIdx.x] = fmaxf(red[threadIdx.x], red[threadIdx.x + s]);
        __syncthreads();
    }
    if (threadIdx.x == 0) surface[l] = f2h(red[0]);
    (void)spatial;
}

}  // namespace

hipError_t launch_gather_columns(const uint16_t *surface, int channels, int spatial, int lanes, uint16_t *out16, float *out32, hipStream_t s) {
    hipLaunchKernelGGL(gather_columns_kernel, dim3((channels + 255) / 256, lanes), dim3(256), 0, s, surface, channels, spatial, lanes, out16, out32);
    return hipGetLastError();
}
hipError_t launch_scatter_columns(const float *in, int channels, int spatial, int lanes, uint16_t *surface, hipStream_t s) {
    hipLaunchKernelGGL(scatter_columns_kernel, dim3((channels + 255) / 256, lanes), dim3(256), 0, s, in, channels, spatial, lanes, surface);
    return hipGetLastError();
}
hipError_t launch_row_max(const float *in, int channels, int spatial, int lanes, uint16_t *surface, hipStream_t s) {
    hipLaunchKernelGGL(row_max_kernel, dim3(lanes), dim3(256), 0, s, in, channels, spatial, surface);
    return hipGetLastError();
}

}  // namespace esp
