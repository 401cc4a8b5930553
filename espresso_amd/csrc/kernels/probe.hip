// A plain streaming read of a large buffer: the bandwidth a kernel that does nothing but 128-bit loads reaches
// on this machine.  Reported next to the GEMV figures so that "fraction of the published HBM peak" can be read
// against what the memory system delivers to the simplest possible reader.
#include "../common.h"

namespace esp {
namespace {

__global__ __launch_bounds__(256) void stream_read_kernel(const uint4 *src, size_t n, unsigned *sink) {
    unsigned acc = 0;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i + 3 * stride < n; i += 4 * stride) {
        const uint4 a = src[i], b = src[i + stride], c = src[i + 2 * stride], d = src[i + 3 * stride];
        acc += a.x ^ b.y ^ c.z ^ d.w;
    }
    for (; i < n; i += stride) acc += src[i].x;
    if (acc == 0x12345678u) sink[0] = acc;   // keeps the loads alive; practically never true
}

}  // namespace

hipError_t launch_stream_read(const void *src, size_t bytes, unsigned *sink, hipStream_t stream) {
    hipLaunchKernelGGL(stream_read_kernel, dim3(8192), dim3(256), 0, stream, static_cast<const uint4 *>(src), bytes / 16, sink);
    return hipGetLastError();
}

}  // namespace esp
