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

// The same bytes read the way the persistent Q4_K GEMVs read them, and nothing else: workgroups of four or eight wavefronts, a
// wavefront takes items of `pair_bytes` contiguous bytes (a weight tile of the matrix-core kernel, a pair of rows of the
// dot-product kernel) team, team + n_teams, ..., every lane issues its 128-bit loads of the next item before it consumes the
// current one.  What this kernel reaches for a launch of N bytes is the ceiling for a GEMV launch over the same N bytes: same
// grid, same loads in flight, no arithmetic, no staging, no epilogue.
template <int PER_LANE>
__global__ __launch_bounds__(512) void stream_read_pairs_kernel(const uint8_t *src, int pairs, int pair_bytes, unsigned *sink) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, n16 = pair_bytes / 16, waves = blockDim.x >> 6;
    const int n_teams = gridDim.x * waves;
    unsigned acc = 0;
    uint4 cur[PER_LANE], nxt[PER_LANE];
    auto load = [&](int pair, uint4 (&buf)[PER_LANE]) {
        const uint4 *p = reinterpret_cast<const uint4 *>(src + (size_t)pair * pair_bytes);
#pragma unroll
        for (int k = 0; k < PER_LANE; k++) buf[k] = p[lane + 64 * k < n16 ? lane + 64 * k : n16 - 1];
    };
    int pair = blockIdx.x * waves + wave;
    if (pair < pairs) load(pair, cur);
    for (; pair < pairs; pair += n_teams) {
        if (pair + n_teams < pairs) load(pair + n_teams, nxt);
#pragma unroll
        for (int k = 0; k < PER_LANE; k++) acc += cur[k].x ^ cur[k].y ^ cur[k].z ^ cur[k].w;
#pragma unroll
        for (int k = 0; k < PER_LANE; k++) cur[k] = nxt[k];
    }
    if (acc == 0x12345678u) sink[0] = acc;   // keeps the loads alive; practically never true
}

}  // namespace

hipError_t launch_stream_read_pairs(const void *src, size_t bytes, int pair_bytes, int grid, int wavefronts, unsigned *sink, hipStream_t stream) {
    if (pair_bytes <= 0 || pair_bytes % 16 != 0 || bytes % pair_bytes != 0 || grid <= 0 || (wavefronts != 4 && wavefronts != 8)) return hipErrorInvalidValue;
    const int pairs = (int)(bytes / pair_bytes), per_lane = (pair_bytes / 16 + 63) / 64;
    const uint8_t *p = static_cast<const uint8_t *>(src);
    if (per_lane <= 5) hipLaunchKernelGGL(stream_read_pairs_kernel<5>, dim3(grid), dim3(64 * wavefronts), 0, stream, p, pairs, pair_bytes, sink);
    else if (per_lane <= 16) hipLaunchKernelGGL(stream_read_pairs_kernel<16>, dim3(grid), dim3(64 * wavefronts), 0, stream, p, pairs, pair_bytes, sink);
    else return hipErrorInvalidValue;
    return hipGetLastError();
}

hipError_t launch_stream_read(const void *src, size_t bytes, unsigned *sink, hipStream_t stream) {
    hipLaunchKernelGGL(stream_read_kernel, dim3(8192), dim3(256), 0, stream, static_cast<const uint4 *>(src), bytes / 16, sink);
    return hipGetLastError();
}

}  // namespace esp
