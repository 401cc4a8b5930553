// GGUF block dequantisation to fp32 and the upload-time re-layout of Q8_0 / Q4_0 into planes.
//
// Stands in for the absent Edgerunner package's DequantDispatcher.dequantize(tensor:device:)
// (call sites: Sources/EspressoGGUF/GGUFModelLoader.swift:359-372).  Results are bit-exact to the
// public ggml block definitions: every product is rounded to fp32 before the next operation
// (__fmul_rn / __fsub_rn are never contracted into a fused multiply-add).
#include "../common.h"

namespace esp {
namespace {

__device__ __forceinline__ float half_at(const uint8_t *p) {
    uint16_t bits = (uint16_t)(p[0] | (p[1] << 8));
    return (float)__builtin_bit_cast(_Float16, bits);
}

// one thread per element, blocks addressed in the GGUF byte layout
__global__ void dequant_q8_0_kernel(const uint8_t *blocks, size_t elems, float *out) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= elems) return;
    const uint8_t *blk = blocks + (i >> 5) * 34;
    float d = half_at(blk);
    int q = (int8_t)blk[2 + (i & 31)];
    out[i] = __fmul_rn((float)q, d);
}

__global__ void dequant_q4_0_kernel(const uint8_t *blocks, size_t elems, float *out) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= elems) return;
    const uint8_t *blk = blocks + (i >> 5) * 18;
    float d = half_at(blk);
    int j = (int)(i & 31);
    uint8_t byte = blk[2 + (j & 15)];
    int n = j < 16 ? (byte & 0x0F) : (byte >> 4);
    out[i] = __fmul_rn((float)(n - 8), d);
}

__device__ __forceinline__ void q4k_scale_min(int j, const uint8_t *s, int &sc, int &m) {
    if (j < 4) {
        sc = s[j] & 63;
        m = s[j + 4] & 63;
    } else {
        sc = (s[j + 4] & 0x0F) | ((s[j - 4] >> 6) << 4);
        m = (s[j + 4] >> 4) | ((s[j] >> 6) << 4);
    }
}

__global__ void dequant_q4_k_kernel(const uint8_t *blocks, size_t elems, float *out) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= elems) return;
    const uint8_t *blk = blocks + (i >> 8) * 144;
    int e = (int)(i & 255);
    int sub = e >> 5, l = e & 31, chunk = sub >> 1;
    float d = half_at(blk), dmin = half_at(blk + 2);
    int sc, m;
    q4k_scale_min(sub, blk + 4, sc, m);
    uint8_t byte = blk[16 + chunk * 32 + l];
    int n = (sub & 1) ? (byte >> 4) : (byte & 0x0F);
    float d1 = __fmul_rn(d, (float)sc);
    float m1 = __fmul_rn(dmin, (float)m);
    out[i] = __fsub_rn(__fmul_rn(d1, (float)n), m1);
}

__global__ void dequant_f16_kernel(const uint8_t *blocks, size_t elems, float *out) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= elems) return;
    out[i] = half_at(blocks + 2 * i);
}

__global__ void copy_f32_kernel(const uint8_t *blocks, size_t elems, float *out) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= elems) return;
    out[i] = reinterpret_cast<const float *>(blocks)[i];
}

// GGUF 34-byte Q8_0 / 18-byte Q4_0 blocks -> (quant plane, scale plane).  One thread per block.
__global__ void repack_q8_0_kernel(const uint8_t *blocks, size_t nblocks, uint8_t *qs, uint16_t *scales) {
    size_t b = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblocks) return;
    const uint8_t *blk = blocks + b * 34;
    scales[b] = (uint16_t)(blk[0] | (blk[1] << 8));
    for (int j = 0; j < 32; j++) qs[b * 32 + j] = blk[2 + j];
}

__global__ void repack_q4_0_kernel(const uint8_t *blocks, size_t nblocks, uint8_t *qs, uint16_t *scales) {
    size_t b = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblocks) return;
    const uint8_t *blk = blocks + b * 18;
    scales[b] = (uint16_t)(blk[0] | (blk[1] << 8));
    for (int j = 0; j < 16; j++) qs[b * 16 + j] = blk[2 + j];
}

// plane layouts -> fp32, same arithmetic as the block kernels
__global__ void dequant_planes_q8_0_kernel(const uint8_t *qs, const uint16_t *scales, size_t elems, float *out) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= elems) return;
    float d = (float)__builtin_bit_cast(_Float16, scales[i >> 5]);
    out[i] = __fmul_rn((float)(int8_t)qs[i], d);
}

__global__ void dequant_planes_q4_0_kernel(const uint8_t *qs, const uint16_t *scales, size_t elems, float *out) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= elems) return;
    float d = (float)__builtin_bit_cast(_Float16, scales[i >> 5]);
    int j = (int)(i & 31);
    uint8_t byte = qs[(i >> 5) * 16 + (j & 15)];
    int n = j < 16 ? (byte & 0x0F) : (byte >> 4);
    out[i] = __fmul_rn((float)(n - 8), d);
}

// One thread per 16-byte piece of the tiled copy: tile (rb, sb) = sixteen headers, then piece (g, n) first halves, then
// second halves (see the matrix-core GEMV).  Rows past the matrix are zero blocks.
__global__ void q4k_tile_kernel(const uint8_t *blocks, int rows, int nsb, size_t pieces, uint8_t *tiled) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= pieces) return;
    const size_t tile = i / 144;
    const int p = (int)(i - tile * 144);
    const int rb = (int)(tile / nsb), sb = (int)(tile - (size_t)rb * nsb);
    int n, src;           // row inside the block, byte offset inside the 144-byte super-block
    if (p < 16) { n = p; src = 0; }
    else {
        const int q = p - 16, half = q >> 6, gn = q & 63;   // piece (g, n) of half `half`
        n = gn & 15;
        src = 16 + 32 * (gn >> 4) + 16 * half;
    }
    const int row = rb * 16 + n;
    uint4 v = make_uint4(0, 0, 0, 0);
    if (row < rows) v = *reinterpret_cast<const uint4 *>(blocks + ((size_t)row * nsb + sb) * 144 + src);
    *reinterpret_cast<uint4 *>(tiled + i * 16) = v;
}

// Q4_0 planes -> the tiled copy of the matrix-core GEMV: tile (rb, t) = sixteen rows x 512 columns = [j][lane] 16 bytes of nibbles
// (lane (n, g) = g * 16 + n owns block 16 t + 4 j + g of row n), then [lane][j] fp16 scales.  320 threads per tile; rows past the
// matrix are zero blocks with zero scales.
__global__ void q40_tile_kernel(const uint8_t *qs, const uint16_t *scales, int rows, int tpr, size_t tiles, uint8_t *tiled) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t tile = i / 320;
    if (tile >= tiles) return;
    const int p = (int)(i - tile * 320);
    const int rb = (int)(tile / tpr), t = (int)(tile - (size_t)rb * tpr);
    uint8_t *dst = tiled + tile * 4608;
    const int blocks_per_row = tpr * 16;
    if (p < 256) {
        const int j = p >> 6, lane = p & 63, g = lane >> 4, n = lane & 15, row = rb * 16 + n;
        uint4 v = make_uint4(0, 0, 0, 0);
        if (row < rows) v = *reinterpret_cast<const uint4 *>(qs + ((size_t)row * blocks_per_row + 16 * t + 4 * j + g) * 16);
        *reinterpret_cast<uint4 *>(dst + 1024 * j + 16 * lane) = v;
    } else {
        const int lane = p - 256, g = lane >> 4, n = lane & 15, row = rb * 16 + n;
        uint16_t d[4] = {0, 0, 0, 0};
        if (row < rows)
            for (int j = 0; j < 4; j++) d[j] = scales[(size_t)row * blocks_per_row + 16 * t + 4 * j + g];
        *reinterpret_cast<uint2 *>(dst + 4096 + 8 * lane) = make_uint2(d[0] | ((unsigned)d[1] << 16), d[2] | ((unsigned)d[3] << 16));
    }
}

// Q8_0 planes -> the tiled copy of the matrix-core GEMV: tile (rb, t) = sixteen rows x 256 columns = [j][half][lane] 16 bytes of
// quants (lane (n, g) = g * 16 + n owns block 8 t + 4 j + g of row n; half = its first or last sixteen bytes), then [lane][j] fp16
// scales.  320 threads per tile; rows past the matrix are zero blocks with zero scales.
__global__ void q80_tile_kernel(const uint8_t *qs, const uint16_t *scales, int rows, int tpr, size_t tiles, uint8_t *tiled) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t tile = i / 320;
    if (tile >= tiles) return;
    const int p = (int)(i - tile * 320);
    const int rb = (int)(tile / tpr), t = (int)(tile - (size_t)rb * tpr);
    uint8_t *dst = tiled + tile * 4352;
    const int blocks_per_row = tpr * 8;
    if (p < 256) {
        const int j = p >> 7, half = (p >> 6) & 1, lane = p & 63, g = lane >> 4, n = lane & 15, row = rb * 16 + n;
        uint4 v = make_uint4(0, 0, 0, 0);
        if (row < rows) v = *reinterpret_cast<const uint4 *>(qs + ((size_t)row * blocks_per_row + 8 * t + 4 * j + g) * 32 + 16 * half);
        *reinterpret_cast<uint4 *>(dst + 1024 * (2 * j + half) + 16 * lane) = v;
    } else {
        const int lane = p - 256, g = lane >> 4, n = lane & 15, row = rb * 16 + n;
        unsigned d0 = 0, d1 = 0;
        if (row < rows) {
            d0 = scales[(size_t)row * blocks_per_row + 8 * t + g];
            d1 = scales[(size_t)row * blocks_per_row + 8 * t + 4 + g];
        }
        *reinterpret_cast<unsigned *>(dst + 4096 + 4 * lane) = d0 | (d1 << 16);
    }
}

// fp16 weights -> the tiled copy of the matrix-core GEMV: tile (rb, t) = sixteen rows x 256 columns = [j][m][lane] 16 bytes (lane
// (n, g) = g * 16 + n owns columns 32 (4 j + g) .. + 31 of the tile, row n; m = which eight of them), the middle two of every four
// weights exchanged (the order in which the kernels stage activations).  512 threads per tile; rows past the matrix are zeros.
__global__ void f16_tile_kernel(const uint16_t *w, int rows, int cols, size_t tiles, uint8_t *tiled) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t tile = i / 512;
    if (tile >= tiles) return;
    const int p = (int)(i - tile * 512), tpr = cols / 256;
    const int rb = (int)(tile / tpr), t = (int)(tile - (size_t)rb * tpr);
    const int j = p >> 8, m = (p >> 6) & 3, lane = p & 63, g = lane >> 4, n = lane & 15, row = rb * 16 + n;
    uint4 v = make_uint4(0, 0, 0, 0);
    if (row < rows) v = *reinterpret_cast<const uint4 *>(w + (size_t)row * cols + 256 * t + 32 * (4 * j + g) + 8 * m);
    uint4 s;
    s.x = __builtin_amdgcn_perm(v.y, v.x, 0x05040100u); s.y = __builtin_amdgcn_perm(v.y, v.x, 0x07060302u);
    s.z = __builtin_amdgcn_perm(v.w, v.z, 0x05040100u); s.w = __builtin_amdgcn_perm(v.w, v.z, 0x07060302u);
    *reinterpret_cast<uint4 *>(tiled + tile * 8192 + 1024 * (4 * j + m) + 16 * lane) = s;
}

inline dim3 grid_for(size_t n, int threads) { return dim3((unsigned)((n + threads - 1) / threads)); }

}  // namespace

hipError_t launch_dequant(int format, const uint8_t *blocks, size_t elems, float *out, hipStream_t stream) {
    if (!blocks || !out) return hipErrorInvalidValue;
    if (elems == 0) return hipSuccess;
    if (elems % format_block_elems(format) != 0) return hipErrorInvalidValue;
    const int t = 256;
    switch (format) {
    case FMT_Q8_0: hipLaunchKernelGGL(dequant_q8_0_kernel, grid_for(elems, t), dim3(t), 0, stream, blocks, elems, out); break;
    case FMT_Q4_0: hipLaunchKernelGGL(dequant_q4_0_kernel, grid_for(elems, t), dim3(t), 0, stream, blocks, elems, out); break;
    case FMT_Q4_K: hipLaunchKernelGGL(dequant_q4_k_kernel, grid_for(elems, t), dim3(t), 0, stream, blocks, elems, out); break;
    case FMT_F16: hipLaunchKernelGGL(dequant_f16_kernel, grid_for(elems, t), dim3(t), 0, stream, blocks, elems, out); break;
    case FMT_F32: hipLaunchKernelGGL(copy_f32_kernel, grid_for(elems, t), dim3(t), 0, stream, blocks, elems, out); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_repack(int format, const uint8_t *blocks, int rows, int cols, const DeviceMatrix &dst,
                         hipStream_t stream) {
    if (!blocks || !dst.qs || rows <= 0 || cols <= 0) return hipErrorInvalidValue;
    const size_t elems = (size_t)rows * cols;
    const int t = 256;
    switch (format) {
    case FMT_Q8_0:
        hipLaunchKernelGGL(repack_q8_0_kernel, grid_for(elems / 32, t), dim3(t), 0, stream, blocks, elems / 32, dst.qs, dst.scales);
        break;
    case FMT_Q4_0:
        hipLaunchKernelGGL(repack_q4_0_kernel, grid_for(elems / 32, t), dim3(t), 0, stream, blocks, elems / 32, dst.qs, dst.scales);
        break;
    case FMT_Q4_K:
    case FMT_F16:
    case FMT_F32: {
        hipError_t e = hipMemcpyAsync(dst.qs, blocks, format_bytes(format, elems), hipMemcpyDeviceToDevice, stream);
        if (e != hipSuccess) return e;
        break;
    }
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_q4k_tile(const uint8_t *blocks, int rows, int cols, uint8_t *tiled, hipStream_t stream) {
    if (!blocks || !tiled || rows <= 0 || cols <= 0 || cols % 256 != 0) return hipErrorInvalidValue;
    const int nsb = cols / 256;
    const size_t pieces = (size_t)((rows + 15) / 16) * nsb * 144;
    hipLaunchKernelGGL(q4k_tile_kernel, grid_for(pieces, 256), dim3(256), 0, stream, blocks, rows, nsb, pieces, tiled);
    return hipGetLastError();
}

hipError_t launch_q40_tile(const uint8_t *qs, const uint16_t *scales, int rows, int cols, uint8_t *tiled, hipStream_t stream) {
    if (!qs || !scales || !tiled || rows <= 0 || cols <= 0 || cols % 512 != 0) return hipErrorInvalidValue;
    const int tpr = cols / 512;
    const size_t tiles = (size_t)((rows + 15) / 16) * tpr;
    hipLaunchKernelGGL(q40_tile_kernel, grid_for(tiles * 320, 320), dim3(320), 0, stream, qs, scales, rows, tpr, tiles, tiled);
    return hipGetLastError();
}

hipError_t launch_q80_tile(const uint8_t *qs, const uint16_t *scales, int rows, int cols, uint8_t *tiled, hipStream_t stream) {
    if (!qs || !scales || !tiled || rows <= 0 || cols <= 0 || cols % 256 != 0) return hipErrorInvalidValue;
    const int tpr = cols / 256;
    const size_t tiles = (size_t)((rows + 15) / 16) * tpr;
    hipLaunchKernelGGL(q80_tile_kernel, grid_for(tiles * 320, 320), dim3(320), 0, stream, qs, scales, rows, tpr, tiles, tiled);
    return hipGetLastError();
}

hipError_t launch_f16_tile(const uint8_t *weights, int rows, int cols, uint8_t *tiled, hipStream_t stream) {
    if (!weights || !tiled || rows <= 0 || cols <= 0 || cols % 256 != 0) return hipErrorInvalidValue;
    const size_t tiles = (size_t)((rows + 15) / 16) * (cols / 256);
    hipLaunchKernelGGL(f16_tile_kernel, grid_for(tiles * 512, 512), dim3(512), 0, stream, reinterpret_cast<const uint16_t *>(weights), rows, cols, tiles, tiled);
    return hipGetLastError();
}

hipError_t launch_dequant_matrix(const DeviceMatrix &m, float *out, hipStream_t stream) {
    const size_t elems = (size_t)m.rows * m.cols;
    const int t = 256;
    switch (m.format) {
    case FMT_Q8_0:
        hipLaunchKernelGGL(dequant_planes_q8_0_kernel, grid_for(elems, t), dim3(t), 0, stream, m.qs, m.scales, elems, out);
        return hipGetLastError();
    case FMT_Q4_0:
        hipLaunchKernelGGL(dequant_planes_q4_0_kernel, grid_for(elems, t), dim3(t), 0, stream, m.qs, m.scales, elems, out);
        return hipGetLastError();
    default: return launch_dequant(m.format, m.qs, elems, out, stream);
    }
}

}  // namespace esp
