// INT4 output head: logits[r] = scale[r] * sum_j nibble[r][j] * x[j] + bias[r] * sum_j x[j]
// (INT4Classifier.rowDotProduct, Sources/Espresso/INT4Classifier.swift:40-71) over the packing of
// TensorBufferINT4 (Sources/ANETypes/TensorBufferINT4.swift:53-135): two nibbles per byte, HIGH nibble first,
// (dim + 1) / 2 bytes per row, per-row fp32 scale and bias.
//
// One wavefront per row at a time, four wavefronts per workgroup; the fp32 input sits in LDS with its sum; a
// lane reads 16 packed bytes (32 weights) per step when rows are 16-byte aligned, single bytes otherwise (odd
// or small dims).  Products nibble * x are exact in fp32; rows reduce with DPP.  HBM-bound: 0.5 byte per weight.
#include "../common.h"
#include "gemv_device.h"

namespace esp {
namespace {

using namespace detail;

__global__ __launch_bounds__(kThreads) void int4_matvec_kernel(const uint8_t *packed, const float *scales, const float *biases,
                                                               const float *input, int vocab, int dim, float *logits) {
    extern __shared__ float xs[];   // [dim] input, then [kWaves] partial sums
    float *red = xs + ((dim + 3) & ~3);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    float s = 0.0f;
    for (int i = tid; i < dim; i += kThreads) { const float v = input[i]; xs[i] = v; s += v; }
    const float input_sum = workgroup_sum(s, red);   // includes the barrier that publishes xs
    const int bpr = (dim + 1) / 2, pairs = dim / 2;
    const bool wide = bpr % 16 == 0;
    for (int row = blockIdx.x * kWaves + wave; row < vocab; row += gridDim.x * kWaves) {
        const uint8_t *rp = packed + (size_t)row * bpr;
        float dot = 0.0f;
        if (wide) {
            for (int b0 = lane * 16; b0 < bpr; b0 += 64 * 16) {
                const uint4 q = *reinterpret_cast<const uint4 *>(rp + b0);
                const float *x = xs + 2 * b0;
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const u32 w = dword_of(q, k);
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        const u32 byte = (w >> (8 * j)) & 0xFFu;
                        dot = __builtin_fmaf((float)(byte >> 4), x[8 * k + 2 * j], dot);
                        dot = __builtin_fmaf((float)(byte & 0xFu), x[8 * k + 2 * j + 1], dot);
                    }
                }
            }
        } else {
            for (int i = lane; i < pairs; i += 64) {
                const u32 byte = rp[i];
                dot = __builtin_fmaf((float)(byte >> 4), xs[2 * i], dot);
                dot = __builtin_fmaf((float)(byte & 0xFu), xs[2 * i + 1], dot);
            }
            if ((dim & 1) && lane == 0) dot = __builtin_fmaf((float)(rp[pairs] >> 4), xs[dim - 1], dot);
        }
        dot = wave_sum(dot);
        if (lane == 0) logits[row] = __fadd_rn(__fmul_rn(scales[row], dot), __fmul_rn(biases[row], input_sum));
    }
}

}  // namespace

hipError_t launch_int4_matvec(const uint8_t *packed, const float *scales, const float *biases, const float *input, int vocab, int dim,
                              float *logits, hipStream_t stream) {
    if (!packed || !scales || !biases || !input || !logits || vocab <= 0 || dim <= 0) return hipErrorInvalidValue;
    const size_t lds = ((size_t)((dim + 3) & ~3) + kWaves) * sizeof(float);
    if (lds > 64 * 1024) return hipErrorInvalidValue;
    int grid = (vocab + kWaves - 1) / kWaves;
    if (grid > 4096) grid = 4096;
    hipLaunchKernelGGL(int4_matvec_kernel, dim3(grid), dim3(kThreads), lds, stream, packed, scales, biases, input, vocab, dim, logits);
    return hipGetLastError();
}

}  // namespace esp
