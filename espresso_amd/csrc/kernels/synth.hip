// Seeded synthetic weights generated and quantised on the GPU: N(0, std) draws from a counter-based
// generator (SplitMix64 finaliser + Box-Muller, so a value depends only on (seed, element index)),
// packed into GGUF-layout blocks.  Used to fill benchmark-sized models (8e9 weights) in seconds;
// the packed bytes are handed back to the host and travel the normal upload path, so the CPU
// baseline and the parity checks see exactly the bytes the kernels run on.
//
// Quantisers: Q8_0 and Q4_0 follow ggml's quantize_row_q8_0_ref / quantize_row_q4_0_ref; Q4_K is a
// plain min/max fit per sub-block with 6-bit super-block scales (a valid Q4_K packing, not ggml's
// iterative search).
#include "../common.h"

namespace esp {
namespace {

__device__ __forceinline__ uint64_t splitmix64(uint64_t x) {
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}

// standard normal for element `i` of stream `seed`
__device__ __forceinline__ float normal_at(uint64_t seed, uint64_t i) {
    const uint64_t r = splitmix64(seed * 0xD1342543DE82EF95ull + i);
    const float u1 = ((float)(uint32_t)(r >> 40) + 1.0f) * (1.0f / 16777216.0f);  // (0, 1]
    const float u2 = (float)(uint32_t)((r >> 8) & 0xFFFFFFu) * (1.0f / 16777216.0f);
    return sqrtf(-2.0f * logf(u1)) * cosf(6.28318530718f * u2);
}

__device__ __forceinline__ uint16_t half_bits(float v) { return __builtin_bit_cast(uint16_t, (_Float16)v); }
__device__ __forceinline__ float half_round(float v) { return (float)(_Float16)v; }

template <int WIDTH>
__device__ __forceinline__ float group_max(float v) {
#pragma unroll
    for (int off = WIDTH / 2; off >= 1; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}
template <int WIDTH>
__device__ __forceinline__ float group_min(float v) {
#pragma unroll
    for (int off = WIDTH / 2; off >= 1; off >>= 1) v = fminf(v, __shfl_xor(v, off, 64));
    return v;
}

// One wavefront per 256 consecutive elements; lane l holds elements 4l..4l+3, so a 32-element
// block lives in 8 consecutive lanes.
template <int FMT>
__global__ __launch_bounds__(256) void synth_kernel(uint64_t seed, float std_dev, size_t elems, uint8_t *out) {
    const int lane = threadIdx.x & 63;
    const size_t group = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (group * 256 >= elems) return;
    float x[4];
#pragma unroll
    for (int k = 0; k < 4; k++) x[k] = std_dev * normal_at(seed, group * 256 + lane * 4 + k);
    const int blk = lane >> 3, l8 = lane & 7;  // block within the group, lane within the block

    if (FMT == FMT_F16) {
        uint16_t *o = reinterpret_cast<uint16_t *>(out) + group * 256 + lane * 4;
#pragma unroll
        for (int k = 0; k < 4; k++) o[k] = half_bits(x[k]);
    } else if (FMT == FMT_Q8_0) {
        float amax = fmaxf(fmaxf(fabsf(x[0]), fabsf(x[1])), fmaxf(fabsf(x[2]), fabsf(x[3])));
        amax = group_max<8>(amax);
        const float d = amax / 127.0f, id = d != 0.0f ? 1.0f / d : 0.0f;
        uint8_t *b = out + (group * 8 + blk) * 34;
        if (l8 == 0) *reinterpret_cast<uint16_t *>(b) = half_bits(d);
#pragma unroll
        for (int k = 0; k < 4; k++) b[2 + l8 * 4 + k] = (uint8_t)(int8_t)roundf(x[k] * id);
    } else if (FMT == FMT_Q4_0) {
        // value of the element with the largest magnitude (first one on ties)
        float amax = 0.0f, vmax = 0.0f;
#pragma unroll
        for (int k = 0; k < 4; k++) if (amax < fabsf(x[k])) { amax = fabsf(x[k]); vmax = x[k]; }
#pragma unroll
        for (int off = 1; off < 8; off <<= 1) {
            const float oa = __shfl_xor(amax, off, 64), ov = __shfl_xor(vmax, off, 64);
            const bool other_first = (lane ^ off) < lane;
            if (oa > amax || (oa == amax && other_first)) { amax = oa; vmax = ov; }
        }
        const float d = vmax / -8.0f, id = d != 0.0f ? 1.0f / d : 0.0f;
        uint8_t *b = out + (group * 8 + blk) * 18;
        if (l8 == 0) *reinterpret_cast<uint16_t *>(b) = half_bits(d);
        int q[4];
#pragma unroll
        for (int k = 0; k < 4; k++) {
            int v = (int)(int8_t)(x[k] * id + 8.5f);
            q[k] = v > 15 ? 15 : v;
        }
        // element e of the block is the low nibble of byte e (e < 16) or the high nibble of byte e-16
        const int partner = lane ^ 4;
        int pq[4];
#pragma unroll
        for (int k = 0; k < 4; k++) pq[k] = __shfl(q[k], partner, 64);
        if (l8 < 4) {
#pragma unroll
            for (int k = 0; k < 4; k++) b[2 + l8 * 4 + k] = (uint8_t)(q[k] | (pq[k] << 4));
        }
    } else {  // FMT_Q4_K
        float lo = fminf(fminf(x[0], x[1]), fminf(x[2], x[3])), hi = fmaxf(fmaxf(x[0], x[1]), fmaxf(x[2], x[3]));
        lo = group_min<8>(lo);
        hi = group_max<8>(hi);
        if (lo > 0.0f) lo = 0.0f;
        const float scale = (hi - lo) / 15.0f, mn = -lo;
        const float max_scale = group_max<64>(scale), max_min = group_max<64>(mn);
        const float inv_scale = max_scale > 0.0f ? 63.0f / max_scale : 0.0f;
        const float inv_min = max_min > 0.0f ? 63.0f / max_min : 0.0f;
        int ls = (int)rintf(inv_scale * scale), lm = (int)rintf(inv_min * mn);
        ls = ls > 63 ? 63 : ls;
        lm = lm > 63 ? 63 : lm;
        const float d = half_round(max_scale / 63.0f), dmin = half_round(max_min / 63.0f);
        const float dd = d * (float)ls, dm = dmin * (float)lm;
        int q[4];
#pragma unroll
        for (int k = 0; k < 4; k++) {
            int v = 0;
            if (dd != 0.0f) {
                v = (int)rintf((x[k] + dm) / dd);
                v = v < 0 ? 0 : (v > 15 ? 15 : v);
            }
            q[k] = v;
        }
        uint8_t *b = out + group * 144;
        if (lane == 0) {
            *reinterpret_cast<uint16_t *>(b) = half_bits(max_scale / 63.0f);
            *reinterpret_cast<uint16_t *>(b + 2) = half_bits(max_min / 63.0f);
        }
        // 6-bit scales/mins: lane 8j holds sub-block j's pair; gather the eight pairs and pack
        int sc8[8], m8[8];
#pragma unroll
        for (int j = 0; j < 8; j++) { sc8[j] = __shfl(ls, 8 * j, 64); m8[j] = __shfl(lm, 8 * j, 64); }
        if (lane < 4) {
            b[4 + lane] = (uint8_t)(sc8[lane] | ((sc8[lane + 4] >> 4) << 6));
            b[8 + lane] = (uint8_t)(m8[lane] | ((m8[lane + 4] >> 4) << 6));
            b[12 + lane] = (uint8_t)((sc8[lane + 4] & 0xF) | ((m8[lane + 4] & 0xF) << 4));
        }
        // sub-block 2c (low nibbles) pairs with sub-block 2c+1 (high nibbles): partner lane is 8 away
        int pq[4];
#pragma unroll
        for (int k = 0; k < 4; k++) pq[k] = __shfl(q[k], lane ^ 8, 64);
        if ((blk & 1) == 0) {
            uint8_t *qs = b + 16 + (blk >> 1) * 32 + l8 * 4;
#pragma unroll
            for (int k = 0; k < 4; k++) qs[k] = (uint8_t)(q[k] | (pq[k] << 4));
        }
    }
}

}  // namespace

hipError_t launch_synth(int format, uint64_t seed, float std_dev, size_t elems, uint8_t *out, hipStream_t stream) {
    if (!out || elems == 0 || elems % 256 != 0) return hipErrorInvalidValue;
    const unsigned grid = (unsigned)((elems / 256 + 3) / 4);
    switch (format) {
    case FMT_F16: hipLaunchKernelGGL(synth_kernel<FMT_F16>, dim3(grid), dim3(256), 0, stream, seed, std_dev, elems, out); break;
    case FMT_Q8_0: hipLaunchKernelGGL(synth_kernel<FMT_Q8_0>, dim3(grid), dim3(256), 0, stream, seed, std_dev, elems, out); break;
    case FMT_Q4_0: hipLaunchKernelGGL(synth_kernel<FMT_Q4_0>, dim3(grid), dim3(256), 0, stream, seed, std_dev, elems, out); break;
    case FMT_Q4_K: hipLaunchKernelGGL(synth_kernel<FMT_Q4_K>, dim3(grid), dim3(256), 0, stream, seed, std_dev, elems, out); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace esp
