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

__global__ void scatter_columns_strided_kernel(const float *in, int in_stride, int channels, int spatial, int lanes, uint16_t *surface) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x, l = blockIdx.y;
    if (c >= channels || l >= lanes) return;
    surface[(size_t)c * spatial + l] = f2h(in[(size_t)l * in_stride + c]);
}

// rope_decode (MetalAttentionKernel.swift:1756-1795): pairs (d, d + headDim/2), freq = theta^(-pair / half), fp16 in and out
__global__ void surface_rope_kernel(uint16_t *q, uint16_t *k, int n_heads, int n_kv_heads, int head_dim, int position, float theta, int lane_stride) {
    const int pair = blockIdx.x * blockDim.x + threadIdx.x, head = blockIdx.y, half = head_dim / 2;
    if (pair >= half) return;
    const float freq = powf(theta, -(float)pair / (float)half);
    const float angle = (float)position * freq;
    const float c = cosf(angle), sn = sinf(angle);
    auto rotate = [&](uint16_t *t) {
        const size_t i0 = (size_t)(head * head_dim + pair) * lane_stride, i1 = (size_t)(head * head_dim + pair + half) * lane_stride;
        const float v0 = h2f(t[i0]), v1 = h2f(t[i1]);
        t[i0] = f2h(__fsub_rn(__fmul_rn(v0, c), __fmul_rn(v1, sn)));
        t[i1] = f2h(__fadd_rn(__fmul_rn(v0, sn), __fmul_rn(v1, c)));
    };
    if (head < n_heads) rotate(q);
    if (head < n_kv_heads) rotate(k);
}

__global__ void surface_kv_scatter_kernel(const uint16_t *k_src, const uint16_t *v_src, uint16_t *k_cache, uint16_t *v_cache, int kv_dim, int token_index,
                                          int cache_stride, int lane_stride) {
    const int ch = blockIdx.x * blockDim.x + threadIdx.x;
    if (ch >= kv_dim) return;
    k_cache[(size_t)ch * cache_stride + token_index] = k_src[(size_t)ch * lane_stride];
    v_cache[(size_t)ch * cache_stride + token_index] = v_src[(size_t)ch * lane_stride];
}

// fused_decode_sdpa (MetalAttentionKernel.swift:1824-1886): one workgroup per query head; scores over the visible tokens in
// LDS, max-subtracted softmax, weighted sum of V per channel.  kvHead = head / (heads / kvHeads).
__global__ __launch_bounds__(256) void surface_sdpa_kernel(const uint16_t *q, const uint16_t *k_cache, const uint16_t *v_cache, uint16_t *context, int heads,
                                                           int kv_heads, int head_dim, int visible, int token_base, int cache_stride, int lane_stride) {
    extern __shared__ float scores[];   // [visible] + 256 for the reductions
    float *red = scores + visible;
    const int head = blockIdx.x, tid = threadIdx.x, kv_head = head / (heads / kv_heads);
    const float scale = 1.0f / sqrtf((float)head_dim);
    for (int t = tid; t < visible; t += 256) {
        float dot = 0.0f;
        for (int d = 0; d < head_dim; d++)
            dot += h2f(q[(size_t)(head * head_dim + d) * lane_stride]) * h2f(k_cache[(size_t)(kv_head * head_dim + d) * cache_stride + token_base + t]);
        scores[t] = dot * scale;
    }
    __syncthreads();
    float m = -INFINITY;
    for (int t = tid; t < visible; t += 256) m = fmaxf(m, scores[t]);
    red[tid] = m;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) { if (tid < s) red[tid] = fmaxf(red[tid], red[tid + s]); __syncthreads(); }
    m = red[0];
    __syncthreads();
    float sum = 0.0f;
    for (int t = tid; t < visible; t += 256) { const float e = expf(scores[t] - m); scores[t] = e; sum += e; }
    red[tid] = sum;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) { if (tid < s) red[tid] += red[tid + s]; __syncthreads(); }
    const float inv = red[0] > 0.0f ? 1.0f / red[0] : 0.0f;
    for (int d = tid; d < head_dim; d += 256) {
        const uint16_t *v = v_cache + (size_t)(kv_head * head_dim + d) * cache_stride + token_base;
        float acc = 0.0f;
        for (int t = 0; t < visible; t++) acc += (scores[t] * inv) * h2f(v[t]);
        context[(size_t)(head * head_dim + d) * lane_stride] = f2h(acc);
    }
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


// ---- factored output head: expansion [bottleneck -> vocab] fused with the arg-max ----
// logit[c] = sum_k proj[g * cpg + k][lane] * w[c][k], g = c / (vocab / groups), one fused multiply-add per term in k order, in fp16
// (the arithmetic of surface_io.c:1521-1700) or in fp32 (MetalExpansionArgmax.swift:1104-1140); no logit is stored.  A thread owns
// whole channels, so a channel's chain is sequential whatever the grid; candidates compare by (value, lowest channel).
template <bool FP32>
__device__ __forceinline__ void expansion_take(float &best, int &best_i, float v, int i) {
    if (v > best || (v == best && i < best_i)) { best = v; best_i = i; }
}

template <bool FP32, bool VEC>
__global__ __launch_bounds__(256) void expansion_argmax_kernel(const uint16_t *proj, int spatial, const uint16_t *w, int cpg, int ch_per_group, int vocab,
                                                               int bottleneck, float *cand_v, int *cand_i) {
    extern __shared__ uint16_t proj_lds[];                         // [bottleneck] of this lane
    const int lane_col = blockIdx.y, tid = threadIdx.x;
    for (int j = tid; j < bottleneck; j += 256) proj_lds[j] = proj[(size_t)j * spatial + lane_col];
    __syncthreads();
    // the running first maximum starts where the reference's does: fp16's most negative finite value (fp32: -inf) at channel 0
    float best = FP32 ? -INFINITY : -65504.0f;
    int best_i = 0;
    for (int c = blockIdx.x * 256 + tid; c < vocab; c += gridDim.x * 256) {
        const uint16_t *wr = w + (size_t)c * cpg;
        const uint16_t *pg = proj_lds + (c / ch_per_group) * cpg;
        float value;
        if constexpr (FP32) {
            float acc = 0.0f;
            if constexpr (VEC) {
                for (int k = 0; k < cpg; k += 8) {
                    const uint4 q = *reinterpret_cast<const uint4 *>(wr + k);
                    const uint32_t qw[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
                    for (int t = 0; t < 4; t++) {
                        acc = __builtin_fmaf(h2f(pg[k + 2 * t]), h2f((uint16_t)(qw[t] & 0xFFFFu)), acc);
                        acc = __builtin_fmaf(h2f(pg[k + 2 * t + 1]), h2f((uint16_t)(qw[t] >> 16)), acc);
                    }
                }
            } else {
                for (int k = 0; k < cpg; k++) acc = __builtin_fmaf(h2f(pg[k]), h2f(wr[k]), acc);
            }
            value = acc;
        } else {
            _Float16 acc = (_Float16)0.0f;
            if constexpr (VEC) {
                for (int k = 0; k < cpg; k += 8) {
                    const uint4 q = *reinterpret_cast<const uint4 *>(wr + k);
                    const uint32_t qw[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
                    for (int t = 0; t < 4; t++) {
                        acc = __builtin_fmaf16(__builtin_bit_cast(_Float16, (uint16_t)(qw[t] & 0xFFFFu)), __builtin_bit_cast(_Float16, pg[k + 2 * t]), acc);
                        acc = __builtin_fmaf16(__builtin_bit_cast(_Float16, (uint16_t)(qw[t] >> 16)), __builtin_bit_cast(_Float16, pg[k + 2 * t + 1]), acc);
                    }
                }
            } else {
                for (int k = 0; k < cpg; k++) acc = __builtin_fmaf16(__builtin_bit_cast(_Float16, wr[k]), __builtin_bit_cast(_Float16, pg[k]), acc);
            }
            value = (float)acc;
        }
        if (value > best) { best = value; best_i = c; }            // a thread's channels only grow: strict > keeps the first maximum
    }
    __shared__ float sv[256];
    __shared__ int si[256];
    sv[tid] = best; si[tid] = best_i;
    __syncthreads();
    for (int off = 128; off > 0; off >>= 1) {
        if (tid < off) expansion_take<FP32>(sv[tid], si[tid], sv[tid + off], si[tid + off]);
        __syncthreads();
    }
    if (tid == 0) {
        cand_v[(size_t)lane_col * gridDim.x + blockIdx.x] = sv[0];
        cand_i[(size_t)lane_col * gridDim.x + blockIdx.x] = si[0];
    }
}

__global__ __launch_bounds__(64) void expansion_argmax_final_kernel(const float *cand_v, const int *cand_i, int blocks, int *out_i, float *out_v) {
    const int lane_col = blockIdx.x, tid = threadIdx.x;
    float best = cand_v[(size_t)lane_col * blocks];
    int best_i = cand_i[(size_t)lane_col * blocks];
    for (int b = tid; b < blocks; b += 64) expansion_take<true>(best, best_i, cand_v[(size_t)lane_col * blocks + b], cand_i[(size_t)lane_col * blocks + b]);
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(best, off);
        const int oi = __shfl_xor(best_i, off);
        expansion_take<true>(best, best_i, ov, oi);
    }
    if (tid == 0) { out_i[lane_col] = best_i; out_v[lane_col] = best; }
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
hipError_t launch_scatter_columns_strided(const float *in, int in_stride, int channels, int spatial, int lanes, uint16_t *surface, hipStream_t s) {
    hipLaunchKernelGGL(scatter_columns_strided_kernel, dim3((channels + 255) / 256, lanes), dim3(256), 0, s, in, in_stride, channels, spatial, lanes, surface);
    return hipGetLastError();
}
hipError_t launch_surface_rope(uint16_t *q, uint16_t *k, int n_heads, int n_kv_heads, int head_dim, int position, float theta, int lane_stride, hipStream_t s) {
    const int half = head_dim / 2, heads = n_heads > n_kv_heads ? n_heads : n_kv_heads;
    hipLaunchKernelGGL(surface_rope_kernel, dim3((half + 63) / 64, heads), dim3(64), 0, s, q, k, n_heads, n_kv_heads, head_dim, position, theta, lane_stride);
    return hipGetLastError();
}
hipError_t launch_surface_kv_scatter(const uint16_t *k_src, const uint16_t *v_src, uint16_t *k_cache, uint16_t *v_cache, int kv_dim, int token_index,
                                     int cache_stride, int lane_stride, hipStream_t s) {
    hipLaunchKernelGGL(surface_kv_scatter_kernel, dim3((kv_dim + 255) / 256), dim3(256), 0, s, k_src, v_src, k_cache, v_cache, kv_dim, token_index, cache_stride,
                       lane_stride);
    return hipGetLastError();
}
hipError_t launch_surface_sdpa(const uint16_t *q, const uint16_t *k_cache, const uint16_t *v_cache, uint16_t *context, int heads, int kv_heads, int head_dim,
                               int visible_tokens, int token_base, int cache_stride, int lane_stride, hipStream_t s) {
    // one score per visible token in LDS: up to 48 KB without raising the kernel's limit, i.e. 12032 tokens
    const size_t lds = ((size_t)visible_tokens + 256) * 4;
    if (lds > 48 * 1024) return hipErrorInvalidValue;
    hipLaunchKernelGGL(surface_sdpa_kernel, dim3(heads), dim3(256), lds, s, q, k_cache, v_cache, context, heads, kv_heads, head_dim, visible_tokens, token_base,
                       cache_stride, lane_stride);
    return hipGetLastError();
}
hipError_t launch_row_max(const float *in, int channels, int spatial, int lanes, uint16_t *surface, hipStream_t s) {
    hipLaunchKernelGGL(row_max_kernel, dim3(lanes), dim3(256), 0, s, in, channels, spatial, surface);
    return hipGetLastError();
}

hipError_t launch_expansion_argmax(const uint16_t *proj, int spatial, int lanes, const uint16_t *w, int bottleneck, int groups, int vocab, bool fp32_sums,
                                   int blocks, float *cand_v, int *cand_i, int *out_i, float *out_v, hipStream_t s) {
    const int cpg = bottleneck / groups, ch_per_group = vocab / groups;
    const size_t lds = (size_t)bottleneck * 2;
    if (lds > 48 * 1024 || blocks <= 0) return hipErrorInvalidValue;
    const dim3 grid(blocks, lanes);
    const bool vec = cpg % 8 == 0;
    if (fp32_sums) {
        if (vec) hipLaunchKernelGGL((expansion_argmax_kernel<true, true>), grid, dim3(256), lds, s, proj, spatial, w, cpg, ch_per_group, vocab, bottleneck, cand_v, cand_i);
        else hipLaunchKernelGGL((expansion_argmax_kernel<true, false>), grid, dim3(256), lds, s, proj, spatial, w, cpg, ch_per_group, vocab, bottleneck, cand_v, cand_i);
    } else {
        if (vec) hipLaunchKernelGGL((expansion_argmax_kernel<false, true>), grid, dim3(256), lds, s, proj, spatial, w, cpg, ch_per_group, vocab, bottleneck, cand_v, cand_i);
        else hipLaunchKernelGGL((expansion_argmax_kernel<false, false>), grid, dim3(256), lds, s, proj, spatial, w, cpg, ch_per_group, vocab, bottleneck, cand_v, cand_i);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(expansion_argmax_final_kernel, dim3(lanes), dim3(64), 0, s, cand_v, cand_i, blocks, out_i, out_v);
    return hipGetLastError();
}

}  // namespace esp
