// The small per-token kernels around the GEMVs of one llama decode step:
// embedding lookup, RMSNorm, per-head q/k norm + RoPE + KV-cache scatter, single-query attention,
// SwiGLU and first-max argmax.  Each follows the order of operations of the reference's CPU-exact
// path (Sources/RealModelInference/RealModelInferenceEngine.swift:6221-6347, helpers :6648-6827) so
// that the only differences from it are the order of parallel sums and the fp16 rounding of GEMV
// inputs.  Products that the reference rounds separately are never contracted into fused
// multiply-adds here (__fmul_rn / __fadd_rn / __fsub_rn).
#include "../common.h"
#include "decode_ops.h"

namespace esp {
namespace {

constexpr int kBlock = 256;

__device__ __forceinline__ float wave_sum_f(float v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}
__device__ __forceinline__ float wave_max_f(float v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}
// block-wide sum for blockDim.x <= 1024 (multiple of 64); `scratch` holds >= 16 floats
__device__ __forceinline__ float block_sum(float v, float *scratch) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = (blockDim.x + 63) >> 6;
    v = wave_sum_f(v);
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float t = 0.0f;
    for (int w = 0; w < waves; w++) t += scratch[w];
    return t;
}
__device__ __forceinline__ float block_max(float v, float *scratch) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = (blockDim.x + 63) >> 6;
    v = wave_max_f(v);
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float t = scratch[0];
    for (int w = 1; w < waves; w++) t = fmaxf(t, scratch[w]);
    return t;
}

__device__ __forceinline__ uint16_t to_half_bits(float v) { return __builtin_bit_cast(uint16_t, (_Float16)v); }
__device__ __forceinline__ float from_half_bits(uint16_t b) { return (float)__builtin_bit_cast(_Float16, b); }

// hidden[m][:] = embedding[token[m]][:]                       (:6222)
__global__ void embed_kernel(const void *table, int table_is_f16, const int *tokens, int d, float *hidden) {
    const int m = blockIdx.y;
    const size_t row = (size_t)tokens[m] * d;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < d; i += gridDim.x * blockDim.x) {
        hidden[(size_t)m * d + i] = table_is_f16 ? from_half_bits(reinterpret_cast<const uint16_t *>(table)[row + i])
                                                 : reinterpret_cast<const float *>(table)[row + i];
    }
}

// out[m][i] = fp16( (x[m][i] * inv) * w[i] ),  inv = 1/sqrt(sum x^2 / d + eps)      (:6724-6743)
// One workgroup per row.  Also clears the row's argmax cell when one is given.
__global__ __launch_bounds__(kBlock) void rmsnorm_kernel(const float *x, const float *w, float eps, int d,
                                                         uint16_t *out_f16, unsigned long long *argmax_cells) {
    __shared__ float scratch[16];
    const int m = blockIdx.x;
    const float *xr = x + (size_t)m * d;
    constexpr int kVec = 8;  // float4 per thread held in registers: rows up to 8192 wide in one pass
    if (d % 4 == 0 && d <= kVec * 4 * kBlock) {
        // every load is issued before the first use, so the row costs one memory round trip
        const float4 *x4 = reinterpret_cast<const float4 *>(xr), *w4 = reinterpret_cast<const float4 *>(w);
        const int n4 = d / 4;
        float4 v[kVec], g[kVec];
#pragma unroll
        for (int k = 0; k < kVec; k++) {
            const int i = threadIdx.x + k * kBlock;
            v[k] = i < n4 ? x4[i] : make_float4(0.f, 0.f, 0.f, 0.f);
            g[k] = i < n4 ? w4[i] : make_float4(0.f, 0.f, 0.f, 0.f);
        }
        float s = 0.0f;
#pragma unroll
        for (int k = 0; k < kVec; k++) s += v[k].x * v[k].x + v[k].y * v[k].y + v[k].z * v[k].z + v[k].w * v[k].w;
        const float inv = 1.0f / sqrtf(block_sum(s, scratch) / (float)d + eps);
#pragma unroll
        for (int k = 0; k < kVec; k++) {
            const int i = threadIdx.x + k * kBlock;
            if (i < n4) {
                uint2 o;
                o.x = to_half_bits(__fmul_rn(__fmul_rn(v[k].x, inv), g[k].x)) | ((uint32_t)to_half_bits(__fmul_rn(__fmul_rn(v[k].y, inv), g[k].y)) << 16);
                o.y = to_half_bits(__fmul_rn(__fmul_rn(v[k].z, inv), g[k].z)) | ((uint32_t)to_half_bits(__fmul_rn(__fmul_rn(v[k].w, inv), g[k].w)) << 16);
                reinterpret_cast<uint2 *>(out_f16 + (size_t)m * d)[i] = o;
            }
        }
    } else {
        float s = 0.0f;
        for (int i = threadIdx.x; i < d; i += kBlock) s += xr[i] * xr[i];
        const float inv = 1.0f / sqrtf(block_sum(s, scratch) / (float)d + eps);
        for (int i = threadIdx.x; i < d; i += kBlock)
            out_f16[(size_t)m * d + i] = to_half_bits(__fmul_rn(__fmul_rn(xr[i], inv), w[i]));
    }
    if (argmax_cells && threadIdx.x == 0) argmax_cells[m] = 0ull;
}

// Per (row m, head slot): optional per-head RMSNorm of q/k (:6648-6672), half-split RoPE from a
// host-built cos/sin table (:6745-6772), then q -> q_out, k/v -> caches at (seq[m], pos[m]) (:6297-6300).
// `qkv` rows are in the fused matrix's order: q and k as RoPE pairs (j, j+half) side by side, v natural.
template <bool KV_F16>
__global__ void qkv_post_kernel(QkvPostArgs a) {
    __shared__ float scratch[16];
    const int m = blockIdx.y, slot = blockIdx.x;
    const int half = a.head_dim / 2, nh = a.n_head, nkv = a.n_kv_head;
    const int ad = nh * a.head_dim, kd = nkv * a.head_dim;
    const float *row = a.qkv + (size_t)m * (ad + 2 * kd);
    const int pos = a.pos[m];
    const size_t seq_base = (size_t)a.seq[m] * a.cache_seq_stride;
    const int j = threadIdx.x;  // pair index; blockDim.x is `half` rounded up to whole wavefronts
    const bool live = j < half;
    if (slot < nh + nkv) {
        const bool is_q = slot < nh;
        const int h = is_q ? slot : slot - nh;
        const float *src = row + (is_q ? 0 : ad) + (size_t)h * a.head_dim;
        float v0 = live ? src[2 * j] : 0.0f, v1 = live ? src[2 * j + 1] : 0.0f;
        const float *norm_w = is_q ? a.q_norm : a.k_norm;
        if (norm_w) {
            const float sum_sq = block_sum(v0 * v0 + v1 * v1, scratch);
            const float inv = 1.0f / sqrtf(sum_sq / (float)a.head_dim + a.norm_eps);
            if (live) {
                v0 = __fmul_rn(v0, __fmul_rn(inv, norm_w[j]));
                v1 = __fmul_rn(v1, __fmul_rn(inv, norm_w[j + half]));
            }
        }
        if (!live) return;
        const float c = a.rope_cos[(size_t)pos * half + j], s = a.rope_sin[(size_t)pos * half + j];
        const float r0 = __fsub_rn(__fmul_rn(v0, c), __fmul_rn(v1, s));
        const float r1 = __fadd_rn(__fmul_rn(v0, s), __fmul_rn(v1, c));
        if (is_q) {
            float *q = a.q_out + (size_t)m * ad + (size_t)h * a.head_dim;
            q[j] = r0;
            q[j + half] = r1;
        } else {
            // K cache is token-major [maxSeq][kvDim], like V
            const size_t c0 = seq_base + (size_t)pos * kd + (size_t)h * a.head_dim + j;
            const size_t c1 = c0 + half;
            if (KV_F16) {
                reinterpret_cast<uint16_t *>(a.k_cache)[c0] = to_half_bits(r0);
                reinterpret_cast<uint16_t *>(a.k_cache)[c1] = to_half_bits(r1);
            } else {
                reinterpret_cast<float *>(a.k_cache)[c0] = r0;
                reinterpret_cast<float *>(a.k_cache)[c1] = r1;
            }
        }
    } else {
        // V cache is token-major [maxSeq][kvDim]
        const int h = slot - nh - nkv;
        const float *src = row + ad + kd + (size_t)h * a.head_dim;
        const size_t c0 = seq_base + (size_t)pos * kd + (size_t)h * a.head_dim;
        for (int i = j; i < a.head_dim; i += blockDim.x) {
            if (KV_F16) reinterpret_cast<uint16_t *>(a.v_cache)[c0 + i] = to_half_bits(src[i]);
            else reinterpret_cast<float *>(a.v_cache)[c0 + i] = src[i];
        }
    }
}

// Single-query attention over the visible prefix of one sequence's KV cache (:6774-6823): the
// general kernel, one workgroup per (head, row), any head size.  Scores use the reference's exact
// per-token sum (dims ascending, separate multiply and add); the softmax sums and the value sums
// run in parallel order.
template <bool KV_F16>
__global__ __launch_bounds__(kBlock) void attention_decode_kernel(AttentionArgs a) {
    extern __shared__ float smem[];
    float *q_s = smem;                     // [head_dim]
    float *p_s = smem + a.head_dim;        // [max_seq]
    float *part = p_s + a.max_seq;         // [kBlock] partial value sums
    __shared__ float scratch[16];
    const int h = blockIdx.x, m = blockIdx.y, hd = a.head_dim;
    const int group = a.n_head / a.n_kv_head;
    const int kvh = h / group < a.n_kv_head - 1 ? h / group : a.n_kv_head - 1;
    const int visible = a.pos[m] + 1;
    const size_t seq_base = (size_t)a.seq[m] * a.cache_seq_stride;
    const int kd = a.n_kv_head * hd;
    const float scale = 1.0f / sqrtf((float)hd);
    for (int i = threadIdx.x; i < hd; i += kBlock) q_s[i] = a.q[(size_t)m * a.n_head * hd + (size_t)h * hd + i];
    __syncthreads();

    float local_max = -INFINITY;
    for (int t = threadIdx.x; t < visible; t += kBlock) {
        float dot = 0.0f;
        const size_t kbase = seq_base + (size_t)t * kd + (size_t)kvh * hd;
        for (int dch = 0; dch < hd; dch++) {
            const float kv = KV_F16 ? from_half_bits(reinterpret_cast<const uint16_t *>(a.k_cache)[kbase + dch])
                                    : reinterpret_cast<const float *>(a.k_cache)[kbase + dch];
            dot = __fadd_rn(dot, __fmul_rn(q_s[dch], kv));
        }
        const float sc = __fmul_rn(dot, scale);
        p_s[t] = sc;
        local_max = fmaxf(local_max, sc);
    }
    const float max_score = block_max(local_max, scratch);
    float local_sum = 0.0f;
    for (int t = threadIdx.x; t < visible; t += kBlock) {
        const float e = expf(p_s[t] - max_score);
        p_s[t] = e;
        local_sum += e;
    }
    const float denom = block_sum(local_sum, scratch);
    const float inv_denom = denom > 0.0f ? 1.0f / denom : 0.0f;
    __syncthreads();

    // value sums: thread = (token slice, channel); slices combined through LDS
    const int slices = kBlock / hd > 0 ? kBlock / hd : 1;
    for (int d0 = 0; d0 < hd; d0 += kBlock) {
        const int dch = d0 + (int)(threadIdx.x % (hd < kBlock ? hd : kBlock));
        const int slice = threadIdx.x / (hd < kBlock ? hd : kBlock);
        float acc = 0.0f;
        if (dch < hd && slice < slices) {
            const size_t vbase = seq_base + (size_t)kvh * hd + dch;
            for (int t = slice; t < visible; t += slices) {
                const float vv = KV_F16 ? from_half_bits(reinterpret_cast<const uint16_t *>(a.v_cache)[vbase + (size_t)t * kd])
                                        : reinterpret_cast<const float *>(a.v_cache)[vbase + (size_t)t * kd];
                acc += __fmul_rn(p_s[t], inv_denom) * vv;
            }
        }
        part[threadIdx.x] = acc;
        __syncthreads();
        if (slice == 0 && dch < hd) {
            float total = 0.0f;
            for (int s = 0; s < slices; s++) total += part[s * (hd < kBlock ? hd : kBlock) + (dch - d0)];
            a.ctx_f16[(size_t)m * a.n_head * hd + (size_t)h * hd + dch] = to_half_bits(total);
        }
        __syncthreads();
    }
}


// Single-query attention, grouped-query form: one workgroup of 16 wavefronts per (KV head, row)
// serves the G query heads that share the KV head, so K and V are read once.  Both caches are
// token-major; a token's head vector is contiguous (HD fp16 = 256 bytes at HD 128).
//   scores: HD/16 lanes per token, 16 dims (two 128-bit loads) per lane, partial dots reduced over
//           those lanes; 64/(HD/16) tokens per wavefront pass;
//   values: HD/8 lanes per token, 8 dims (one 128-bit load) per lane, fp32 accumulators per query
//           head, reduced over the token slots of the wavefront and then over the 16 wavefronts.
template <int HD, int G, bool KV_F16>
__global__ __launch_bounds__(1024) void attention_gqa_kernel(AttentionArgs a) {
    extern __shared__ float smem[];
    float *sc = smem;                                  // [G][max_seq] scores, then probabilities
    float *part = smem + (size_t)G * a.max_seq;        // [16][G][HD] per-wavefront value sums
    __shared__ float red[16 * G];
    constexpr int LPT = HD / 16, TPI = 64 / LPT;       // score phase: lanes per token, tokens per pass
    constexpr int LPV = HD / 8, TPV = 64 / LPV;        // value phase
    const int kvh = blockIdx.x, m = blockIdx.y;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int visible = a.pos[m] + 1;
    const int kd = a.n_kv_head * HD;
    const size_t seq_base = (size_t)a.seq[m] * a.cache_seq_stride;
    const float scale = 1.0f / sqrtf((float)HD);

    {   // ---- scores ----
        const int seg = (lane % LPT) * 16;
        float q[G][16];
#pragma unroll
        for (int g = 0; g < G; g++)
#pragma unroll
            for (int i = 0; i < 16; i++) q[g][i] = a.q[(size_t)m * a.n_head * HD + (size_t)(kvh * G + g) * HD + seg + i];
        for (int t0 = wave * TPI; t0 < visible; t0 += 16 * TPI) {
            const int t = t0 + lane / LPT;
            const bool valid = t < visible;
            const size_t off = seq_base + (size_t)(valid ? t : 0) * kd + (size_t)kvh * HD + seg;
            float k[16];
            if (KV_F16) {
                const uint4 *p = reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(a.k_cache) + off);
                const uint4 v0 = p[0], v1 = p[1];
                const uint32_t w[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
#pragma unroll
                for (int i = 0; i < 8; i++) { k[2 * i] = from_half_bits((uint16_t)(w[i] & 0xFFFFu)); k[2 * i + 1] = from_half_bits((uint16_t)(w[i] >> 16)); }
            } else {
                const float4 *p = reinterpret_cast<const float4 *>(reinterpret_cast<const float *>(a.k_cache) + off);
#pragma unroll
                for (int i = 0; i < 4; i++) { const float4 v = p[i]; k[4 * i] = v.x; k[4 * i + 1] = v.y; k[4 * i + 2] = v.z; k[4 * i + 3] = v.w; }
            }
            float dot[G];
#pragma unroll
            for (int g = 0; g < G; g++) {
                float d = 0.0f;
#pragma unroll
                for (int i = 0; i < 16; i++) d += q[g][i] * k[i];
#pragma unroll
                for (int o = LPT / 2; o >= 1; o >>= 1) d += __shfl_xor(d, o, 64);
                dot[g] = d;
            }
            if (valid && lane % LPT == 0) {
#pragma unroll
                for (int g = 0; g < G; g++) sc[(size_t)g * a.max_seq + t] = dot[g] * scale;
            }
        }
    }
    __syncthreads();
    // ---- softmax over the visible tokens, per query head ----
    float inv_denom[G];
    {
        float mx[G], sm[G];
#pragma unroll
        for (int g = 0; g < G; g++) {
            float v = -INFINITY;
            for (int t = tid; t < visible; t += 1024) v = fmaxf(v, sc[(size_t)g * a.max_seq + t]);
            v = wave_max_f(v);
            if (lane == 0) red[wave * G + g] = v;
        }
        __syncthreads();
#pragma unroll
        for (int g = 0; g < G; g++) {
            float v = red[g];
            for (int w = 1; w < 16; w++) v = fmaxf(v, red[w * G + g]);
            mx[g] = v;
        }
        __syncthreads();
#pragma unroll
        for (int g = 0; g < G; g++) {
            float s = 0.0f;
            for (int t = tid; t < visible; t += 1024) {
                const float e = expf(sc[(size_t)g * a.max_seq + t] - mx[g]);
                sc[(size_t)g * a.max_seq + t] = e;
                s += e;
            }
            s = wave_sum_f(s);
            if (lane == 0) red[wave * G + g] = s;
        }
        __syncthreads();
#pragma unroll
        for (int g = 0; g < G; g++) {
            float s = 0.0f;
            for (int w = 0; w < 16; w++) s += red[w * G + g];
            sm[g] = s;
            inv_denom[g] = s > 0.0f ? 1.0f / s : 0.0f;
        }
        (void)sm;
    }
    // ---- values ----
    {
        const int seg = (lane % LPV) * 8;
        float acc[G][8];
#pragma unroll
        for (int g = 0; g < G; g++)
#pragma unroll
            for (int i = 0; i < 8; i++) acc[g][i] = 0.0f;
        for (int t0 = wave * TPV; t0 < visible; t0 += 16 * TPV) {
            const int t = t0 + lane / LPV;
            const bool valid = t < visible;
            const size_t off = seq_base + (size_t)(valid ? t : 0) * kd + (size_t)kvh * HD + seg;
            float v[8];
            if (KV_F16) {
                const uint4 r = *reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(a.v_cache) + off);
                const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
                for (int i = 0; i < 4; i++) { v[2 * i] = from_half_bits((uint16_t)(w[i] & 0xFFFFu)); v[2 * i + 1] = from_half_bits((uint16_t)(w[i] >> 16)); }
            } else {
                const float4 *p = reinterpret_cast<const float4 *>(reinterpret_cast<const float *>(a.v_cache) + off);
                const float4 r0 = p[0], r1 = p[1];
                v[0] = r0.x; v[1] = r0.y; v[2] = r0.z; v[3] = r0.w; v[4] = r1.x; v[5] = r1.y; v[6] = r1.z; v[7] = r1.w;
            }
#pragma unroll
            for (int g = 0; g < G; g++) {
                const float p = valid ? sc[(size_t)g * a.max_seq + t] * inv_denom[g] : 0.0f;
#pragma unroll
                for (int i = 0; i < 8; i++) acc[g][i] += p * v[i];
            }
        }
#pragma unroll
        for (int g = 0; g < G; g++)
#pragma unroll
            for (int i = 0; i < 8; i++) {
                float x = acc[g][i];
#pragma unroll
                for (int o = LPV; o < 64; o <<= 1) x += __shfl_xor(x, o, 64);
                if (lane < LPV) part[((size_t)wave * G + g) * HD + seg + i] = x;
            }
    }
    __syncthreads();
    for (int i = tid; i < G * HD; i += 1024) {
        float total = 0.0f;
        for (int w = 0; w < 16; w++) total += part[(size_t)w * G * HD + i];
        const int g = i / HD, dch = i % HD;
        a.ctx_f16[(size_t)m * a.n_head * HD + (size_t)(kvh * G + g) * HD + dch] = to_half_bits(total);
    }
}

template <int HD, int G>
hipError_t launch_attention_gqa(const AttentionArgs &a, int rows, bool kv_f16, hipStream_t s) {
    const size_t lds = ((size_t)G * a.max_seq + (size_t)16 * G * HD) * sizeof(float);
    dim3 grid(a.n_kv_head, rows);
    if (kv_f16) {
        auto kernel = attention_gqa_kernel<HD, G, true>;
        if (lds > 48 * 1024) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return e;
        }
        hipLaunchKernelGGL(kernel, grid, dim3(1024), lds, s, a);
    } else {
        auto kernel = attention_gqa_kernel<HD, G, false>;
        if (lds > 48 * 1024) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return e;
        }
        hipLaunchKernelGGL(kernel, grid, dim3(1024), lds, s, a);
    }
    return hipGetLastError();
}

// act[m][i] = fp16( silu_tanh(gate) * up ), gate/up interleaved in `gu` as (g0,u0,g1,u1,...)   (:6825-6827, :6337)
__global__ void swiglu_kernel(const float *gu, int hidden, uint16_t *act_f16) {
    const int m = blockIdx.y;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= hidden) return;
    const float g = gu[(size_t)m * 2 * hidden + 2 * i], u = gu[(size_t)m * 2 * hidden + 2 * i + 1];
    const float hg = __fmul_rn(0.5f, g);
    const float silu = __fmul_rn(hg, __fadd_rn(1.0f, tanhf(hg)));
    act_f16[(size_t)m * hidden + i] = to_half_bits(__fmul_rn(silu, u));
}

// First-max argmax of logits[m][0..vocab): lowest index wins ties (:8219-8275, neon_convert.c:36-101).
__global__ __launch_bounds__(kBlock) void argmax_kernel(const float *logits, int vocab, int *out_token, float *out_value) {
    __shared__ float bv[kBlock];
    __shared__ int bi[kBlock];
    const int m = blockIdx.x;
    const float *row = logits + (size_t)m * vocab;
    float best = -INFINITY;
    int best_i = 0x7FFFFFFF;
    for (int i = threadIdx.x; i < vocab; i += kBlock) {
        const float v = row[i];
        if (v > best) { best = v; best_i = i; }   // ascending i per thread: strict > keeps the first
    }
    bv[threadIdx.x] = best;
    bi[threadIdx.x] = best_i;
    __syncthreads();
    for (int s = kBlock / 2; s > 0; s >>= 1) {
        if (threadIdx.x < s) {
            const float ov = bv[threadIdx.x + s];
            const int oi = bi[threadIdx.x + s];
            if (ov > bv[threadIdx.x] || (ov == bv[threadIdx.x] && oi < bi[threadIdx.x])) { bv[threadIdx.x] = ov; bi[threadIdx.x] = oi; }
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        out_token[m] = bi[0] == 0x7FFFFFFF ? 0 : bi[0];
        if (out_value) out_value[m] = bv[0];
    }
}

__global__ void set_rows_kernel(StepRows rows, int *tokens, int *pos, int *seq) {
    const int i = threadIdx.x;
    if (i < rows.count) {
        tokens[i] = rows.token[i];
        pos[i] = rows.pos[i];
        seq[i] = rows.seq[i];
    }
}

// Device-side bookkeeping of one greedy step inside a captured graph: the token chosen by the head
// becomes row 0 of the next trunk pass at the sequence's visible position, is appended to the token
// log, and the visible length grows by one.
__global__ void greedy_feed_kernel(const int *next_token, int seq, int *visible, int *tokens, int *pos, int *seqs,
                                   int *log, int *log_count, int log_capacity) {
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    const int t = *next_token;
    tokens[0] = t;
    pos[0] = visible[seq];
    seqs[0] = seq;
    const int n = *log_count;
    if (n < log_capacity) log[n] = t;
    *log_count = n + 1;
    visible[seq] += 1;
}

__global__ void set_ints_kernel(int *dst0, int v0, int *dst1, int v1) {
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        if (dst0) *dst0 = v0;
        if (dst1) *dst1 = v1;
    }
}

// hidden[dst] = hidden[src] rows of d floats (keeps the last hidden state of a sequence)
__global__ void copy_rows_kernel(const float *src, float *dst, int d) {
    const int m = blockIdx.y;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < d; i += gridDim.x * blockDim.x) dst[(size_t)m * d + i] = src[(size_t)m * d + i];
}

}  // namespace

hipError_t launch_embed(const void *table, bool table_is_f16, const int *tokens, int rows, int d, float *hidden, hipStream_t s) {
    hipLaunchKernelGGL(embed_kernel, dim3((d + 255) / 256, rows), dim3(256), 0, s, table, table_is_f16 ? 1 : 0, tokens, d, hidden);
    return hipGetLastError();
}

hipError_t launch_rmsnorm(const float *x, const float *w, float eps, int rows, int d, uint16_t *out_f16,
                          unsigned long long *argmax_cells, hipStream_t s) {
    hipLaunchKernelGGL(rmsnorm_kernel, dim3(rows), dim3(kBlock), 0, s, x, w, eps, d, out_f16, argmax_cells);
    return hipGetLastError();
}

hipError_t launch_qkv_post(const QkvPostArgs &a, int rows, bool kv_f16, hipStream_t s) {
    const int half = a.head_dim / 2;
    if (half <= 0 || half > 1024 || a.head_dim % 2 != 0) return hipErrorInvalidValue;
    const int threads = (half + 63) / 64 * 64;  // whole wavefronts: the per-head norm reduces across them
    dim3 grid(a.n_head + 2 * a.n_kv_head, rows);
    if (kv_f16) hipLaunchKernelGGL(qkv_post_kernel<true>, grid, dim3(threads), 0, s, a);
    else hipLaunchKernelGGL(qkv_post_kernel<false>, grid, dim3(threads), 0, s, a);
    return hipGetLastError();
}

hipError_t launch_attention(const AttentionArgs &a, int rows, bool kv_f16, hipStream_t s) {
    // grouped-query kernel for the common head shapes; everything else takes the general kernel
    const int group = a.n_head / a.n_kv_head;
    const size_t fast_lds = ((size_t)group * a.max_seq + (size_t)16 * group * a.head_dim) * sizeof(float);
    if (a.n_head % a.n_kv_head == 0 && fast_lds <= 150 * 1024) {
        if (a.head_dim == 128) {
            if (group == 1) return launch_attention_gqa<128, 1>(a, rows, kv_f16, s);
            if (group == 2) return launch_attention_gqa<128, 2>(a, rows, kv_f16, s);
            if (group == 4) return launch_attention_gqa<128, 4>(a, rows, kv_f16, s);
        } else if (a.head_dim == 64) {
            if (group == 1) return launch_attention_gqa<64, 1>(a, rows, kv_f16, s);
            if (group == 2) return launch_attention_gqa<64, 2>(a, rows, kv_f16, s);
            if (group == 4) return launch_attention_gqa<64, 4>(a, rows, kv_f16, s);
        }
    }
    if (a.head_dim > kBlock && a.head_dim % kBlock != 0) return hipErrorInvalidValue;
    if (a.head_dim < kBlock && kBlock % a.head_dim != 0) return hipErrorInvalidValue;
    const size_t lds = ((size_t)a.head_dim + a.max_seq + kBlock) * sizeof(float);
    if (lds > 60 * 1024) return hipErrorInvalidValue;
    dim3 grid(a.n_head, rows);
    if (kv_f16) hipLaunchKernelGGL(attention_decode_kernel<true>, grid, dim3(kBlock), lds, s, a);
    else hipLaunchKernelGGL(attention_decode_kernel<false>, grid, dim3(kBlock), lds, s, a);
    return hipGetLastError();
}

hipError_t launch_swiglu(const float *gu, int rows, int hidden, uint16_t *act_f16, hipStream_t s) {
    hipLaunchKernelGGL(swiglu_kernel, dim3((hidden + 255) / 256, rows), dim3(256), 0, s, gu, hidden, act_f16);
    return hipGetLastError();
}

hipError_t launch_argmax(const float *logits, int rows, int vocab, int *out_token, float *out_value, hipStream_t s) {
    hipLaunchKernelGGL(argmax_kernel, dim3(rows), dim3(kBlock), 0, s, logits, vocab, out_token, out_value);
    return hipGetLastError();
}

hipError_t launch_set_rows(const StepRows &rows, int *tokens, int *pos, int *seq, hipStream_t s) {
    hipLaunchKernelGGL(set_rows_kernel, dim3(1), dim3(64), 0, s, rows, tokens, pos, seq);
    return hipGetLastError();
}

hipError_t launch_greedy_feed(const int *next_token, int seq, int *visible, int *tokens, int *pos, int *seqs, int *log,
                              int *log_count, int log_capacity, hipStream_t s) {
    hipLaunchKernelGGL(greedy_feed_kernel, dim3(1), dim3(64), 0, s, next_token, seq, visible, tokens, pos, seqs, log, log_count,
                       log_capacity);
    return hipGetLastError();
}

hipError_t launch_set_ints(int *dst0, int v0, int *dst1, int v1, hipStream_t s) {
    hipLaunchKernelGGL(set_ints_kernel, dim3(1), dim3(64), 0, s, dst0, v0, dst1, v1);
    return hipGetLastError();
}

hipError_t launch_copy_rows(const float *src, float *dst, int rows, int d, hipStream_t s) {
    hipLaunchKernelGGL(copy_rows_kernel, dim3((d + 255) / 256, rows), dim3(256), 0, s, src, dst, d);
    return hipGetLastError();
}

}  // namespace esp
