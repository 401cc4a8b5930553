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

// DPP row operations (no LDS traffic).  group_sum<N>: sum over aligned groups of N lanes (N = 8 or 16),
// result in every lane of the group.
template <int CTRL>
__device__ __forceinline__ float dpp_get(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xF, 0xF, false));
}
template <int N>
__device__ __forceinline__ float group_sum(float v) {
    v += dpp_get<0xB1>(v);                 // quad_perm [1,0,3,2]
    v += dpp_get<0x4E>(v);                 // quad_perm [2,3,0,1]
    v += dpp_get<0x141>(v);                // row_half_mirror
    if (N == 16) v += dpp_get<0x140>(v);   // row_mirror
    return v;
}
// maximum over the first lane of every group of N lanes, as a wave-uniform value
template <int N>
__device__ __forceinline__ float max_over_groups(float v) {
    float m = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));
#pragma unroll
    for (int l = N; l < 64; l += N) m = fmaxf(m, __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), l)));
    return m;
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
    auto value = [&](const float *p) {   // the GEMM's result, or the sum of its split-K partial sums in split order
        float s = p[0];
        for (int sp = 1; sp < a.splits; sp++) s += p[(size_t)sp * a.plane];
        return s;
    };
    if (slot < nh + nkv) {
        const bool is_q = slot < nh;
        const int h = is_q ? slot : slot - nh;
        const float *src = row + (is_q ? 0 : ad) + (size_t)h * a.head_dim;
        float v0 = live ? value(src + 2 * j) : 0.0f, v1 = live ? value(src + 2 * j + 1) : 0.0f;
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
            const float v = value(src + i);
            if (KV_F16) reinterpret_cast<uint16_t *>(a.v_cache)[c0 + i] = to_half_bits(v);
            else reinterpret_cast<float *>(a.v_cache)[c0 + i] = v;
        }
    }
}

// rmsnorm_kernel for a row whose values are still split-K partial sums of a GEMM: x = (residual +) partial[0] + partial[1]
// + ... in split order (the sum gemm_reduce_kernel forms), written to y, then normalised as above.  One workgroup per row,
// d a multiple of four and at most 8192.
__global__ __launch_bounds__(kBlock) void rmsnorm_reduce_kernel(const float *partial, int splits, size_t plane, const float *residual, float *y,
                                                                const float *w, float eps, int d, uint16_t *out_f16) {
    __shared__ float scratch[16];
    const int m = blockIdx.x;
    constexpr int kVec = 8;
    const int n4 = d / 4;
    const float4 *w4 = reinterpret_cast<const float4 *>(w);
    float4 v[kVec], g[kVec];
#pragma unroll
    for (int k = 0; k < kVec; k++) {
        const int i = threadIdx.x + k * kBlock;
        v[k] = make_float4(0.f, 0.f, 0.f, 0.f);
        g[k] = v[k];
        if (i < n4) {
            const size_t o = (size_t)m * n4 + i;
            float4 s = reinterpret_cast<const float4 *>(partial)[o];
            for (int sp = 1; sp < splits; sp++) {
                const float4 t = reinterpret_cast<const float4 *>(partial + (size_t)sp * plane)[o];
                s.x += t.x; s.y += t.y; s.z += t.z; s.w += t.w;
            }
            if (residual) {
                const float4 r = reinterpret_cast<const float4 *>(residual)[o];
                s.x = r.x + s.x; s.y = r.y + s.y; s.z = r.z + s.z; s.w = r.w + s.w;
            }
            reinterpret_cast<float4 *>(y)[o] = s;
            v[k] = s;
            g[k] = w4[i];
        }
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


// Single-query attention, grouped-query form with a one-pass ("online") softmax.
// grid (KV heads, rows, splits), 4 wavefronts per workgroup.  The G query heads that share a KV head
// are served together, so K and V are read once.  Both caches are token-major: a token's head
// vector is contiguous (HD fp16 = 256 bytes at HD 128).
//   * a wavefront owns chunks of 4 tokens, round-robin over all wavefronts of the KV head;
//     16 lanes per token, 8 dims per lane, the same lane mapping for K and V;
//   * per chunk: K and V rows are loaded first (one 128-bit load each for fp16 caches), the partial
//     dots are all-reduced over a token's 16 lanes, the running maximum m, the per-slot denominators
//     l and the value sums acc are updated (acc *= exp(m_old - m_new));
//   * the token slots and wavefronts of the workgroup are combined through LDS with the usual
//     (m, l, acc) merge; with more than one split the workgroup writes its partial state and
//     attention_merge_kernel combines the splits in split order.
template <int HD, int G, bool KV_F16>
__global__ __launch_bounds__(256) void attention_flash_kernel(AttentionArgs a) {
    constexpr int WAVES = 4, LPT = HD / 8, SLOTS = 64 / LPT;   // lanes per token, tokens per chunk
    constexpr int KW = KV_F16 ? 1 : 2;                         // 128-bit loads per 8 values
    __shared__ float wm[WAVES][G], wl[WAVES][SLOTS][G];
    __shared__ float wacc[WAVES][SLOTS][G][HD];
    const int kvh = blockIdx.x, m = blockIdx.y, split = blockIdx.z, splits = gridDim.z;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int visible = a.pos[m] + 1;
    const int kd = a.n_kv_head * HD;
    const size_t seq_base = (size_t)a.seq[m] * a.cache_seq_stride;
    const float scale = 1.0f / sqrtf((float)HD);
    const int slot = lane / LPT, seg = (lane % LPT) * 8;

    float q[G][8];
#pragma unroll
    for (int g = 0; g < G; g++) {
        const float4 *qp = reinterpret_cast<const float4 *>(a.q + (size_t)m * a.n_head * HD + (size_t)(kvh * G + g) * HD + seg);
        const float4 q0 = qp[0], q1 = qp[1];
        q[g][0] = q0.x; q[g][1] = q0.y; q[g][2] = q0.z; q[g][3] = q0.w;
        q[g][4] = q1.x; q[g][5] = q1.y; q[g][6] = q1.z; q[g][7] = q1.w;
    }
    float mx[G], l[G], acc[G][8];
#pragma unroll
    for (int g = 0; g < G; g++) {
        mx[g] = -INFINITY;
        l[g] = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; i++) acc[g][i] = 0.0f;
    }

    auto unpack8 = [](const uint4 *r, float *out) {
        if (KV_F16) {
            const uint32_t w[4] = {r[0].x, r[0].y, r[0].z, r[0].w};
#pragma unroll
            for (int i = 0; i < 4; i++) { out[2 * i] = from_half_bits((uint16_t)(w[i] & 0xFFFFu)); out[2 * i + 1] = from_half_bits((uint16_t)(w[i] >> 16)); }
        } else {
            out[0] = __uint_as_float(r[0].x); out[1] = __uint_as_float(r[0].y); out[2] = __uint_as_float(r[0].z); out[3] = __uint_as_float(r[0].w);
            out[4] = __uint_as_float(r[KW - 1].x); out[5] = __uint_as_float(r[KW - 1].y); out[6] = __uint_as_float(r[KW - 1].z); out[7] = __uint_as_float(r[KW - 1].w);
        }
    };

    constexpr int U = 2;   // chunks whose loads are in flight together
    const int stride = splits * WAVES * SLOTS;
    for (int t0 = (split * WAVES + wave) * SLOTS; t0 < visible; t0 += stride * U) {
        uint4 kr[U][KW], vr[U][KW];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int t = t0 + u * stride + slot;
            const size_t off = seq_base + (size_t)(t < visible ? t : 0) * kd + (size_t)kvh * HD + seg;
            const uint4 *kp = KV_F16 ? reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(a.k_cache) + off)
                                     : reinterpret_cast<const uint4 *>(reinterpret_cast<const float *>(a.k_cache) + off);
            const uint4 *vp = KV_F16 ? reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(a.v_cache) + off)
                                     : reinterpret_cast<const uint4 *>(reinterpret_cast<const float *>(a.v_cache) + off);
#pragma unroll
            for (int i = 0; i < KW; i++) { kr[u][i] = kp[i]; vr[u][i] = vp[i]; }
        }
        // every load above is issued before the first use below: one memory round trip for all U chunks
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int t = t0 + u * stride + slot;
            const bool valid = t < visible;
            if (t0 + u * stride >= visible) break;   // whole chunk beyond the prefix (uniform)
            float k[8], v[8];
            unpack8(kr[u], k);
            unpack8(vr[u], v);
#pragma unroll
            for (int g = 0; g < G; g++) {
                float d = 0.0f;
#pragma unroll
                for (int i = 0; i < 8; i++) d = __builtin_fmaf(q[g][i], k[i], d);
                d = group_sum<LPT>(d);                                  // all lanes of the token
                const float sc = valid ? __fmul_rn(d, scale) : -INFINITY;
                const float cm = max_over_groups<LPT>(sc);              // over the chunk's tokens
                const float m_new = fmaxf(mx[g], cm);      // finite: the chunk holds at least one visible token
                const float alpha = expf(mx[g] - m_new);   // exp(-inf) = 0 on the first chunk
                const float p = valid ? expf(sc - m_new) : 0.0f;
                l[g] = __builtin_fmaf(l[g], alpha, p);
#pragma unroll
                for (int i = 0; i < 8; i++) acc[g][i] = __builtin_fmaf(p, v[i], __fmul_rn(acc[g][i], alpha));
                mx[g] = m_new;
            }
        }
    }
    // ---- every (wavefront, token slot) publishes its partial state; m is the same in all lanes ----
#pragma unroll
    for (int g = 0; g < G; g++) {
#pragma unroll
        for (int i = 0; i < 8; i++) wacc[wave][slot][g][seg + i] = acc[g][i];
        if (lane % LPT == 0) wl[wave][slot][g] = l[g];
        if (lane == 0) wm[wave][g] = mx[g];
    }
    __syncthreads();
    // ---- merge over wavefronts and slots: thread (g, dim) ----
    float *scratch = a.split_scratch + (((size_t)m * a.n_kv_head + kvh) * splits) * G * (HD + 2);
    for (int i = tid; i < G * HD; i += 256) {
        const int g = i / HD, dch = i % HD;
        float M = wm[0][g];
#pragma unroll
        for (int w = 1; w < WAVES; w++) M = fmaxf(M, wm[w][g]);
        float L = 0.0f, A = 0.0f;
#pragma unroll
        for (int w = 0; w < WAVES; w++) {
            const float f = wm[w][g] == -INFINITY ? 0.0f : expf(wm[w][g] - M);
            float lw = 0.0f, aw = 0.0f;
#pragma unroll
            for (int sl = 0; sl < SLOTS; sl++) { lw += wl[w][sl][g]; aw += wacc[w][sl][g][dch]; }
            L = __builtin_fmaf(lw, f, L);
            A = __builtin_fmaf(aw, f, A);
        }
        if (splits == 1) {
            a.ctx_f16[(size_t)m * a.n_head * HD + (size_t)(kvh * G + g) * HD + dch] = to_half_bits(L > 0.0f ? A / L : 0.0f);
        } else {
            float *ps = scratch + ((size_t)split * G + g) * (HD + 2);
            ps[2 + dch] = A;
            if (dch == 0) { ps[0] = M; ps[1] = L; }
        }
    }
}

// Merges the per-split partial states (m, l, acc) of attention_flash_kernel in split order.
// grid (query heads, rows).  A kernel boundary, not a device-scope fence, orders it after the partial
// writes: fences plus arrival counters in every workgroup cost far more than this launch.
template <int HD, int G>
__global__ __launch_bounds__(HD) void attention_merge_kernel(AttentionArgs a, int splits) {
    // one workgroup per query head, one thread per channel
    const int head = blockIdx.x, m = blockIdx.y, kvh = head / G, g = head % G, dch = threadIdx.x;
    const float *scratch = a.split_scratch + (((size_t)m * a.n_kv_head + kvh) * splits) * G * (HD + 2);
    // all partials are fetched before the first is used (one memory round trip)
    float pm[kAttentionMaxSplits], pl[kAttentionMaxSplits], pa[kAttentionMaxSplits];
#pragma unroll
    for (int sp = 0; sp < kAttentionMaxSplits; sp++) {
        const float *ps = scratch + ((size_t)(sp < splits ? sp : 0) * G + g) * (HD + 2);
        pm[sp] = ps[0]; pl[sp] = ps[1]; pa[sp] = ps[2 + dch];
    }
    float M = -INFINITY;
#pragma unroll
    for (int sp = 0; sp < kAttentionMaxSplits; sp++) if (sp < splits) M = fmaxf(M, pm[sp]);
    float L = 0.0f, A = 0.0f;
#pragma unroll
    for (int sp = 0; sp < kAttentionMaxSplits; sp++) {
        const float f = (sp < splits && pm[sp] != -INFINITY) ? expf(pm[sp] - M) : 0.0f;
        L = __builtin_fmaf(pl[sp], f, L);
        A = __builtin_fmaf(pa[sp], f, A);
    }
    a.ctx_f16[(size_t)m * a.n_head * HD + (size_t)head * HD + dch] = to_half_bits(L > 0.0f ? A / L : 0.0f);
}

// Causal attention of a block of prompt rows on the matrix cores (v_mfma_f32_32x32x16_f16), for rows that are one
// sequence at consecutive positions (pos[m0 + i] = pos[m0] + i), which is what a prompt block is.  Replaces the per-row
// loop of the reference's attention (:6774-6823) over a block: the single-query kernels above read a row's whole prefix
// once per row, this one reads a key tile once per 32 rows.
// grid (KV heads, tiles of 32 rows, sets of G query heads); wavefront g of a workgroup serves query head kvh * group + G z + g,
// so G heads that share a KV head share the value tiles.  Per tile of 32 keys:
//   * S^T = K Q^T: keys are the A rows (a lane loads eight consecutive dims of its key straight from the cache, two
//     tiles ahead), queries the B columns (fragments kept in registers); a lane's 16 accumulators are
//     16 keys of ONE query, so the row maximum and sum of the online softmax are in-lane plus one exchange with lane ^ 32;
//   * O^T += V^T P: the probabilities a lane holds are already a B fragment (column = its query, k slots = its keys), and
//     the A operand is the value tile transposed in LDS (written once per workgroup, double-buffered: one barrier per tile),
//     read so that k slot (lane / 32, i) is key 16 j + 8 (i / 4) + 4 (lane / 32) + i % 4, the key of accumulator 8 j + i.
// Q, K, V and the probabilities enter the matrix cores as fp16, sums are fp32.
// SPLIT: queries and probabilities go in as hi / lo pairs (v = hi + lo / 2048: two MFMAs each against the same keys / values, which
// the fp16 cache holds exactly), and the context comes out as split rows for the GEMM that consumes it.
typedef _Float16 attn_half8 __attribute__((ext_vector_type(8)));
typedef _Float16 attn_half4 __attribute__((ext_vector_type(4)));
typedef float attn_floatx16 __attribute__((ext_vector_type(16)));

// KP = 2: the workgroup has two sets of G wavefronts; set p takes the key tiles p, p + 2, ... with value tiles of its own, and the two
// (maximum, sum, context) states of a head are merged through LDS at the end.  A workgroup's time is the length of its chain of key
// tiles (a tile of arithmetic is shorter than the trip to memory behind it), and the last row tile of a 512-row block has sixteen.
template <int HD, int G, bool KV_F16, bool SPLIT, int KP>
__global__ __launch_bounds__(G * KP * 64) void attention_prompt_kernel(AttentionArgs a, int rows) {
    constexpr int THREADS = G * 64, QT = 32, KS = HD / 16, MTILES = HD / 32, LDV = 32 + 8;   // THREADS: of one set; LDV: fp16 per row of V^T
    constexpr int VP = 32 * (HD / 8) / THREADS;                                            // 8-dim pieces of V per thread
    static_assert(VP >= 1 && 32 * (HD / 8) % THREADS == 0, "value tile divides over a set of wavefronts");
    static_assert(KP == 1 || KP == 2, "one or two sets");
    __shared__ _Float16 vt_all[KP][2][HD * LDV];
    const int kvh = blockIdx.x, m0 = blockIdx.y * QT;
    const int phase = KP == 1 ? 0 : (int)threadIdx.x / THREADS;
    const int tid = (int)threadIdx.x - phase * THREADS, lane = tid & 63, wave = tid >> 6, half = lane >> 5, col = lane & 31;
    _Float16 (*vt)[HD * LDV] = vt_all[phase];
    const int head = kvh * (a.n_head / a.n_kv_head) + (int)blockIdx.z * G + wave;   // grid z: sets of G query heads of the KV head
    const int pos0 = a.pos[m0];
    const int last_row = rows - 1 - m0 < QT - 1 ? rows - 1 - m0 : QT - 1;
    const int t_max = pos0 + last_row;             // last key any row of the tile sees
    const int kd = a.n_kv_head * HD;
    const size_t seq_base = (size_t)a.seq[m0] * a.cache_seq_stride;
    const float scale = 1.0f / sqrtf((float)HD);

    auto to_half8 = [](const float4 &x0, const float4 &x1) {
        return attn_half8{(_Float16)x0.x, (_Float16)x0.y, (_Float16)x0.z, (_Float16)x0.w, (_Float16)x1.x, (_Float16)x1.y, (_Float16)x1.z, (_Float16)x1.w};
    };
    // query fragments: column = query `col` (rows beyond the block repeat its last row, never stored), dims 16 ks + 8 half ..
    attn_half8 qf[KS], ql[SPLIT ? KS : 1];
    {
        const float *qp = a.q + (size_t)(m0 + (col <= last_row ? col : last_row)) * a.n_head * HD + (size_t)head * HD + 8 * half;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            const float4 x0 = *reinterpret_cast<const float4 *>(qp + 16 * ks), x1 = *reinterpret_cast<const float4 *>(qp + 16 * ks + 4);
            qf[ks] = to_half8(x0, x1);
            if constexpr (SPLIT) {
                const float v[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
#pragma unroll
                for (int e = 0; e < 8; e++) ql[ks][e] = (_Float16)__fmul_rn(__fsub_rn(v[e], (float)qf[ks][e]), 2048.0f);
            }
        }
    }
    // keys beyond t_max are clamped to it: in bounds, and masked below
    auto load_k = [&](int t0, attn_half8 (&kf)[KS]) {
        const int t = t0 + col < t_max ? t0 + col : t_max;
        const size_t off = seq_base + (size_t)t * kd + (size_t)kvh * HD + 8 * half;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            if (KV_F16) kf[ks] = *reinterpret_cast<const attn_half8 *>(reinterpret_cast<const uint16_t *>(a.k_cache) + off + 16 * ks);
            else {
                const float *kp = reinterpret_cast<const float *>(a.k_cache) + off + 16 * ks;
                kf[ks] = to_half8(*reinterpret_cast<const float4 *>(kp), *reinterpret_cast<const float4 *>(kp + 4));
            }
        }
    };
    // value tile: piece = (key, group of eight dims); consecutive lanes take consecutive keys so that the transposed
    // two-byte LDS writes of a wavefront spread over the banks
    auto load_v = [&](int t0, attn_half8 (&vreg)[VP]) {
#pragma unroll
        for (int i = 0; i < VP; i++) {
            const int piece = tid + i * THREADS, key = piece & 31, dg = piece >> 5;
            const int t = t0 + key < t_max ? t0 + key : t_max;
            const size_t off = seq_base + (size_t)t * kd + (size_t)kvh * HD + 8 * dg;
            if (KV_F16) vreg[i] = *reinterpret_cast<const attn_half8 *>(reinterpret_cast<const uint16_t *>(a.v_cache) + off);
            else {
                const float *vp = reinterpret_cast<const float *>(a.v_cache) + off;
                vreg[i] = to_half8(*reinterpret_cast<const float4 *>(vp), *reinterpret_cast<const float4 *>(vp + 4));
            }
        }
    };
    auto store_v = [&](int buf, const attn_half8 (&vreg)[VP]) {
#pragma unroll
        for (int i = 0; i < VP; i++) {
            const int piece = tid + i * THREADS, key = piece & 31, dg = piece >> 5;
#pragma unroll
            for (int e = 0; e < 8; e++) vt[buf][(8 * dg + e) * LDV + key] = vreg[i][e];
        }
    };

    attn_floatx16 o[MTILES], ol[SPLIT ? MTILES : 1];
#pragma unroll
    for (int mt = 0; mt < MTILES; mt++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[mt][r] = 0.0f;
#pragma unroll
    for (int mt = 0; mt < (SPLIT ? MTILES : 1); mt++)
#pragma unroll
        for (int r = 0; r < 16; r++) ol[mt][r] = 0.0f;
    float mx = -INFINITY, l = 0.0f;
    const int qpos = pos0 + col;

    // Keys and values are fetched two tiles ahead: one tile of arithmetic is shorter than a trip to memory.
    constexpr int STEP = 32 * KP;   // keys between a set's tiles
    attn_half8 kf[KS], k1[KS], k2[KS], v1[VP], v2[VP];
    load_k(32 * phase, kf);
    load_v(32 * phase, v1);
    store_v(0, v1);
    load_k(32 * phase + STEP, k1);      // tiles beyond t_max are clamped to it, in bounds and masked
    load_v(32 * phase + STEP, v1);
    __syncthreads();
    for (int base = 0, buf = 0; base <= t_max; base += STEP, buf ^= 1) {   // the same number of rounds for both sets
        const int t0 = base + 32 * phase;
        const bool more = base + STEP <= t_max;
        load_k(t0 + 2 * STEP, k2);
        load_v(t0 + 2 * STEP, v2);
        attn_floatx16 sc;
#pragma unroll
        for (int r = 0; r < 16; r++) sc[r] = 0.0f;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) sc = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[ks], qf[ks], sc, 0, 0, 0);
        if constexpr (SPLIT) {
            attn_floatx16 sl;
#pragma unroll
            for (int r = 0; r < 16; r++) sl[r] = 0.0f;
#pragma unroll
            for (int ks = 0; ks < KS; ks++) sl = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[ks], ql[ks], sl, 0, 0, 0);
#pragma unroll
            for (int r = 0; r < 16; r++) sc[r] = __builtin_fmaf(sl[r], 1.0f / 2048.0f, sc[r]);
        }
        // accumulator r: key t0 + 8 (r / 4) + 4 half + r % 4 against query `col`
        float tile_max = -INFINITY;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int key = t0 + 8 * (r >> 2) + 4 * half + (r & 3);
            sc[r] = key <= qpos ? __fmul_rn(sc[r], scale) : -INFINITY;
            tile_max = fmaxf(tile_max, sc[r]);
        }
        tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32));
        // finite from the first tile on in set 0 (key 0 is visible to every query); set 1 may see only masked keys for a while:
        // its state then stays (-inf, 0, 0) (exponents taken against 0 instead of -inf)
        const float m_new = fmaxf(mx, tile_max);
        const float m_ref = (KP > 1 && m_new == -INFINITY) ? 0.0f : m_new;
        const float alpha = __expf(mx - m_ref);      // exp(-inf) = 0 on the first tile
        float psum = 0.0f;
        _Float16 ph[16], pl[SPLIT ? 16 : 1];
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const float pr = __expf(sc[r] - m_ref);  // masked keys: exp(-inf) = 0
            psum += pr;
            ph[r] = (_Float16)pr;
            if constexpr (SPLIT) pl[r] = (_Float16)__fmul_rn(__fsub_rn(pr, (float)ph[r]), 2048.0f);
        }
        l = __builtin_fmaf(l, alpha, psum);
        mx = m_new;
        const attn_half8 pf[2] = {attn_half8{ph[0], ph[1], ph[2], ph[3], ph[4], ph[5], ph[6], ph[7]},
                                  attn_half8{ph[8], ph[9], ph[10], ph[11], ph[12], ph[13], ph[14], ph[15]}};
        attn_half8 pfl[2];
        if constexpr (SPLIT) {
#pragma unroll
            for (int e = 0; e < 8; e++) { pfl[0][e] = pl[e]; pfl[1][e] = pl[8 + e]; }
        }
#pragma unroll
        for (int mt = 0; mt < MTILES; mt++) {
#pragma unroll
            for (int r = 0; r < 16; r++) o[mt][r] *= alpha;
            if constexpr (SPLIT) {
#pragma unroll
                for (int r = 0; r < 16; r++) ol[mt][r] *= alpha;
            }
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const _Float16 *vrow = vt[buf] + (32 * mt + col) * LDV + 16 * j + 4 * half;
                const attn_half4 lo = *reinterpret_cast<const attn_half4 *>(vrow), hi = *reinterpret_cast<const attn_half4 *>(vrow + 8);
                const attn_half8 vf = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                o[mt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf, pf[j], o[mt], 0, 0, 0);
                if constexpr (SPLIT) ol[mt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf, pfl[j], ol[mt], 0, 0, 0);
            }
        }
        if (more) store_v(buf ^ 1, v1);
#pragma unroll
        for (int ks = 0; ks < KS; ks++) { kf[ks] = k1[ks]; k1[ks] = k2[ks]; }
#pragma unroll
        for (int i = 0; i < VP; i++) v1[i] = v2[i];
        __syncthreads();
    }
    if constexpr (KP == 2) {
        // set 1 hands (maximum, sum, context) to set 0 through the value tiles' LDS, 32 dims at a time: [wave][value][lane]
        float *mb = reinterpret_cast<float *>(&vt_all[0][0][0]);
        constexpr int kPerWave = (SPLIT ? 32 : 16) * 64, kStateBase = G * kPerWave;
        static_assert((size_t)(kStateBase + G * 2 * 64) * 4 <= sizeof(vt_all), "the merge fits the value tiles");
        float f0 = 1.0f, f1 = 0.0f;
        if (phase == 1) { mb[kStateBase + (wave * 2) * 64 + lane] = mx; mb[kStateBase + (wave * 2 + 1) * 64 + lane] = l; }
#pragma unroll
        for (int mt = 0; mt < MTILES; mt++) {
            if (phase == 1) {
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    mb[wave * kPerWave + r * 64 + lane] = o[mt][r];
                    if constexpr (SPLIT) mb[wave * kPerWave + (16 + r) * 64 + lane] = ol[mt][r];
                }
            }
            __syncthreads();
            if (phase == 0) {
                if (mt == 0) {
                    const float m1 = mb[kStateBase + (wave * 2) * 64 + lane], l1 = mb[kStateBase + (wave * 2 + 1) * 64 + lane];
                    const float m_all = fmaxf(mx, m1);   // finite: set 0 saw key 0
                    f0 = __expf(mx - m_all); f1 = __expf(m1 - m_all);
                    l = __builtin_fmaf(l, f0, __fmul_rn(l1, f1));
                }
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    o[mt][r] = __builtin_fmaf(o[mt][r], f0, __fmul_rn(mb[wave * kPerWave + r * 64 + lane], f1));
                    if constexpr (SPLIT) ol[mt][r] = __builtin_fmaf(ol[mt][r], f0, __fmul_rn(mb[wave * kPerWave + (16 + r) * 64 + lane], f1));
                }
            }
            __syncthreads();
        }
        if (phase == 1) return;
    }
    l += __shfl_xor(l, 32);
    if constexpr (SPLIT) {
        // context = (o + ol / 2048) / l as split rows; dims 32 mt .. 32 mt + 31 of a head are one sub-block of the row, half of it in
        // this lane and half in lane ^ 32
        const float inv = 1.0f / l;
        const size_t row = (size_t)(m0 + (col <= last_row ? col : last_row));
        const int ad = a.n_head * HD;
#pragma unroll
        for (int mt = 0; mt < MTILES; mt++) {
            float s = 0.0f;
#pragma unroll
            for (int q4 = 0; q4 < 4; q4++) {
                attn_half4 vh, vl;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const float v = __fmul_rn(__builtin_fmaf(ol[mt][4 * q4 + e], 1.0f / 2048.0f, o[mt][4 * q4 + e]), inv);
                    vh[e] = (_Float16)v;
                    vl[e] = (_Float16)__fmul_rn(__fsub_rn(v, (float)vh[e]), 2048.0f);
                    s += __builtin_fmaf((float)vl[e], 1.0f / 2048.0f, (float)vh[e]);
                }
                if (col <= last_row) {   // the planes' order inside fours: (0, 2, 1, 3)
                    const size_t o16 = row * ad + (size_t)head * HD + 32 * mt + 8 * q4 + 4 * half;
                    *reinterpret_cast<attn_half4 *>(a.ctx_hi + o16) = attn_half4{vh[0], vh[2], vh[1], vh[3]};
                    *reinterpret_cast<attn_half4 *>(a.ctx_lo + o16) = attn_half4{vl[0], vl[2], vl[1], vl[3]};
                }
            }
            s += __shfl_xor(s, 32);
            if (half == 0 && col <= last_row) {
                const int sub = head * (HD / 32) + mt;
                uint16_t *p = a.ctx_sums + (row * (size_t)(ad / 256) + (sub >> 3)) * 16 + (sub & 7);
                const _Float16 h = (_Float16)s;
                p[0] = __builtin_bit_cast(uint16_t, h);
                p[8] = __builtin_bit_cast(uint16_t, (_Float16)__fmul_rn(__fsub_rn(s, (float)h), 2048.0f));
            }
        }
        return;
    }
    if (col <= last_row) {
        const float inv = 1.0f / l;
        uint16_t *out = a.ctx_f16 + (size_t)(m0 + col) * a.n_head * HD + (size_t)head * HD;
#pragma unroll
        for (int mt = 0; mt < MTILES; mt++)
#pragma unroll
            for (int q4 = 0; q4 < 4; q4++) {
                const attn_half4 v = {(_Float16)(o[mt][4 * q4] * inv), (_Float16)(o[mt][4 * q4 + 1] * inv), (_Float16)(o[mt][4 * q4 + 2] * inv), (_Float16)(o[mt][4 * q4 + 3] * inv)};
                *reinterpret_cast<attn_half4 *>(out + 32 * mt + 8 * q4 + 4 * half) = v;
            }
    }
}

// Single-query attention whose merge is left to the consumer: grid (query heads, rows, kAttentionHeadSplits),
// WAVES wavefronts per workgroup, one query head each.  Chunks, lane mapping and the (m, l, acc) arithmetic are
// those of attention_flash_kernel; a wavefront keeps U chunks of loads in flight, so kAttentionHeadSplits *
// WAVES * U chunks of the prefix cost one memory round trip and longer prefixes loop.  The arithmetic per
// chunk is what a wavefront spends its time on, hence many wavefronts with few chunks each.  Every workgroup writes its
// state to `head_partials` as [row][head][split][HD values, m, l, 2 pad] (16-byte aligned rows); the GEMV
// that consumes the context merges the splits while it stages its input, so no merge launch follows.
// Workgroups x, x + kvHeads, ... serve the query heads of KV head x: with eight KV heads the group shares
// one L2, which then reads K and V from memory once.
template <int HD, bool KV_F16, int WAVES, int U>
__global__ __launch_bounds__(WAVES * 64) void attention_partial_kernel(const float *q_rows, const void *k_cache, const void *v_cache, const int *pos,
                                                                       const int *seq, float *head_partials, unsigned cache_seq_stride, unsigned heads) {
    // Fourteen 32-bit words of scalar arguments (heads = query heads | key/value heads << 16): all of them are
    // preloaded into registers with the wavefront's launch, so the first loads do not wait for an argument fetch
    // from memory, which the fields of a structure passed by value would need.
    AttentionArgs a = {};
    a.q = q_rows; a.k_cache = k_cache; a.v_cache = v_cache; a.pos = pos; a.seq = seq; a.head_partials = head_partials;
    a.cache_seq_stride = cache_seq_stride; a.n_head = (int)(heads & 0xFFFFu); a.n_kv_head = (int)(heads >> 16);
    constexpr int LPT = HD / 8, SLOTS = 64 / LPT, KW = KV_F16 ? 1 : 2, STRIDE = HD + 4;
    __shared__ float wm[WAVES], wl[WAVES];
    __shared__ float wacc[WAVES][HD];
    const int group = a.n_head / a.n_kv_head;
    const int kvh = blockIdx.x % a.n_kv_head, head = kvh * group + blockIdx.x / a.n_kv_head, m = blockIdx.y;
    const int split = blockIdx.z;
    constexpr int splits = kAttentionHeadSplits;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // both row descriptors are fetched in one round trip, before anything branches on the first
    const int row_pos = a.pos[m], row_seq = a.seq[m];
    asm volatile("" ::"s"(row_pos), "s"(row_seq));
    const int visible = row_pos + 1;
    const int kd = a.n_kv_head * HD;
    const size_t seq_base = (size_t)row_seq * a.cache_seq_stride;
    const float scale = 1.0f / sqrtf((float)HD);
    const int slot = lane / LPT, seg = (lane % LPT) * 8;

    float q[8];
    {
        const float4 *qp = reinterpret_cast<const float4 *>(a.q + (size_t)m * a.n_head * HD + (size_t)head * HD + seg);
        const float4 q0 = qp[0], q1 = qp[1];
        q[0] = q0.x; q[1] = q0.y; q[2] = q0.z; q[3] = q0.w;
        q[4] = q1.x; q[5] = q1.y; q[6] = q1.z; q[7] = q1.w;
    }
    float mx = -INFINITY, l = 0.0f, acc[8];
#pragma unroll
    for (int i = 0; i < 8; i++) acc[i] = 0.0f;

    auto unpack8 = [](const uint4 *r, float *out) {
        if (KV_F16) {
            const uint32_t w[4] = {r[0].x, r[0].y, r[0].z, r[0].w};
#pragma unroll
            for (int i = 0; i < 4; i++) { out[2 * i] = from_half_bits((uint16_t)(w[i] & 0xFFFFu)); out[2 * i + 1] = from_half_bits((uint16_t)(w[i] >> 16)); }
        } else {
            out[0] = __uint_as_float(r[0].x); out[1] = __uint_as_float(r[0].y); out[2] = __uint_as_float(r[0].z); out[3] = __uint_as_float(r[0].w);
            out[4] = __uint_as_float(r[KW - 1].x); out[5] = __uint_as_float(r[KW - 1].y); out[6] = __uint_as_float(r[KW - 1].z); out[7] = __uint_as_float(r[KW - 1].w);
        }
    };

    const int stride = splits * WAVES * SLOTS;
    for (int t0 = (split * WAVES + wave) * SLOTS; t0 < visible; t0 += stride * U) {
        uint4 kr[U][KW], vr[U][KW];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int t = t0 + u * stride + slot;
            const size_t off = seq_base + (size_t)(t < visible ? t : 0) * kd + (size_t)kvh * HD + seg;
            const uint4 *kp = KV_F16 ? reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(a.k_cache) + off)
                                     : reinterpret_cast<const uint4 *>(reinterpret_cast<const float *>(a.k_cache) + off);
            const uint4 *vp = KV_F16 ? reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(a.v_cache) + off)
                                     : reinterpret_cast<const uint4 *>(reinterpret_cast<const float *>(a.v_cache) + off);
#pragma unroll
            for (int i = 0; i < KW; i++) { kr[u][i] = kp[i]; vr[u][i] = vp[i]; }
        }
        // every load above is issued before the first use below: one memory round trip for all U chunks
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int t = t0 + u * stride + slot;
            const bool valid = t < visible;
            // a chunk wholly beyond the prefix changes nothing (alpha = 1, p = 0): no branch, so the loop unrolls and
            // all U chunks stay in registers
            float k[8], v[8];
            unpack8(kr[u], k);
            unpack8(vr[u], v);
            float d = 0.0f;
#pragma unroll
            for (int i = 0; i < 8; i++) d = __builtin_fmaf(q[i], k[i], d);
            d = group_sum<LPT>(d);                                  // all lanes of the token
            const float sc = valid ? __fmul_rn(d, scale) : -INFINITY;
            const float cm = max_over_groups<LPT>(sc);              // over the chunk's tokens
            const float m_new = fmaxf(mx, cm);         // finite: the chunk holds at least one visible token
            const float alpha = expf(mx - m_new);      // exp(-inf) = 0 on the first chunk
            const float p = valid ? expf(sc - m_new) : 0.0f;
            l = __builtin_fmaf(l, alpha, p);
#pragma unroll
            for (int i = 0; i < 8; i++) acc[i] = __builtin_fmaf(p, v[i], __fmul_rn(acc[i], alpha));
            mx = m_new;
        }
    }
    // ---- the wavefront's token slots share one m: their sums and accumulators add up across the lanes that differ in the slot
    // index only, and the wavefront publishes one state ----
#pragma unroll
    for (int off = LPT; off < 64; off <<= 1) {
        l += __shfl_xor(l, off);
#pragma unroll
        for (int i = 0; i < 8; i++) acc[i] += __shfl_xor(acc[i], off);
    }
    if (slot == 0) {
#pragma unroll
        for (int i = 0; i < 8; i++) wacc[wave][seg + i] = acc[i];
    }
    if (lane == 0) { wl[wave] = l; wm[wave] = mx; }
    __syncthreads();
    // ---- merge over wavefronts in wavefront order: thread = channel ----
    float *ps = a.head_partials + (((size_t)m * a.n_head + head) * splits + split) * STRIDE;
    for (int dch = tid; dch < HD; dch += WAVES * 64) {
        float M = wm[0];
#pragma unroll
        for (int w = 1; w < WAVES; w++) M = fmaxf(M, wm[w]);
        float L = 0.0f, A = 0.0f;
#pragma unroll
        for (int w = 0; w < WAVES; w++) {
            const float f = wm[w] == -INFINITY ? 0.0f : expf(wm[w] - M);
            L = __builtin_fmaf(wl[w], f, L);
            A = __builtin_fmaf(wacc[w][dch], f, A);
        }
        ps[dch] = A;
        if (dch == 0) { ps[HD] = M; ps[HD + 1] = L; }
    }
}

template <int HD, int G>
hipError_t launch_attention_gqa(const AttentionArgs &a, int rows, bool kv_f16, hipStream_t s) {
    // enough workgroups to spread a long prefix over the chip; fixed per runtime so that a captured
    // graph stays valid as the prefix grows
    // each wavefront keeps two chunks of loads in flight: with max_seq / (2 chunks * 4 wavefronts * tokens per
    // chunk) splits, a prefix of any length up to max_seq costs every wavefront one memory round trip
    int splits = attention_split_count(a.max_seq, HD);
    // blocks of prompt rows already fill the chip: fewer slices per row, down to one (no merge launch)
    while (splits > 1 && (long)rows * a.n_kv_head * (splits / 2) >= 2048) splits /= 2;
    if (!a.split_scratch) splits = 1;
    dim3 grid(a.n_kv_head, rows, splits);
    if (kv_f16) hipLaunchKernelGGL((attention_flash_kernel<HD, G, true>), grid, dim3(256), 0, s, a);
    else hipLaunchKernelGGL((attention_flash_kernel<HD, G, false>), grid, dim3(256), 0, s, a);
    if (splits > 1) hipLaunchKernelGGL((attention_merge_kernel<HD, G>), dim3(a.n_head, rows), dim3(HD), 0, s, a, splits);
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
// Two launches: argmax_partial_kernel, grid (slices, rows), scans one slice per workgroup and writes
// (value, index); argmax_final_kernel, grid (rows), reduces the slices in slice order.
constexpr int kArgmaxBlocks = 128;

__device__ __forceinline__ bool better(float v, int i, float bv, int bi) { return v > bv || (v == bv && i < bi); }

__device__ __forceinline__ void argmax_block_reduce(float &best, int &best_i, float *bv, int *bi) {
    bv[threadIdx.x] = best;
    bi[threadIdx.x] = best_i;
    __syncthreads();
    for (int s = kBlock / 2; s > 0; s >>= 1) {
        if (threadIdx.x < s && better(bv[threadIdx.x + s], bi[threadIdx.x + s], bv[threadIdx.x], bi[threadIdx.x])) {
            bv[threadIdx.x] = bv[threadIdx.x + s];
            bi[threadIdx.x] = bi[threadIdx.x + s];
        }
        __syncthreads();
    }
    best = bv[0];
    best_i = bi[0];
}

__global__ __launch_bounds__(kBlock) void argmax_partial_kernel(const float *logits, int vocab, float *part_value, int *part_index) {
    __shared__ float bv[kBlock];
    __shared__ int bi[kBlock];
    const int m = blockIdx.y, blk = blockIdx.x, nblk = gridDim.x;
    const float *row = logits + (size_t)m * vocab;
    const int per = (vocab + nblk - 1) / nblk;
    const int lo = blk * per, hi = lo + per < vocab ? lo + per : vocab;
    float best = -INFINITY;
    int best_i = 0x7FFFFFFF;
    for (int i = lo + threadIdx.x; i < hi; i += kBlock) {
        const float v = row[i];
        if (v > best) { best = v; best_i = i; }   // ascending i per thread: strict > keeps the first
    }
    argmax_block_reduce(best, best_i, bv, bi);
    if (threadIdx.x == 0) {
        part_value[(size_t)m * nblk + blk] = best;
        part_index[(size_t)m * nblk + blk] = best_i;
    }
}

__global__ __launch_bounds__(kBlock) void argmax_final_kernel(const float *part_value, const int *part_index, int nblk,
                                                              int *out_token, float *out_value) {
    __shared__ float bv[kBlock];
    __shared__ int bi[kBlock];
    const int m = blockIdx.x;
    float best = -INFINITY;
    int best_i = 0x7FFFFFFF;
    for (int i0 = threadIdx.x; i0 < nblk; i0 += 4 * kBlock) {   // four candidates per thread in flight; past the end the first again
        float v[4];
        int idx[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int i = i0 + u * kBlock, j = i < nblk ? i : i0;
            v[u] = part_value[(size_t)m * nblk + j];
            idx[u] = part_index[(size_t)m * nblk + j];
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < 4; u++)
            if (better(v[u], idx[u], best, best_i)) { best = v[u]; best_i = idx[u]; }
    }
    argmax_block_reduce(best, best_i, bv, bi);
    if (threadIdx.x == 0) {
        out_token[m] = best_i == 0x7FFFFFFF ? 0 : best_i;
        if (out_value) out_value[m] = best;
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

// One embedding row into `hidden` (d floats), by a whole workgroup of `threads` threads: up to four loads per thread are in flight
// before the first store (a load after a store through an unrelated pointer would have to wait for it), eight values per load
// where the row allows.
__device__ __forceinline__ void embed_row(const void *table, int table_is_f16, int token, int d, float *hidden, int threads) {
    if (table_is_f16 && d % 8 == 0) {
        const uint4 *src = reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(table) + (size_t)token * d);
        const int groups = d / 8;
        for (int g0 = threadIdx.x; g0 < groups; g0 += 4 * threads) {
            uint4 v[4];
#pragma unroll
            for (int u = 0; u < 4; u++) v[u] = src[g0 + u * threads < groups ? g0 + u * threads : g0];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                if (g0 + u * threads >= groups) break;
                const uint32_t w[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
                float4 lo, hi;
                lo.x = from_half_bits((uint16_t)(w[0] & 0xFFFFu)); lo.y = from_half_bits((uint16_t)(w[0] >> 16));
                lo.z = from_half_bits((uint16_t)(w[1] & 0xFFFFu)); lo.w = from_half_bits((uint16_t)(w[1] >> 16));
                hi.x = from_half_bits((uint16_t)(w[2] & 0xFFFFu)); hi.y = from_half_bits((uint16_t)(w[2] >> 16));
                hi.z = from_half_bits((uint16_t)(w[3] & 0xFFFFu)); hi.w = from_half_bits((uint16_t)(w[3] >> 16));
                float4 *dst = reinterpret_cast<float4 *>(hidden + (size_t)(g0 + u * threads) * 8);
                dst[0] = lo;
                dst[1] = hi;
            }
        }
        return;
    }
    const size_t row = (size_t)token * d;
    for (int i0 = threadIdx.x; i0 < d; i0 += 4 * threads) {
        float v[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int i = i0 + u * threads < d ? i0 + u * threads : i0;
            v[u] = table_is_f16 ? from_half_bits(reinterpret_cast<const uint16_t *>(table)[row + i]) : reinterpret_cast<const float *>(table)[row + i];
        }
#pragma unroll
        for (int u = 0; u < 4; u++)
            if (i0 + u * threads < d) hidden[i0 + u * threads] = v[u];
    }
}

// The end of a greedy step in one launch: reduce the argmax slices of row 0 (argmax_final_kernel), feed the token
// (greedy_feed_kernel) and fetch its embedding row as the next trunk pass's input (embed_kernel).
struct GreedyTailArgs {
    const float *part_value;
    const int *part_index;
    int nblk;
    int *out_token;
    int seq;
    int *visible, *tokens, *pos, *seqs, *log, *log_count;   // log_count: [tokens logged, stopped, stop at the stop token (set by the host)]
    int log_capacity;
    const void *table;
    int table_is_f16, d;
    float *hidden;
    int eos;
};
__global__ __launch_bounds__(kBlock) void greedy_tail_kernel(GreedyTailArgs a) {
    __shared__ float bv[kBlock];
    __shared__ int bi[kBlock];
    // The loop state the bookkeeping below branches on is requested first, all of it at once: read where it is needed, its five
    // words would be a chain of trips to memory behind the reduction (every replay finds them written by the replay before).
    // (Through pointers the compiler must keep in vector registers: vector loads share a counter with the candidates' loads below and
    // are in flight together with them, scalar loads would be waited for together with the kernel's arguments, before anything else.)
    typedef const __attribute__((address_space(1))) int *global_ints;   // global, not generic: generic loads count as LDS traffic too
    global_ints state = (global_ints)a.log_count, fed = (global_ints)a.tokens, vis = (global_ints)(a.visible + a.seq);
    asm volatile("" : "+v"(state), "+v"(fed), "+v"(vis));
    int logged = state[0], stopped = state[1], stop_armed = state[2];
    int fed_before = fed[0], visible_before = vis[0];
    float best = -INFINITY;
    int best_i = 0x7FFFFFFF;
    auto take_four = [&](int i0) {   // four candidates per thread in flight; past the end candidate 0 again, which changes nothing
        float v[4];
        int idx[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int i = i0 + u * kBlock, j = i < a.nblk ? i : 0;
            v[u] = a.part_value[j];
            idx[u] = a.part_index[j];
        }
        __builtin_amdgcn_sched_barrier(0);   // every load is issued before the first comparison waits for one
#pragma unroll
        for (int u = 0; u < 4; u++)
            if (better(v[u], idx[u], best, best_i)) { best = v[u]; best_i = idx[u]; }
    };
    take_four(threadIdx.x);   // outside the loop: a loop's entry would wait for the state loads above
    for (int i0 = threadIdx.x + 4 * kBlock; i0 < a.nblk; i0 += 4 * kBlock) take_four(i0);
    asm volatile("" : "+v"(logged), "+v"(stopped), "+v"(stop_armed), "+v"(fed_before), "+v"(visible_before));   // here at the latest
    argmax_block_reduce(best, best_i, bv, bi);
    int t = best_i == 0x7FFFFFFF ? 0 : best_i;
    __shared__ int feed;   // the token whose embedding the trunk after this kernel runs on
    if (threadIdx.x == 0) {
        if (stopped) {
            // stopped in an earlier replay: nothing is emitted, and the trunk recomputes the row it computed last (same token, same
            // position, same values), so replays past the stop change nothing
            feed = fed_before;
        } else {
            a.out_token[0] = t;
            if (logged < a.log_capacity) a.log[logged] = t;
            a.log_count[0] = logged + 1;
            if (a.eos >= 0 && stop_armed && t == a.eos) {   // the stop token is emitted, not consumed (:6385-6388)
                a.log_count[1] = 1;
                feed = fed_before;
            } else {
                a.tokens[0] = t;
                a.pos[0] = visible_before;
                a.seqs[0] = a.seq;
                a.visible[a.seq] = visible_before + 1;
                feed = t;
            }
        }
    }
    __syncthreads();
    embed_row(a.table, a.table_is_f16, feed, a.d, a.hidden, kBlock);
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

// Rows 0 and 1 of `hidden` = embedding rows of the two tokens (every thread of a 256-thread workgroup calls this).
__device__ __forceinline__ void embed_two_rows(const EmbedTarget &e, int t0, int t1) {
    if (e.keep_row1) {
        for (int i = threadIdx.x; i < e.d; i += 256) e.keep_row1[i] = e.hidden[e.d + i];
        __syncthreads();   // row 1 is read by other threads than those that overwrite it below
    }
    embed_row(e.table, e.table_is_f16, t0, e.d, e.hidden, 256);
    embed_row(e.table, e.table_is_f16, t1, e.d, e.hidden + e.d, 256);
}

// Thread 0: see launch_two_token_verify_rows; then the workgroup embeds the target's two rows.
__global__ __launch_bounds__(256) void two_token_verify_rows_kernel(TwoTokenState *st, const int *draft_head, int *tokens, int *pos, EmbedTarget embed) {
    __shared__ int row_token[2];
    if (threadIdx.x == 0) {
        if (!st->done) {
            // row 0 of the draft's step was the row it owed after an accepted pass: its successor is the reference's second
            // comparison of that pass (:6156-6163)
            if (st->accepted_prev && st->reference_accounting && draft_head[0] == st->exact1_prev) st->reference_accepted_total += 1;
            const int proposed = draft_head[1];
            st->proposed = proposed;
            tokens[0] = st->current; pos[0] = st->full_pos;
            tokens[1] = proposed;    pos[1] = st->full_pos + 1;
        }
        // after the end the rows stay what they were: the trunk then recomputes what it computed last
        row_token[0] = tokens[0]; row_token[1] = tokens[1];
    }
    if (!embed.hidden) return;
    __syncthreads();
    embed_two_rows(embed, row_token[0], row_token[1]);
}

// Thread 0 runs one iteration of the reference loop's bookkeeping (:6109-6186), then the workgroup keeps the hidden row.
__global__ __launch_bounds__(256) void two_token_accept_kernel(TwoTokenState *st, const int *head, int *log, int log_capacity, const float *hidden_rows,
                                                                float *last_hidden, int d, int *draft_tokens, int *draft_pos, EmbedTarget draft_embed) {
    __shared__ int keep;
    __shared__ int draft_row_token[2];
    if (threadIdx.x == 0) {
        keep = -1;
        if (!st->done) {
            const int e0 = head[0], e1 = head[1], proposed = st->proposed;
            st->passes += 1;
            if (st->emitted < log_capacity) log[st->emitted] = e0;
            st->emitted += 1; st->all += 1; st->committed_total += 1;
            if (st->reference_accounting && proposed == e0) st->reference_accepted_total += 1;
            const bool stop0 = (st->eos >= 0 && e0 == st->eos) || st->emitted >= st->budget || st->all >= st->max_seq;
            if (stop0 || proposed != e0) {
                st->full_pos += 1; st->current = e0; st->accepted_prev = 0;
                keep = 0;
                if (stop0) { st->done = 1; st->stopped = 1; }
            } else {
                // the proposal was right: row 1 ran on the exact token, its column and its successor stand
                st->accepted_total += 1; st->committed_total += 1;
                st->full_pos += 2;
                keep = 1;
                if (st->emitted < log_capacity) log[st->emitted] = e1;
                st->emitted += 1; st->all += 1; st->current = e1;
                st->accepted_prev = 1; st->proposed_prev = proposed; st->exact1_prev = e1;
                if (st->eos >= 0 && e1 == st->eos) { st->done = 1; st->stopped = 1; }
            }
            // the next pass runs here only if it is a full one: two tokens of budget and two positions of context left
            if (!st->done && (st->budget - st->emitted < 2 || st->all + 1 >= st->max_seq || st->emitted >= st->budget || st->all >= st->max_seq)) st->done = 1;
            if (!st->done) {
                if (st->accepted_prev) {
                    draft_tokens[0] = st->proposed_prev; draft_pos[0] = st->full_pos - 1;
                    draft_tokens[1] = st->current;       draft_pos[1] = st->full_pos;
                } else {   // nothing owed: both rows are the same row, which writes the same cache column twice
                    draft_tokens[0] = draft_tokens[1] = st->current;
                    draft_pos[0] = draft_pos[1] = st->full_pos;
                }
            }
        }
        draft_row_token[0] = draft_tokens[0]; draft_row_token[1] = draft_tokens[1];   // changed or not: what the draft's next step runs on
    }
    __syncthreads();
    if (keep >= 0)
        for (int i = threadIdx.x; i < d; i += 256) last_hidden[i] = hidden_rows[(size_t)keep * d + i];
    if (draft_embed.hidden) embed_two_rows(draft_embed, draft_row_token[0], draft_row_token[1]);
}

// One thread per sequence: see launch_two_token_batch_verify_rows.
__global__ void two_token_batch_verify_rows_kernel(TwoTokenBatchState *st, const int *draft_head, int *tokens, int *pos) {
    const int s = threadIdx.x;
    if (s >= st->n_seq) return;
    const bool live = st->emitted[s] < st->budget;
    st->live[s] = live ? 1 : 0;
    if (!live) return;                       // finished: its rows stay what they were, the pass recomputes the same values
    const int proposed = draft_head[2 * s + 1];
    const bool can_two = st->budget - st->emitted[s] >= 2;
    st->proposed[s] = proposed;
    st->can_two[s] = can_two ? 1 : 0;
    tokens[2 * s] = st->current[s];                            pos[2 * s] = st->full_pos[s];
    tokens[2 * s + 1] = can_two ? proposed : st->current[s];   pos[2 * s + 1] = st->full_pos[s] + (can_two ? 1 : 0);
}

// One workgroup per sequence: thread 0 runs the sequence's bookkeeping, then the workgroup keeps its hidden row.
__global__ __launch_bounds__(256) void two_token_batch_accept_kernel(TwoTokenBatchState *st, const int *head, int *log, const float *hidden_rows,
                                                                      float *last_hidden, int d, int *draft_tokens, int *draft_pos) {
    __shared__ int keep;
    const int s = blockIdx.x;
    if (threadIdx.x == 0) {
        keep = -1;
        if (s == 0) {
            int any = 0;
            for (int i = 0; i < st->n_seq; i++) any |= st->live[i];
            if (any) st->passes += 1;
        }
        if (st->live[s]) {
            const int e0 = head[2 * s], e1 = head[2 * s + 1], proposed = st->proposed[s];
            int *out = log + (size_t)s * st->budget;
            out[st->emitted[s]] = e0;
            st->emitted[s] += 1; st->committed[s] += 1;
            if (!(st->can_two[s] && proposed == e0)) {
                st->full_pos[s] += 1; st->current[s] = e0; st->accepted_prev[s] = 0;
                keep = 2 * s;
            } else {
                st->accepted[s] += 1; st->committed[s] += 1;
                st->full_pos[s] += 2;
                out[st->emitted[s]] = e1;
                st->emitted[s] += 1; st->current[s] = e1;
                st->accepted_prev[s] = 1; st->proposed_prev[s] = proposed;
                keep = 2 * s + 1;
            }
            if (st->emitted[s] < st->budget) {   // the draft's rows of the next pass
                if (st->accepted_prev[s]) {
                    draft_tokens[2 * s] = st->proposed_prev[s]; draft_pos[2 * s] = st->full_pos[s] - 1;
                    draft_tokens[2 * s + 1] = st->current[s];   draft_pos[2 * s + 1] = st->full_pos[s];
                } else {
                    draft_tokens[2 * s] = draft_tokens[2 * s + 1] = st->current[s];
                    draft_pos[2 * s] = draft_pos[2 * s + 1] = st->full_pos[s];
                }
            }
        }
    }
    __syncthreads();
    if (keep >= 0)
        for (int i = threadIdx.x; i < d; i += 256) last_hidden[(size_t)s * d + i] = hidden_rows[(size_t)keep * d + i];
}

__global__ void batch_greedy_feed_kernel(const int *head_tokens, int n, int *tokens, int *pos, int *log, int *step, int capacity_steps) {
    const int s = threadIdx.x, at = *step;
    __syncthreads();
    if (s < n) {
        const int t = head_tokens[s];
        tokens[s] = t;
        pos[s] += 1;
        if (at < capacity_steps) log[(size_t)at * n + s] = t;
    }
    if (s == 0) *step = at + 1;
}

}  // namespace

hipError_t launch_two_token_batch_verify_rows(TwoTokenBatchState *state, const int *draft_head_tokens, int *target_tokens, int *target_pos, hipStream_t s) {
    hipLaunchKernelGGL(two_token_batch_verify_rows_kernel, dim3(1), dim3(64), 0, s, state, draft_head_tokens, target_tokens, target_pos);
    return hipGetLastError();
}

hipError_t launch_two_token_batch_accept(TwoTokenBatchState *state, int n_seq, const int *target_head_tokens, int *log, const float *hidden_rows,
                                         float *last_hidden, int d, int *draft_tokens, int *draft_pos, hipStream_t s) {
    if (n_seq < 1 || n_seq > kMaxLoopSequences) return hipErrorInvalidValue;
    hipLaunchKernelGGL(two_token_batch_accept_kernel, dim3(n_seq), dim3(256), 0, s, state, target_head_tokens, log, hidden_rows, last_hidden, d,
                       draft_tokens, draft_pos);
    return hipGetLastError();
}

hipError_t launch_batch_greedy_feed(const int *head_tokens, int n, int *tokens, int *pos, int *log, int *step, int capacity_steps, hipStream_t s) {
    if (n < 1 || n > kMaxStepRows) return hipErrorInvalidValue;
    hipLaunchKernelGGL(batch_greedy_feed_kernel, dim3(1), dim3(64), 0, s, head_tokens, n, tokens, pos, log, step, capacity_steps);
    return hipGetLastError();
}

hipError_t launch_two_token_verify_rows(TwoTokenState *state, const int *draft_head_tokens, int *target_tokens, int *target_pos, const EmbedTarget &embed,
                                        hipStream_t s) {
    hipLaunchKernelGGL(two_token_verify_rows_kernel, dim3(1), dim3(256), 0, s, state, draft_head_tokens, target_tokens, target_pos, embed);
    return hipGetLastError();
}

hipError_t launch_two_token_accept(TwoTokenState *state, const int *target_head_tokens, int *log, int log_capacity, const float *hidden_rows,
                                   float *last_hidden, int d, int *draft_tokens, int *draft_pos, const EmbedTarget &draft_embed, hipStream_t s) {
    hipLaunchKernelGGL(two_token_accept_kernel, dim3(1), dim3(256), 0, s, state, target_head_tokens, log, log_capacity, hidden_rows, last_hidden, d,
                       draft_tokens, draft_pos, draft_embed);
    return hipGetLastError();
}

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

int attention_split_count(int max_seq, int head_dim) {
    const int tokens_per_wg = 2 * 4 * (64 / (head_dim / 8));
    int splits = (max_seq + tokens_per_wg - 1) / tokens_per_wg;
    return splits < 1 ? 1 : (splits > kAttentionMaxSplits ? kAttentionMaxSplits : splits);
}

hipError_t launch_attention(const AttentionArgs &a, int rows, bool kv_f16, hipStream_t s) {
    // grouped-query kernel for the common head shapes; everything else takes the general kernel
    const int group = a.n_head / a.n_kv_head;
    if (a.n_head % a.n_kv_head == 0) {
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

bool attention_prompt_supported(int n_head, int n_kv_head, int head_dim) {
    if (n_kv_head <= 0 || n_head % n_kv_head != 0) return false;
    const int group = n_head / n_kv_head;
    return (head_dim == 128 || head_dim == 64) && (group == 1 || group == 2 || group == 4);
}

template <int HD, int G>
hipError_t launch_attention_prompt_shape(const AttentionArgs &a, int rows, bool kv_f16, int key_sets, hipStream_t s) {
    dim3 grid(a.n_kv_head, (rows + 31) / 32);
    // Two sets of wavefronts per workgroup (alternate key tiles) for 128-dim heads: the workgroup keeps its size (the kernel needs more
    // than 256 registers, one wavefront per SIMD), so half of the KV head's query heads go to a second workgroup (grid z).
    constexpr bool kTwoSets = HD == 128;
    constexpr int GS = G >= 2 ? G / 2 : 1;
    dim3 grid2(a.n_kv_head, (rows + 31) / 32, G / GS);
    if (a.ctx_hi) {   // split rows out: fp16 caches only (they hold keys and values exactly)
        if (!kv_f16 || !a.ctx_lo || !a.ctx_sums || (a.n_head * HD) % 256 != 0) return hipErrorInvalidValue;
        if constexpr (kTwoSets) {
            if (key_sets == 2) {
                hipLaunchKernelGGL((attention_prompt_kernel<HD, GS, true, true, 2>), grid2, dim3(GS * 128), 0, s, a, rows);
                return hipGetLastError();
            }
        }
        hipLaunchKernelGGL((attention_prompt_kernel<HD, G, true, true, 1>), grid, dim3(G * 64), 0, s, a, rows);
        return hipGetLastError();
    }
    if constexpr (kTwoSets) {
        if (key_sets == 2 && kv_f16) {
            hipLaunchKernelGGL((attention_prompt_kernel<HD, GS, true, false, 2>), grid2, dim3(GS * 128), 0, s, a, rows);
            return hipGetLastError();
        }
    }
    if (kv_f16) hipLaunchKernelGGL((attention_prompt_kernel<HD, G, true, false, 1>), grid, dim3(G * 64), 0, s, a, rows);
    else hipLaunchKernelGGL((attention_prompt_kernel<HD, G, false, false, 1>), grid, dim3(G * 64), 0, s, a, rows);
    return hipGetLastError();
}

// 0 (default): two sets of wavefronts for blocks of more than 64 rows; 1 / 2: always that many (tests, measurements)
static int g_prompt_attention_key_sets = 0;
void attention_prompt_set_key_sets(int sets) { g_prompt_attention_key_sets = sets == 1 || sets == 2 ? sets : 0; }

hipError_t launch_attention_prompt(const AttentionArgs &a, int rows, bool kv_f16, hipStream_t s) {
    if (rows <= 0 || !attention_prompt_supported(a.n_head, a.n_kv_head, a.head_dim)) return hipErrorInvalidValue;
    const int group = a.n_head / a.n_kv_head;
    const int sets = g_prompt_attention_key_sets ? g_prompt_attention_key_sets : (rows > 64 ? 2 : 1);
    if (a.head_dim == 128) {
        if (group == 1) return launch_attention_prompt_shape<128, 1>(a, rows, kv_f16, sets, s);
        if (group == 2) return launch_attention_prompt_shape<128, 2>(a, rows, kv_f16, sets, s);
        return launch_attention_prompt_shape<128, 4>(a, rows, kv_f16, sets, s);
    }
    if (group == 1) return launch_attention_prompt_shape<64, 1>(a, rows, kv_f16, sets, s);
    if (group == 2) return launch_attention_prompt_shape<64, 2>(a, rows, kv_f16, sets, s);
    return launch_attention_prompt_shape<64, 4>(a, rows, kv_f16, sets, s);
}

int attention_head_splits(int) { return kAttentionHeadSplits; }

template <int HD, int WAVES, int U>
void launch_attention_partial_shape(const AttentionArgs &a, dim3 grid, bool kv_f16, unsigned heads, hipStream_t s) {
    if (kv_f16) hipLaunchKernelGGL((attention_partial_kernel<HD, true, WAVES, U>), grid, dim3(WAVES * 64), 0, s, a.q, a.k_cache, a.v_cache, a.pos, a.seq, a.head_partials, (unsigned)a.cache_seq_stride, heads);
    else hipLaunchKernelGGL((attention_partial_kernel<HD, false, WAVES, U>), grid, dim3(WAVES * 64), 0, s, a.q, a.k_cache, a.v_cache, a.pos, a.seq, a.head_partials, (unsigned)a.cache_seq_stride, heads);
}

hipError_t launch_attention_partials(const AttentionArgs &a, int rows, bool kv_f16, hipStream_t s) {
    if (!a.head_partials || (a.head_dim != 128 && a.head_dim != 64) || a.n_head % a.n_kv_head != 0 || rows < 1 || rows > kMaxStepRows)
        return hipErrorInvalidValue;
    if (a.cache_seq_stride > 0xFFFFFFFFull || a.n_head > 0xFFFF || a.n_kv_head > 0xFFFF) return hipErrorInvalidValue;
    const unsigned heads = (unsigned)a.n_head | ((unsigned)a.n_kv_head << 16);
    dim3 grid(a.n_head, rows, attention_head_splits(a.max_seq));
    // Wavefronts per workgroup x chunks in flight per wavefront.  One pass of a wavefront's loop covers splits x wavefronts x
    // (tokens per chunk: 4 at head size 128, 8 at 64) x chunks tokens of the prefix and costs one trip to memory, with the loads of
    // chunks past the prefix issued all the same (clamped, masked).  The shape is fixed per runtime (a captured graph replays it),
    // so it follows the context size: the smallest that covers half of it in one pass.  Measured at head size 128, prefix 512-776:
    // 4 x 12 6.2 us, 8 x 6 5.0 us, 16 x 3 4.7 us but a slower step.  At head size 64, prefix 16-144 of 256 (6-layer model, tok/s):
    // 8 x 4 7.6 k, 8 x 1 7.9 k, 2 x 8 7.7 k, 1 x 8 7.8 k, 2 x 4 8.0 k, 4 x 2 8.0 k, 1 x 4 8.0 k, 2 x 2 8.1 k.
    if (a.head_dim == 128) {
        if (a.max_seq <= 256) launch_attention_partial_shape<128, 2, 4>(a, grid, kv_f16, heads, s);        // 128 tokens per pass
        else if (a.max_seq <= 512) launch_attention_partial_shape<128, 4, 4>(a, grid, kv_f16, heads, s);   // 256
        else launch_attention_partial_shape<128, 8, 6>(a, grid, kv_f16, heads, s);                         // 768
    } else {
        if (a.max_seq <= 256) launch_attention_partial_shape<64, 2, 2>(a, grid, kv_f16, heads, s);         // 128 tokens per pass
        else if (a.max_seq <= 512) launch_attention_partial_shape<64, 2, 4>(a, grid, kv_f16, heads, s);    // 256
        else if (a.max_seq <= 1024) launch_attention_partial_shape<64, 4, 4>(a, grid, kv_f16, heads, s);   // 512
        else launch_attention_partial_shape<64, 8, 4>(a, grid, kv_f16, heads, s);                          // 1024
    }
    return hipGetLastError();
}

bool rmsnorm_reduce_supported(int d) { return d % 4 == 0 && d <= 8 * 4 * kBlock; }

hipError_t launch_rmsnorm_reduce(const float *partial, int splits, size_t plane, const float *residual, float *y, const float *w, float eps,
                                 int rows, int d, uint16_t *out_f16, hipStream_t s) {
    if (!rmsnorm_reduce_supported(d) || splits < 1 || plane % 4 != 0) return hipErrorInvalidValue;
    hipLaunchKernelGGL(rmsnorm_reduce_kernel, dim3(rows), dim3(kBlock), 0, s, partial, splits, plane, residual, y, w, eps, d, out_f16);
    return hipGetLastError();
}

hipError_t launch_swiglu(const float *gu, int rows, int hidden, uint16_t *act_f16, hipStream_t s) {
    hipLaunchKernelGGL(swiglu_kernel, dim3((hidden + 255) / 256, rows), dim3(256), 0, s, gu, hidden, act_f16);
    return hipGetLastError();
}

hipError_t launch_argmax(const float *logits, int rows, int vocab, int *out_token, float *out_value, const ArgmaxScratch &scratch,
                         hipStream_t s) {
    if (!scratch.part_value || !scratch.part_index || rows > kMaxStepRows) return hipErrorInvalidValue;
    const int blocks = vocab < kArgmaxBlocks * kBlock ? (vocab + kBlock - 1) / kBlock : kArgmaxBlocks;
    hipLaunchKernelGGL(argmax_partial_kernel, dim3(blocks, rows), dim3(kBlock), 0, s, logits, vocab, scratch.part_value, scratch.part_index);
    hipLaunchKernelGGL(argmax_final_kernel, dim3(rows), dim3(kBlock), 0, s, scratch.part_value, scratch.part_index, blocks, out_token,
                       out_value);
    return hipGetLastError();
}

hipError_t launch_argmax_final(const ArgmaxScratch &scratch, int blocks, int rows, int *out_token, hipStream_t s) {
    if (!scratch.part_value || !scratch.part_index || blocks < 1 || rows < 1) return hipErrorInvalidValue;
    hipLaunchKernelGGL(argmax_final_kernel, dim3(rows), dim3(kBlock), 0, s, scratch.part_value, scratch.part_index, blocks, out_token,
                       static_cast<float *>(nullptr));
    return hipGetLastError();
}

hipError_t launch_greedy_tail(const ArgmaxScratch &scratch, int blocks, int *out_token, int seq, int *visible, int *tokens, int *pos, int *seqs,
                              int *log, int *log_count, int log_capacity, const void *table, bool table_is_f16, int d, float *hidden, int eos,
                              hipStream_t s) {
    if (!scratch.part_value || !scratch.part_index || blocks < 1) return hipErrorInvalidValue;
    GreedyTailArgs a{scratch.part_value, scratch.part_index, blocks, out_token, seq, visible, tokens, pos, seqs, log, log_count, log_capacity,
                     table, table_is_f16 ? 1 : 0, d, hidden, eos};
    hipLaunchKernelGGL(greedy_tail_kernel, dim3(1), dim3(kBlock), 0, s, a);
    return hipGetLastError();
}

hipError_t launch_greedy_step_tail(const float *logits, int vocab, int *out_token, const ArgmaxScratch &scratch, int seq, int *visible,
                                   int *tokens, int *pos, int *seqs, int *log, int *log_count, int log_capacity, const void *table,
                                   bool table_is_f16, int d, float *hidden, int eos, hipStream_t s) {
    if (!scratch.part_value || !scratch.part_index) return hipErrorInvalidValue;
    const int blocks = vocab < kArgmaxBlocks * kBlock ? (vocab + kBlock - 1) / kBlock : kArgmaxBlocks;
    hipLaunchKernelGGL(argmax_partial_kernel, dim3(blocks, 1), dim3(kBlock), 0, s, logits, vocab, scratch.part_value, scratch.part_index);
    GreedyTailArgs a{scratch.part_value, scratch.part_index, blocks, out_token, seq, visible, tokens, pos, seqs, log, log_count, log_capacity,
                     table, table_is_f16 ? 1 : 0, d, hidden, eos};
    hipLaunchKernelGGL(greedy_tail_kernel, dim3(1), dim3(kBlock), 0, s, a);
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
