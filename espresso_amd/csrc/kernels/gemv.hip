// Dequant-fused GEMV for batch-1/2 decode on gfx950:  y[b][r] = sum_c dequant(W)[r][c] * x[b][c].
//
// Replaces the seven vDSP_mmul GEMVs per layer of the reference's CPU-exact path
// (RealModelInferenceEngine.swift:6674-6697) with kernels that read the *packed* weights once.
//
// Shape of the kernels
//   * one workgroup = 4 wavefronts of 64 lanes; a wavefront (or, for long Q4_K rows, a team of four) owns a pair
//     of consecutive rows at a time - a RoPE pair or a (gate, up) pair, so the epilogues stay in registers;
//   * a lane's unit of work ("item") is built from aligned 128-bit loads of packed weights; consecutive lanes read
//     consecutive pieces of the row, so a wavefront load covers 1 KiB+ of contiguous HBM;
//   * the activations are staged once per workgroup in LDS as fp16 - copied, computed on the spot as
//     fp16((x * inv_rms) * w) from the fp32 residual stream (fused RMSNorm), or merged from the partial softmax
//     states the attention kernel left per query head (the wo GEMV).  For the integer formats they are stored
//     with the two middle elements of every group of four swapped, (x0,x2,x1,x3): masking a weight dword with
//     0x000F000F / 0x00FF00FF yields elements 0 and 2 of a group, so the matching activation pair is one LDS dword;
//   * nibbles / bytes become exact fp16 values with exponent tricks (Q4_0, Q8_0: 0x6400 | n = 1024 + n, then an
//     exact packed subtract; Q4_K: in place under 0x5400 / 0x4400 with the offset removed per sub-block through
//     precomputed sums of x), and v_dot2_f32_f16 forms exact products accumulated in fp32;
//   * block scales multiply the per-block partial sums, never the individual weights; Q4_K minimums use the same
//     per-32 sums of x:  sum (d*sc*n - dmin*m) x = d*sc*sum(n x) - dmin*m*sum(x);
//   * DPP row operations reduce a row over the wavefront; one lane applies the epilogue
//     (store / + residual / SiLU(gate)*up -> fp16 / RoPE + KV-cache write).
//
// HBM traffic per launch = packed weight bytes + batch*cols*2 (x) + batch*rows*4 (y): measured 1.006x the
// algorithmic bytes; x is re-read from L2 once per workgroup.
//
// The Q4_K kernels for the llama family's widths are persistent: the grid is what the chip holds at once, teams
// take row pairs round by round with the next pair's loads in flight, and the ragged last round goes to the
// workgroups that were dispatched first (they get their first weights first and stay ahead).
#include <cstdlib>

#include <string>
#include <type_traits>

#include "../common.h"

#include <hip/hip_ext.h>
#include "gemv_device.h"

namespace esp {
namespace {

using namespace detail;

// Eight nibbles of `w` against the activation pairs of their elements.
// Low nibbles of bytes (0,2) and (1,3) meet (xl02, xl13); high nibbles meet (xh02, xh13).
// High nibbles are left multiplied by 16 (they sit in mantissa bits 4..7): callers fold 1/16.
template <int SUB_LO, int SUB_HI>
__device__ __forceinline__ void nibble_dword(u32 w, h2 xl02, h2 xl13, h2 xh02, h2 xh13, float &dlo, float &dhi) {
    const h2 sub_lo = {(_Float16)SUB_LO, (_Float16)SUB_LO};
    const h2 sub_hi = {(_Float16)SUB_HI, (_Float16)SUB_HI};
    const u32 w8 = w >> 8;
    h2 l02 = as_h2((w & 0x000F000Fu) | 0x64006400u) - sub_lo;
    h2 h02 = as_h2((w & 0x00F000F0u) | 0x64006400u) - sub_hi;
    h2 l13 = as_h2((w8 & 0x000F000Fu) | 0x64006400u) - sub_lo;
    h2 h13 = as_h2((w8 & 0x00F000F0u) | 0x64006400u) - sub_hi;
    dlo = fdot2(l02, xl02, dlo);
    dlo = fdot2(l13, xl13, dlo);
    dhi = fdot2(h02, xh02, dhi);
    dhi = fdot2(h13, xh13, dhi);
}

// Four signed bytes of `w` against (x02, x13).
__device__ __forceinline__ void byte_dword(u32 w, h2 x02, h2 x13, float &d) {
    const h2 sub = {(_Float16)1152.0f, (_Float16)1152.0f};  // 1024 + 128
    const u32 t = w ^ 0x80808080u;                            // signed -> biased unsigned
    // fp16 little-endian: low byte = mantissa bits 0..7, high byte 0x64 -> value 1024 + byte
    h2 f02 = as_h2(__builtin_amdgcn_perm(0x64646464u, t, 0x04020400u)) - sub;
    h2 f13 = as_h2(__builtin_amdgcn_perm(0x64646464u, t, 0x04030401u)) - sub;
    d = fdot2(f02, x02, d);
    d = fdot2(f13, x13, d);
}

template <int FMT>
struct Traits;
template <>
struct Traits<FMT_Q4_0> { static constexpr int kItemElems = 32; static constexpr bool kPermuteX = true; static constexpr bool kXSums = false; };
template <>
struct Traits<FMT_Q8_0> { static constexpr int kItemElems = 16; static constexpr bool kPermuteX = true; static constexpr bool kXSums = false; };
template <>
struct Traits<FMT_F32> { static constexpr int kItemElems = 4; static constexpr bool kPermuteX = false; static constexpr bool kXSums = false; };
template <>
struct Traits<FMT_F16> { static constexpr int kItemElems = 8; static constexpr bool kPermuteX = false; static constexpr bool kXSums = false; };

struct KernelArgs {
    QkvEpilogue qkv;
    uint16_t *out_f16;
    const uint8_t *qs;
    const uint8_t *tiled;     // Q4_K: the copy tiled by (sixteen rows, super-block), or null
    const uint16_t *scales;
    size_t qs_row_bytes;
    int rows, cols;
    const uint16_t *x;
    float *y;
    const float *residual;
    int epilogue;
    // when norm_x is set the activations are rmsnorm(norm_x) * norm_w computed while staging (x is unused)
    const float *norm_x, *norm_w;
    float norm_eps;
    // when merge_partials is set the activations are the attention context merged from per-split partial states
    // while staging (x and norm_x unused): [batch][cols / head_dim heads][kMergeSplits][head_dim values, m, l, 2 pad]
    const float *merge_partials;
    int merge_head_dim;
    // EPI_ARGMAX: one (value, index) pair per workgroup and batch row, [batch][gridDim.x]
    float *part_value;
    int *part_index;
    // split activations (matrix-core Q4_K kernel): x holds two fp16 rows per activation row, hi and lo (see split_group); with
    // the fused norm or the merged attention states the staging makes both.  split_out: the SiLU(gate)*up epilogue writes such
    // row pairs.
    int split_x, split_out;
    // measurement only (null otherwise; read by the stamped instantiations alone): four 100 MHz wall-clock stamps per
    // wavefront, [wavefront][4] = start, activations staged, first weights consumed, end; stamp_capacity wavefronts have room
    unsigned long long *stamps;
    int stamp_capacity;
};
template <bool STAMPS>
__device__ __forceinline__ void stamp(const KernelArgs &a, int which) {
    if constexpr (STAMPS) {
        const int w = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
        if (a.stamps && (threadIdx.x & 63) == 0 && w < a.stamp_capacity) a.stamps[(size_t)w * 4 + which] = wall_clock64();
    }
}

// First-max rule of the reference's output head (RealModelInferenceEngine.swift:8219-8275, neon_convert.c:36-101): a larger
// value wins, equal values keep the lower index, NaN never wins.
__device__ __forceinline__ void argmax_take(float &best, int &best_i, float v, int i) {
    if (v > best || (v == best && i < best_i)) { best = v; best_i = i; }
}
// The workgroup's result from one candidate per wavefront and batch row (lane 0 of each wavefront holds it).
// Every thread of the workgroup must call this.  `bv` / `bi`: kWaves * B entries of LDS nobody else uses.
template <int B>
__device__ __forceinline__ void argmax_workgroup(const KernelArgs &a, const float (&best)[B], const int (&best_i)[B], float *bv, int *bi) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) {
#pragma unroll
        for (int b = 0; b < B; b++) { bv[b * kWaves + wave] = best[b]; bi[b * kWaves + wave] = best_i[b]; }
    }
    __syncthreads();
    if (threadIdx.x < B) {
        const int b = threadIdx.x;
        float v = bv[b * kWaves];
        int i = bi[b * kWaves];
#pragma unroll
        for (int w = 1; w < kWaves; w++) argmax_take(v, i, bv[b * kWaves + w], bi[b * kWaves + w]);
        a.part_value[(size_t)b * gridDim.x + blockIdx.x] = v;
        a.part_index[(size_t)b * gridDim.x + blockIdx.x] = i;
    }
}

// ---- attention context merged from per-split partial states -------------------------------------------
// The arithmetic of attention_merge_kernel: M = max m, f = exp(m - M) (0 for an empty split), L = fma(l, f, L),
// A = fma(acc, f, A) in split order, context = A / L, rounded to fp16.  Eight channels of one query head.
constexpr int kMergeSplits = kAttentionHeadSplits;
__device__ __forceinline__ void merge_group_values(const float2 (&ml)[kMergeSplits], const float4 (&a0)[kMergeSplits], const float4 (&a1)[kMergeSplits],
                                                   float (&c)[8]) {
    float M = ml[0].x;
#pragma unroll
    for (int sp = 1; sp < kMergeSplits; sp++) M = fmaxf(M, ml[sp].x);
    float L = 0.0f, A[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int sp = 0; sp < kMergeSplits; sp++) {
        const float f = ml[sp].x != -INFINITY ? expf(ml[sp].x - M) : 0.0f;
        L = __builtin_fmaf(ml[sp].y, f, L);
        const float v[8] = {a0[sp].x, a0[sp].y, a0[sp].z, a0[sp].w, a1[sp].x, a1[sp].y, a1[sp].z, a1[sp].w};
#pragma unroll
        for (int i = 0; i < 8; i++) A[i] = __builtin_fmaf(v[i], f, A[i]);
    }
#pragma unroll
    for (int i = 0; i < 8; i++) c[i] = L > 0.0f ? A[i] / L : 0.0f;
}
__device__ __forceinline__ uint4 merge_group(const float2 (&ml)[kMergeSplits], const float4 (&a0)[kMergeSplits], const float4 (&a1)[kMergeSplits]) {
    float c[8];
    merge_group_values(ml, a0, a1, c);
    uint4 h;
    h.x = pack_half2(c[0], c[1]); h.y = pack_half2(c[2], c[3]); h.z = pack_half2(c[4], c[5]); h.w = pack_half2(c[6], c[7]);
    return h;
}
// Loads of group g (eight channels) of row b; head size known at run time.
__device__ __forceinline__ void merge_group_load(const KernelArgs &a, int b, int g, int cols, float2 (&ml)[kMergeSplits],
                                                 float4 (&a0)[kMergeSplits], float4 (&a1)[kMergeSplits]) {
    const int hd = a.merge_head_dim, stride = hd + 4, per_head = hd / 8;
    const int head = g / per_head, d0 = (g - head * per_head) * 8;
    const float *base = a.merge_partials + ((size_t)b * (cols / hd) + head) * kMergeSplits * stride;
#pragma unroll
    for (int sp = 0; sp < kMergeSplits; sp++) {
        const float *ps = base + sp * stride;
        a0[sp] = *reinterpret_cast<const float4 *>(ps + d0);
        a1[sp] = *reinterpret_cast<const float4 *>(ps + d0 + 4);
        ml[sp] = *reinterpret_cast<const float2 *>(ps + hd);
    }
}

// 1 / sqrt(mean(x^2) + eps) of row b of norm_x (any cols that is a multiple of 8); `red` as above.
__device__ __forceinline__ float row_inverse_rms(const KernelArgs &a, int b, int cols, float *red) {
    const float4 *x4 = reinterpret_cast<const float4 *>(a.norm_x + (size_t)b * cols);
    float s = 0.0f;
    for (int g = threadIdx.x; g < cols / 8; g += kThreads) s += sum_squares(x4[2 * g], x4[2 * g + 1]);
    return 1.0f / sqrtf(workgroup_sum(s, red) / (float)cols + a.norm_eps);
}
// Group g (eight consecutive elements) of row b of the activations, as fp16.
__device__ __forceinline__ uint4 activation_group(const KernelArgs &a, int b, int g, int cols, float inv) {
    if (a.merge_partials) {
        float2 ml[kMergeSplits];
        float4 a0[kMergeSplits], a1[kMergeSplits];
        merge_group_load(a, b, g, cols, ml, a0, a1);
        return merge_group(ml, a0, a1);
    }
    if (!a.norm_x) return reinterpret_cast<const uint4 *>(a.x)[(size_t)b * (cols / 8) + g];
    const float4 *x4 = reinterpret_cast<const float4 *>(a.norm_x + (size_t)b * cols);
    const float4 *w4 = reinterpret_cast<const float4 *>(a.norm_w);
    return normalized_group(x4[2 * g], x4[2 * g + 1], w4[2 * g], w4[2 * g + 1], inv);
}

// What a wavefront does with the two row sums (rows 2p and 2p+1) of each batch column.
template <int B>
__device__ __forceinline__ void pair_epilogue(const KernelArgs &a, int pair, const float va[B], const float vb[B]) {
    const int r0 = 2 * pair, r1 = 2 * pair + 1;
    if (a.epilogue == EPI_SWIGLU_F16) {
        // rows are (gate_i, up_i): act_i = silu_tanh(gate) * up, rounded to fp16 for the next GEMV
        // (RealModelInferenceEngine.swift:6825-6827, :6337)
        if (r1 < a.rows) {
#pragma unroll
            for (int b = 0; b < B; b++) {
                const float hg = __fmul_rn(0.5f, va[b]);
                const float silu = __fmul_rn(hg, __fadd_rn(1.0f, tanhf(hg)));
                const float act = __fmul_rn(silu, vb[b]);
                if (a.split_out) {   // hi and lo rows for a consumer that takes split activations
                    const _Float16 hi = (_Float16)act;
                    a.out_f16[(size_t)(2 * b) * (a.rows / 2) + pair] = __builtin_bit_cast(uint16_t, hi);
                    a.out_f16[(size_t)(2 * b + 1) * (a.rows / 2) + pair] =
                        __builtin_bit_cast(uint16_t, (_Float16)__fmul_rn(__fsub_rn(act, (float)hi), kSplitScale));
                } else {
                    a.out_f16[(size_t)b * (a.rows / 2) + pair] = __builtin_bit_cast(uint16_t, (_Float16)act);
                }
            }
        }
        return;
    }
    if (a.epilogue == EPI_QKV_ROPE) {
        // rows of the fused q|k|v matrix: q and k as RoPE pairs (j, j + half), v in natural order.
        // Half-split RoPE from the host-built table (:6745-6772), then q -> q_out, k/v -> caches at
        // (seq, pos), both token-major (:6297-6300).
        const QkvEpilogue &q = a.qkv;
        const int half = q.head_dim / 2, ad = q.n_head * q.head_dim, kd = q.n_kv_head * q.head_dim;
        if (r1 >= a.rows) return;
#pragma unroll
        for (int b = 0; b < B; b++) {
            const int pos = q.pos[b];
            const size_t seq_base = (size_t)q.seq[b] * q.cache_seq_stride;
            if (r0 < ad + kd) {
                const bool is_q = r0 < ad;
                const int pr = is_q ? pair : pair - ad / 2;
                const int h = pr / half, j = pr - h * half;
                const float c = q.rope_cos[(size_t)pos * half + j], sn = q.rope_sin[(size_t)pos * half + j];
                const float o0 = __fsub_rn(__fmul_rn(va[b], c), __fmul_rn(vb[b], sn));
                const float o1 = __fadd_rn(__fmul_rn(va[b], sn), __fmul_rn(vb[b], c));
                if (is_q) {
                    float *dst = q.q_out + (size_t)b * ad + (size_t)h * q.head_dim + j;
                    dst[0] = o0;
                    dst[half] = o1;
                } else {
                    const size_t o = seq_base + (size_t)pos * kd + (size_t)h * q.head_dim + j;
                    if (q.kv_f16) {
                        uint16_t *kc = reinterpret_cast<uint16_t *>(q.k_cache);
                        kc[o] = __builtin_bit_cast(uint16_t, (_Float16)o0);
                        kc[o + half] = __builtin_bit_cast(uint16_t, (_Float16)o1);
                    } else {
                        float *kc = reinterpret_cast<float *>(q.k_cache);
                        kc[o] = o0;
                        kc[o + half] = o1;
                    }
                }
            } else {
                const size_t o = seq_base + (size_t)pos * kd + (size_t)(r0 - ad - kd);
                if (q.kv_f16) {
                    uint16_t *vc = reinterpret_cast<uint16_t *>(q.v_cache);
                    vc[o] = __builtin_bit_cast(uint16_t, (_Float16)va[b]);
                    vc[o + 1] = __builtin_bit_cast(uint16_t, (_Float16)vb[b]);
                } else {
                    float *vc = reinterpret_cast<float *>(q.v_cache);
                    vc[o] = va[b];
                    vc[o + 1] = vb[b];
                }
            }
        }
        return;
    }
#pragma unroll
    for (int b = 0; b < B; b++) {
        if (r0 < a.rows) {
            const size_t o = (size_t)b * a.rows + r0;
            a.y[o] = a.epilogue == EPI_ADD_RESIDUAL ? a.residual[o] + va[b] : va[b];
        }
        if (r1 < a.rows) {
            const size_t o = (size_t)b * a.rows + r1;
            a.y[o] = a.epilogue == EPI_ADD_RESIDUAL ? a.residual[o] + vb[b] : vb[b];
        }
    }
}

// The scalar arguments that the first loads of a GEMV kernel need.  Leading scalar arguments are preloaded
// into registers with the wavefront's launch; the fields of a structure passed by value are fetched from
// memory first, which costs the start of every kernel a memory round trip.
// mode: 0 = fp16 activations, 1 = RMSNorm fused into the staging, 2 = attention partial states (head size in bits 8..).
__device__ __forceinline__ KernelArgs with_leading_args(const KernelArgs &rest, const uint8_t *qs, const uint16_t *scales, const void *activations,
                                                        const float *norm_w, int rows, int cols, int row_bytes, int mode, float norm_eps) {
    KernelArgs a = rest;
    a.qs = qs;
    a.scales = scales;
    a.rows = rows;
    a.cols = cols;
    a.qs_row_bytes = (size_t)row_bytes;
    a.norm_w = norm_w;
    a.norm_eps = norm_eps;
    a.x = (mode & 0xFF) == 0 ? static_cast<const uint16_t *>(activations) : nullptr;
    a.norm_x = (mode & 0xFF) == 1 ? static_cast<const float *>(activations) : nullptr;
    a.merge_partials = (mode & 0xFF) == 2 ? static_cast<const float *>(activations) : nullptr;
    a.merge_head_dim = mode >> 8;
    return a;
}
inline const void *leading_activations(const KernelArgs &a) {
    return a.merge_partials ? static_cast<const void *>(a.merge_partials) : a.norm_x ? static_cast<const void *>(a.norm_x) : static_cast<const void *>(a.x);
}
inline int leading_mode(const KernelArgs &a) { return a.merge_partials ? (2 | (a.merge_head_dim << 8)) : a.norm_x ? 1 : 0; }

template <int FMT, int B, int R>
__global__ __launch_bounds__(kThreads) void gemv_kernel(const uint8_t *qs, const uint16_t *scales, const void *activations, const float *norm_w, int rows,
                                                        int cols_arg, int row_bytes, int mode, float norm_eps, KernelArgs rest) {
    const KernelArgs a = with_leading_args(rest, qs, scales, activations, norm_w, rows, cols_arg, row_bytes, mode, norm_eps);
    using T = Traits<FMT>;
    extern __shared__ uint4 smem_raw[];
    uint16_t *xs = reinterpret_cast<uint16_t *>(smem_raw);                 // [B][cols] fp16
    float *xsum = reinterpret_cast<float *>(xs + (size_t)B * a.cols);      // [B][cols/16] (Q4_K)
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int cols = a.cols;

    // ---- the wavefront's rows and the first 128 bits of weights per lane: in flight while the activations are staged ----
    const int row0 = (blockIdx.x * kWaves + wave) * R;
    const int items = cols / T::kItemElems;
    const uint8_t *rowp[R];
    const uint16_t *scalep[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int row = row0 + r < a.rows ? row0 + r : a.rows - 1;  // clamp: never read past the matrix
        rowp[r] = a.qs + (size_t)row * a.qs_row_bytes;
        scalep[r] = (FMT == FMT_Q4_0 || FMT == FMT_Q8_0) ? a.scales + (size_t)row * (cols / 32) : nullptr;
    }
    struct Item { uint4 q[R]; uint16_t d[R]; };
    auto load_item = [&](int item) {
        Item it;
#pragma unroll
        for (int r = 0; r < R; r++) {
            it.q[r] = *reinterpret_cast<const uint4 *>(rowp[r] + (size_t)item * 16);
            if constexpr (FMT == FMT_Q4_0) it.d[r] = scalep[r][item];
            else if constexpr (FMT == FMT_Q8_0) it.d[r] = scalep[r][item >> 1];
            else it.d[r] = 0;
        }
        return it;
    };
    Item cur = load_item(lane < items ? lane : items - 1);

    // ---- stage activations: 128-bit loads (or the fused RMSNorm), middle elements of each group of
    // four swapped for the integer formats ----
    {
        __shared__ float norm_red[B * kWaves];
        uint4 *dst = reinterpret_cast<uint4 *>(xs);
        const int per_row = cols / 8;
#pragma unroll
        for (int b = 0; b < B; b++) {
            const float inv = a.norm_x ? row_inverse_rms(a, b, cols, norm_red + b * kWaves) : 0.0f;
            for (int g = tid; g < per_row; g += kThreads) {
                const uint4 v = activation_group(a, b, g, cols, inv);
                dst[(size_t)b * per_row + g] = T::kPermuteX ? swap_middle(v) : v;
            }
        }
    }
    __syncthreads();
    if (T::kXSums) {
        const int groups = B * cols / 16;
        for (int g = tid; g < groups; g += kThreads) {
            const h2 *p = reinterpret_cast<const h2 *>(xs + (size_t)g * 16);
            float s = 0.0f;
#pragma unroll
            for (int i = 0; i < 8; i++) s += (float)p[i].x + (float)p[i].y;
            xsum[g] = s;
        }
        __syncthreads();
    }

    if (row0 >= a.rows && a.epilogue != EPI_ARGMAX) return;   // (the arg-max epilogue ends with a workgroup barrier)

    float acc[R][B];
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int b = 0; b < B; b++) acc[r][b] = 0.0f;

    for (int item = lane; item < items; item += 64) {
        Item nxt = cur;
        if (item + 64 < items) nxt = load_item(item + 64);   // one step ahead of the arithmetic
        if constexpr (FMT == FMT_Q4_0) {
            const int e_lo = item * 32;
            uint4 xl[B][2], xh[B][2];
#pragma unroll
            for (int b = 0; b < B; b++) {
                const uint4 *px = reinterpret_cast<const uint4 *>(xs + (size_t)b * cols + e_lo);
                xl[b][0] = px[0]; xl[b][1] = px[1];
                xh[b][0] = px[2]; xh[b][1] = px[3];
            }
#pragma unroll
            for (int r = 0; r < R; r++) {
                const uint4 q = cur.q[r];
                const float d = half_bits_to_float(cur.d[r]);
#pragma unroll
                for (int b = 0; b < B; b++) {
                    float dlo = 0.0f, dhi = 0.0f;
#pragma unroll
                    for (int k = 0; k < 4; k++) {
                        const u32 w = dword_of(q, k);
                        const uint4 &vl = xl[b][k >> 1];
                        const uint4 &vh = xh[b][k >> 1];
                        // (n - 8): subtract 1024 + 8; high nibbles carry x16: subtract 1024 + 128
                        nibble_dword<1032, 1152>(w, as_h2(dword_of(vl, (k & 1) * 2)), as_h2(dword_of(vl, (k & 1) * 2 + 1)),
                                                 as_h2(dword_of(vh, (k & 1) * 2)), as_h2(dword_of(vh, (k & 1) * 2 + 1)),
                                                 dlo, dhi);
                    }
                    acc[r][b] += d * (dlo + dhi * 0.0625f);
                }
            }
        } else if constexpr (FMT == FMT_Q8_0) {
            const int e0 = item * 16;
            uint4 xv[B][2];
#pragma unroll
            for (int b = 0; b < B; b++) {
                const uint4 *px = reinterpret_cast<const uint4 *>(xs + (size_t)b * cols + e0);
                xv[b][0] = px[0]; xv[b][1] = px[1];
            }
#pragma unroll
            for (int r = 0; r < R; r++) {
                const uint4 q = cur.q[r];
                const float d = half_bits_to_float(cur.d[r]);
#pragma unroll
                for (int b = 0; b < B; b++) {
                    float dot = 0.0f;
#pragma unroll
                    for (int k = 0; k < 4; k++) {
                        const uint4 &v = xv[b][k >> 1];
                        byte_dword(dword_of(q, k), as_h2(dword_of(v, (k & 1) * 2)), as_h2(dword_of(v, (k & 1) * 2 + 1)), dot);
                    }
                    acc[r][b] += d * dot;
                }
            }
        } else if constexpr (FMT == FMT_F32) {
            // exact fp32 weights (float32 sidecars): four weights per 128-bit load, plain fp32 multiply-adds
            const int e0 = item * 4;
            uint2 xv[B];
#pragma unroll
            for (int b = 0; b < B; b++) xv[b] = *reinterpret_cast<const uint2 *>(xs + (size_t)b * cols + e0);
#pragma unroll
            for (int r = 0; r < R; r++) {
                const uint4 q = cur.q[r];
#pragma unroll
                for (int b = 0; b < B; b++) {
                    const h2 x01 = as_h2(xv[b].x), x23 = as_h2(xv[b].y);
                    float dot = __uint_as_float(q.x) * (float)x01.x;
                    dot += __uint_as_float(q.y) * (float)x01.y;
                    dot += __uint_as_float(q.z) * (float)x23.x;
                    dot += __uint_as_float(q.w) * (float)x23.y;
                    acc[r][b] += dot;
                }
            }
        } else {  // FMT_F16
            const int e0 = item * 8;
            uint4 xv[B];
#pragma unroll
            for (int b = 0; b < B; b++) xv[b] = *reinterpret_cast<const uint4 *>(xs + (size_t)b * cols + e0);
#pragma unroll
            for (int r = 0; r < R; r++) {
                const uint4 q = cur.q[r];
#pragma unroll
                for (int b = 0; b < B; b++) {
                    float dot = 0.0f;
#pragma unroll
                    for (int k = 0; k < 4; k++) dot = fdot2(as_h2(dword_of(q, k)), as_h2(dword_of(xv[b], k)), dot);
                    acc[r][b] += dot;
                }
            }
        }
        cur = nxt;
    }

#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int b = 0; b < B; b++) acc[r][b] = wave_sum(acc[r][b]);

    static_assert(R % 2 == 0, "the epilogues work on row pairs");
    if (a.epilogue == EPI_ARGMAX) {
        __shared__ float bv[B * kWaves];
        __shared__ int bi[B * kWaves];
        float best[B];
        int best_i[B];
#pragma unroll
        for (int b = 0; b < B; b++) {
            best[b] = -INFINITY;
            best_i[b] = 0x7FFFFFFF;
#pragma unroll
            for (int r = 0; r < R; r++)
                if (row0 + r < a.rows) argmax_take(best[b], best_i[b], acc[r][b], row0 + r);   // ascending rows
        }
        argmax_workgroup<B>(a, best, best_i, bv, bi);
        return;
    }
    if (lane == 0) {
#pragma unroll
        for (int p = 0; p < R / 2; p++) {
            if (row0 + 2 * p >= a.rows) break;
            float va[B], vb[B];
#pragma unroll
            for (int b = 0; b < B; b++) { va[b] = acc[2 * p][b]; vb[b] = acc[2 * p + 1][b]; }
            pair_epilogue<B>(a, row0 / 2 + p, va, vb);
        }
    }
}

// cols known only at run time (a multiple of 256, so every quad of lanes is inside the row)
template <int B>
__device__ __forceinline__ void q4k_stage_x(const KernelArgs &a, int cols, int xstride, uint4 *xs4, float *xsum, float *red) {
#pragma unroll
    for (int b = 0; b < B; b++) {
        const float inv = a.norm_x ? row_inverse_rms(a, b, cols, red + b * kWaves) : 0.0f;
        for (int g = threadIdx.x; g < cols / 8; g += kThreads) q4k_store_group(activation_group(a, b, g, cols, inv), b, g, cols, xstride, xs4, xsum);
    }
}

// cols = 64 * IPR: every load of the row is issued before the first use, so staging costs one memory
// round trip (two with the fused RMSNorm: values, then nothing else - the weights ride along).
// NATURAL: the LDS layout of the matrix-core kernel (q4k_store_group_natural) instead of the transposed one.
template <bool NATURAL>
__device__ __forceinline__ void q4k_store(const uint4 &v, int b, int g, int cols, int xstride, uint4 *xs4, float *xsum) {
    if constexpr (NATURAL) q4k_store_group_natural(v, b, g, cols, xs4, xsum);
    else q4k_store_group(v, b, g, cols, xstride, xs4, xsum);
}

template <int B, int IPR, bool NORM, bool NATURAL = false, int THREADS = kThreads>
struct Q4KStage {
    static_assert(!NORM || THREADS == kThreads, "the fused RMSNorm adds four wavefronts' sums");
    static_assert(IPR % 4 == 0, "whole super-blocks per row");
    static constexpr int GROUPS = IPR * 8, K = (GROUPS + THREADS - 1) / THREADS, cols = IPR * 64, XSTRIDE = IPR | 1;
    // Threads past the last group load group 0 and drop it: a guarded load becomes a branch, and
    // each branch waits for its own round trip to the L2, while clamped loads all issue at once.
    static constexpr bool FULL = GROUPS % THREADS == 0;
    float4 v0[NORM ? B : 1][K], v1[NORM ? B : 1][K], g0[K], g1[K];   // NORM: fp32 values and norm weights
    uint4 v[NORM ? 1 : B][K];                                        // otherwise: fp16 values

    // Issues the loads.  Called before the first weight loads: memory returns in order, so the
    // activations (L2 hits) must not queue behind weight lines that come from HBM.
    __device__ __forceinline__ void issue(const KernelArgs &a) {
        const int tid = threadIdx.x;
        if constexpr (NORM) {
            const float4 *w4 = reinterpret_cast<const float4 *>(a.norm_w);
            const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
            for (int k = 0; k < K; k++) {
                const bool in = FULL || tid + k * THREADS < GROUPS;   // whole quads of lanes: GROUPS is a multiple of 32
                const int g = in ? tid + k * THREADS : 0;
                g0[k] = w4[2 * g];
                g1[k] = w4[2 * g + 1];
#pragma unroll
                for (int b = 0; b < B; b++) {
                    const float4 *x4 = reinterpret_cast<const float4 *>(a.norm_x + (size_t)b * cols);
                    v0[b][k] = x4[2 * g];
                    v1[b][k] = x4[2 * g + 1];
                    if (!in) v0[b][k] = v1[b][k] = zero;   // no part in the sum of squares
                }
            }
        } else {
#pragma unroll
            for (int b = 0; b < B; b++)
#pragma unroll
                for (int k = 0; k < K; k++)
                    v[b][k] = reinterpret_cast<const uint4 *>(a.x)[(size_t)b * (cols / 8) + (FULL || tid + k * THREADS < GROUPS ? tid + k * THREADS : 0)];
        }
    }

    // Normalises (NORM) and writes the fp16 groups and their sums to LDS; the caller's barrier follows.
    __device__ __forceinline__ void finish(const KernelArgs &a, uint4 *xs4, float *xsum, float *red) {
        const int tid = threadIdx.x;
        if constexpr (NORM) {
#pragma unroll
            for (int b = 0; b < B; b++) {
                float s = 0.0f;
#pragma unroll
                for (int k = 0; k < K; k++) s += sum_squares(v0[b][k], v1[b][k]);
                const float inv = 1.0f / sqrtf(workgroup_sum(s, red + b * kWaves) / (float)cols + a.norm_eps);
#pragma unroll
                for (int k = 0; k < K; k++)
                    if (FULL || tid + k * THREADS < GROUPS)
                        q4k_store<NATURAL>(normalized_group(v0[b][k], v1[b][k], g0[k], g1[k], inv), b, tid + k * THREADS, cols, XSTRIDE, xs4, xsum);
            }
        } else {
#pragma unroll
            for (int b = 0; b < B; b++)
#pragma unroll
                for (int k = 0; k < K; k++)
                    if (FULL || tid + k * THREADS < GROUPS) q4k_store<NATURAL>(v[b][k], b, tid + k * THREADS, cols, XSTRIDE, xs4, xsum);
        }
    }
};

// Staging of the persistent kernel when its input is the attention context left as partial states (merge_group
// above).  Row 0's loads are issued with issue(), before the first weight loads; further rows take one more
// round trip each inside finish().
template <int B, int IPR, bool NATURAL = false>
struct Q4KMergeStage {
    static constexpr int GROUPS = IPR * 8, K = GROUPS / kThreads, cols = IPR * 64, XSTRIDE = IPR | 1;
    static_assert(GROUPS % kThreads == 0, "whole groups per thread");
    float4 a0[K][kMergeSplits], a1[K][kMergeSplits];
    float2 ml[K][kMergeSplits];

    __device__ __forceinline__ void load_row(const KernelArgs &a, int b) {
#pragma unroll
        for (int k = 0; k < K; k++) merge_group_load(a, b, threadIdx.x + k * kThreads, cols, ml[k], a0[k], a1[k]);
    }
    __device__ __forceinline__ void store_row(int b, uint4 *xs4, float *xsum) {
#pragma unroll
        for (int k = 0; k < K; k++) q4k_store<NATURAL>(merge_group(ml[k], a0[k], a1[k]), b, threadIdx.x + k * kThreads, cols, XSTRIDE, xs4, xsum);
    }
    __device__ __forceinline__ void issue(const KernelArgs &a) { load_row(a, 0); }
    __device__ __forceinline__ void finish(const KernelArgs &a, uint4 *xs4, float *xsum, float *) {
        store_row(0, xs4, xsum);
#pragma unroll
        for (int b = 1; b < B; b++) {
            load_row(a, b);
            store_row(b, xs4, xsum);
        }
    }
};

// Persistent kernel for cols = 64 * IPR.  TEAM wavefronts share one row pair at a time (TEAM = 1: a
// wavefront streams whole pairs on its own; TEAM = 4: the workgroup splits a long row pair and adds
// the four partial sums through LDS).  Teams take pairs team, team + n_teams, ...: the chip reads
// one contiguous band of rows at a time, the activations are staged once per workgroup however many
// pairs it handles, and the loads of a team's next pair are issued before the arithmetic of the
// current one, so weight traffic never waits for the arithmetic.  Every workgroup runs `iters`
// rounds, so the barriers of the TEAM > 1 reduction line up even when the last round is ragged.
constexpr int kDeferredRounds = 16;   // rounds whose team reductions wait for one barrier at the end of the kernel

// MODE: 0 = fp16 activations as given, 1 = RMSNorm fused into the staging, 2 = attention partial states merged in the staging.
// WAVES: wavefronts per workgroup (more than four only with activations given as fp16, MODE 0, and TEAM > 1): the activations are
// staged once per workgroup, so with eight wavefronts a long row's 28 KB of them are read by a third as many workgroups.
template <int B, int IPR, int TEAM, int MODE, int WAVES = kWaves>
__global__ __launch_bounds__(WAVES * 64) void gemv_q4k_kernel(const uint8_t *qs, const void *activations, const float *norm_w, int rows, int row_bytes,
                                                            int iters, int workgroups, float norm_eps, KernelArgs rest) {
    // The arguments that the first loads need come as leading scalars: those can be preloaded into registers
    // with the wavefront's launch, where fields of a structure passed by value are fetched from memory first.
    KernelArgs a = rest;
    a.qs = qs;
    a.rows = rows;
    a.qs_row_bytes = (size_t)row_bytes;
    if constexpr (MODE == 1) { a.norm_x = static_cast<const float *>(activations); a.norm_w = norm_w; a.norm_eps = norm_eps; }
    else if constexpr (MODE == 2) a.merge_partials = static_cast<const float *>(activations);
    else a.x = static_cast<const uint16_t *>(activations);
    constexpr int cols = IPR * 64, XSTRIDE = IPR | 1, TOTAL = 2 * IPR, TEAM_LANES = TEAM * 64;
    constexpr int PASSES = (TOTAL + TEAM_LANES - 1) / TEAM_LANES, TEAMS = WAVES / TEAM;
    static_assert(WAVES == kWaves || (MODE == 0 && TEAM > 1), "more wavefronts: fp16 activations, teams");
    static_assert(PASSES <= 2 && WAVES % TEAM == 0, "pick TEAM so that a lane holds at most two items per pair");
    extern __shared__ uint4 smem_raw[];
    uint4 *xs4 = smem_raw;                                                       // [B][8][XSTRIDE] x 8 fp16
    float *xsum = reinterpret_cast<float *>(smem_raw + (size_t)B * 8 * XSTRIDE);  // [B][cols/32]
    float *red = xsum + (size_t)B * (cols / 32);                                  // [kDeferredRounds][WAVES][2 * B]
    float *norm_red = red + kDeferredRounds * WAVES * 2 * B;                     // [B][kWaves]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int tl = (wave % TEAM) * 64 + lane;
    const int n_teams = workgroups * TEAMS, npairs = (a.rows + 1) / 2;
    const Q4KLane L = q4k_lane_constants(lane);

    // Issued unconditionally, also for pairs past the end (those read the matrix's first 48 bytes, shared by every lane): a load
    // under a branch makes the compiler wait for every load in flight wherever it needs one of them, which would tie the staging
    // of the activations to the arrival of the first weights.
    auto load_pair = [&](int pair, Q4KItem (&buf)[PASSES]) {
        const bool real = pair < npairs;
        const int row_a = 2 * pair < a.rows ? 2 * pair : a.rows - 1;   // clamped: loads stay inside the matrix
        const int row_b = 2 * pair + 1 < a.rows ? 2 * pair + 1 : a.rows - 1;
        const uint8_t *base_a = a.qs + (real ? (size_t)row_a * a.qs_row_bytes : 0), *base_b = a.qs + (real ? (size_t)row_b * a.qs_row_bytes : 0);
#pragma unroll
        for (int p = 0; p < PASSES; p++) {
            const int t = tl + p * TEAM_LANES, tt = t < TOTAL && real ? t : 0;
            const bool second = tt >= IPR;
            const int i = tt - (second ? IPR : 0);
            const uint8_t *bp = (second ? base_b : base_a) + (size_t)(i >> 2) * 144;
            buf[p].hdr = *reinterpret_cast<const uint4 *>(bp);
            const uint4 *q = reinterpret_cast<const uint4 *>(bp + 16 + (i & 3) * 32);
            buf[p].q0 = q[0];
            buf[p].q1 = q[1];
        }
    };

    // TEAM > 1: the partial sums of a round go to LDS.  With few rounds every round has its own slot and the
    // wavefronts run all rounds without meeting; one barrier after the last round, then the first lanes of each
    // team add the partial sums (wavefront order) and run the epilogues, one round per lane.  With more
    // rounds than slots the team meets after every round (two slots, alternating).
    const bool deferred = TEAM > 1 && iters <= kDeferredRounds;
    auto team_sum = [&](const float *slot, float (&sa)[B], float (&sb)[B]) {
        const int w0 = (wave / TEAM) * TEAM;   // first wavefront of the team
#pragma unroll
        for (int b = 0; b < B; b++) {
            float ta = slot[w0 * 2 * B + 2 * b], tb = slot[w0 * 2 * B + 2 * b + 1];
#pragma unroll
            for (int w = 1; w < TEAM; w++) { ta += slot[(w0 + w) * 2 * B + 2 * b]; tb += slot[(w0 + w) * 2 * B + 2 * b + 1]; }
            sa[b] = ta;
            sb[b] = tb;
        }
    };

    float best[B];     // EPI_ARGMAX (TEAM == 1): the wavefront's running first maximum, valid in lane 0
    int best_i[B];
#pragma unroll
    for (int b = 0; b < B; b++) { best[b] = -INFINITY; best_i[b] = 0x7FFFFFFF; }

    auto process = [&](const Q4KItem (&buf)[PASSES], int pair, int round) {
        float acc_a[B], acc_b[B];
#pragma unroll
        for (int b = 0; b < B; b++) acc_a[b] = acc_b[b] = 0.0f;
        if (pair < npairs) {
#pragma unroll
            for (int p = 0; p < PASSES; p++) {
                const int t = tl + p * TEAM_LANES;
                const bool valid = t < TOTAL;
                const int tt = valid ? t : 0;
                const bool second = tt >= IPR;
                float v[B];
                q4k_item_dots<B, XSTRIDE>(buf[p], L, xs4, xsum, tt - (second ? IPR : 0), XSTRIDE, cols, v);
#pragma unroll
                for (int b = 0; b < B; b++) {
                    const float vv = valid ? v[b] : 0.0f;
                    acc_a[b] += second ? 0.0f : vv;
                    acc_b[b] += second ? vv : 0.0f;
                }
            }
#pragma unroll
            for (int b = 0; b < B; b++) {
                acc_a[b] = wave_sum(acc_a[b]);
                acc_b[b] = wave_sum(acc_b[b]);
            }
        }
        if constexpr (TEAM == 1) {
            if (a.epilogue == EPI_ARGMAX) {
                if (pair < npairs) {
#pragma unroll
                    for (int b = 0; b < B; b++) {
                        argmax_take(best[b], best_i[b], acc_a[b], 2 * pair);
                        if (2 * pair + 1 < a.rows) argmax_take(best[b], best_i[b], acc_b[b], 2 * pair + 1);
                    }
                }
            } else if (pair < npairs && lane == 0) pair_epilogue<B>(a, pair, acc_a, acc_b);
        } else {
            float *slot = red + (size_t)(deferred ? round : (round & 1)) * WAVES * 2 * B;
            if (lane == 0) {
#pragma unroll
                for (int b = 0; b < B; b++) { slot[wave * 2 * B + 2 * b] = acc_a[b]; slot[wave * 2 * B + 2 * b + 1] = acc_b[b]; }
            }
            if (deferred) return;
            __syncthreads();
            if (pair < npairs && tl == 0) {
                team_sum(slot, acc_a, acc_b);
                pair_epilogue<B>(a, pair, acc_a, acc_b);
            }
        }
    };

    Q4KItem buf0[PASSES], buf1[PASSES];
    typename std::conditional<MODE == 2, Q4KMergeStage<B, MODE == 2 ? IPR : 32>, Q4KStage<B, IPR, MODE == 1, false, WAVES * 64>>::type stage;
    const int first_pair = blockIdx.x * TEAMS + wave / TEAM;
    int pair = first_pair;
    stage.issue(a);
    load_pair(pair, buf0);
    stage.finish(a, xs4, xsum, norm_red);
    __syncthreads();
    for (int j = 0; j < iters; j += 2) {
        int next = pair + n_teams;
        load_pair(next, buf1);
        process(buf0, pair, j);
        pair = next;
        if (j + 1 < iters) {
            next = pair + n_teams;
            load_pair(next, buf0);
            process(buf1, pair, j + 1);
            pair = next;
        }
    }
    if constexpr (TEAM == 1) {
        if (a.epilogue == EPI_ARGMAX) argmax_workgroup<B>(a, best, best_i, red, reinterpret_cast<int *>(red + B * kWaves));
    }
    if constexpr (TEAM > 1) {
        if (deferred) {
            __syncthreads();
            const int round = tl;   // lane `round` of the team finishes that round's pair
            const int p = first_pair + round * n_teams;
            if (round < iters && p < npairs) {
                float sa[B], sb[B];
                team_sum(red + (size_t)round * WAVES * 2 * B, sa, sb);
                pair_epilogue<B>(a, p, sa, sb);
            }
        }
    }
}

// Any cols that is a multiple of 256: one workgroup per eight rows, a wavefront per row pair, loads
// one pass ahead of the arithmetic.
template <int B>
__global__ __launch_bounds__(kThreads) void gemv_q4k_generic_kernel(const uint8_t *qs, const void *activations, const float *norm_w, int rows, int cols_arg,
                                                                    int row_bytes, int mode, float norm_eps, KernelArgs rest) {
    const KernelArgs a = with_leading_args(rest, qs, nullptr, activations, norm_w, rows, cols_arg, row_bytes, mode, norm_eps);
    extern __shared__ uint4 smem_raw[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int cols = a.cols, ipr = cols >> 6, xstride = ipr | 1, total = 2 * ipr;
    uint4 *xs4 = smem_raw;
    float *xsum = reinterpret_cast<float *>(smem_raw + (size_t)B * 8 * xstride);
    float *norm_red = xsum + (size_t)B * (cols / 32);   // [B][kWaves]
    const int pair = blockIdx.x * kWaves + wave;
    const int row_a = 2 * pair < a.rows ? 2 * pair : a.rows - 1;
    const int row_b = 2 * pair + 1 < a.rows ? 2 * pair + 1 : a.rows - 1;
    const uint8_t *base_a = a.qs + (size_t)row_a * a.qs_row_bytes, *base_b = a.qs + (size_t)row_b * a.qs_row_bytes;
    const Q4KLane L = q4k_lane_constants(lane);

    auto load_item = [&](int t) {
        Q4KItem it;
        const int tt = t < total ? t : 0;
        const bool second = tt >= ipr;
        const int i = tt - (second ? ipr : 0);
        const uint8_t *bp = (second ? base_b : base_a) + (size_t)(i >> 2) * 144;
        it.hdr = *reinterpret_cast<const uint4 *>(bp);
        const uint4 *q = reinterpret_cast<const uint4 *>(bp + 16 + (i & 3) * 32);
        it.q0 = q[0];
        it.q1 = q[1];
        return it;
    };

    float acc_a[B], acc_b[B];
#pragma unroll
    for (int b = 0; b < B; b++) acc_a[b] = acc_b[b] = 0.0f;
    Q4KItem cur = load_item(lane);
    q4k_stage_x<B>(a, cols, xstride, xs4, xsum, norm_red);
    __syncthreads();
    for (int t0 = 0; t0 < total; t0 += 64) {
        Q4KItem nxt = cur;
        if (t0 + 64 < total) nxt = load_item(t0 + 64 + lane);
        const int t = t0 + lane;
        const bool valid = t < total;
        const int tt = valid ? t : 0;
        const bool second = tt >= ipr;
        float v[B];
        q4k_item_dots<B, 0>(cur, L, xs4, xsum, tt - (second ? ipr : 0), xstride, cols, v);
#pragma unroll
        for (int b = 0; b < B; b++) {
            const float vv = valid ? v[b] : 0.0f;
            acc_a[b] += second ? 0.0f : vv;
            acc_b[b] += second ? vv : 0.0f;
        }
        cur = nxt;
    }
#pragma unroll
    for (int b = 0; b < B; b++) {
        acc_a[b] = wave_sum(acc_a[b]);
        acc_b[b] = wave_sum(acc_b[b]);
    }
    if (a.epilogue == EPI_ARGMAX) {
        __shared__ float bv[B * kWaves];
        __shared__ int bi[B * kWaves];
        float best[B];
        int best_i[B];
#pragma unroll
        for (int b = 0; b < B; b++) {
            best[b] = -INFINITY;
            best_i[b] = 0x7FFFFFFF;
            if (2 * pair < a.rows) argmax_take(best[b], best_i[b], acc_a[b], 2 * pair);
            if (2 * pair + 1 < a.rows) argmax_take(best[b], best_i[b], acc_b[b], 2 * pair + 1);
        }
        argmax_workgroup<B>(a, best, best_i, bv, bi);
        return;
    }
    if (lane == 0) pair_epilogue<B>(a, pair, acc_a, acc_b);
}


// ---------------------------------------------------------------------------------------------------------------
// Q4_K GEMV on the matrix cores: up to four activation rows for the price of one.
//
// v_mfma_f32_16x16x32_f16 computes D[i][j] += sum_k A[i][k] B[k][j] with lane l supplying A[l % 16][8 (l / 16) ..+7] and
// B[8 (l / 16) ..+7][l % 16], and holding D[4 (l / 16) + r][l % 16], r = 0..3.  Here j is a weight row: a wavefront owns
// sixteen consecutive rows, and lane (n = l % 16, g = l / 16) works on chunk g (64 weights: sub-blocks 2g in the low
// nibbles, 2g + 1 in the high ones) of every super-block of row n.  The nibbles go into the B operand under an fp16
// exponent (64 + n/16, 4 + n/16), exactly as in the dot-product kernels.  The four lane groups of one instruction hold
// four different sub-blocks, whose scales differ, so their products must not meet in one sum: the sixteen i are used as
// 4 lane groups x 4 activation rows, and slot i = 4 g + b carries activation row b in lane group g ONLY (zeros in the
// other three groups).  D[4 g + b][n] is then the sum over lane group g's eight weights alone, and it lands in lane
// (n, g) - the lane that loaded those weights and holds their super-block header.  Four instructions cover a
// sub-block; scale, minimum and the exponent offsets are folded per lane as in q4k_item_dots.  Only 4 * NB lanes of an A
// operand are not zero: those read the staged activations from LDS, the others read a block of zeros with the same
// offsets.  The vector ALU is left with the nibble masks and the scale arithmetic (about one operation per weight
// whatever the number of activation rows); the dot products cost it nothing, and a row's sum needs no reduction over
// the wavefront because a lane keeps adding to its own row.
//
// The weights come from the matrix's TILED copy (DeviceMatrix::tiled): a tile is (block of sixteen rows, super-block),
// 2304 bytes: sixteen 16-byte headers, then piece (g, n) = the first sixteen bytes of chunk g of row n at 256 + 16 (16 g
// + n), then the second sixteen bytes at 1280 + 16 (16 g + n).  A wavefront's three loads of a step are then three
// contiguous runs (256 B, 1 KiB, 1 KiB); from the row-major GGUF layout the same lanes would touch sixteen different
// cache lines per quarter wavefront, which measures 25 % slower.  Rows are padded to a multiple of sixteen with zero
// blocks (d = dmin = 0), so no load is clamped.
//
// Work: a workgroup of WAVES wavefronts takes WAVES / KS blocks of sixteen rows per round, KS wavefronts sharing a block
// and splitting its super-blocks between them; their partial sums meet in LDS after the last round (one barrier).  The
// grid is persistent; DEPTH super-block steps of packed weights are in flight per wavefront, across rounds.
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
constexpr int kMfmaRounds = 8;   // rounds whose partial sums have an LDS slot of their own (KS > 1)

// Sum over the workgroup's WAVES wavefronts, added in wavefront order; `red` holds WAVES floats.
template <int WAVES>
__device__ __forceinline__ float workgroup_sum_waves(float v, float *red) {
    v = wave_sum(v);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    float t = red[0];
#pragma unroll
    for (int w = 1; w < WAVES; w++) t += red[w];
    return t;
}

// Activations of a row (fp16 as given, RMSNorm fused, or attention states merged) into LDS for the matrix-core kernel:
// every load is issued before the first use, as in Q4KStage; THREADS threads take groups tid, tid + THREADS, ...
// SPLIT (Q4_K): the staged rows are hi / lo pairs (rows 2b and 2b + 1 of the LDS copy, see split_group); fp16 activations given
// (MODE 0) then arrive as such pairs, 2 NB rows.
template <int NB, int IPR, int THREADS, int MODE, bool Q40 = false, bool SPLIT = false>
struct MfmaStage {
    static constexpr int GROUPS = IPR * 8, K = (GROUPS + THREADS - 1) / THREADS, cols = IPR * 64, WAVES = THREADS / 64;
    static constexpr int NBX = SPLIT ? 2 * NB : NB;
    static constexpr bool FULL = GROUPS % THREADS == 0;
    static_assert(!(Q40 && SPLIT), "split activations: Q4_K only");
    float4 v0[MODE == 1 ? NB : 1][K], v1[MODE == 1 ? NB : 1][K], g0[K], g1[K];
    uint4 v[MODE == 0 ? NBX : 1][K];
    float4 a0[MODE == 2 ? K : 1][kMergeSplits], a1[MODE == 2 ? K : 1][kMergeSplits];
    float2 ml[MODE == 2 ? K : 1][kMergeSplits];

    __device__ __forceinline__ int group(int k) const { return FULL || (int)threadIdx.x + k * THREADS < GROUPS ? (int)threadIdx.x + k * THREADS : 0; }
    __device__ __forceinline__ bool mine(int k) const { return FULL || (int)threadIdx.x + k * THREADS < GROUPS; }

    __device__ __forceinline__ void load_merge_row(const KernelArgs &a, int b) {
#pragma unroll
        for (int k = 0; k < K; k++) merge_group_load(a, b, group(k), cols, ml[k], a0[k], a1[k]);
    }
    __device__ __forceinline__ void issue(const KernelArgs &a) {
        if constexpr (MODE == 1) {
            const float4 *w4 = reinterpret_cast<const float4 *>(a.norm_w);
            const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
            for (int k = 0; k < K; k++) {
                const int g = group(k);
                g0[k] = w4[2 * g];
                g1[k] = w4[2 * g + 1];
#pragma unroll
                for (int b = 0; b < NB; b++) {
                    const float4 *x4 = reinterpret_cast<const float4 *>(a.norm_x + (size_t)b * cols);
                    v0[b][k] = x4[2 * g];
                    v1[b][k] = x4[2 * g + 1];
                    if (!mine(k)) v0[b][k] = v1[b][k] = zero;
                }
            }
        } else if constexpr (MODE == 2) {
            load_merge_row(a, 0);
        } else {
#pragma unroll
            for (int b = 0; b < NBX; b++)
#pragma unroll
                for (int k = 0; k < K; k++) v[b][k] = reinterpret_cast<const uint4 *>(a.x)[(size_t)b * (cols / 8) + group(k)];
        }
    }
    __device__ __forceinline__ void finish(const KernelArgs &a, uint4 *xs4, float *xsum, float *red) {
        if constexpr (MODE == 1) {
#pragma unroll
            for (int b = 0; b < NB; b++) {
                float s = 0.0f;
#pragma unroll
                for (int k = 0; k < K; k++) s += sum_squares(v0[b][k], v1[b][k]);
                const float inv = 1.0f / sqrtf(workgroup_sum_waves<WAVES>(s, red + b * WAVES) / (float)cols + a.norm_eps);
#pragma unroll
                for (int k = 0; k < K; k++) {
                    if (!mine(k)) continue;
                    if constexpr (SPLIT) {
                        float c[8];
                        normalized_values(v0[b][k], v1[b][k], g0[k], g1[k], inv, c);
                        q4k_store_split_natural(split_group(c), b, group(k), cols, xs4, xsum);
                    } else {
                        q4k_store_group_natural<Q40>(normalized_group(v0[b][k], v1[b][k], g0[k], g1[k], inv), b, group(k), cols, xs4, xsum);
                    }
                }
            }
        } else if constexpr (MODE == 2) {
#pragma unroll
            for (int b = 0; b < NB; b++) {
                if (b > 0) load_merge_row(a, b);
#pragma unroll
                for (int k = 0; k < K; k++) {
                    if (!mine(k)) continue;
                    if constexpr (SPLIT) {
                        float c[8];
                        merge_group_values(ml[k], a0[k], a1[k], c);
                        q4k_store_split_natural(split_group(c), b, group(k), cols, xs4, xsum);
                    } else {
                        q4k_store_group_natural<Q40>(merge_group(ml[k], a0[k], a1[k]), b, group(k), cols, xs4, xsum);
                    }
                }
            }
        } else {
#pragma unroll
            for (int b = 0; b < NB; b++)
#pragma unroll
                for (int k = 0; k < K; k++) {
                    if (!mine(k)) continue;
                    if constexpr (SPLIT) q4k_store_split_natural(SplitGroup{v[2 * b][k], v[2 * b + 1][k]}, b, group(k), cols, xs4, xsum);
                    else q4k_store_group_natural<Q40>(v[b][k], b, group(k), cols, xs4, xsum);
                }
        }
    }
};

constexpr size_t kQ4KTileBytes = 2304;

template <int NB, int IPR, int WAVES, int KS, int MODE, bool SPLIT = false, bool STAMPS = false>
__global__ __launch_bounds__(WAVES * 64) void gemv_q4k_mfma_kernel(const uint8_t *tiled, const void *activations, const float *norm_w, int rows, int iters,
                                                                   int workgroups, float norm_eps, KernelArgs rest) {
    KernelArgs a = rest;
    a.rows = rows;
    if constexpr (MODE == 1) { a.norm_x = static_cast<const float *>(activations); a.norm_w = norm_w; a.norm_eps = norm_eps; }
    else if constexpr (MODE == 2) a.merge_partials = static_cast<const float *>(activations);
    else a.x = static_cast<const uint16_t *>(activations);
    constexpr int THREADS = WAVES * 64, cols = IPR * 64, NSB = IPR / 4, S = NSB / KS, RB = WAVES / KS, GROUPS = cols / 8;
    constexpr int DEPTH = S % 4 == 0 ? 4 : (S % 7 == 0 ? 7 : (S % 2 == 0 ? 2 : 1));   // divides S: a step's slot in the ring is a constant
    constexpr int NBX = SPLIT ? 2 * NB : NB;   // staged fp16 rows: with split activations row b is the pair (2b: hi, 2b + 1: lo)
    constexpr int SETS = (NBX + 3) / 4;   // staged rows 4 s .. 4 s + 3 ride in the slots of A operand set s; every set meets the same B operand
    static_assert(NSB % KS == 0 && WAVES % KS == 0 && NB >= 1 && NBX <= 8, "whole super-blocks per wavefront");
    extern __shared__ uint4 smem_raw[];
    uint4 *xs4 = smem_raw;                                        // [NBX][GROUPS] groups of eight fp16, (0,2,1,3) order inside fours
    uint4 *zero4 = xs4 + (size_t)NBX * GROUPS;                    // eight groups of zeros
    float *xsum = reinterpret_cast<float *>(zero4 + 8);           // [NB][cols / 32]
    float *red = xsum + (size_t)NB * (cols / 32);                 // [kMfmaRounds][WAVES][NB][16]   (KS > 1)
    float *misc = red + (KS > 1 ? kMfmaRounds * WAVES * NB * 16 : 0);   // [NB][WAVES] norm sums, later [2][NB][WAVES] arg-max candidates
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n = lane & 15, g = lane >> 4, ks = wave % KS, team = wave / KS;
    const int row_blocks = (a.rows + 15) >> 4;
    const Q4KLane L = q4k_chunk_constants(g);
    // constants of the nibble trick, hidden from the optimiser so that (w & mask) | magic stays one v_and_or_b32
    u32 mask_lo = 0x000F000Fu, mask_hi = 0x00F000F0u, magic_lo = 0x54005400u, magic_hi = 0x44004400u;
    asm volatile("" : "+s"(mask_lo), "+s"(mask_hi));
    asm volatile("" : "+v"(magic_lo), "+v"(magic_hi));

    // ---- packed weights: step f of this wavefront = (round f / S, super-block ks * S + f % S of its row block) ----
    // The last round is ragged and goes to the workgroups with the lowest indices: they are dispatched first, get their first
    // weights first (the opening burst of loads is served roughly in order) and stay ahead to the end, so one round more for
    // them evens the finish.
    {
        const int units = (row_blocks + RB - 1) / RB;   // a unit = the RB row blocks a workgroup takes per round
        iters = (units - (int)blockIdx.x + workgroups - 1) / workgroups;
        if (iters < 0) iters = 0;
    }
    const int total_steps = iters * S;
    auto block_of = [&](int round) { return (round * workgroups + (int)blockIdx.x) * RB + team; };
    // Every load of the ring is issued unconditionally: a load under a branch makes the compiler wait for all loads in flight
    // wherever it needs any of them (it cannot count what was issued), which would tie the staging of the activations and every
    // step of the ring to the arrival of the newest weights.  Steps past the end read sixteen bytes that every lane shares.
    auto load_step = [&](int f) {
        Q4KItem it;
        const bool real = f < total_steps;
        const int round = f / S, step = f - round * S;
        const int rb = block_of(round) < row_blocks ? block_of(round) : row_blocks - 1;   // blocks past the end repeat the last one; never stored
        const uint8_t *tp = real ? tiled + ((size_t)rb * NSB + (ks * S + step)) * kQ4KTileBytes : tiled;
        const int spread = real ? 16 : 0;
        it.hdr = *reinterpret_cast<const uint4 *>(tp + spread * n);
        it.q0 = *reinterpret_cast<const uint4 *>(tp + (real ? 256 : 0) + spread * lane);
        it.q1 = *reinterpret_cast<const uint4 *>(tp + (real ? 1280 : 0) + spread * lane);
        return it;
    };

    stamp<STAMPS>(a, 0);
    // Activations given as fp16 and K split over all wavefronts of the workgroup: a wavefront needs only its own S super-block columns
    // of them, stages those by itself and waits for no other wavefront (LDS operations of one wavefront complete in order).  Used at
    // 14336 columns (4096 x 14336 in a train: 9.0 against 9.3 us for one row, 10.1 against 10.4 for two) and for two and more rows;
    // at 4096 columns the common staging measures better for one row (14336 x 4096: 9.4 against 9.8 us; two rows 10.2 against 10.4-10.7).
    constexpr bool PRIVATE = MODE == 0 && KS == WAVES && (IPR >= 128 || NBX >= 2);
    constexpr int SLICE = S * 32, KW = (SLICE + 63) / 64;          // groups of eight columns in a wavefront's share
    MfmaStage<NB, IPR, THREADS, MODE, false, SPLIT> stage;
    uint4 own[PRIVATE ? NBX : 1][PRIVATE ? KW : 1];
    if constexpr (PRIVATE) {
#pragma unroll
        for (int b = 0; b < NBX; b++)
#pragma unroll
            for (int k = 0; k < KW; k++) {
                const int gi = lane + 64 * k;
                own[b][k] = reinterpret_cast<const uint4 *>(a.x)[(size_t)b * GROUPS + SLICE * ks + (gi < SLICE ? gi : 0)];
            }
    } else {
        stage.issue(a);
    }
    // AHEAD steps (of 2.3 KB per wavefront) are in flight per wavefront.  The ring has a slot per step of a round, up to seven (14336
    // columns), so that a step's slot is a constant; but a compute unit's memory pipeline takes about 50-70 KB at once, and what is
    // issued beyond that blocks the issuing wavefront - and with it the barrier below and the start of the arithmetic - until the
    // first weights have arrived.  Measured in the 8B decode step (same box, alternating): one step ahead instead of two for the
    // 4096-column kernels with eight wavefronts (two workgroups per compute unit: 37 KB in flight instead of 74) 723 against 711
    // tok/s; three steps ahead instead of seven at 14336 columns (55 KB per compute unit instead of 129) 9.3 against 11.4 us per
    // launch, two or four steps ahead measure the same or slightly worse.  Four-step rings stay full: they belong to four-wavefront
    // workgroups (37 KB per workgroup), and the 128256-row head measures 54.3 us with four steps ahead, 57.0 with two, 67.3 with one.
    constexpr int AHEAD = DEPTH == 2 ? 1 : DEPTH == 7 ? 3 : DEPTH;
    Q4KItem ring[DEPTH];
#pragma unroll
    for (int d = 0; d < AHEAD; d++) ring[d] = load_step(d);
    if constexpr (PRIVATE) {
        if (lane < 8) zero4[lane] = make_uint4(0, 0, 0, 0);        // every wavefront writes the same zeros
#pragma unroll
        for (int b = 0; b < NB; b++)
#pragma unroll
            for (int k = 0; k < KW; k++)
                if (SLICE % 64 == 0 || lane + 64 * k < SLICE) {
                    if constexpr (SPLIT) q4k_store_split_natural(SplitGroup{own[2 * b][k], own[2 * b + 1][k]}, b, SLICE * ks + lane + 64 * k, cols, xs4, xsum);
                    else q4k_store_group_natural(own[b][k], b, SLICE * ks + lane + 64 * k, cols, xs4, xsum);
                }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    } else {
        if (tid < 8) zero4[tid] = make_uint4(0, 0, 0, 0);
        stage.finish(a, xs4, xsum, misc);
        __syncthreads();
    }
    stamp<STAMPS>(a, 1);

    // ---- the A operand: slot i = lane % 16 carries staged row i % 4 in lane group i / 4 only ----
    const int slot = lane & 15;
    const uint4 *a_base[SETS];
    int a_stride[SETS];                                            // groups per super-block step
#pragma unroll
    for (int set = 0; set < SETS; set++) {
        const bool feeds = (slot >> 2) == g && 4 * set + (slot & 3) < NBX;
        a_base[set] = feeds ? xs4 + (size_t)(4 * set + (slot & 3)) * GROUPS + 32 * (ks * S) + 8 * g : zero4;
        a_stride[set] = feeds ? 32 : 0;
    }
    const float *xsum_base = xsum + 8 * (ks * S) + 2 * g;

    float v[NB];
    auto step_compute = [&](const Q4KItem &it, int i) {            // i: step inside the round (a constant where unrolled)
        const uint4 *ap[SETS];
        floatx4 lo[SETS], hi[SETS];
#pragma unroll
        for (int set = 0; set < SETS; set++) {
            ap[set] = a_base[set] + i * a_stride[set];
            lo[set] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
            hi[set] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
        }
        const u32 qd[8] = {it.q0.x, it.q0.y, it.q0.z, it.q0.w, it.q1.x, it.q1.y, it.q1.z, it.q1.w};
#pragma unroll
        for (int jj = 0; jj < 4; jj++) {
            const u32 w0 = qd[2 * jj], w1 = qd[2 * jj + 1];
            const uint4 pl = make_uint4((w0 & mask_lo) | magic_lo, ((w0 >> 8) & mask_lo) | magic_lo, (w1 & mask_lo) | magic_lo, ((w1 >> 8) & mask_lo) | magic_lo);
            const uint4 ph = make_uint4((w0 & mask_hi) | magic_hi, ((w0 >> 8) & mask_hi) | magic_hi, (w1 & mask_hi) | magic_hi, ((w1 >> 8) & mask_hi) | magic_hi);
#pragma unroll
            for (int set = 0; set < SETS; set++) {
                lo[set] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, ap[set][jj]), __builtin_bit_cast(half8, pl), lo[set], 0, 0, 0);
                hi[set] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, ap[set][4 + jj]), __builtin_bit_cast(half8, ph), hi[set], 0, 0, 0);
            }
        }
        // 6-bit (scale, min) of sub-blocks 2g and 2g + 1, as in q4k_item_dots
        const u32 src_sc = L.upper ? it.hdr.w : it.hdr.y, src_min = L.upper ? it.hdr.w : it.hdr.z;
        const u32 scp = ((src_sc >> L.sh_sc) & L.mask_low) | ((it.hdr.y >> L.sh_top) & L.mask_top);
        const u32 mp = ((src_min >> L.sh_min) & L.mask_low) | ((it.hdr.z >> L.sh_top) & L.mask_top);
        const float sc_lo = (float)(scp & 0xFFu), sc_hi = (float)((scp >> 8) & 0xFFu);
        const float m_lo = (float)(mp & 0xFFu), m_hi = (float)((mp >> 8) & 0xFFu);
        const float d16 = 16.0f * half_bits_to_float(it.hdr.x & 0xFFFFu), dmin = half_bits_to_float(it.hdr.x >> 16);
#pragma unroll
        for (int b = 0; b < NB; b++) {
            const float2 xsp = *reinterpret_cast<const float2 *>(xsum_base + (size_t)b * (cols >> 5) + 8 * i);
            float raw_lo, raw_hi;
            if constexpr (SPLIT) {   // the sums over the hi and the lo row of the pair
                const int r0 = 2 * b, r1 = 2 * b + 1;
                raw_lo = __builtin_fmaf(lo[r1 >> 2][r1 & 3], kSplitUnscale, lo[r0 >> 2][r0 & 3]);
                raw_hi = __builtin_fmaf(hi[r1 >> 2][r1 & 3], kSplitUnscale, hi[r0 >> 2][r0 & 3]);
            } else {
                raw_lo = lo[b >> 2][b & 3];
                raw_hi = hi[b >> 2][b & 3];
            }
            const float nx_lo = raw_lo - 64.0f * xsp.x, nx_hi = raw_hi - 4.0f * xsp.y;
            v[b] += d16 * (sc_lo * nx_lo + sc_hi * nx_hi) - dmin * (m_lo * xsp.x + m_hi * xsp.y);
        }
    };

    // rows n = 2q, 2q + 1 of a block are a pair: the even lane of each pair among lanes 0..15 runs the epilogue.  The
    // arg-max epilogue keeps a running first maximum per lane instead (rows only grow from round to round).
    float best[NB];
    int best_i[NB];
#pragma unroll
    for (int b = 0; b < NB; b++) { best[b] = -INFINITY; best_i[b] = 0x7FFFFFFF; }
    auto finish_block = [&](int rb, float (&sum)[NB]) {            // sum[b]: the row's total, valid in lanes 0..15
        if (a.epilogue == EPI_ARGMAX) {
            const int row = rb * 16 + lane;
            if (lane < 16 && row < a.rows) {
#pragma unroll
                for (int b = 0; b < NB; b++) argmax_take(best[b], best_i[b], sum[b], row);
            }
            return;
        }
        float other[NB];
#pragma unroll
        for (int b = 0; b < NB; b++) other[b] = dpp_term<0xB1, 0xF>(sum[b]);   // the neighbouring lane's row
        if (lane < 16 && (lane & 1) == 0 && rb < row_blocks) pair_epilogue<NB>(a, rb * 8 + (lane >> 1), sum, other);
    };

    for (int round = 0; round < iters; round++) {
#pragma unroll
        for (int b = 0; b < NB; b++) v[b] = 0.0f;
#pragma unroll
        for (int i = 0; i < S; i++) {
            const Q4KItem it = ring[i % DEPTH];
            ring[(i + AHEAD) % DEPTH] = load_step(round * S + i + AHEAD);
            step_compute(it, i);
            // long rounds (the head's sixteen steps): without a fence between the unrolled steps the scheduler interleaves them all and
            // the kernel spills (1.3 KB of scratch per lane, 270 us instead of 47 us for the 128256-row head)
            if constexpr (S > 8) __builtin_amdgcn_sched_barrier(0);
            if constexpr (STAMPS) { if (a.stamps && round == 0 && i == 0 && v[0] != 12345.678f) stamp<STAMPS>(a, 2); }   // after the first weights were needed
        }
#pragma unroll
        for (int b = 0; b < NB; b++) {          // the four lane groups of a row: every lane ends up with the row's share
            v[b] += __shfl_xor(v[b], 16);
            v[b] += __shfl_xor(v[b], 32);
        }
        if constexpr (KS == 1) {
            finish_block(block_of(round), v);
        } else {
            float *slot_base = red + ((size_t)(round % kMfmaRounds) * WAVES + wave) * NB * 16;
            if (lane < 16) {
#pragma unroll
                for (int b = 0; b < NB; b++) slot_base[b * 16 + lane] = v[b];
            }
        }
    }

    if constexpr (KS > 1) {
        __syncthreads();
        // wavefront ks == 0 of each team adds the team's shares (wavefront order, lane groups in order) and finishes its blocks
        if (ks == 0) {
            for (int round = 0; round < iters; round++) {
                float sum[NB];
#pragma unroll
                for (int b = 0; b < NB; b++) {
                    float t = 0.0f;
                    if (lane < 16) {
#pragma unroll
                        for (int w = 0; w < KS; w++) t += red[((size_t)(round % kMfmaRounds) * WAVES + wave + w) * NB * 16 + b * 16 + lane];
                    }
                    sum[b] = t;
                }
                finish_block(block_of(round), sum);
            }
        }
    }

    stamp<STAMPS>(a, 3);
    if (a.epilogue == EPI_ARGMAX) {
        // lanes 0..15 of the finishing wavefronts hold candidates: first within the wavefront, then over the workgroup
        float *cv = misc;
        int *ci = reinterpret_cast<int *>(misc + NB * WAVES);
        __syncthreads();   // misc was the norm's scratch
#pragma unroll
        for (int b = 0; b < NB; b++) {
#pragma unroll
            for (int off = 8; off >= 1; off >>= 1) {
                const float ov = __shfl_xor(best[b], off);
                const int oi = __shfl_xor(best_i[b], off);
                argmax_take(best[b], best_i[b], ov, oi);
            }
            if (lane == 0) { cv[b * WAVES + wave] = ks == 0 ? best[b] : -INFINITY; ci[b * WAVES + wave] = ks == 0 ? best_i[b] : 0x7FFFFFFF; }
        }
        __syncthreads();
        if (tid < NB) {
            float bv = cv[tid * WAVES];
            int bi = ci[tid * WAVES];
#pragma unroll
            for (int w = 1; w < WAVES; w++) argmax_take(bv, bi, cv[tid * WAVES + w], ci[tid * WAVES + w]);
            a.part_value[(size_t)tid * gridDim.x + blockIdx.x] = bv;
            a.part_index[(size_t)tid * gridDim.x + blockIdx.x] = bi;
        }
    }
}


// ---- Q4_K, five to eight activation rows in one pass over the tiled copy ----------------------------------------------------------
// The slot trick above spends three quarters of the A operand on keeping lane groups apart, so that each lane can fold its own
// sub-block's scale after the MFMA: four rows per MFMA set, and the fold's vector work grows with the rows (eight rows: 18.7 us at
// 14336 x 4096 where four take 10.5).  Here the scale is folded into the B operand instead: the nibble becomes the exact integer
// sc * q (at most 63 * 15, exact in fp16) with one v_and_or_b32 and one packed fused multiply-add per two weights
// ((1024 + q) * sc - 1024 * sc for low nibbles, (64 + q) * sc - 64 * sc for high ones), the rows of A carry activation rows, one
// accumulator runs over the whole super-block and d is applied to it once.  The minimum term d_min * sum_k x_k * m_sub(k) comes from
// a second MFMA chain over the same A fragments whose B operand is the lane's own sub-block minimum, repeated (the k values a lane
// feeds all belong to its chunk's two sub-blocks).  Products are exact and sums fp32, as in the kernels above; the vector work per
// tile does not depend on the number of rows.  Lane (i, g) of the A operand needs the 64 columns of chunk g of activation row i,
// each group of four in the order in which nibbles unpack (0, 2, 1, 3).  Read straight from memory those are sixteen-byte pieces
// 128 bytes apart within an instruction, and the cache-line accesses, not the bytes, bound the kernel (15-18 us at eight rows); so
// the activations go through LDS, in one of two ways:
//   XMODE 1 (4096 columns, tall matrices): the workgroup stages all rows once (eight rows: 64 KB; rows 16 bytes apart in the banks,
//           so that the reads of a lane group do not collide) and every round reuses them;
//   XMODE 2 (any width): the wavefront fetches its tile's 8 x 256 activations with four fully coalesced loads (two rows of 512 bytes
//           per instruction, one step ahead like the weights), writes them to four kilobytes of LDS of its own and reads the fragments
//           from there: no workgroup barrier, nothing resident beyond the tile.
// Rows of A past the batch repeat live rows; their products land in accumulator rows that are never stored.
//
// Q40: the same kernel for Q4_0 (tiled copy of sixteen rows x 512 columns, see gemv_q40_mfma_kernel below; a step here is half a
// tile).  A block's one scale is an arbitrary fp16 number and cannot go into the B operand exactly, so every MFMA contracts exactly
// one 32-weight block for all sixteen weight rows: lane (n, g) needs dword g of each of the half tile's eight blocks of row n, which it
// gets from the whole blocks the four lane groups loaded by a transpose in registers (v_permlane32_swap / v_permlane16_swap; as
// four-byte loads the same bytes cost sixteen memory instructions per step instead of seven and the kernel 15.4 / 16.5 us instead of
// 11.4 / 12.3 at 14336 x 4096 / 4096 x 14336, eight rows); B is the exact integer q - 8 ((1024 + q) - 1032,
// (64 + q) - 72: one v_and_or_b32 and one packed add per two weights), and the block's scale multiplies the four accumulator
// registers afterwards.  A lane's eight k values are weights 4 g .. 4 g + 3 and 16 + 4 g .. 16 + 4 g + 3 of the block: two eight-byte
// reads of the staged activations.
constexpr int kWideRounds = 4;            // rounds whose partial sums have an LDS slot of their own
constexpr size_t kQ40TileBytes = 4608;
// XMODE 2: bytes between the rows of a wavefront's tile of activations in LDS; the pad spreads the eight rows over the banks for
// sixteen-byte (Q4_K) and eight-byte (Q4_0) reads
constexpr int wide_row_bytes(bool q40) { return 512 + (q40 ? 32 : 16); }

// v_permlane32_swap exchanges the upper 32 lanes of its first operand with the lower 32 of its second, v_permlane16_swap the odd
// sixteen-lane rows of the first with the even rows of the second: two of each transpose four registers over the four lane groups.
__device__ __forceinline__ uint4 transpose_lane_groups(const uint4 &q) {
    const auto a = __builtin_amdgcn_permlane32_swap(q.x, q.z, false, false);
    const auto b = __builtin_amdgcn_permlane32_swap(q.y, q.w, false, false);
    const auto c = __builtin_amdgcn_permlane16_swap(a[0], b[0], false, false);
    const auto d = __builtin_amdgcn_permlane16_swap(a[1], b[1], false, false);
    return make_uint4(c[0], c[1], d[0], d[1]);
}
// .x .. .w = the value that lane groups 0 .. 3 hold in the same lane % 16
__device__ __forceinline__ uint4 gather_lane_groups(u32 v) {
    const auto a = __builtin_amdgcn_permlane32_swap(v, v, false, false);      // rows (v0 v1 v0 v1), (v2 v3 v2 v3)
    const auto c = __builtin_amdgcn_permlane16_swap(a[0], a[0], false, false);
    const auto d = __builtin_amdgcn_permlane16_swap(a[1], a[1], false, false);
    return make_uint4(c[0], c[1], d[0], d[1]);
}

template <int XMODE>
struct Q4KWideItem {
    uint4 q0, q1, hdr;              // Q4_0: q0, q1 = the lane's two blocks of the half tile, hdr.x = their scales
    uint4 xa[XMODE == 2 ? 4 : 1];   // XMODE 2: sixteen bytes of row 2 j + lane / 32 at 16 (lane % 32), j = 0..3
};

template <int IPR, int WAVES, int KS, int XMODE, bool Q40 = false>
__global__ __launch_bounds__(WAVES * 64, 4) void gemv_q4k_wide_kernel(const uint8_t *tiled, const uint16_t *x, int rows, int batch, int workgroups,
                                                                      KernelArgs rest) {
    KernelArgs a = rest;
    a.rows = rows;
    constexpr int cols = IPR * 64, NSB = IPR / 4, S = NSB / KS, RB = WAVES / KS, THREADS = WAVES * 64;
    constexpr int XROW = cols * 2 + (Q40 ? 32 : 16);                // XMODE 1: bytes between staged rows
    constexpr int kWideRowBytes = wide_row_bytes(Q40);
    static_assert(NSB % KS == 0 && WAVES % KS == 0 && (XMODE == 1 || XMODE == 2), "whole super-blocks per wavefront");
    extern __shared__ float4 wide_red[];                            // [kWideRounds][WAVES][64] partial sums (four rows per lane)
    // XMODE 1: [8 rows][XROW]; XMODE 2: [WAVES][8 rows][kWideRowBytes]
    uint8_t *xs = reinterpret_cast<uint8_t *>(wide_red + (size_t)kWideRounds * WAVES * 64);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n = lane & 15, g = lane >> 4, ks = wave % KS, team = wave / KS;
    const int row_blocks = (a.rows + 15) >> 4;
    const Q4KLane L = q4k_chunk_constants(g);
    u32 mask_lo = 0x000F000Fu, mask_hi = 0x00F000F0u, magic_lo = 0x64006400u, magic_hi = 0x54005400u;
    asm volatile("" : "+s"(mask_lo), "+s"(mask_hi));
    asm volatile("" : "+v"(magic_lo), "+v"(magic_hi));

    const int units = (row_blocks + RB - 1) / RB;
    int iters = (units - (int)blockIdx.x + workgroups - 1) / workgroups;
    if (iters < 0) iters = 0;
    const int total_steps = iters * S;
    auto block_of = [&](int round) { return (round * workgroups + (int)blockIdx.x) * RB + team; };
    // XMODE 2: rows 2 j + lane / 32 of the batch (rows past it repeat the last one)
    const uint8_t *xtile = reinterpret_cast<const uint8_t *>(x) + (size_t)ks * S * 512 + 16 * (lane & 31);
    size_t xrow2[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int r = 2 * j + (lane >> 5);
        xrow2[j] = (size_t)(r < batch ? r : batch - 1) * cols * 2;
    }
    uint8_t *xw = xs + (size_t)wave * 8 * kWideRowBytes;            // XMODE 2: this wavefront's tile
    auto load_step = [&](int f) {                                   // every load unconditional, addresses clamped (as above)
        Q4KWideItem<XMODE> it;
        const bool real = f < total_steps;
        const int round = f / S, step = f - round * S;
        const int rb = block_of(round) < row_blocks ? block_of(round) : row_blocks - 1;
        if constexpr (Q40) {
            // whole blocks as the tile holds them: lane (n, g) gets blocks (2 half, g) and (2 half + 1, g) of row n and their two scales
            const int unit = ks * S + step, half = unit & 1;
            const uint8_t *tp = real ? tiled + ((size_t)rb * (NSB / 2) + (unit >> 1)) * kQ40TileBytes + 2048 * half : tiled;
            const int spread = real ? 16 : 0;
            it.q0 = *reinterpret_cast<const uint4 *>(tp + spread * lane);
            it.q1 = *reinterpret_cast<const uint4 *>(tp + (real ? 1024 : 0) + spread * lane);
            it.hdr.x = *reinterpret_cast<const u32 *>(tp + (real ? 4096 - 2048 * half + 4 * half : 0) + (real ? 8 : 0) * lane);
        } else {
            const uint8_t *tp = real ? tiled + ((size_t)rb * NSB + (ks * S + step)) * kQ4KTileBytes : tiled;
            const int spread = real ? 16 : 0;
            it.hdr = *reinterpret_cast<const uint4 *>(tp + spread * n);
            it.q0 = *reinterpret_cast<const uint4 *>(tp + (real ? 256 : 0) + spread * lane);
            it.q1 = *reinterpret_cast<const uint4 *>(tp + (real ? 1280 : 0) + spread * lane);
        }
        if constexpr (XMODE == 2) {
            const uint8_t *xp = xtile + (real ? step * 512 : 0);
#pragma unroll
            for (int j = 0; j < 4; j++) it.xa[j] = *reinterpret_cast<const uint4 *>(xp + xrow2[j]);
        }
        return it;
    };

    float v[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    auto nibble_order = [](const uint4 &t) {                        // (x0 x1)(x2 x3)(x4 x5)(x6 x7) -> (x0 x2)(x1 x3)(x4 x6)(x5 x7)
        uint4 r;
        r.x = __builtin_amdgcn_perm(t.y, t.x, 0x05040100u);
        r.y = __builtin_amdgcn_perm(t.y, t.x, 0x07060302u);
        r.z = __builtin_amdgcn_perm(t.w, t.z, 0x05040100u);
        r.w = __builtin_amdgcn_perm(t.w, t.z, 0x07060302u);
        return r;
    };
    // lane (i = n, g) of the A operand: chunk g of row i % 8.  XMODE 1: of the staged rows, by super-block column; XMODE 2: of the tile
    const int xg = Q40 ? 8 * g : 128 * g;
    const uint8_t *xl = XMODE == 1 ? xs + (n & 7) * XROW + xg + ks * S * 512 : xw + (n & 7) * kWideRowBytes + xg;
    auto step_compute = [&](const Q4KWideItem<XMODE> &it, int f) {
        const int round = f / S, step = f - round * S;
        if constexpr (XMODE == 2) {
            // LDS operations of one wavefront complete in order: the reads of the previous step are done before these writes land
#pragma unroll
            for (int j = 0; j < 4; j++)
                *reinterpret_cast<uint4 *>(xw + (2 * j + (lane >> 5)) * kWideRowBytes + 16 * (lane & 31)) = nibble_order(it.xa[j]);
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
        const uint8_t *xp = XMODE == 1 ? xl + step * 512 : xl;
        if constexpr (Q40) {
            // dword g of every block of the half tile, and every block's scale, from the lanes that loaded them: a 4 x 4 transpose
            // over the four lane groups (register r of group g <-> register g of group r) and an all-gather of the scale dword
            const uint4 t0 = transpose_lane_groups(it.q0), t1 = transpose_lane_groups(it.q1);
            const u32 qd[8] = {t0.x, t0.y, t0.z, t0.w, t1.x, t1.y, t1.z, t1.w};
            const uint4 ds4 = gather_lane_groups(it.hdr.x);
            const u32 dsc[4] = {ds4.x, ds4.y, ds4.z, ds4.w};
            const h2 c_lo = {(_Float16)-1032.0f, (_Float16)-1032.0f}, c_hi = {(_Float16)-72.0f, (_Float16)-72.0f};
#pragma unroll
            for (int b = 0; b < 8; b++) {
                const u32 w = qd[b];
                uint4 pb;
                pb.x = __builtin_bit_cast(u32, as_h2((w & mask_lo) | magic_lo) + c_lo);           // weights 4 g, 4 g + 2
                pb.y = __builtin_bit_cast(u32, as_h2(((w >> 8) & mask_lo) | magic_lo) + c_lo);    // 4 g + 1, 4 g + 3
                pb.z = __builtin_bit_cast(u32, as_h2((w & mask_hi) | magic_hi) + c_hi);           // 16 + 4 g, 16 + 4 g + 2
                pb.w = __builtin_bit_cast(u32, as_h2(((w >> 8) & mask_hi) | magic_hi) + c_hi);    // 16 + 4 g + 1, 16 + 4 g + 3
                const uint2 x_lo = *reinterpret_cast<const uint2 *>(xp + 64 * b), x_hi = *reinterpret_cast<const uint2 *>(xp + 64 * b + 32);
                const uint4 pa = make_uint4(x_lo.x, x_lo.y, x_hi.x, x_hi.y);
                const floatx4 acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, pa), __builtin_bit_cast(half8, pb),
                                                                           floatx4{0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
                const float d = half_bits_to_float(b < 4 ? dsc[b] & 0xFFFFu : dsc[b - 4] >> 16);
#pragma unroll
                for (int r = 0; r < 4; r++) v[r] = __builtin_fmaf(d, acc[r], v[r]);
            }
        } else {
        const u32 qd[8] = {it.q0.x, it.q0.y, it.q0.z, it.q0.w, it.q1.x, it.q1.y, it.q1.z, it.q1.w};
        const u32 src_sc = L.upper ? it.hdr.w : it.hdr.y, src_min = L.upper ? it.hdr.w : it.hdr.z;
        const u32 scp = ((src_sc >> L.sh_sc) & L.mask_low) | ((it.hdr.y >> L.sh_top) & L.mask_top);
        const u32 mp = ((src_min >> L.sh_min) & L.mask_low) | ((it.hdr.z >> L.sh_top) & L.mask_top);
        const _Float16 s0 = (_Float16)(unsigned short)(scp & 0xFFu), s1 = (_Float16)(unsigned short)((scp >> 8) & 0xFFu);
        const _Float16 m0 = (_Float16)(unsigned short)(mp & 0xFFu), m1 = (_Float16)(unsigned short)((mp >> 8) & 0xFFu);
        const h2 s_lo = {s0, s0}, s_hi = {s1, s1};
        const h2 o_lo = s_lo * (h2){(_Float16)-1024.0f, (_Float16)-1024.0f}, o_hi = s_hi * (h2){(_Float16)-64.0f, (_Float16)-64.0f};
        const u32 mm0 = __builtin_bit_cast(u32, (h2){m0, m0}), mm1 = __builtin_bit_cast(u32, (h2){m1, m1});
        const uint4 bm_lo = make_uint4(mm0, mm0, mm0, mm0), bm_hi = make_uint4(mm1, mm1, mm1, mm1);
        floatx4 acc = {0.0f, 0.0f, 0.0f, 0.0f}, accm = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int jj = 0; jj < 4; jj++) {
            const u32 w0 = qd[2 * jj], w1 = qd[2 * jj + 1];
            uint4 pl, ph;
            pl.x = __builtin_bit_cast(u32, __builtin_elementwise_fma(as_h2((w0 & mask_lo) | magic_lo), s_lo, o_lo));
            pl.y = __builtin_bit_cast(u32, __builtin_elementwise_fma(as_h2(((w0 >> 8) & mask_lo) | magic_lo), s_lo, o_lo));
            pl.z = __builtin_bit_cast(u32, __builtin_elementwise_fma(as_h2((w1 & mask_lo) | magic_lo), s_lo, o_lo));
            pl.w = __builtin_bit_cast(u32, __builtin_elementwise_fma(as_h2(((w1 >> 8) & mask_lo) | magic_lo), s_lo, o_lo));
            ph.x = __builtin_bit_cast(u32, __builtin_elementwise_fma(as_h2((w0 & mask_hi) | magic_hi), s_hi, o_hi));
            ph.y = __builtin_bit_cast(u32, __builtin_elementwise_fma(as_h2(((w0 >> 8) & mask_hi) | magic_hi), s_hi, o_hi));
            ph.z = __builtin_bit_cast(u32, __builtin_elementwise_fma(as_h2((w1 & mask_hi) | magic_hi), s_hi, o_hi));
            ph.w = __builtin_bit_cast(u32, __builtin_elementwise_fma(as_h2(((w1 >> 8) & mask_hi) | magic_hi), s_hi, o_hi));
            // low nibbles of the chunk: columns 8 jj .. 8 jj + 7 of its first half, high nibbles: of its second half
            const half8 a_lo = *reinterpret_cast<const half8 *>(xp + 16 * jj), a_hi = *reinterpret_cast<const half8 *>(xp + 64 + 16 * jj);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a_lo, __builtin_bit_cast(half8, pl), acc, 0, 0, 0);
            accm = __builtin_amdgcn_mfma_f32_16x16x32_f16(a_lo, __builtin_bit_cast(half8, bm_lo), accm, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a_hi, __builtin_bit_cast(half8, ph), acc, 0, 0, 0);
            accm = __builtin_amdgcn_mfma_f32_16x16x32_f16(a_hi, __builtin_bit_cast(half8, bm_hi), accm, 0, 0, 0);
        }
        const float d = half_bits_to_float(it.hdr.x & 0xFFFFu), dmin = half_bits_to_float(it.hdr.x >> 16);
#pragma unroll
        for (int r = 0; r < 4; r++) v[r] += d * acc[r] - dmin * accm[r];
        }
        if (step == S - 1) {                                        // the round's last step: this wavefront's share of sixteen rows x sixteen
            wide_red[((size_t)(round % kWideRounds) * WAVES + wave) * 64 + lane] = make_float4(v[0], v[1], v[2], v[3]);
            v[0] = v[1] = v[2] = v[3] = 0.0f;
        }
    };

    // two slots, each filled while the other is consumed
    Q4KWideItem<XMODE> even = load_step(0);
    if constexpr (XMODE == 1) {
        // the first weights are on their way; every thread stages its share of the batch's rows, in nibble order
        constexpr int GROUPS = cols / 8;
        for (int idx = tid; idx < 8 * GROUPS; idx += THREADS) {
            const int row = idx / GROUPS, grp = idx - row * GROUPS;
            const uint4 t = reinterpret_cast<const uint4 *>(x)[(size_t)(row < batch ? row : batch - 1) * GROUPS + grp];
            *reinterpret_cast<uint4 *>(xs + row * XROW + 16 * grp) = nibble_order(t);
        }
        __syncthreads();
    }
    for (int f = 0; f < total_steps; f += 2) {
        Q4KWideItem<XMODE> odd = load_step(f + 1);
        step_compute(even, f);
        even = load_step(f + 2);
        if (f + 1 < total_steps) step_compute(odd, f + 1);
    }
    __syncthreads();
    // wavefront ks == 0 of each team adds the team's shares in wavefront order and stores: lane (n, g) holds weight row n of the
    // block for activation rows 4 g .. 4 g + 3
    if (ks == 0) {
        for (int round = 0; round < iters; round++) {
            const int rb = block_of(round);
            float4 t = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
#pragma unroll
            for (int w = 0; w < KS; w++) {
                const float4 p = wide_red[((size_t)(round % kWideRounds) * WAVES + wave + w) * 64 + lane];
                t.x += p.x; t.y += p.y; t.z += p.z; t.w += p.w;
            }
            const int row = rb * 16 + n;
            if (rb < row_blocks && row < a.rows) {
                const float out[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int b = 4 * g + r;
                    if (b < batch) {
                        const size_t o = (size_t)b * a.rows + row;
                        a.y[o] = a.epilogue == EPI_ADD_RESIDUAL ? a.residual[o] + out[r] : out[r];
                    }
                }
            }
        }
    }
}


// ---- Q4_0 on the matrix cores ---------------------------------------------------------------------------------------------------
// The same scheme as gemv_q4k_mfma_kernel for Q4_0's 32-weight blocks.  The tiled copy holds, per (sixteen rows, 512 columns),
// four kilobytes of nibbles as [j][lane] 16 bytes (lane (n, g) owns blocks 4 j + g, j = 0..3, of row n) and then [lane][j] fp16
// scales: four contiguous 1 KB loads and one of 512 bytes per wavefront and tile.  The four MFMAs of a block (low and high nibbles
// of its two byte halves) share the block's one scale and hence one accumulator: w = d (n - 8) = d (16 acc - 1032 Sx_first16 -
// 72 Sx_last16) with the low nibbles read as 64 + n / 16 and the high ones as 4 + n / 16 (staged beside the activations per block).
// rounds whose partial sums have an LDS slot of their own (KS > 1): sixteen at 4096 columns (a 128256-row head needs eleven), eight
// at 14336 columns, where four activation rows leave no room for more
constexpr int q40_rounds(int tpr) { return tpr >= 28 ? 8 : 16; }
struct Q40Item { uint4 q[4]; uint2 d; };

template <int NB, int TPR, int WAVES, int KS, int MODE>
__global__ __launch_bounds__(WAVES * 64) void gemv_q40_mfma_kernel(const uint8_t *tiled, const void *activations, const float *norm_w, int rows, int iters,
                                                                   int workgroups, float norm_eps, KernelArgs rest) {
    KernelArgs a = rest;
    a.rows = rows;
    if constexpr (MODE == 1) { a.norm_x = static_cast<const float *>(activations); a.norm_w = norm_w; a.norm_eps = norm_eps; }
    else if constexpr (MODE == 2) a.merge_partials = static_cast<const float *>(activations);
    else a.x = static_cast<const uint16_t *>(activations);
    constexpr int THREADS = WAVES * 64, cols = TPR * 512, IPR = cols / 64, S = TPR / KS, RB = WAVES / KS, GROUPS = cols / 8;
    constexpr int DEPTH = S % 4 == 0 ? 4 : (S % 7 == 0 ? 7 : (S % 2 == 0 ? 2 : 1));   // divides S: a step's slot in the ring is a constant
    constexpr int SETS = (NB + 3) / 4;
    static_assert(TPR % KS == 0 && WAVES % KS == 0 && NB >= 1 && NB <= 8, "whole tiles per wavefront");
    extern __shared__ uint4 smem_raw[];
    uint4 *xs4 = smem_raw;                                        // [NB][GROUPS] groups of eight fp16, (0,2,1,3) order inside fours
    uint4 *zero4 = xs4 + (size_t)NB * GROUPS;                     // eight groups of zeros
    float *xsum = reinterpret_cast<float *>(zero4 + 8);           // [NB][cols / 32]: the offset term of every block
    float *red = xsum + (size_t)NB * (cols / 32);                 // [q40_rounds(TPR)][WAVES][NB][16]   (KS > 1)
    float *misc = red + (KS > 1 ? q40_rounds(TPR) * WAVES * NB * 16 : 0);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int g = lane >> 4, ks = wave % KS, team = wave / KS;
    const int row_blocks = (a.rows + 15) >> 4;
    u32 mask_lo = 0x000F000Fu, mask_hi = 0x00F000F0u, magic_lo = 0x54005400u, magic_hi = 0x44004400u;
    asm volatile("" : "+s"(mask_lo), "+s"(mask_hi));
    asm volatile("" : "+v"(magic_lo), "+v"(magic_hi));

    {
        const int units = (row_blocks + RB - 1) / RB;
        iters = (units - (int)blockIdx.x + workgroups - 1) / workgroups;   // ragged last round for the lowest workgroups
        if (iters < 0) iters = 0;
    }
    const int total_steps = iters * S;
    auto block_of = [&](int round) { return (round * workgroups + (int)blockIdx.x) * RB + team; };
    auto load_step = [&](int f) {   // unconditional: steps past the end read bytes that every lane shares
        Q40Item it;
        const bool real = f < total_steps;
        const int round = f / S, step = f - round * S;
        const int rb = block_of(round) < row_blocks ? block_of(round) : row_blocks - 1;
        const uint8_t *tp = real ? tiled + ((size_t)rb * TPR + (ks * S + step)) * kQ40TileBytes : tiled;
        const int spread = real ? 16 : 0;
#pragma unroll
        for (int j = 0; j < 4; j++) it.q[j] = *reinterpret_cast<const uint4 *>(tp + (real ? 1024 * j : 0) + spread * lane);
        it.d = *reinterpret_cast<const uint2 *>(tp + (real ? 4096 : 0) + (real ? 8 : 0) * lane);
        return it;
    };

    // fp16 activations and K split over all wavefronts: a wavefront stages its own S tiles' columns and waits for no other
    // (as in gemv_q4k_mfma_kernel; 14336 columns only)
    // (4096 x 14336: one row 8.9 against 8.7 us, so one row keeps the common staging; two rows 9.4 against 9.8, four 11.0 against 12.0)
    constexpr bool PRIVATE = MODE == 0 && KS == WAVES && TPR >= 16 && NB >= 2;
    constexpr int SLICE = S * 64, KW = (SLICE + 63) / 64;          // groups of eight columns in a wavefront's share
    MfmaStage<NB, IPR, THREADS, MODE, true> stage;
    uint4 own[PRIVATE ? NB : 1][PRIVATE ? KW : 1];
    if constexpr (PRIVATE) {
#pragma unroll
        for (int b = 0; b < NB; b++)
#pragma unroll
            for (int k = 0; k < KW; k++) own[b][k] = reinterpret_cast<const uint4 *>(a.x)[(size_t)b * GROUPS + SLICE * ks + lane + 64 * k];
    } else {
        stage.issue(a);
    }
    // steps in flight, as in gemv_q4k_mfma_kernel: with fourteen wavefronts a two-step ring filled up front has 129 KB on its
    // way before the staging barrier (4096 x 14336: 10.5 / 11.4 / 13.7 us for one / two / four rows; one step ahead 8.7 / 9.8 / 12.1)
    constexpr int AHEAD = DEPTH == 2 ? 1 : DEPTH;
    Q40Item ring[DEPTH];
#pragma unroll
    for (int d = 0; d < AHEAD; d++) ring[d] = load_step(d);
    if constexpr (PRIVATE) {
        if (lane < 8) zero4[lane] = make_uint4(0, 0, 0, 0);        // every wavefront writes the same zeros
#pragma unroll
        for (int b = 0; b < NB; b++)
#pragma unroll
            for (int k = 0; k < KW; k++) q4k_store_group_natural<true>(own[b][k], b, SLICE * ks + lane + 64 * k, cols, xs4, xsum);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    } else {
        if (tid < 8) zero4[tid] = make_uint4(0, 0, 0, 0);
        stage.finish(a, xs4, xsum, misc);
        __syncthreads();
    }

    // A operand: slot i = lane % 16 carries activation row i % 4 in lane group i / 4 only; group index of (tile step, j, fragment f)
    // = 64 step + 16 j + 4 g + f
    const int slot = lane & 15;
    const uint4 *a_base[SETS];
    int a_stride[SETS], a_jstride[SETS];
#pragma unroll
    for (int set = 0; set < SETS; set++) {
        const bool feeds = (slot >> 2) == g && 4 * set + (slot & 3) < NB;
        a_base[set] = feeds ? xs4 + (size_t)(4 * set + (slot & 3)) * GROUPS + 64 * (ks * S) + 4 * g : zero4;
        a_stride[set] = feeds ? 64 : 0;
        a_jstride[set] = feeds ? 16 : 0;
    }
    const float *xsum_base = xsum + 16 * (ks * S) + g;

    float v[NB];
    auto step_compute = [&](const Q40Item &it, int i) {
        const u32 dw[2] = {it.d.x, it.d.y};
#pragma unroll
        for (int j = 0; j < 4; j++) {
            floatx4 acc[SETS];
#pragma unroll
            for (int set = 0; set < SETS; set++) acc[set] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
            const u32 w0 = it.q[j].x, w1 = it.q[j].y, w2 = it.q[j].z, w3 = it.q[j].w;
            const uint4 pl0 = make_uint4((w0 & mask_lo) | magic_lo, ((w0 >> 8) & mask_lo) | magic_lo, (w1 & mask_lo) | magic_lo, ((w1 >> 8) & mask_lo) | magic_lo);
            const uint4 pl1 = make_uint4((w2 & mask_lo) | magic_lo, ((w2 >> 8) & mask_lo) | magic_lo, (w3 & mask_lo) | magic_lo, ((w3 >> 8) & mask_lo) | magic_lo);
            const uint4 ph0 = make_uint4((w0 & mask_hi) | magic_hi, ((w0 >> 8) & mask_hi) | magic_hi, (w1 & mask_hi) | magic_hi, ((w1 >> 8) & mask_hi) | magic_hi);
            const uint4 ph1 = make_uint4((w2 & mask_hi) | magic_hi, ((w2 >> 8) & mask_hi) | magic_hi, (w3 & mask_hi) | magic_hi, ((w3 >> 8) & mask_hi) | magic_hi);
#pragma unroll
            for (int set = 0; set < SETS; set++) {
                const uint4 *ap = a_base[set] + i * a_stride[set] + j * a_jstride[set];
                acc[set] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, ap[0]), __builtin_bit_cast(half8, pl0), acc[set], 0, 0, 0);
                acc[set] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, ap[1]), __builtin_bit_cast(half8, pl1), acc[set], 0, 0, 0);
                acc[set] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, ap[2]), __builtin_bit_cast(half8, ph0), acc[set], 0, 0, 0);
                acc[set] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, ap[3]), __builtin_bit_cast(half8, ph1), acc[set], 0, 0, 0);
            }
            const float d = half_bits_to_float((dw[j >> 1] >> (16 * (j & 1))) & 0xFFFFu);
#pragma unroll
            for (int b = 0; b < NB; b++) {
                const float c = xsum_base[(size_t)b * (cols >> 5) + 16 * i + 4 * j];
                v[b] += d * (16.0f * acc[b >> 2][b & 3] - c);
            }
        }
    };

    float best[NB];
    int best_i[NB];
#pragma unroll
    for (int b = 0; b < NB; b++) { best[b] = -INFINITY; best_i[b] = 0x7FFFFFFF; }
    auto finish_block = [&](int rb, float (&sum)[NB]) {
        if (a.epilogue == EPI_ARGMAX) {
            const int row = rb * 16 + lane;
            if (lane < 16 && row < a.rows) {
#pragma unroll
                for (int b = 0; b < NB; b++) argmax_take(best[b], best_i[b], sum[b], row);
            }
            return;
        }
        float other[NB];
#pragma unroll
        for (int b = 0; b < NB; b++) other[b] = dpp_term<0xB1, 0xF>(sum[b]);
        if (lane < 16 && (lane & 1) == 0 && rb < row_blocks) pair_epilogue<NB>(a, rb * 8 + (lane >> 1), sum, other);
    };

    for (int round = 0; round < iters; round++) {
#pragma unroll
        for (int b = 0; b < NB; b++) v[b] = 0.0f;
#pragma unroll
        for (int i = 0; i < S; i++) {
            const Q40Item it = ring[i % DEPTH];
            ring[(i + AHEAD) % DEPTH] = load_step(round * S + i + AHEAD);
            step_compute(it, i);
        }
#pragma unroll
        for (int b = 0; b < NB; b++) {
            v[b] += __shfl_xor(v[b], 16);
            v[b] += __shfl_xor(v[b], 32);
        }
        if constexpr (KS == 1) {
            finish_block(block_of(round), v);
        } else {
            float *slot_base = red + ((size_t)(round % q40_rounds(TPR)) * WAVES + wave) * NB * 16;
            if (lane < 16) {
#pragma unroll
                for (int b = 0; b < NB; b++) slot_base[b * 16 + lane] = v[b];
            }
        }
    }
    if constexpr (KS > 1) {
        __syncthreads();
        if (ks == 0) {   // the team's shares in wavefront order, then the epilogue
            for (int round = 0; round < iters; round++) {
                float sum[NB];
#pragma unroll
                for (int b = 0; b < NB; b++) {
                    float t = 0.0f;
                    if (lane < 16) {
#pragma unroll
                        for (int w = 0; w < KS; w++) t += red[((size_t)(round % q40_rounds(TPR)) * WAVES + wave + w) * NB * 16 + b * 16 + lane];
                    }
                    sum[b] = t;
                }
                finish_block(block_of(round), sum);
            }
        }
    }
    if (a.epilogue == EPI_ARGMAX) {
        float *cv = misc;
        int *ci = reinterpret_cast<int *>(misc + NB * WAVES);
        __syncthreads();
#pragma unroll
        for (int b = 0; b < NB; b++) {
#pragma unroll
            for (int off = 8; off >= 1; off >>= 1) {
                const float ov = __shfl_xor(best[b], off);
                const int oi = __shfl_xor(best_i[b], off);
                argmax_take(best[b], best_i[b], ov, oi);
            }
            if (lane == 0) { cv[b * WAVES + wave] = ks == 0 ? best[b] : -INFINITY; ci[b * WAVES + wave] = ks == 0 ? best_i[b] : 0x7FFFFFFF; }
        }
        __syncthreads();
        if (tid < NB) {
            float bv = cv[tid * WAVES];
            int bi = ci[tid * WAVES];
#pragma unroll
            for (int w = 1; w < WAVES; w++) argmax_take(bv, bi, cv[tid * WAVES + w], ci[tid * WAVES + w]);
            a.part_value[(size_t)tid * gridDim.x + blockIdx.x] = bv;
            a.part_index[(size_t)tid * gridDim.x + blockIdx.x] = bi;
        }
    }
}

// ---- Q8_0 on the matrix cores ---------------------------------------------------------------------------------------------------
// The same scheme for Q8_0's 32-byte blocks with one fp16 scale.  The tiled copy holds, per (sixteen rows, 256 columns), four
// kilobytes of quants as [j][half][lane] 16 bytes (lane (n, g) owns blocks 4 j + g, j = 0, 1, of row n; half = its first or last
// sixteen bytes) and then [lane][j] fp16 scales: four contiguous 1 KB loads and one of 256 bytes per wavefront and tile.  A signed
// byte b becomes the fp16 number 1152 + b without arithmetic (v_perm puts b ^ 0x80 under the exponent byte 0x64: 1024 + 128 + b,
// exact), two bytes per v_perm; the four MFMAs of a block share its scale and one accumulator, and w = d b folds as
// d (acc - 1152 Sx) with Sx the sum of the block's activations, staged beside them.  Exact products, fp32 sums.
// F16 = true: the same kernel for fp16 weights.  Their tiled copy holds the weights themselves, [j][m][lane] 16 bytes per (sixteen
// rows, 256 columns) = eight 1 KB loads per wavefront and tile, already in the order the activations are staged in: a lane's sixteen
// bytes ARE its B operand, and one accumulator runs over the whole round.
constexpr size_t kQ80TileBytes = 4352, kF16TileBytes = 8192;
constexpr int kQ80Rounds = 8;   // rounds whose partial sums have an LDS slot of their own (KS > 1)
template <bool F16> struct Q80Item { uint4 q[F16 ? 8 : 4]; u32 d; };

template <int NB, int TPR, int WAVES, int KS, int MODE, bool F16 = false>
__global__ __launch_bounds__(WAVES * 64) void gemv_q80_mfma_kernel(const uint8_t *tiled, const void *activations, const float *norm_w, int rows, int iters,
                                                                   int workgroups, float norm_eps, KernelArgs rest) {
    KernelArgs a = rest;
    a.rows = rows;
    if constexpr (MODE == 1) { a.norm_x = static_cast<const float *>(activations); a.norm_w = norm_w; a.norm_eps = norm_eps; }
    else if constexpr (MODE == 2) a.merge_partials = static_cast<const float *>(activations);
    else a.x = static_cast<const uint16_t *>(activations);
    constexpr int THREADS = WAVES * 64, cols = TPR * 256, IPR = cols / 64, S = TPR / KS, RB = WAVES / KS, GROUPS = cols / 8;
    constexpr int DEPTH = S % 4 == 0 ? 4 : (S % 2 == 0 ? 2 : 1);   // divides S: a step's slot in the ring is a constant
    static_assert(TPR % KS == 0 && WAVES % KS == 0 && NB >= 1 && NB <= 4, "whole tiles per wavefront, one set of A slots");
    extern __shared__ uint4 smem_raw[];
    uint4 *xs4 = smem_raw;                                        // [NB][GROUPS] groups of eight fp16, (0,2,1,3) order inside fours
    uint4 *zero4 = xs4 + (size_t)NB * GROUPS;                     // eight groups of zeros
    float *xsum = reinterpret_cast<float *>(zero4 + 8);           // [NB][cols / 32]: the sum of every block's activations
    float *red = xsum + (size_t)NB * (cols / 32);                 // [kQ80Rounds][WAVES][NB][16]   (KS > 1)
    float *misc = red + (KS > 1 ? kQ80Rounds * WAVES * NB * 16 : 0);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int g = lane >> 4, ks = wave % KS, team = wave / KS;
    const int row_blocks = (a.rows + 15) >> 4;
    {
        const int units = (row_blocks + RB - 1) / RB;
        iters = (units - (int)blockIdx.x + workgroups - 1) / workgroups;   // ragged last round for the lowest workgroups
        if (iters < 0) iters = 0;
    }
    const int total_steps = iters * S;
    auto block_of = [&](int round) { return (round * workgroups + (int)blockIdx.x) * RB + team; };
    auto load_step = [&](int f) {   // unconditional: steps past the end read bytes that every lane shares
        Q80Item<F16> it;
        const bool real = f < total_steps;
        const int round = f / S, step = f - round * S;
        const int rb = block_of(round) < row_blocks ? block_of(round) : row_blocks - 1;
        const uint8_t *tp = real ? tiled + ((size_t)rb * TPR + (ks * S + step)) * (F16 ? kF16TileBytes : kQ80TileBytes) : tiled;
        const int spread = real ? 16 : 0;
#pragma unroll
        for (int j = 0; j < (F16 ? 8 : 4); j++) it.q[j] = *reinterpret_cast<const uint4 *>(tp + (real ? 1024 * j : 0) + spread * lane);
        if constexpr (F16) it.d = 0;
        else it.d = *reinterpret_cast<const u32 *>(tp + (real ? 4096 : 0) + (real ? 4 : 0) * lane);
        return it;
    };

    MfmaStage<NB, IPR, THREADS, MODE> stage;
    stage.issue(a);
    constexpr int AHEAD = DEPTH == 2 ? 1 : DEPTH;
    Q80Item<F16> ring[DEPTH];
#pragma unroll
    for (int d = 0; d < AHEAD; d++) ring[d] = load_step(d);
    if (tid < 8) zero4[tid] = make_uint4(0, 0, 0, 0);
    stage.finish(a, xs4, xsum, misc);
    __syncthreads();

    // A operand: slot i = lane % 16 carries activation row i % 4 in lane group i / 4 only; group index of (tile step, j, fragment m)
    // = 32 step + 16 j + 4 g + m
    const int slot = lane & 15;
    const bool feeds = (slot >> 2) == g && (slot & 3) < NB;
    const uint4 *a_base = feeds ? xs4 + (size_t)(slot & 3) * GROUPS + 32 * (ks * S) + 4 * g : zero4;
    const int a_stride = feeds ? 32 : 0, a_jstride = feeds ? 16 : 0;
    const float *xsum_base = xsum + 8 * (ks * S) + g;

    float v[NB];
    floatx4 run = floatx4{0.0f, 0.0f, 0.0f, 0.0f};   // fp16 weights: the round's sums (no scale stands between the blocks)
    auto step_compute = [&](const Q80Item<F16> &it, int i) {
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const uint4 *ap = a_base + i * a_stride + j * a_jstride;
            if constexpr (F16) {
#pragma unroll
                for (int m = 0; m < 4; m++)
                    run = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, ap[m]), __builtin_bit_cast(half8, it.q[4 * j + m]), run, 0, 0, 0);
                continue;
            }
            floatx4 acc = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int m = 0; m < 4; m++) {
                if constexpr (F16) continue;
                const uint4 &q = it.q[F16 ? 0 : 2 * j + (m >> 1)];
                const u32 t0 = ((m & 1) ? q.z : q.x) ^ 0x80808080u, t1 = ((m & 1) ? q.w : q.y) ^ 0x80808080u;   // signed -> biased
                const uint4 p = make_uint4(__builtin_amdgcn_perm(0x64646464u, t0, 0x04020400u), __builtin_amdgcn_perm(0x64646464u, t0, 0x04030401u),
                                           __builtin_amdgcn_perm(0x64646464u, t1, 0x04020400u), __builtin_amdgcn_perm(0x64646464u, t1, 0x04030401u));
                acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, ap[m]), __builtin_bit_cast(half8, p), acc, 0, 0, 0);
            }
            const float d = half_bits_to_float((it.d >> (16 * j)) & 0xFFFFu);
#pragma unroll
            for (int b = 0; b < NB; b++) {
                const float sx = xsum_base[(size_t)b * (cols >> 5) + 8 * i + 4 * j];
                v[b] += d * (acc[b] - 1152.0f * sx);
            }
        }
    };

    float best[NB];
    int best_i[NB];
#pragma unroll
    for (int b = 0; b < NB; b++) { best[b] = -INFINITY; best_i[b] = 0x7FFFFFFF; }
    auto finish_block = [&](int rb, float (&sum)[NB]) {
        if (a.epilogue == EPI_ARGMAX) {
            const int row = rb * 16 + lane;
            if (lane < 16 && row < a.rows) {
#pragma unroll
                for (int b = 0; b < NB; b++) argmax_take(best[b], best_i[b], sum[b], row);
            }
            return;
        }
        float other[NB];
#pragma unroll
        for (int b = 0; b < NB; b++) other[b] = dpp_term<0xB1, 0xF>(sum[b]);
        if (lane < 16 && (lane & 1) == 0 && rb < row_blocks) pair_epilogue<NB>(a, rb * 8 + (lane >> 1), sum, other);
    };

    for (int round = 0; round < iters; round++) {
#pragma unroll
        for (int b = 0; b < NB; b++) v[b] = 0.0f;
#pragma unroll
        for (int i = 0; i < S; i++) {
            const Q80Item<F16> it = ring[i % DEPTH];
            ring[(i + AHEAD) % DEPTH] = load_step(round * S + i + AHEAD);
            step_compute(it, i);
            if constexpr (S >= 3) __builtin_amdgcn_sched_barrier(0);   // rounds of several steps: keep the unrolled steps apart (registers)
        }
        if constexpr (F16) {
#pragma unroll
            for (int b = 0; b < NB; b++) v[b] = run[b];
            run = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
        }
#pragma unroll
        for (int b = 0; b < NB; b++) {
            v[b] += __shfl_xor(v[b], 16);
            v[b] += __shfl_xor(v[b], 32);
        }
        if constexpr (KS == 1) {
            finish_block(block_of(round), v);
        } else {
            float *slot_base = red + ((size_t)(round % kQ80Rounds) * WAVES + wave) * NB * 16;
            if (lane < 16) {
#pragma unroll
                for (int b = 0; b < NB; b++) slot_base[b * 16 + lane] = v[b];
            }
        }
    }
    if constexpr (KS > 1) {
        __syncthreads();
        if (ks == 0) {   // the team's shares in wavefront order, then the epilogue
            for (int round = 0; round < iters; round++) {
                float sum[NB];
#pragma unroll
                for (int b = 0; b < NB; b++) {
                    float t = 0.0f;
                    if (lane < 16) {
#pragma unroll
                        for (int w = 0; w < KS; w++) t += red[((size_t)(round % kQ80Rounds) * WAVES + wave + w) * NB * 16 + b * 16 + lane];
                    }
                    sum[b] = t;
                }
                finish_block(block_of(round), sum);
            }
        }
    }
    if (a.epilogue == EPI_ARGMAX) {
        float *cv = misc;
        int *ci = reinterpret_cast<int *>(misc + NB * WAVES);
        __syncthreads();
#pragma unroll
        for (int b = 0; b < NB; b++) {
#pragma unroll
            for (int off = 8; off >= 1; off >>= 1) {
                const float ov = __shfl_xor(best[b], off);
                const int oi = __shfl_xor(best_i[b], off);
                argmax_take(best[b], best_i[b], ov, oi);
            }
            if (lane == 0) { cv[b * WAVES + wave] = ks == 0 ? best[b] : -INFINITY; ci[b * WAVES + wave] = ks == 0 ? best_i[b] : 0x7FFFFFFF; }
        }
        __syncthreads();
        if (tid < NB) {
            float bv = cv[tid * WAVES];
            int bi = ci[tid * WAVES];
#pragma unroll
            for (int w = 1; w < WAVES; w++) argmax_take(bv, bi, cv[tid * WAVES + w], ci[tid * WAVES + w]);
            a.part_value[(size_t)tid * gridDim.x + blockIdx.x] = bv;
            a.part_index[(size_t)tid * gridDim.x + blockIdx.x] = bi;
        }
    }
}

// Launch through the extension entry point when the caller gave the launch a pair of events of its own: they
// take the kernel's own start and end times (what a kernel trace reports), without the gaps between launches.
static thread_local hipEvent_t tl_start_event = nullptr, tl_stop_event = nullptr;
static thread_local int tl_argmax_capacity = 0;   // EPI_ARGMAX: slots per batch row the caller provided
static thread_local unsigned tl_last_grid = 0;    // workgroups of the most recent launch
template <typename K, typename... Args>
inline void launch_kernel(K kernel, dim3 grid, dim3 block, size_t lds, hipStream_t stream, Args... args) {
    tl_last_grid = grid.x;
    if (tl_argmax_capacity > 0 && grid.x > (unsigned)tl_argmax_capacity) return;   // the caller reports the shortfall
    if (tl_start_event && tl_stop_event) hipExtLaunchKernelGGL(kernel, grid, block, (uint32_t)lds, stream, tl_start_event, tl_stop_event, 0, args...);
    else hipLaunchKernelGGL(kernel, grid, block, lds, stream, args...);
}

inline hipError_t ensure_lds(const void *kernel, size_t lds, size_t *configured) {
    if (lds > 160 * 1024) return hipErrorInvalidValue;
    if (lds > 48 * 1024 && lds > *configured) {
        hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        *configured = lds;
    }
    return hipSuccess;
}

// Workgroups resident per compute unit that the persistent grid is sized for.
int q4k_wgs_per_cu() {
    static int v = [] {
        const char *e = getenv("ESPRESSO_HIP_Q4K_WGS_PER_CU");
        const int n = e ? atoi(e) : 0;
        return n >= 1 && n <= 16 ? n : 16;
    }();
    return v;
}
int compute_units() {
    static int v = [] {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        return n;
    }();
    return v;
}

template <int B, int IPR, int TEAM, int MODE, int WAVES = kWaves>
hipError_t launch_q4k_persistent(const KernelArgs &a, hipStream_t stream) {
    constexpr int TEAMS = WAVES / TEAM;
    const size_t lds = (size_t)B * 8 * (IPR | 1) * 16 + (size_t)B * (IPR * 2) * 4 + (size_t)(kDeferredRounds * WAVES * 2 * B + B * WAVES) * 4;
    auto kernel = gemv_q4k_kernel<B, IPR, TEAM, MODE, WAVES>;
    static size_t configured_lds = 0;
    hipError_t e = ensure_lds(reinterpret_cast<const void *>(kernel), lds, &configured_lds);
    if (e != hipSuccess) return e;
    // the persistent grid never exceeds what the chip holds at once
    static int resident_per_cu = 0;
    if (resident_per_cu == 0) {
        int n = 0;
        e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kernel, WAVES * 64, lds);
        if (e != hipSuccess) return e;
        const int limit = q4k_wgs_per_cu();
        resident_per_cu = n < 1 ? 1 : (n > limit ? limit : n);
    }
    const int npairs = (a.rows + 1) / 2;
    const int want = (npairs + TEAMS - 1) / TEAMS;            // one round
    const int cap = compute_units() * resident_per_cu;
    int grid = want < cap ? want : cap;
    // Just one round with every slot of the chip taken (the 8B q|k|v matrix) is slower than a round and a half at
    // one workgroup fewer per compute unit: 5.9 against 5.4 us; grids that are not whole multiples of the compute
    // units lose more than that (6.3-6.9 us).
    if (resident_per_cu >= 3 && want > cap - compute_units() && want <= cap) grid = cap - compute_units();
    // The last round is ragged and goes to the workgroups with the lowest indices.  Those are dispatched first and
    // get their first weights first (the memory system serves the opening burst roughly in order), and they stay
    // ahead by one to three microseconds to the end: one pair less for the later workgroups evens the finish.
    const int iters = (npairs + grid * TEAMS - 1) / (grid * TEAMS);
    const void *activations = MODE == 1 ? static_cast<const void *>(a.norm_x) : MODE == 2 ? static_cast<const void *>(a.merge_partials) : static_cast<const void *>(a.x);
    launch_kernel(kernel, dim3(grid), dim3(WAVES * 64), lds, stream, a.qs, activations, a.norm_w, a.rows, (int)a.qs_row_bytes, iters, grid, a.norm_eps, a);
    return hipGetLastError();
}


// The matrix-core Q4_K GEMV: ESPRESSO_HIP_Q4K_MFMA = 0 never, 1 wherever an instantiation exists, unset: the default table below.
// The matrix-core Q4_K GEMV.  "q4k_mfma" (ESPRESSO_HIP_Q4K_MFMA): 0 never, 1 wherever an instantiation exists, -1 the
// default (activation batches of two and more rows).  "q4k_mfma_ks" / "q4k_mfma_waves" override the table below.
int g_q4k_mfma_ragged = -2;
int g_q4k_mfma_mode = -2, g_q4k_mfma_split = -2, g_q4k_mfma_waves = -2;   // -2: not read from the environment yet
int env_int(const char *name, int fallback) {
    const char *e = getenv(name);
    return e ? atoi(e) : fallback;
}
int q4k_mfma_mode() {
    if (g_q4k_mfma_mode == -2) g_q4k_mfma_mode = env_int("ESPRESSO_HIP_Q4K_MFMA", -1);
    return g_q4k_mfma_mode;
}
int q4k_mfma_split() {
    if (g_q4k_mfma_split == -2) g_q4k_mfma_split = env_int("ESPRESSO_HIP_Q4K_MFMA_KS", 0);
    return g_q4k_mfma_split;
}
// five to eight activation rows: matrices with more weight rows stay on the nibble-B GEMM kernel
int g_q4k_mfma_rows8_max = -2;
int q4k_mfma_rows8_max() {
    if (g_q4k_mfma_rows8_max == -2) g_q4k_mfma_rows8_max = env_int("ESPRESSO_HIP_Q4K_MFMA_ROWS8_MAX", 8192);
    return g_q4k_mfma_rows8_max;
}
int g_q4k_mfma_max_rows = -2;   // single activation rows: matrices with more rows stay on the dot-product kernel (0: no limit)
int q4k_mfma_max_rows() {
    if (g_q4k_mfma_max_rows == -2) g_q4k_mfma_max_rows = env_int("ESPRESSO_HIP_Q4K_MFMA_MAX_ROWS", 0);
    return g_q4k_mfma_max_rows;
}
// one activation row at 14336 columns: 0 (default) = the matrix-core kernel, 8 or 4 = the dot-product kernel with that many wavefronts per workgroup
int g_q4k_long_row_waves = -2;
int q4k_long_row_waves() {
    if (g_q4k_long_row_waves == -2) g_q4k_long_row_waves = env_int("ESPRESSO_HIP_Q4K_LONG_ROW_WAVES", 0);
    return g_q4k_long_row_waves;
}
int q4k_mfma_waves() {
    if (g_q4k_mfma_waves == -2) g_q4k_mfma_waves = env_int("ESPRESSO_HIP_Q4K_MFMA_WAVES", 0);
    return g_q4k_mfma_waves;
}

// widths beside 4096 and 14336 that have matrix-core instantiations (one and two activation rows)
inline bool q4k_registry_width(int cols) { return cols == 1024 || cols == 2048 || cols == 3072 || cols == 8192; }

template <int NB, int IPR, int WAVES, int KS, int MODE, bool SPLIT = false, bool STAMPS = false>
hipError_t launch_q4k_mfma(const KernelArgs &a, hipStream_t stream, bool *launched) {
    constexpr int RB = WAVES / KS, cols = IPR * 64, THREADS = WAVES * 64, NBX = SPLIT ? 2 * NB : NB;
    *launched = false;
    const size_t lds = ((size_t)NBX * (cols / 8) + 8) * 16 + (size_t)NB * (cols / 32) * 4 + (KS > 1 ? (size_t)kMfmaRounds * WAVES * NB * 16 * 4 : 0) +
                       (size_t)2 * NB * WAVES * 4;
    if (lds > 160 * 1024) return hipSuccess;   // not launched
    auto kernel = gemv_q4k_mfma_kernel<NB, IPR, WAVES, KS, MODE, SPLIT, STAMPS>;
    static size_t configured_lds = 0;
    hipError_t e = ensure_lds(reinterpret_cast<const void *>(kernel), lds, &configured_lds);
    if (e != hipSuccess) return e;
    static int resident_per_cu = 0;
    if (resident_per_cu == 0) {
        int n = 0;
        e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kernel, THREADS, lds);
        if (e != hipSuccess) return e;
        // sixteen wavefronts per compute unit: with one step in flight each, a third workgroup of eight fits the registers, and
        // the 8B decode step measures 726 tok/s with it against 730 without (gate|up 13.75 against 13.4 us)
        const int by_waves = WAVES >= 16 ? 1 : 16 / WAVES;
        const int limit = q4k_wgs_per_cu() < by_waves ? q4k_wgs_per_cu() : by_waves;
        resident_per_cu = n < 1 ? 1 : (n > limit ? limit : n);
    }
    const int row_blocks = (a.rows + 15) / 16;
    const int want = (row_blocks + RB - 1) / RB;
    const int cap = compute_units() * resident_per_cu;
    if (g_q4k_mfma_ragged == -2) g_q4k_mfma_ragged = env_int("ESPRESSO_HIP_Q4K_MFMA_RAGGED", 1);
    // "q4k_mfma_ragged" 0: every workgroup runs the same number of rounds (the smallest grid that needs no more rounds than the
    // chip-filling one); 1 (default): the grid fills the chip and the ragged last round goes to the first workgroups
    int iters = (want + cap - 1) / cap;
    int grid = g_q4k_mfma_ragged ? (want < cap ? want : cap) : (want + iters - 1) / iters;
    iters = (want + grid - 1) / grid;
    if (KS > 1 && iters > kMfmaRounds) return hipSuccess;   // not launched: the caller takes the other kernel
    const void *activations = MODE == 1 ? static_cast<const void *>(a.norm_x) : MODE == 2 ? static_cast<const void *>(a.merge_partials) : static_cast<const void *>(a.x);
    launch_kernel(kernel, dim3(grid), dim3(THREADS), lds, stream, a.tiled, activations, a.norm_w, a.rows, iters, grid, a.norm_eps, a);
    *launched = true;
    return hipGetLastError();
}

// Five to eight rows (gemv_q4k_wide_kernel): fp16 activations given, store / residual epilogues, 4096 and 14336 columns.
int g_q4k_wide_mode = -2;
int q4k_wide_mode() {
    if (g_q4k_wide_mode == -2) g_q4k_wide_mode = env_int("ESPRESSO_HIP_Q4K_WIDE", 1);
    return g_q4k_wide_mode;
}
template <int IPR, int WAVES, int KS, int XMODE, bool Q40 = false>
hipError_t launch_q4k_wide(const KernelArgs &a, int batch, hipStream_t stream, bool *launched) {
    constexpr int RB = WAVES / KS, THREADS = WAVES * 64;
    *launched = false;
    const size_t lds = (size_t)kWideRounds * WAVES * 64 * sizeof(float4) +
                       (XMODE == 1 ? (size_t)8 * (IPR * 128 + (Q40 ? 32 : 16)) : (size_t)WAVES * 8 * wide_row_bytes(Q40));
    auto kernel = gemv_q4k_wide_kernel<IPR, WAVES, KS, XMODE, Q40>;
    static size_t configured_lds = 0;
    hipError_t e = ensure_lds(reinterpret_cast<const void *>(kernel), lds, &configured_lds);
    if (e != hipSuccess) return e;
    static int resident_per_cu = 0;
    if (resident_per_cu == 0) {
        int n = 0;
        e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kernel, THREADS, lds);
        if (e != hipSuccess) return e;
        const int by_waves = WAVES >= 16 ? 1 : 16 / WAVES;
        resident_per_cu = n < 1 ? 1 : (n > by_waves ? by_waves : n);
    }
    const int row_blocks = (a.rows + 15) / 16;
    const int want = (row_blocks + RB - 1) / RB;
    const int cap = compute_units() * resident_per_cu;
    const int grid = want < cap ? want : cap;
    const int iters = (want + grid - 1) / grid;
    if (iters > kWideRounds) return hipSuccess;   // not launched
    launch_kernel(kernel, dim3(grid), dim3(THREADS), lds, stream, a.tiled, a.x, a.rows, batch, grid, a);
    *launched = true;
    return hipGetLastError();
}
// Measured (us, eight rows; nibble-B GEMM kernel in brackets): 14336 x 4096 staged rows 11.3, own tiles 12.75 (15.5); 28672 x 4096 18.7,
// 21.05 (27.4); 4096 x 4096 7.0, 5.9 (7.6); 4096 x 14336 own tiles 12.0 (22.3).  Q4_0: 11.3, 12.8 (17.1); 18.9, 21.5 (29.6); 7.2, 5.8 (8.3); 12.3 (24.0).  Tuning key "q4k_wide": 0 off, 1 this table, 2 / 3 own tiles / staged rows wherever both exist.
hipError_t try_q4k_wide(const KernelArgs &a, int batch, hipStream_t stream, bool *launched) {
    *launched = false;
    if (!a.tiled || !a.x || a.norm_x || a.merge_partials || a.split_x || batch < 5 || batch > 8) return hipSuccess;
    if (a.epilogue != EPI_STORE_F32 && a.epilogue != EPI_ADD_RESIDUAL) return hipSuccess;
    const int form = q4k_wide_mode();
    if (a.cols == 4096) {
        if (form == 2 || (form != 3 && a.rows <= 8192)) return launch_q4k_wide<64, 8, 8, 2>(a, batch, stream, launched);
        return launch_q4k_wide<64, 16, 8, 1>(a, batch, stream, launched);
    }
    if (a.cols == 14336) return launch_q4k_wide<224, 8, 8, 2>(a, batch, stream, launched);
    // the registry's other widths (see try_q4k_mfma): own tiles, the K split that leaves whole super-blocks per wavefront
    if (a.cols == 1024) return launch_q4k_wide<16, 8, 4, 2>(a, batch, stream, launched);
    if (a.cols == 2048) return launch_q4k_wide<32, 8, 8, 2>(a, batch, stream, launched);
    if (a.cols == 3072) return launch_q4k_wide<48, 8, 4, 2>(a, batch, stream, launched);
    if (a.cols == 8192) return launch_q4k_wide<128, 8, 8, 2>(a, batch, stream, launched);
    return hipSuccess;
}
hipError_t try_q40_wide(const KernelArgs &a, int batch, hipStream_t stream, bool *launched) {
    *launched = false;
    if (!a.tiled || !a.x || a.norm_x || a.merge_partials || a.split_x || batch < 5 || batch > 8) return hipSuccess;
    if (a.epilogue != EPI_STORE_F32 && a.epilogue != EPI_ADD_RESIDUAL) return hipSuccess;
    const int form = q4k_wide_mode();
    if (a.cols == 4096) {
        if (form == 2 || (form != 3 && a.rows <= 8192)) return launch_q4k_wide<64, 8, 8, 2, true>(a, batch, stream, launched);
        return launch_q4k_wide<64, 16, 8, 1, true>(a, batch, stream, launched);
    }
    if (a.cols == 14336) return launch_q4k_wide<224, 8, 8, 2, true>(a, batch, stream, launched);
    return hipSuccess;
}

// Picks the instantiation; *launched stays false when there is none for this shape.
template <int NB>
hipError_t try_q4k_mfma(const KernelArgs &a, hipStream_t stream, bool *launched) {
    *launched = false;
    if (!a.tiled) return hipSuccess;
    const int mode = a.merge_partials ? 2 : a.norm_x ? 1 : 0;
    int waves = q4k_mfma_waves(), ks = q4k_mfma_split();
    if (a.cols == 4096) {
        // measured on the Llama-3-8B shapes (kernel duration / back-to-back, microseconds, one activation row):
        //   4096 rows: 16 x 16 5.5 / 6.1, 8 x 8 5.8 / 6.5;  6144 rows: 8 x 8 6.3 / 7.0, 16 x 16 6.4 / 7.2;
        //   28672 rows: 8 x 8 13.8 / 15.4, 4 x 2 14.7 / 15.8; with two rows and more the long matrices prefer 4 x 2
        //   two rows: 14336 rows 8 x 8 9.8, 4 x 2 10.0; 28672 rows 4 x 2 16.4, 8 x 8 17.6.  Eight rows: 4096 rows 8 x 8 8.7, 16 x 16 10.9
        //   second sweep (another box; one / two / four rows): 28672 rows 8 x 8 14.7 / 15.5 / 17.5, 4 x 2 15.9 / 16.6 / 19.9; 128256 rows
        //   (the output head; splits of K decline it, too many rounds) 4 x 1 53.9 / 57.2 / 67.2, dot-product kernel 60.6 / 71.1 / 92.6
        if (waves == 0 && ks == 0) {
            if (a.rows <= 4096 && NB <= 4) waves = ks = 16;
            else if (a.rows <= 32768) waves = ks = 8;
            else { waves = 4; ks = 1; }
        }
        if (waves == 0) waves = 8;
        if (ks == 0 || ks > waves) ks = waves;
        // split activations: one and two rows; the stamped instantiations: fp16 activations given, not split
#define ESP_MFMA_CASE(W_, KS_)                                                                                   \
        if (waves == W_ && ks == KS_) {                                                                          \
            if constexpr (NB <= 2) if (a.split_x) {                                                              \
                if (mode == 0) return launch_q4k_mfma<NB, 64, W_, KS_, 0, true>(a, stream, launched);             \
                if (mode == 1) return launch_q4k_mfma<NB, 64, W_, KS_, 1, true>(a, stream, launched);             \
                return launch_q4k_mfma<NB, 64, W_, KS_, 2, true>(a, stream, launched);                            \
            }                                                                                                    \
            if (a.split_x) return hipSuccess;                                                                    \
            if constexpr (NB <= 2) if (a.stamps && mode == 0) return launch_q4k_mfma<NB, 64, W_, KS_, 0, false, true>(a, stream, launched); \
            if (mode == 0) return launch_q4k_mfma<NB, 64, W_, KS_, 0>(a, stream, launched);                       \
            if (mode == 1) return launch_q4k_mfma<NB, 64, W_, KS_, 1>(a, stream, launched);                       \
            if constexpr (NB <= 2) return launch_q4k_mfma<NB, 64, W_, KS_, 2>(a, stream, launched);               \
        }
        ESP_MFMA_CASE(4, 1)
        ESP_MFMA_CASE(8, 8)
        ESP_MFMA_CASE(16, 16)
#undef ESP_MFMA_CASE
        return hipSuccess;
    }
    if (a.cols == 14336 && mode == 0) {
        if (waves == 0) waves = 8;
        if (ks == 0) ks = waves == 16 ? 8 : waves;
        if (waves == 8 && ks == 8) {
            if constexpr (NB <= 2) if (a.split_x) return launch_q4k_mfma<NB, 224, 8, 8, 0, true>(a, stream, launched);
            if (a.split_x) return hipSuccess;
            if constexpr (NB <= 2) if (a.stamps) return launch_q4k_mfma<NB, 224, 8, 8, 0, false, true>(a, stream, launched);
            return launch_q4k_mfma<NB, 224, 8, 8, 0>(a, stream, launched);
        }
        if (a.split_x) return hipSuccess;
        if (waves == 4 && ks == 4) return launch_q4k_mfma<NB, 224, 4, 4, 0>(a, stream, launched);
        if (waves == 16 && ks == 8) return launch_q4k_mfma<NB, 224, 16, 8, 0>(a, stream, launched);
        return hipSuccess;
    }
    // The other widths of the reference's model registry (Sources/ModelSupport/ModelRegistry.swift:59-107: llama3.2-1B d 2048, llama3.2-3B
    // d 3072, both FFN 8192; Qwen3-0.6B d 1024, FFN 3072), one and two activation rows: a wavefront takes one super-block column per step
    // at the model widths (all wavefronts of a workgroup share a row block), two at 8192 columns.  No tuning variants.
    if constexpr (NB <= 2) {
        if (waves != 0 || ks != 0) return hipSuccess;
#define ESP_MFMA_WIDTH(COLS_, W_)                                                                                   \
        if (a.cols == COLS_) {                                                                                     \
            if (a.split_x) {                                                                                       \
                if (mode == 0) return launch_q4k_mfma<NB, COLS_ / 64, W_, W_, 0, true>(a, stream, launched);       \
                if (mode == 1) return launch_q4k_mfma<NB, COLS_ / 64, W_, W_, 1, true>(a, stream, launched);       \
                return launch_q4k_mfma<NB, COLS_ / 64, W_, W_, 2, true>(a, stream, launched);                      \
            }                                                                                                      \
            if (mode == 0) return launch_q4k_mfma<NB, COLS_ / 64, W_, W_, 0>(a, stream, launched);                 \
            if (mode == 1) return launch_q4k_mfma<NB, COLS_ / 64, W_, W_, 1>(a, stream, launched);                 \
            return launch_q4k_mfma<NB, COLS_ / 64, W_, W_, 2>(a, stream, launched);                                \
        }
        ESP_MFMA_WIDTH(1024, 4)
        ESP_MFMA_WIDTH(2048, 8)
        ESP_MFMA_WIDTH(3072, 12)
#undef ESP_MFMA_WIDTH
        if (a.cols == 8192 && mode == 0) {
            if (a.split_x) return launch_q4k_mfma<NB, 128, 16, 16, 0, true>(a, stream, launched);
            return launch_q4k_mfma<NB, 128, 16, 16, 0>(a, stream, launched);
        }
    }
    return hipSuccess;
}

// Column counts with a compile-time instantiation of the persistent kernel (items per row, wavefronts per
// row pair): the model widths and FFN sizes of the llama family (2048, 4096, 8192; 11008, 14336).
template <int B>
hipError_t launch_q4k(const KernelArgs &a, hipStream_t stream) {
    const bool norm = a.norm_x != nullptr;
    // By default the matrix-core kernel takes two rows and more, and single rows of the 4096- and 14336-column matrices (14336
    // columns, 4096 rows, one row, in the 8B decode step: 8.3 us on the matrix cores with three steps in flight, 9.3 us on the
    // eight-wavefront dot-product kernel below, which "q4k_long_row_waves" = 8 or 4 selects).
    const bool one_row_on_the_matrix_cores = (a.cols == 4096 && (q4k_mfma_max_rows() <= 0 || a.rows <= q4k_mfma_max_rows())) ||
                                             (a.cols == 14336 && q4k_long_row_waves() == 0) || q4k_registry_width(a.cols);
    if (q4k_mfma_mode() == 1 || (q4k_mfma_mode() < 0 && (B >= 2 || one_row_on_the_matrix_cores))) {
        bool launched = false;
        const hipError_t e = try_q4k_mfma<B>(a, stream, &launched);
        if (e != hipSuccess || launched) return e;
    }
    if (a.split_x) return hipErrorInvalidValue;   // only the matrix-core kernel reads hi / lo rows
    if (a.merge_partials && a.cols == 2048) return launch_q4k_persistent<B, 32, 1, 2>(a, stream);
    if (a.merge_partials && a.cols == 4096) return launch_q4k_persistent<B, 64, 1, 2>(a, stream);
    if (!a.merge_partials) switch (a.cols) {
    case 2048: return norm ? launch_q4k_persistent<B, 32, 1, 1>(a, stream) : launch_q4k_persistent<B, 32, 1, 0>(a, stream);
    case 4096: return norm ? launch_q4k_persistent<B, 64, 1, 1>(a, stream) : launch_q4k_persistent<B, 64, 1, 0>(a, stream);
    case 8192: return norm ? launch_q4k_persistent<B, 128, 2, 1>(a, stream) : launch_q4k_persistent<B, 128, 2, 0>(a, stream);
    case 11008: if (!norm) return launch_q4k_persistent<B, 172, 4, 0>(a, stream); break;
    case 14336:
        if (!norm) {
            // Eight wavefronts (two teams) per workgroup, one workgroup per compute unit: a workgroup stages the row's 28 KB of
            // activations once, and with a third as many workgroups doing so the last of them has them 2.6 us after the launch
            // instead of 6.3 us.  Measured in the 8B decode step: 9.3 against 10.2-10.6 us per launch, 704 against 690 tok/s;
            // twelve and sixteen wavefronts, eight per team and two such workgroups per compute unit (at 128 registers) measure no better
            // than four.  "q4k_long_row_waves" = 4 selects four wavefronts, three workgroups per compute unit.
            if (q4k_long_row_waves() != 4) return launch_q4k_persistent<B, 224, 4, 0, 8>(a, stream);
            return launch_q4k_persistent<B, 224, 4, 0>(a, stream);
        }
        break;
    default: break;
    }
    const size_t lds = (size_t)B * 8 * ((a.cols / 64) | 1) * 16 + (size_t)B * (a.cols / 32) * 4 + (size_t)B * kWaves * 4;
    auto kernel = gemv_q4k_generic_kernel<B>;
    static size_t configured_lds = 0;
    hipError_t e = ensure_lds(reinterpret_cast<const void *>(kernel), lds, &configured_lds);
    if (e != hipSuccess) return e;
    const int pairs = (a.rows + 1) / 2;
    launch_kernel(kernel, dim3((pairs + kWaves - 1) / kWaves), dim3(kThreads), lds, stream, a.qs, leading_activations(a), a.norm_w, a.rows, a.cols,
                       (int)a.qs_row_bytes, leading_mode(a), a.norm_eps, a);
    return hipGetLastError();
}

template <int FMT, int B, int R>
hipError_t launch_one(const KernelArgs &a, hipStream_t stream) {
    using T = Traits<FMT>;
    size_t lds = (size_t)B * a.cols * 2 + (T::kXSums ? (size_t)B * (a.cols / 16) * 4 : 0);
    if (lds > 160 * 1024) return hipErrorInvalidValue;
    auto kernel = gemv_kernel<FMT, B, R>;
    static size_t configured_lds = 0;  // per instantiation
    if (lds > 48 * 1024 && lds > configured_lds) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        configured_lds = lds;
    }
    const int rows_per_wg = kWaves * R;
    const int grid = (a.rows + rows_per_wg - 1) / rows_per_wg;
    launch_kernel(kernel, dim3(grid), dim3(kThreads), lds, stream, a.qs, a.scales, leading_activations(a), a.norm_w, a.rows, a.cols, (int)a.qs_row_bytes,
                       leading_mode(a), a.norm_eps, a);
    return hipGetLastError();
}

template <int FMT>
hipError_t launch_fmt(const KernelArgs &a, int batch, hipStream_t stream) {
    if (batch == 1) {
        // tall matrices (an output head): four rows per wavefront, so that one wave of workgroups covers the matrix (32000 x 768 Q8_0:
        // 2000 workgroups instead of 4000, 8.8 against 10.1 us; eight rows measure the same as four)
        if (a.rows >= 16384) return launch_one<FMT, 1, 4>(a, stream);
        return launch_one<FMT, 1, 2>(a, stream);
    }
    if (batch == 2) return a.rows >= 16384 ? launch_one<FMT, 2, 4>(a, stream) : launch_one<FMT, 2, 2>(a, stream);
    return hipErrorInvalidValue;
}


template <int NB, int TPR, int WAVES, int KS, int MODE>
hipError_t launch_q40_mfma(const KernelArgs &a, hipStream_t stream, bool *launched) {
    constexpr int RB = WAVES / KS, cols = TPR * 512, THREADS = WAVES * 64;
    *launched = false;
    const size_t lds = ((size_t)NB * (cols / 8) + 8) * 16 + (size_t)NB * (cols / 32) * 4 + (KS > 1 ? (size_t)q40_rounds(TPR) * WAVES * NB * 16 * 4 : 0) +
                       (size_t)2 * NB * WAVES * 4;
    if (lds > 160 * 1024) return hipSuccess;   // not launched
    auto kernel = gemv_q40_mfma_kernel<NB, TPR, WAVES, KS, MODE>;
    static size_t configured_lds = 0;
    hipError_t e = ensure_lds(reinterpret_cast<const void *>(kernel), lds, &configured_lds);
    if (e != hipSuccess) return e;
    static int resident_per_cu = 0;
    if (resident_per_cu == 0) {
        int n = 0;
        e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kernel, THREADS, lds);
        if (e != hipSuccess) return e;
        // one activation row: sixteen wavefronts per compute unit, as for Q4_K (14336 x 4096: 8.6 against 9.2 us; two rows 9.5 against 9.4)
        const int by_waves = NB > 1 ? 16 : WAVES >= 16 ? 1 : 16 / WAVES;
        const int limit = q4k_wgs_per_cu() < by_waves ? q4k_wgs_per_cu() : by_waves;
        resident_per_cu = n < 1 ? 1 : (n > limit ? limit : n);
    }
    const int row_blocks = (a.rows + 15) / 16;
    const int want = (row_blocks + RB - 1) / RB;
    const int cap = compute_units() * resident_per_cu;
    const int grid = want < cap ? want : cap;
    const int iters = (want + grid - 1) / grid;
    if (KS > 1 && iters > q40_rounds(TPR)) return hipSuccess;   // not launched: the caller takes the other kernel
    const void *activations = MODE == 1 ? static_cast<const void *>(a.norm_x) : MODE == 2 ? static_cast<const void *>(a.merge_partials) : static_cast<const void *>(a.x);
    launch_kernel(kernel, dim3(grid), dim3(THREADS), lds, stream, a.tiled, activations, a.norm_w, a.rows, iters, grid, a.norm_eps, a);
    *launched = true;
    return hipGetLastError();
}

// "q40_mfma" (ESPRESSO_HIP_Q40_MFMA): 0 never, 1 wherever an instantiation exists, -1 the default (two and more activation rows,
// and single rows of matrices with 2048 rows and more: 1024 x 4096 measures 3.7 against 3.3 us on the dot-product kernel).
int g_q40_mfma_mode = -2;
int q40_mfma_mode() {
    if (g_q40_mfma_mode == -2) g_q40_mfma_mode = env_int("ESPRESSO_HIP_Q40_MFMA", -1);
    return g_q40_mfma_mode;
}

template <int NB>
hipError_t try_q40_mfma(const KernelArgs &a, hipStream_t stream, bool *launched) {
    *launched = false;
    if (!a.tiled) return hipSuccess;
    const int mode = a.merge_partials ? 2 : a.norm_x ? 1 : 0;
    int waves = q4k_mfma_waves(), ks = q4k_mfma_split();
    if (a.cols == 4096) {
        // measured (us, one / two / four rows): 14336 rows 8 x 8 9.2 / 9.5 / 11.0, 8 x 4 9.4 / 9.9 / 11.4, 4 x 2 9.7 / 10.7 / 12.6;
        // 28672 rows 13.6 / 14.3 / 16.1, 14.6 / 15.6 / 18.0, 16.3 / 17.5 / 20.5; the dot-product kernel 9.9 / 12.2 / 15.6 and 17.2 / 22.0 / 28.8
        if (waves == 0) waves = 8;
        if (ks == 0 || ks > waves) ks = waves;
#define ESP_Q40_CASE(W_, KS_)                                                                                    \
        if (waves == W_ && ks == KS_) {                                                                          \
            if (mode == 0) return launch_q40_mfma<NB, 8, W_, KS_, 0>(a, stream, launched);                        \
            if (mode == 1) return launch_q40_mfma<NB, 8, W_, KS_, 1>(a, stream, launched);                        \
            if constexpr (NB <= 2) return launch_q40_mfma<NB, 8, W_, KS_, 2>(a, stream, launched);                \
        }
        ESP_Q40_CASE(4, 2)
        ESP_Q40_CASE(8, 4)
        ESP_Q40_CASE(8, 8)
#undef ESP_Q40_CASE
        return hipSuccess;
    }
    if constexpr (NB <= 4) if (a.cols == 14336 && mode == 0) {
        // 4096 rows: 14 x 14 10.5 / 11.4 / 13.7, 7 x 7 10.4 / 11.6 / 14.6; the dot-product kernel 10.8 / 14.2 / 25.1
        if (waves == 0) waves = 14;
        if (ks == 0) ks = waves == 8 ? 4 : waves;
        if (waves == 7 && ks == 7) return launch_q40_mfma<NB, 28, 7, 7, 0>(a, stream, launched);
        if (waves == 14 && ks == 14) return launch_q40_mfma<NB, 28, 14, 14, 0>(a, stream, launched);
        if (waves == 14 && ks == 7) return launch_q40_mfma<NB, 28, 14, 7, 0>(a, stream, launched);
        if (waves == 8 && ks == 4) return launch_q40_mfma<NB, 28, 8, 4, 0>(a, stream, launched);
        return hipSuccess;
    }
    return hipSuccess;
}

template <int NB, int TPR, int WAVES, int KS, int MODE, bool F16 = false>
hipError_t launch_q80_mfma(const KernelArgs &a, hipStream_t stream, bool *launched) {
    constexpr int RB = WAVES / KS, cols = TPR * 256, THREADS = WAVES * 64;
    *launched = false;
    const size_t lds = ((size_t)NB * (cols / 8) + 8) * 16 + (size_t)NB * (cols / 32) * 4 + (KS > 1 ? (size_t)kQ80Rounds * WAVES * NB * 16 * 4 : 0) +
                       (size_t)2 * NB * WAVES * 4;
    auto kernel = gemv_q80_mfma_kernel<NB, TPR, WAVES, KS, MODE, F16>;
    static size_t configured_lds = 0;
    hipError_t e = ensure_lds(reinterpret_cast<const void *>(kernel), lds, &configured_lds);
    if (e != hipSuccess) return e;
    static int resident_per_cu = 0;
    if (resident_per_cu == 0) {
        int n = 0;
        e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kernel, THREADS, lds);
        if (e != hipSuccess) return e;
        const int by_waves = WAVES >= 16 ? 1 : 16 / WAVES;   // sixteen wavefronts per compute unit, as for the other formats
        resident_per_cu = n < 1 ? 1 : (n > by_waves ? by_waves : n);
    }
    const int row_blocks = (a.rows + 15) / 16;
    const int want = (row_blocks + RB - 1) / RB;
    const int cap = compute_units() * resident_per_cu;
    const int grid = want < cap ? want : cap;
    const int iters = (want + grid - 1) / grid;
    if (KS > 1 && iters > kQ80Rounds) return hipSuccess;   // not launched: the caller takes the other kernel
    const void *activations = MODE == 1 ? static_cast<const void *>(a.norm_x) : MODE == 2 ? static_cast<const void *>(a.merge_partials) : static_cast<const void *>(a.x);
    launch_kernel(kernel, dim3(grid), dim3(THREADS), lds, stream, a.tiled, activations, a.norm_w, a.rows, iters, grid, a.norm_eps, a);
    *launched = true;
    return hipGetLastError();
}

// "q80_mfma" (ESPRESSO_HIP_Q80_MFMA): 0 never, 1 wherever an instantiation exists (768, 2048 and 4096 columns, one and two activation
// rows), -1 the default (see launch_q80).  Tall matrices (an output head) take four wavefronts that each walk whole rows; the others split a row
// block's columns over the wavefronts of a workgroup.
int g_q80_mfma_mode = -2;
int q80_mfma_mode() {
    if (g_q80_mfma_mode == -2) g_q80_mfma_mode = env_int("ESPRESSO_HIP_Q80_MFMA", -1);
    return g_q80_mfma_mode;
}
inline bool q80_mfma_width(int cols) { return cols == 768 || cols == 2048 || cols == 4096; }

template <int NB, bool F16 = false>
hipError_t try_q80_mfma(const KernelArgs &a, hipStream_t stream, bool *launched) {
    *launched = false;
    if (!a.tiled || q80_mfma_mode() == 0) return hipSuccess;
    const int mode = a.merge_partials ? 2 : a.norm_x ? 1 : 0;
    const bool tall = a.rows > 8192;
#define ESP_Q80_WIDTH(COLS_, W_)                                                                                       \
    if (a.cols == COLS_) {                                                                                            \
        if (tall) {                                                                                                   \
            if (mode == 0) return launch_q80_mfma<NB, COLS_ / 256, 4, 1, 0, F16>(a, stream, launched);                \
            if (mode == 1) return launch_q80_mfma<NB, COLS_ / 256, 4, 1, 1, F16>(a, stream, launched);                \
            return hipSuccess;                                                                                        \
        }                                                                                                             \
        if (mode == 0) return launch_q80_mfma<NB, COLS_ / 256, W_, W_, 0, F16>(a, stream, launched);                  \
        if (mode == 1) return launch_q80_mfma<NB, COLS_ / 256, W_, W_, 1, F16>(a, stream, launched);                  \
        return launch_q80_mfma<NB, COLS_ / 256, W_, W_, 2, F16>(a, stream, launched);                                 \
    }
    ESP_Q80_WIDTH(768, 3)
    ESP_Q80_WIDTH(2048, 8)
    if constexpr (!F16) { ESP_Q80_WIDTH(4096, 8) }
#undef ESP_Q80_WIDTH
    return hipSuccess;
}

// fp16 weights (768 and 2048 columns): the same rule
template <int B>
hipError_t launch_f16(const KernelArgs &a, hipStream_t stream) {
    if (q80_mfma_mode() == 1 || (q80_mfma_mode() < 0 && (B >= 2 || a.rows > 8192))) {
        bool launched = false;
        const hipError_t e = try_q80_mfma<B, true>(a, stream, &launched);
        if (e != hipSuccess || launched) return e;
    }
    return launch_fmt<FMT_F16>(a, B, stream);
}

template <int B>
hipError_t launch_q80(const KernelArgs &a, hipStream_t stream) {
    // measured (us, dot-product / matrix cores): one row 2304 x 768 2.74 / 2.96, 4096 x 768 3.08 / 3.22, 768 x 2048 3.01 / 3.00, 4096 x 4096
    // 6.36 / 5.52, 32000 x 768 9.26 / 6.76, 32000 x 4096 31.5 / 26.9; two rows 3.36 / 3.17, 3.77 / 3.31, 3.47 / 3.36, 7.23 / 5.69, 12.1 / 6.8, 32.8 / 27.6:
    // two rows always, one row where the matrix is tall or wide ("q80_mfma" = 1: wherever an instantiation exists)
    if (q80_mfma_mode() == 1 || (q80_mfma_mode() < 0 && (B >= 2 || a.rows > 8192 || a.cols >= 4096))) {
        bool launched = false;
        const hipError_t e = try_q80_mfma<B>(a, stream, &launched);
        if (e != hipSuccess || launched) return e;
    }
    return launch_fmt<FMT_Q8_0>(a, B, stream);
}

template <int B>
hipError_t launch_q40(const KernelArgs &a, hipStream_t stream) {
    if (q40_mfma_mode() == 1 || (q40_mfma_mode() < 0 && (B >= 2 || a.rows >= 2048))) {
        bool launched = false;
        const hipError_t e = try_q40_mfma<B>(a, stream, &launched);
        if (e != hipSuccess || launched) return e;
    }
    return launch_fmt<FMT_Q4_0>(a, B, stream);
}
}  // namespace

bool gemv_merges_attention_partials(const DeviceMatrix &w, int batch, int head_dim) {
    if (batch < 1 || batch > 2 || (head_dim != 64 && head_dim != 128) || w.cols % head_dim != 0) return false;
    // the persistent Q4_K instantiations for the wider inputs have no merging form
    if (w.format == FMT_Q4_K && (w.cols == 8192 || w.cols == 11008 || w.cols == 14336)) return false;
    return true;
}

static unsigned g_tuning_epoch = 0;
unsigned gemv_tuning_epoch() { return g_tuning_epoch; }

bool gemv_set_tuning(const char *key, int value) {
    const std::string k = key ? key : "";
    g_tuning_epoch++;   // runtimes drop the graphs they captured under the old selection
    if (k == "q4k_mfma") { g_q4k_mfma_mode = value; return true; }
    if (k == "q4k_mfma_ks") { g_q4k_mfma_split = value; return true; }
    if (k == "q4k_mfma_waves") { g_q4k_mfma_waves = value; return true; }
    if (k == "q4k_mfma_ragged") { g_q4k_mfma_ragged = value; return true; }
    if (k == "q40_mfma") { g_q40_mfma_mode = value; return true; }
    if (k == "q80_mfma") { g_q80_mfma_mode = value; return true; }
    if (k == "q4k_mfma_max_rows") { g_q4k_mfma_max_rows = value; return true; }
    if (k == "q4k_mfma_rows8_max") { g_q4k_mfma_rows8_max = value; return true; }
    if (k == "q4k_long_row_waves") { g_q4k_long_row_waves = value; return true; }
    if (k == "q4k_wide") { g_q4k_wide_mode = value; return true; }
    if (k == "split_gemm_shared_k") { gemm_split_set_shared_k(value); return true; }
    if (k == "prompt_attention_key_sets") { attention_prompt_set_key_sets(value); return true; }
    return false;
}

// The wide kernel keeps kWideRounds rounds of partial sums in LDS: row blocks / (compute units x workgroups per unit) may not exceed that.
static int q4k_wide_max_rows() { return compute_units() * 2 * 16 * kWideRounds; }

bool gemv_takes_rows(const DeviceMatrix &w, int batch) {
    if (batch <= 2) return true;
    // (eight rows of 14336 columns do not fit the kernel's LDS staging in one pass and stay on the nibble-B GEMM kernel)
    // and so do five to eight rows of the long 4096-column matrices, where that kernel measures faster: 15.3 against 17.1 us at 14336 rows)
    if (w.format == FMT_Q4_0) {
        if (!w.tiled || q40_mfma_mode() == 0) return false;
        if (batch >= 5 && batch <= 8 && q4k_wide_mode() != 0 && (w.cols == 4096 || w.cols == 14336) && w.rows <= q4k_wide_max_rows()) return true;
        // (five to eight rows without the wide kernel: up to 8192 x 4096 8.7 against 10.7 us on the nibble-B kernel, at 14336 rows 18.9 against 17.1)
        return batch <= 4 ? (w.cols == 4096 || w.cols == 14336) : (batch <= 8 && w.cols == 4096 && w.rows <= 8192);
    }
    if (w.format != FMT_Q4_K || !w.tiled || q4k_mfma_mode() == 0) return false;
    if (batch >= 5 && batch <= 8 && q4k_wide_mode() != 0 && (w.cols == 4096 || w.cols == 14336 || q4k_registry_width(w.cols)) && w.rows <= q4k_wide_max_rows())
        return true;
    if (batch > 8) return false;
    return batch <= 4 ? (w.cols == 4096 || w.cols == 14336) : (w.cols == 4096 && w.rows <= q4k_mfma_rows8_max());
}

// Whether launch_gemv takes split activations (GemvParams::split_x) for this matrix and row count: the matrix-core Q4_K kernel
// at one or two rows, under the same conditions as its dispatch.
bool gemv_splits_activations(const DeviceMatrix &w, int batch) {
    if (w.format != FMT_Q4_K || !w.tiled || batch < 1 || batch > 2 || q4k_mfma_mode() == 0) return false;
    if (q4k_mfma_waves() != 0 || q4k_mfma_split() != 0) return false;   // tuning overrides: not every variant has a split form
    if (w.cols == 4096) return batch >= 2 || q4k_mfma_mode() == 1 || q4k_mfma_max_rows() <= 0 || w.rows <= q4k_mfma_max_rows();
    if (w.cols == 14336) return batch >= 2 || q4k_mfma_mode() == 1 || q4k_long_row_waves() == 0;
    return q4k_registry_width(w.cols) && w.rows <= 32768;   // taller matrices would need more rounds than the kernel's LDS slots
}

// Which matrices get the tiled copy the matrix-core GEMVs read, at upload (ESPRESSO_HIP_TILED_COPIES=0: none, the dot-product
// kernels run everywhere and resident weight memory is the packed size).
bool gemv_wants_tiled_copy(int format, int cols) {
    static const int enabled = env_int("ESPRESSO_HIP_TILED_COPIES", 1);
    if (!enabled) return false;
    if (format == FMT_Q4_K) return cols == 4096 || cols == 14336 || q4k_registry_width(cols);
    if (format == FMT_Q4_0) return cols == 4096 || cols == 14336;
    if (format == FMT_Q8_0) return q80_mfma_width(cols);
    if (format == FMT_F16) return cols == 768 || cols == 2048;
    return false;
}

bool gemv_supports_argmax(const DeviceMatrix &w) {
    return !(w.format == FMT_Q4_K && (w.cols == 8192 || w.cols == 11008 || w.cols == 14336));
}

hipError_t launch_gemv(const GemvParams &p, hipStream_t stream) {
    const DeviceMatrix &w = p.w;
    if (!w.qs || (!p.x && !p.norm_x && !p.merge_partials) || (p.norm_x && !p.norm_w) || w.rows <= 0 || w.cols <= 0 || p.batch <= 0) return hipErrorInvalidValue;
    if (p.merge_partials && !gemv_merges_attention_partials(w, p.batch, p.merge_head_dim)) return hipErrorInvalidValue;
    if ((p.epilogue == EPI_STORE_F32 || p.epilogue == EPI_ADD_RESIDUAL) && !p.y) return hipErrorInvalidValue;
    if (p.epilogue == EPI_ADD_RESIDUAL && !p.residual) return hipErrorInvalidValue;
    if (p.epilogue == EPI_SWIGLU_F16 && (!p.out_f16 || w.rows % 2 != 0)) return hipErrorInvalidValue;
    if (p.split_x && (!gemv_splits_activations(w, p.batch) || ((w.cols == 14336 || w.cols == 8192) && (p.norm_x || p.merge_partials)))) return hipErrorInvalidValue;
    if (p.split_out && (p.epilogue != EPI_SWIGLU_F16 || p.batch > 2)) return hipErrorInvalidValue;
    if (p.epilogue == EPI_ARGMAX && (!p.argmax_value || !p.argmax_index || p.argmax_capacity <= 0 || p.batch > 2 || !gemv_supports_argmax(w)))
        return hipErrorInvalidValue;
    if (p.epilogue == EPI_QKV_ROPE) {
        const QkvEpilogue &q = p.qkv;
        if (!q.rope_cos || !q.rope_sin || !q.pos || !q.seq || !q.q_out || !q.k_cache || !q.v_cache || q.head_dim % 2 != 0 ||
            w.rows != (q.n_head + 2 * q.n_kv_head) * q.head_dim)
            return hipErrorInvalidValue;
    }
    const int block = w.format == FMT_F16 ? 8 : w.format == FMT_F32 ? 4 : format_block_elems(w.format);
    if (w.cols % block != 0 || w.qs_row_bytes % 16 != 0 || (p.norm_x && w.cols % 8 != 0)) return hipErrorInvalidValue;
    if ((w.format == FMT_Q8_0 || w.format == FMT_Q4_0) && !w.scales) return hipErrorInvalidValue;

    // events of its own only for a single launch
    struct EventScope {
        EventScope(hipEvent_t a, hipEvent_t b) { tl_start_event = a; tl_stop_event = b; }
        ~EventScope() { tl_start_event = tl_stop_event = nullptr; }
    } scope(p.batch <= 2 ? p.start_event : nullptr, p.batch <= 2 ? p.stop_event : nullptr);
    struct CapacityScope {
        explicit CapacityScope(int n) { tl_argmax_capacity = n; }
        ~CapacityScope() { tl_argmax_capacity = 0; }
    } capacity(p.epilogue == EPI_ARGMAX ? p.argmax_capacity : 0);
    // batches beyond 2 run as successive pairs (each pair re-reads the weights); the matrix-core Q4_K kernel takes four rows at once
    const bool fours = p.batch > 2 && gemv_takes_rows(w, p.batch) && !p.merge_partials;
    for (int b0 = 0, nb = 0; b0 < p.batch; b0 += nb) {
        const bool wide = fours && (w.format == FMT_Q4_K || w.format == FMT_Q4_0) && p.batch - b0 >= 5 && p.batch - b0 <= 8 && q4k_wide_mode() != 0 && w.rows <= q4k_wide_max_rows() &&
                          (p.epilogue == EPI_STORE_F32 || p.epilogue == EPI_ADD_RESIDUAL) && p.x && !p.split_x;
        nb = wide ? p.batch - b0 : fours && p.batch - b0 == 8 ? 8 : fours && p.batch - b0 >= 4 ? 4 : p.batch - b0 >= 2 ? 2 : 1;
        KernelArgs a;
        a.qs = w.qs; a.tiled = w.tiled; a.scales = w.scales; a.qs_row_bytes = w.qs_row_bytes; a.rows = w.rows; a.cols = w.cols;
        a.x = p.x ? p.x + (size_t)b0 * w.cols * (p.split_x ? 2 : 1) : nullptr;
        a.split_x = p.split_x ? 1 : 0;
        a.split_out = p.split_out ? 1 : 0;
        a.merge_partials = p.merge_partials;   // batch <= 2 here: one launch
        a.merge_head_dim = p.merge_head_dim;
        a.y = p.y ? p.y + (size_t)b0 * w.rows : nullptr;
        a.residual = p.residual ? p.residual + (size_t)b0 * w.rows : nullptr;
        a.out_f16 = p.out_f16 ? p.out_f16 + (size_t)b0 * (w.rows / 2) : nullptr;
        a.qkv = p.qkv;
        a.part_value = p.argmax_value;
        a.part_index = p.argmax_index;
        a.stamps = p.stamps;
        a.stamp_capacity = p.stamp_capacity;
        if (p.epilogue == EPI_QKV_ROPE) {
            a.qkv.pos += b0;
            a.qkv.seq += b0;
            a.qkv.q_out += (size_t)b0 * p.qkv.n_head * p.qkv.head_dim;
        }
        a.epilogue = p.epilogue;
        a.norm_x = p.norm_x ? p.norm_x + (size_t)b0 * w.cols : nullptr;
        a.norm_w = p.norm_w;
        a.norm_eps = p.norm_eps;
        hipError_t e;
        switch (w.format) {
        case FMT_Q4_K:
            if (nb >= 5 && wide) {
                bool launched = false;
                e = try_q4k_wide(a, nb, stream, &launched);
                if (e == hipSuccess && !launched) e = hipErrorInvalidValue;
            } else if (nb == 8) {   // only the matrix-core kernel takes eight rows
                bool launched = false;
                e = try_q4k_mfma<8>(a, stream, &launched);
                if (e == hipSuccess && !launched) e = hipErrorInvalidValue;
            } else e = nb == 1 ? launch_q4k<1>(a, stream) : nb == 2 ? launch_q4k<2>(a, stream) : launch_q4k<4>(a, stream);
            break;
        case FMT_Q4_0:
            if (nb >= 5 && wide) {
                bool launched = false;
                e = try_q40_wide(a, nb, stream, &launched);
                if (e == hipSuccess && !launched) e = hipErrorInvalidValue;
            } else if (nb >= 4) {   // four and eight rows only on the matrix cores; where that kernel declines the shape, two rows at a time
                bool launched = false;
                e = nb == 8 ? try_q40_mfma<8>(a, stream, &launched) : try_q40_mfma<4>(a, stream, &launched);
                if (e == hipSuccess && !launched) { nb = 2; e = launch_q40<2>(a, stream); }
            } else e = nb == 1 ? launch_q40<1>(a, stream) : launch_q40<2>(a, stream);
            break;
        case FMT_Q8_0: e = nb == 1 ? launch_q80<1>(a, stream) : launch_q80<2>(a, stream); break;
        case FMT_F16: e = nb == 1 ? launch_f16<1>(a, stream) : launch_f16<2>(a, stream); break;
        case FMT_F32: e = launch_fmt<FMT_F32>(a, nb, stream); break;
        default: e = hipErrorInvalidValue;
        }
        if (e != hipSuccess) return e;
        if (p.epilogue == EPI_ARGMAX) {
            if (p.argmax_blocks) *p.argmax_blocks = (int)tl_last_grid;
            if (tl_last_grid > (unsigned)p.argmax_capacity) return hipErrorInvalidValue;   // nothing was launched
        }
    }
    return hipSuccess;
}

}  // namespace esp
