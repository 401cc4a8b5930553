// The decoder trunk of one batch-1 decode step as a single persistent launch: for every layer,
// RMSNorm + q|k|v GEMV + RoPE + KV write, attention over the cache, Wo GEMV + residual, RMSNorm +
// gate|up GEMV + SiLU*up, down GEMV + residual  (RealModelInferenceEngine.swift:6221-6347), with
// grid-wide barriers between the five phases instead of kernel boundaries.
//
// Idea: a dependent kernel boundary costs 4-5 us on this chip (dispatch, first-load latency, cache
// write-back), six per layer, and HBM idles meanwhile.  Here
//   * every wavefront issues the weight loads of its first row pair of the NEXT phase as it enters the
//     barrier, so the weight stream continues while the barrier completes;
//   * a barrier is two levels of agent-scope relaxed atomics (16 leaf counters, a root, 16 flags) with no
//     cache write-back fences.  Everything one phase hands to the next (hidden state, q, the new K/V rows,
//     attention partials, context, activations) is written with agent-scope stores (write-through) and
//     read with agent-scope loads, which is what makes the fences unnecessary: the eight L2 caches of the
//     chip are not coherent with each other for ordinary accesses;
//   * K/V rows of earlier positions were written by earlier launches and are read with ordinary 128-bit
//     loads; the current position's rows are written here and never read before the barrier that
//     follows, so no cache can hold a stale copy of them;
//   * the grid is sized by the occupancy query so that all workgroups are resident at once, and every
//     spin is bounded: a barrier that does not complete records a time-out, raises an abort flag that
//     cuts all later waits short, and the kernel runs to its end (with wrong results that the host
//     reports as an error) instead of hanging.
//
// Measured on MI355X (8B-architecture Q4_K, batch 1): the results are bit-identical to the separate
// kernels, but a round trip of an agent-scope access to the memory side takes about 0.8 us, a barrier
// plus the staging after it needs five to six of them (4.6 us, as much as the kernel boundary it
// replaces), and the attention phase with its partial hand-off needs about ten (16.7 us against 10.3 us
// for the two separate kernels).  One step takes 2.34 ms against 1.78 ms for the separate kernels, so the
// runtime uses this kernel only when asked to (ESPRESSO_HIP_FUSED_TRUNK=1 or esp_llama_set_fused_trunk).
//
// The arithmetic of each phase is the GEMV / attention code of the separate kernels.
#include "layer_kernel.h"

#include <cstdlib>

#include "gemv_device.h"

namespace esp {
namespace {

using namespace detail;

// ---- agent-scope (cross-XCD coherent) accesses -------------------------------------------------
template <typename T>
__device__ __forceinline__ T ld(const T *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
template <typename T>
__device__ __forceinline__ void st(T *p, T v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ uint4 ld16(const void *p) {
    const uint64_t *q = reinterpret_cast<const uint64_t *>(p);
    const uint64_t a = ld(q), b = ld(q + 1);
    return make_uint4((u32)a, (u32)(a >> 32), (u32)b, (u32)(b >> 32));
}
__device__ __forceinline__ float4 ld_f4(const float *p) { return __builtin_bit_cast(float4, ld16(p)); }

// ---- barrier ---------------------------------------------------------------------------------------
constexpr int kLeaves = 16, kPad = 32;                 // 32 words = 128 bytes between counters
constexpr int kRootWord = kLeaves * kPad;              // 512
constexpr int kFlagWord = kRootWord + kPad;            // 544
constexpr int kAttnWord = kFlagWord + kLeaves * kPad;  // 1056: one counter per KV head, 128 bytes apart
constexpr int kAbortWord = kAttnWord + 16 * kPad;      // 1568
constexpr int kClearWords = kAbortWord + kPad;         // cleared before every launch
constexpr int kTimeoutWord = kTrunkSyncWords - 1;      // cumulative, never cleared
static_assert(kClearWords < kTimeoutWord, "sync state layout");
constexpr unsigned kSpinLimit = 1u << 15;

// `prefetch` issues the weight loads of the next phase.  It runs after this wavefront's stores have drained
// (loads and stores share one counter, so a later wait for the stores would also wait for the loads) and,
// for the wavefront whose first lane runs the atomics, only after the barrier: the value an atomic returns
// arrives behind every load issued before it.
template <typename Prefetch>
__device__ __forceinline__ void grid_barrier(unsigned *sync, unsigned gen, Prefetch prefetch) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // this wavefront's stores have reached memory
    if (threadIdx.x >= 64) prefetch();
    __syncthreads();
    if (threadIdx.x == 0) {
        const unsigned g = gridDim.x, leaf = blockIdx.x % kLeaves;
        const unsigned members = g / kLeaves + (leaf < g % kLeaves ? 1u : 0u), leaves = g < kLeaves ? g : kLeaves;
        const unsigned old = __hip_atomic_fetch_add(&sync[leaf * kPad], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (old + 1 == gen * members) {
            const unsigned r = __hip_atomic_fetch_add(&sync[kRootWord], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (r + 1 == gen * leaves)
                for (unsigned i = 0; i < leaves; i++) st(&sync[kFlagWord + i * kPad], gen);
        }
        unsigned spins = 0;
        while (ld(&sync[kFlagWord + leaf * kPad]) < gen) {
            __builtin_amdgcn_s_sleep(2);
            ++spins;
            if ((spins & 255u) == 0u && ld(&sync[kAbortWord]) != 0u) break;   // another workgroup gave up
            if (spins > kSpinLimit) {
                __hip_atomic_fetch_add(&sync[kTimeoutWord], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                st(&sync[kAbortWord], 1u);
                break;
            }
        }
    }
    __syncthreads();
    if (threadIdx.x < 64) prefetch();
}

// ---- activations into LDS (the Q4_K GEMV layout) ---------------------------------------------------
// x = rmsnorm(hidden) * w, all loads issued before the first use
template <int IPR>
__device__ __forceinline__ void stage_normalized(const float *hidden, const float *w, float eps, uint4 *xs4, float *xsum, float *red) {
    constexpr int K = IPR / 32, cols = IPR * 64, XSTRIDE = IPR | 1;
    const int tid = threadIdx.x;
    float4 v0[K], v1[K], g0[K], g1[K];
#pragma unroll
    for (int k = 0; k < K; k++) {
        const int g = tid + k * kThreads;
        v0[k] = ld_f4(hidden + 8 * g);
        v1[k] = ld_f4(hidden + 8 * g + 4);
        g0[k] = reinterpret_cast<const float4 *>(w)[2 * g];
        g1[k] = reinterpret_cast<const float4 *>(w)[2 * g + 1];
    }
    float s = 0.0f;
#pragma unroll
    for (int k = 0; k < K; k++) s += sum_squares(v0[k], v1[k]);
    const float inv = 1.0f / sqrtf(workgroup_sum(s, red) / (float)cols + eps);
#pragma unroll
    for (int k = 0; k < K; k++) q4k_store_group(normalized_group(v0[k], v1[k], g0[k], g1[k], inv), 0, tid + k * kThreads, cols, XSTRIDE, xs4, xsum);
}
// x = fp16 vector written by the previous phase
template <int IPR>
__device__ __forceinline__ void stage_half(const uint16_t *x, uint4 *xs4, float *xsum) {
    constexpr int K = IPR / 32, cols = IPR * 64, XSTRIDE = IPR | 1;
    const int tid = threadIdx.x;
    uint4 v[K];
#pragma unroll
    for (int k = 0; k < K; k++) v[k] = ld16(x + 8 * (tid + k * kThreads));
#pragma unroll
    for (int k = 0; k < K; k++) q4k_store_group(v[k], 0, tid + k * kThreads, cols, XSTRIDE, xs4, xsum);
}

// ---- one GEMV phase --------------------------------------------------------------------------------
template <int IPR, int TEAM>
__device__ __forceinline__ void load_pair(const uint8_t *qs, size_t row_bytes, int rows, int pair, Q4KItem (&buf)[2]) {
    constexpr int TOTAL = 2 * IPR, TEAM_LANES = TEAM * 64;
    static_assert((TOTAL + TEAM_LANES - 1) / TEAM_LANES <= 2, "two items per lane per pair");
    const int tl = ((threadIdx.x >> 6) % TEAM) * 64 + (threadIdx.x & 63);
    const int row_a = 2 * pair < rows ? 2 * pair : rows - 1, row_b = 2 * pair + 1 < rows ? 2 * pair + 1 : rows - 1;
    const uint8_t *base_a = qs + (size_t)row_a * row_bytes, *base_b = qs + (size_t)row_b * row_bytes;
#pragma unroll
    for (int p = 0; p < 2; p++) {
        const int t = tl + p * TEAM_LANES, tt = t < TOTAL ? t : 0;
        const bool second = tt >= IPR;
        const int i = tt - (second ? IPR : 0);
        const uint8_t *bp = (second ? base_b : base_a) + (size_t)(i >> 2) * 144;
        buf[p].hdr = *reinterpret_cast<const uint4 *>(bp);
        const uint4 *q = reinterpret_cast<const uint4 *>(bp + 16 + (i & 3) * 32);
        buf[p].q0 = q[0];
        buf[p].q1 = q[1];
    }
}
template <int TEAM>
__device__ __forceinline__ int first_pair() { return blockIdx.x * (kWaves / TEAM) + (threadIdx.x >> 6) / TEAM; }

// Issues the loads of this wavefront's first row pair of a matrix (call before the barrier that precedes
// the phase).
template <int IPR, int TEAM>
__device__ __forceinline__ void prefetch_first(const uint8_t *qs, size_t row_bytes, int rows, Q4KItem (&buf0)[2]) {
    const int pair = first_pair<TEAM>();
    if (pair < (rows + 1) / 2) load_pair<IPR, TEAM>(qs, row_bytes, rows, pair, buf0);
}

// rows x (64 * IPR) Q4_K matrix times the staged activations.  buf0 already holds the first pair.
// epilogue(pair, sum_a, sum_b) runs in one lane per row pair.
template <int IPR, int TEAM, typename Epilogue>
__device__ __forceinline__ void gemv_phase(const uint8_t *qs, size_t row_bytes, int rows, Q4KItem (&buf0)[2], const Q4KLane &L,
                                           const uint4 *xs4, const float *xsum, float *red, Epilogue epilogue) {
    constexpr int cols = IPR * 64, XSTRIDE = IPR | 1, TOTAL = 2 * IPR, TEAM_LANES = TEAM * 64, TEAMS = kWaves / TEAM;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, tl = (wave % TEAM) * 64 + lane;
    const int npairs = (rows + 1) / 2, n_teams = gridDim.x * TEAMS;
    const int iters = (npairs + n_teams - 1) / n_teams;   // the same for every workgroup: barriers line up

    auto process = [&](const Q4KItem (&buf)[2], int pair, int parity) {
        float acc_a = 0.0f, acc_b = 0.0f;
        if (pair < npairs) {
#pragma unroll
            for (int p = 0; p < 2; p++) {
                const int t = tl + p * TEAM_LANES;
                const bool valid = t < TOTAL;
                const int tt = valid ? t : 0;
                const bool second = tt >= IPR;
                float v[1];
                q4k_item_dots<1, XSTRIDE>(buf[p], L, xs4, xsum, tt - (second ? IPR : 0), XSTRIDE, cols, v);
                const float vv = valid ? v[0] : 0.0f;
                acc_a += second ? 0.0f : vv;
                acc_b += second ? vv : 0.0f;
            }
            acc_a = wave_sum(acc_a);
            acc_b = wave_sum(acc_b);
        }
        if constexpr (TEAM == 1) {
            if (pair < npairs && lane == 0) epilogue(pair, acc_a, acc_b);
        } else {
            float *slot = red + parity * kWaves * 2;
            if (lane == 0) { slot[wave * 2] = acc_a; slot[wave * 2 + 1] = acc_b; }
            __syncthreads();
            if (pair < npairs && tl == 0) {
                float sa = slot[wave * 2], sb = slot[wave * 2 + 1];
#pragma unroll
                for (int w = 1; w < TEAM; w++) { sa += slot[(wave + w) * 2]; sb += slot[(wave + w) * 2 + 1]; }
                epilogue(pair, sa, sb);
            }
        }
    };

    Q4KItem buf1[2];
    int pair = first_pair<TEAM>();
    for (int j = 0; j < iters; j += 2) {
        int next = pair + n_teams;
        if (next < npairs) load_pair<IPR, TEAM>(qs, row_bytes, rows, next, buf1);
        process(buf0, pair, 0);
        pair = next;
        if (j + 1 < iters) {
            next = pair + n_teams;
            if (next < npairs) load_pair<IPR, TEAM>(qs, row_bytes, rows, next, buf0);
            process(buf1, pair, 1);
            pair = next;
        }
    }
}

// ---- attention of one (KV head, slice of the prefix), then the merge by the last slice to finish ------
constexpr int kMaxSplits = 32;

template <int CTRL>
__device__ __forceinline__ float dpp_get(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xF, 0xF, false));
}
template <int N>
__device__ __forceinline__ float group_sum(float v) {
    v += dpp_get<0xB1>(v);
    v += dpp_get<0x4E>(v);
    v += dpp_get<0x141>(v);
    if (N == 16) v += dpp_get<0x140>(v);
    return v;
}
template <int N>
__device__ __forceinline__ float max_over_groups(float v) {
    float m = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));
#pragma unroll
    for (int l = N; l < 64; l += N) m = fmaxf(m, __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), l)));
    return m;
}
__device__ __forceinline__ float from_half_bits(uint16_t b) { return (float)__builtin_bit_cast(_Float16, b); }
__device__ __forceinline__ uint16_t to_half_bits(float v) { return __builtin_bit_cast(uint16_t, (_Float16)v); }

template <int HD, int G, bool KV_F16>
__device__ __forceinline__ void attention_phase(const TrunkArgs &a, const TrunkLayer &layer, int layer_index, float *lds) {
    constexpr int WAVES = 4, LPT = HD / 8, SLOTS = 64 / LPT, KW = KV_F16 ? 1 : 2;
    const int item = blockIdx.x;
    const int splits = a.splits;
    if (item >= a.n_kv_head * splits) return;        // workgroup-uniform: the others go straight to the barrier
    const int kvh = item % a.n_kv_head, split = item / a.n_kv_head;
    float *wm = lds;                                   // [WAVES][G]
    float *wl = wm + WAVES * G;                        // [WAVES][SLOTS][G]
    float *wacc = wl + WAVES * SLOTS * G;              // [WAVES][SLOTS][G][HD]
    int *last_flag = reinterpret_cast<int *>(wacc + WAVES * SLOTS * G * HD);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int visible = a.pos[0] + 1, kd = a.n_kv_head * HD;
    const size_t seq_base = (size_t)a.seq[0] * a.cache_seq_stride;
    const float scale = 1.0f / sqrtf((float)HD);
    const int slot = lane / LPT, seg = (lane % LPT) * 8;

    float q[G][8];
#pragma unroll
    for (int g = 0; g < G; g++) {
        const float *qp = a.q + (size_t)(kvh * G + g) * HD + seg;
        const float4 q0 = ld_f4(qp), q1 = ld_f4(qp + 4);
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
            const u32 w[4] = {r[0].x, r[0].y, r[0].z, r[0].w};
#pragma unroll
            for (int i = 0; i < 4; i++) { out[2 * i] = from_half_bits((uint16_t)(w[i] & 0xFFFFu)); out[2 * i + 1] = from_half_bits((uint16_t)(w[i] >> 16)); }
        } else {
            out[0] = __uint_as_float(r[0].x); out[1] = __uint_as_float(r[0].y); out[2] = __uint_as_float(r[0].z); out[3] = __uint_as_float(r[0].w);
            out[4] = __uint_as_float(r[KW - 1].x); out[5] = __uint_as_float(r[KW - 1].y); out[6] = __uint_as_float(r[KW - 1].z); out[7] = __uint_as_float(r[KW - 1].w);
        }
    };
    constexpr int U = 2;
    const int stride = splits * WAVES * SLOTS;
    for (int t0 = (split * WAVES + wave) * SLOTS; t0 < visible; t0 += stride * U) {
        uint4 kr[U][KW], vr[U][KW];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int t = t0 + u * stride + slot;
            const size_t off = seq_base + (size_t)(t < visible ? t : 0) * kd + (size_t)kvh * HD + seg;
            const uint4 *kp = KV_F16 ? reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(layer.k_cache) + off)
                                     : reinterpret_cast<const uint4 *>(reinterpret_cast<const float *>(layer.k_cache) + off);
            const uint4 *vp = KV_F16 ? reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(layer.v_cache) + off)
                                     : reinterpret_cast<const uint4 *>(reinterpret_cast<const float *>(layer.v_cache) + off);
#pragma unroll
            for (int i = 0; i < KW; i++) { kr[u][i] = kp[i]; vr[u][i] = vp[i]; }
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int t = t0 + u * stride + slot;
            const bool valid = t < visible;
            if (t0 + u * stride >= visible) break;
            float k[8], v[8];
            unpack8(kr[u], k);
            unpack8(vr[u], v);
#pragma unroll
            for (int g = 0; g < G; g++) {
                float d = 0.0f;
#pragma unroll
                for (int i = 0; i < 8; i++) d = __builtin_fmaf(q[g][i], k[i], d);
                d = group_sum<LPT>(d);
                const float sc = valid ? __fmul_rn(d, scale) : -INFINITY;
                const float cm = max_over_groups<LPT>(sc);
                const float m_new = fmaxf(mx[g], cm);
                const float alpha = expf(mx[g] - m_new);
                const float p = valid ? expf(sc - m_new) : 0.0f;
                l[g] = __builtin_fmaf(l[g], alpha, p);
#pragma unroll
                for (int i = 0; i < 8; i++) acc[g][i] = __builtin_fmaf(p, v[i], __fmul_rn(acc[g][i], alpha));
                mx[g] = m_new;
            }
        }
    }
#pragma unroll
    for (int g = 0; g < G; g++) {
#pragma unroll
        for (int i = 0; i < 8; i++) wacc[((wave * SLOTS + slot) * G + g) * HD + seg + i] = acc[g][i];
        if (lane % LPT == 0) wl[(wave * SLOTS + slot) * G + g] = l[g];
        if (lane == 0) wm[wave * G + g] = mx[g];
    }
    __syncthreads();
    // merge over wavefronts and slots, publish this slice's state
    float *scratch = a.attn_scratch + ((size_t)kvh * splits) * G * (HD + 2);
    for (int i = tid; i < G * HD; i += kThreads) {
        const int g = i / HD, dch = i % HD;
        float M = wm[g];
#pragma unroll
        for (int w = 1; w < WAVES; w++) M = fmaxf(M, wm[w * G + g]);
        float Ls = 0.0f, As = 0.0f;
#pragma unroll
        for (int w = 0; w < WAVES; w++) {
            const float f = wm[w * G + g] == -INFINITY ? 0.0f : expf(wm[w * G + g] - M);
            float lw = 0.0f, aw = 0.0f;
#pragma unroll
            for (int sl = 0; sl < SLOTS; sl++) { lw += wl[(w * SLOTS + sl) * G + g]; aw += wacc[((w * SLOTS + sl) * G + g) * HD + dch]; }
            Ls = __builtin_fmaf(lw, f, Ls);
            As = __builtin_fmaf(aw, f, As);
        }
        float *ps = scratch + ((size_t)split * G + g) * (HD + 2);
        st(ps + 2 + dch, As);
        if (dch == 0) { st(ps, M); st(ps + 1, Ls); }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0) {
        const unsigned old = __hip_atomic_fetch_add(&a.sync[kAttnWord + kvh * kPad], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        *last_flag = old + 1 == (unsigned)splits * (unsigned)(layer_index + 1);
    }
    __syncthreads();
    if (!*last_flag) return;
    // the last slice of this KV head to finish merges all of them, in slice order
    float *pm = lds, *pf = lds + G * kMaxSplits;     // [G][kMaxSplits] maxima and sums of the slices
    if (tid < G * kMaxSplits) {
        const int g = tid / kMaxSplits, sp = tid % kMaxSplits;
        const float *ps = scratch + ((size_t)(sp < splits ? sp : 0) * G + g) * (HD + 2);
        pm[tid] = ld(ps);
        pf[tid] = ld(ps + 1);
    }
    __syncthreads();
    for (int i = tid; i < G * HD; i += kThreads) {
        const int g = i / HD, dch = i % HD;
        float pa[kMaxSplits];
#pragma unroll
        for (int sp = 0; sp < kMaxSplits; sp++) pa[sp] = ld(scratch + ((size_t)(sp < splits ? sp : 0) * G + g) * (HD + 2) + 2 + dch);
        float M = -INFINITY;
#pragma unroll
        for (int sp = 0; sp < kMaxSplits; sp++) if (sp < splits) M = fmaxf(M, pm[g * kMaxSplits + sp]);
        float Lt = 0.0f, At = 0.0f;
#pragma unroll
        for (int sp = 0; sp < kMaxSplits; sp++) {
            const float m = pm[g * kMaxSplits + sp];
            const float f = (sp < splits && m != -INFINITY) ? expf(m - M) : 0.0f;
            Lt = __builtin_fmaf(pf[g * kMaxSplits + sp], f, Lt);
            At = __builtin_fmaf(pa[sp], f, At);
        }
        st(a.ctx + (size_t)(kvh * G + g) * HD + dch, to_half_bits(Lt > 0.0f ? At / Lt : 0.0f));
    }
}

// ---- the kernel ------------------------------------------------------------------------------------
template <int IPR_D, int IPR_H, int HD, int G>
__global__ __launch_bounds__(kThreads, 2) void trunk_kernel(TrunkArgs a) {
    extern __shared__ uint4 smem_raw[];
    constexpr int IPR_MAX = IPR_D > IPR_H ? IPR_D : IPR_H;
    uint4 *xs4 = smem_raw;                                                   // [8][IPR | 1] x 8 fp16
    float *xsum = reinterpret_cast<float *>(smem_raw + 8 * (IPR_MAX | 1));  // [cols / 32]
    float *red = xsum + IPR_MAX * 2;                                         // [2][kWaves][2]
    float *norm_red = red + 2 * kWaves * 2;                                  // [kWaves]
    constexpr int d = IPR_D * 64, hd = IPR_H * 64;
    constexpr size_t row_bytes_d = (size_t)(d / 256) * 144, row_bytes_h = (size_t)(hd / 256) * 144;
    const int ad = a.n_head * HD, kd = a.n_kv_head * HD, qkv_rows = ad + 2 * kd;
    const Q4KLane L = q4k_lane_constants(threadIdx.x & 63);
    const int pos = a.pos[0];
    const size_t seq_base = (size_t)a.seq[0] * a.cache_seq_stride;
    unsigned gen = 0;

    Q4KItem buf0[2];
    prefetch_first<IPR_D, 1>(a.layers[0].wqkv, row_bytes_d, qkv_rows, buf0);
    for (int li = 0; li < a.n_layer; li++) {
        const TrunkLayer layer = a.layers[li];
        // ---- q|k|v: RMSNorm while staging, RoPE and the KV write in the epilogue ----
        stage_normalized<IPR_D>(a.hidden, layer.rms_att, a.norm_eps, xs4, xsum, norm_red);
        __syncthreads();
        gemv_phase<IPR_D, 1>(layer.wqkv, row_bytes_d, qkv_rows, buf0, L, xs4, xsum, red, [&](int pair, float va, float vb) {
            constexpr int half = HD / 2;
            const int r0 = 2 * pair;
            if (r0 < ad + kd) {
                const bool is_q = r0 < ad;
                const int pr = is_q ? pair : pair - ad / 2;
                const int h = pr / half, j = pr - h * half;
                const float c = a.rope_cos[(size_t)pos * half + j], sn = a.rope_sin[(size_t)pos * half + j];
                const float o0 = __fsub_rn(__fmul_rn(va, c), __fmul_rn(vb, sn));
                const float o1 = __fadd_rn(__fmul_rn(va, sn), __fmul_rn(vb, c));
                if (is_q) {
                    st(a.q + (size_t)h * HD + j, o0);
                    st(a.q + (size_t)h * HD + j + half, o1);
                } else {
                    const size_t o = seq_base + (size_t)pos * kd + (size_t)h * HD + j;
                    if (a.kv_f16) {
                        st(reinterpret_cast<uint16_t *>(layer.k_cache) + o, to_half_bits(o0));
                        st(reinterpret_cast<uint16_t *>(layer.k_cache) + o + half, to_half_bits(o1));
                    } else {
                        st(reinterpret_cast<float *>(layer.k_cache) + o, o0);
                        st(reinterpret_cast<float *>(layer.k_cache) + o + half, o1);
                    }
                }
            } else {
                const size_t o = seq_base + (size_t)pos * kd + (size_t)(r0 - ad - kd);
                if (a.kv_f16) {
                    st(reinterpret_cast<u32 *>(reinterpret_cast<uint16_t *>(layer.v_cache) + o), pack_half2(va, vb));
                } else {
                    st(reinterpret_cast<float *>(layer.v_cache) + o, va);
                    st(reinterpret_cast<float *>(layer.v_cache) + o + 1, vb);
                }
            }
        });
        grid_barrier(a.sync, ++gen, [&] { prefetch_first<IPR_D, 1>(layer.wo, row_bytes_d, d, buf0); });

        // ---- attention ----
        if (a.kv_f16) attention_phase<HD, G, true>(a, layer, li, reinterpret_cast<float *>(smem_raw));
        else attention_phase<HD, G, false>(a, layer, li, reinterpret_cast<float *>(smem_raw));
        grid_barrier(a.sync, ++gen, [] {});

        // ---- Wo + residual ----
        stage_half<IPR_D>(a.ctx, xs4, xsum);
        __syncthreads();
        gemv_phase<IPR_D, 1>(layer.wo, row_bytes_d, d, buf0, L, xs4, xsum, red, [&](int pair, float va, float vb) {
            float *h = a.hidden + 2 * pair;
            const float r0 = ld(h), r1 = ld(h + 1);
            st(h, r0 + va);
            st(h + 1, r1 + vb);
        });
        grid_barrier(a.sync, ++gen, [&] { prefetch_first<IPR_D, 1>(layer.w13, row_bytes_d, 2 * hd, buf0); });

        // ---- gate|up: RMSNorm while staging, SiLU(gate) * up in the epilogue ----
        stage_normalized<IPR_D>(a.hidden, layer.rms_ffn, a.norm_eps, xs4, xsum, norm_red);
        __syncthreads();
        gemv_phase<IPR_D, 1>(layer.w13, row_bytes_d, 2 * hd, buf0, L, xs4, xsum, red, [&](int pair, float va, float vb) {
            const float hg = __fmul_rn(0.5f, va);
            const float silu = __fmul_rn(hg, __fadd_rn(1.0f, tanhf(hg)));
            st(a.act + pair, to_half_bits(__fmul_rn(silu, vb)));
        });
        grid_barrier(a.sync, ++gen, [&] { prefetch_first<IPR_H, 4>(layer.w2, row_bytes_h, d, buf0); });

        // ---- down + residual ----
        stage_half<IPR_H>(a.act, xs4, xsum);
        __syncthreads();
        gemv_phase<IPR_H, 4>(layer.w2, row_bytes_h, d, buf0, L, xs4, xsum, red, [&](int pair, float va, float vb) {
            float *h = a.hidden + 2 * pair;
            const float r0 = ld(h), r1 = ld(h + 1);
            st(h, r0 + va);
            st(h + 1, r1 + vb);
        });
        grid_barrier(a.sync, ++gen, [&] {
            if (li + 1 < a.n_layer) prefetch_first<IPR_D, 1>(a.layers[li + 1].wqkv, row_bytes_d, qkv_rows, buf0);
        });
    }
}

__global__ void clear_sync_kernel(unsigned *sync) {
    for (int i = threadIdx.x; i < kClearWords; i += blockDim.x) sync[i] = 0u;
}

template <int IPR_D, int IPR_H, int HD, int G>
hipError_t launch_instance(const TrunkArgs &args, hipStream_t stream) {
    constexpr int IPR_MAX = IPR_D > IPR_H ? IPR_D : IPR_H;
    constexpr size_t gemv_lds = (size_t)8 * (IPR_MAX | 1) * 16 + (size_t)IPR_MAX * 2 * 4 + (size_t)(2 * kWaves * 2 + kWaves) * 4;
    constexpr int LPT = HD / 8, SLOTS = 64 / LPT;
    constexpr size_t attn_lds = (size_t)(4 * G + 4 * SLOTS * G + 4 * SLOTS * G * HD) * 4 + 16;
    constexpr size_t lds = gemv_lds > attn_lds ? gemv_lds : attn_lds;
    auto kernel = trunk_kernel<IPR_D, IPR_H, HD, G>;
    static int grid = 0;
    if (grid == 0) {
        hipError_t e = hipSuccess;
        if (lds > 48 * 1024) e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        int per_cu = 0, dev = 0, cus = 0;
        e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, kThreads, lds);
        if (e == hipSuccess) e = hipGetDevice(&dev);
        if (e == hipSuccess) e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
        if (e != hipSuccess) return e;
        if (per_cu < 1 || cus < 1) return hipErrorLaunchOutOfResources;
        if (per_cu > 4) per_cu = 4;
        const char *env = getenv("ESPRESSO_HIP_TRUNK_WGS_PER_CU");
        if (env && atoi(env) >= 1 && atoi(env) < per_cu) per_cu = atoi(env);
        grid = per_cu * cus;
    }
    if (args.splits < 1 || args.splits > kMaxSplits || args.n_kv_head * args.splits > grid || args.n_kv_head > 16) return hipErrorInvalidValue;
    hipLaunchKernelGGL(clear_sync_kernel, dim3(1), dim3(256), 0, stream, args.sync);
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(kThreads), lds, stream, args);
    return hipGetLastError();
}

}  // namespace

bool trunk_kernel_supports(int d_model, int hidden_dim, int head_dim, int n_head, int n_kv_head) {
    return d_model == 4096 && hidden_dim == 14336 && head_dim == 128 && n_kv_head > 0 && n_head == 4 * n_kv_head && n_head * head_dim == d_model;
}

hipError_t launch_trunk_kernel(const TrunkArgs &args, int d_model, int hidden_dim, hipStream_t stream) {
    if (d_model == 4096 && hidden_dim == 14336) return launch_instance<64, 224, 128, 4>(args, stream);
    return hipErrorInvalidValue;
}

hipError_t trunk_kernel_timeouts(const unsigned *sync, hipStream_t stream, unsigned *out) {
    hipError_t e = hipMemcpyAsync(out, sync + kTimeoutWord, sizeof(unsigned), hipMemcpyDeviceToHost, stream);
    return e == hipSuccess ? hipStreamSynchronize(stream) : e;
}

}  // namespace esp
