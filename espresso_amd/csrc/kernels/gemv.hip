// Dequant-fused GEMV for batch-1/2 decode on gfx950:  y[b][r] = sum_c dequant(W)[r][c] * x[b][c].
//
// Replaces the seven vDSP_mmul GEMVs per layer of the reference's CPU-exact path
// (RealModelInferenceEngine.swift:6674-6697) with kernels that read the *packed* weights once.
//
// Shape of the kernel
//   * one workgroup = 4 wavefronts of 64 lanes; a wavefront owns R consecutive rows at a time;
//   * a lane's unit of work ("item") is one aligned 128-bit load of packed weights
//     (Q4_K/Q4_0: 32 weights, Q8_0: 16, F16: 8); consecutive lanes read consecutive 16-byte
//     pieces of the row, so a wavefront load covers 1 KiB of contiguous HBM;
//   * the fp16 activations are staged once per workgroup in LDS.  For the integer formats they are
//     stored with the two middle elements of every group of four swapped, (x0,x2,x1,x3): masking a
//     weight dword with 0x000F000F / 0x00FF00FF yields elements 0 and 2 of a group, so the matching
//     activation pair is then one aligned LDS dword;
//   * nibbles / bytes become exact fp16 integers with the 0x6400 exponent trick (1024 + n, then an
//     exact packed subtract), and v_dot2_f32_f16 forms exact products accumulated in fp32;
//   * block scales multiply the per-block partial sums, never the individual weights;
//   * Q4_K minimums use per-16-element sums of x precomputed in LDS:  sum (d*sc*n - dmin*m) x
//     = d*sc*sum(n x) - dmin*m*sum(x);
//   * a wavefront butterfly reduction leaves the row sums in every lane; lane 0 applies the epilogue.
//
// HBM traffic per launch = packed weight bytes + batch*cols*2 (x) + batch*rows*4 (y): the kernel is
// bound by HBM bandwidth; x is re-read from L2 once per workgroup.
#include "../common.h"

namespace esp {
namespace {

typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32;

constexpr int kThreads = 256;
constexpr int kWaves = 4;

__device__ __forceinline__ h2 as_h2(u32 v) { return __builtin_bit_cast(h2, v); }
__device__ __forceinline__ float fdot2(h2 a, h2 b, float c) { return __builtin_amdgcn_fdot2(a, b, c, false); }
__device__ __forceinline__ float half_bits_to_float(u32 bits16) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)bits16);
}
// (a & mask) | magic in one VALU op.  The compiler splits this into v_and + v_or when both constants
// are literals (a VOP3 instruction may read one scalar/literal operand), so the mask is pinned to a
// scalar register and the magic to a vector register.
__device__ __forceinline__ u32 and_or(u32 a, u32 mask, u32 magic) {
    u32 r;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "s"(mask), "v"(magic));
    return r;
}
__device__ __forceinline__ u32 dword_of(const uint4 &v, int k) {
    return k == 0 ? v.x : k == 1 ? v.y : k == 2 ? v.z : v.w;
}

// Sum over the 64 lanes with DPP row operations; the total is returned in every lane.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_term(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, ROW_MASK, 0xF, false));
}
__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_term<0xB1, 0xF>(v);   // quad_perm [1,0,3,2]
    v += dpp_term<0x4E, 0xF>(v);   // quad_perm [2,3,0,1]
    v += dpp_term<0x141, 0xF>(v);  // row_half_mirror: the other quad of each 8
    v += dpp_term<0x140, 0xF>(v);  // row_mirror: the other half of each 16
    v += dpp_term<0x142, 0xA>(v);  // row_bcast15 into rows 1 and 3
    v += dpp_term<0x143, 0xC>(v);  // row_bcast31 into rows 2 and 3
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

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
    const uint16_t *scales;
    size_t qs_row_bytes;
    int rows, cols;
    const uint16_t *x;
    float *y;
    const float *residual;
    int epilogue;
};

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
                a.out_f16[(size_t)b * (a.rows / 2) + pair] = __builtin_bit_cast(uint16_t, (_Float16)__fmul_rn(silu, vb[b]));
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


template <int FMT, int B, int R>
__global__ __launch_bounds__(kThreads) void gemv_kernel(KernelArgs a) {
    using T = Traits<FMT>;
    extern __shared__ uint4 smem_raw[];
    uint16_t *xs = reinterpret_cast<uint16_t *>(smem_raw);                 // [B][cols] fp16
    float *xsum = reinterpret_cast<float *>(xs + (size_t)B * a.cols);      // [B][cols/16] (Q4_K)
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int cols = a.cols;

    // ---- stage activations: 128-bit loads, middle elements of each group of four swapped ----
    {
        const uint4 *src = reinterpret_cast<const uint4 *>(a.x);
        uint4 *dst = reinterpret_cast<uint4 *>(xs);
        const int n16 = B * cols / 8;
        for (int i = tid; i < n16; i += kThreads) {
            uint4 v = src[i];
            if (T::kPermuteX) {
                uint4 p;
                p.x = __builtin_amdgcn_perm(v.y, v.x, 0x05040100u);
                p.y = __builtin_amdgcn_perm(v.y, v.x, 0x07060302u);
                p.z = __builtin_amdgcn_perm(v.w, v.z, 0x05040100u);
                p.w = __builtin_amdgcn_perm(v.w, v.z, 0x07060302u);
                v = p;
            }
            dst[i] = v;
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

    const int row0 = (blockIdx.x * kWaves + wave) * R;
    if (row0 >= a.rows) return;
    const int items = cols / T::kItemElems;

    float acc[R][B];
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int b = 0; b < B; b++) acc[r][b] = 0.0f;

    const uint8_t *rowp[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        int row = row0 + r < a.rows ? row0 + r : a.rows - 1;  // clamp: never read past the matrix
        rowp[r] = a.qs + (size_t)row * a.qs_row_bytes;
    }

    for (int item = lane; item < items; item += 64) {
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
                const uint4 q = *reinterpret_cast<const uint4 *>(rowp[r] + (size_t)item * 16);
                const int row = row0 + r < a.rows ? row0 + r : a.rows - 1;
                const float d = half_bits_to_float(a.scales[(size_t)row * (cols / 32) + item]);
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
                const uint4 q = *reinterpret_cast<const uint4 *>(rowp[r] + (size_t)item * 16);
                const int row = row0 + r < a.rows ? row0 + r : a.rows - 1;
                const float d = half_bits_to_float(a.scales[(size_t)row * (cols / 32) + (item >> 1)]);
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
                const uint4 q = *reinterpret_cast<const uint4 *>(rowp[r] + (size_t)item * 16);
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
                const uint4 q = *reinterpret_cast<const uint4 *>(rowp[r] + (size_t)item * 16);
#pragma unroll
                for (int b = 0; b < B; b++) {
                    float dot = 0.0f;
#pragma unroll
                    for (int k = 0; k < 4; k++) dot = fdot2(as_h2(dword_of(q, k)), as_h2(dword_of(xv[b], k)), dot);
                    acc[r][b] += dot;
                }
            }
        }
    }

#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int b = 0; b < B; b++) acc[r][b] = wave_sum(acc[r][b]);

    static_assert(R == 2, "the epilogues work on row pairs");
    if (lane == 0) {
        float va[B], vb[B];
#pragma unroll
        for (int b = 0; b < B; b++) { va[b] = acc[0][b]; vb[b] = acc[1][b]; }
        pair_epilogue<B>(a, row0 / 2, va, vb);
    }
}

// ---------------------------------------------------------------------------------------------
// Q4_K.  A lane's item is one 64-weight chunk of a super-block: 32 bytes of nibbles (two 128-bit
// loads) whose low nibbles are sub-block 2c and whose high nibbles are sub-block 2c+1, plus the
// block's 16-byte header (d, dmin, twelve scale bytes; the four lanes of a block read the same
// 16 bytes).  A wavefront owns two consecutive rows and walks their items as one flat range, so
// every lane is busy whenever cols is a multiple of 2048 (4096 -> 2 passes, 14336 -> 7 passes).
// Weight loads run two passes ahead of the arithmetic and the first ones are issued before the
// activations are staged.  Because rows hold a multiple of four items, a lane keeps the same chunk
// index c = lane & 3 for the whole kernel, so everything the 6-bit scale unpacking needs besides
// the header itself (shift counts, masks, which header word to read) is computed once.
//
// Nibbles are turned into fp16 with the exponent trick at offset 64: a nibble placed in mantissa
// bits 4..7 under exponent 0x5400 reads as 64 + n exactly.  v_dot2_f32_f16 then accumulates
// sum (64 + n) x in fp32 with exact products, and the offset is removed once per sub-block with
// the precomputed sum of its 32 activations:  sum n x = raw - 64 * sum x.
struct Q4KItem {
    uint4 q0, q1, hdr;
};

struct Q4KLane {   // per-lane constants of the scale unpacking
    bool upper;    // sub-blocks 4..7: six-bit values are split over two header words
    u32 sh_sc, sh_min, sh_top, mask_low, mask_top;
};

template <int B, int XSTRIDE>
__device__ __forceinline__ void q4k_item_dots(const Q4KItem &it, const Q4KLane &L, const uint4 *xs4, const float *xsum, int i,
                                              int xstride_rt, int cols, float v[B]) {
    const int xstride = XSTRIDE ? XSTRIDE : xstride_rt;
    // 6-bit (scale, min) of sub-blocks 2c and 2c+1, two at a time in the low 16 bits
    const u32 src_sc = L.upper ? it.hdr.w : it.hdr.y, src_min = L.upper ? it.hdr.w : it.hdr.z;
    const u32 scp = ((src_sc >> L.sh_sc) & L.mask_low) | ((it.hdr.y >> L.sh_top) & L.mask_top);
    const u32 mp = ((src_min >> L.sh_min) & L.mask_low) | ((it.hdr.z >> L.sh_top) & L.mask_top);
    const float sc_lo = (float)(scp & 0xFFu), sc_hi = (float)((scp >> 8) & 0xFFu);
    const float m_lo = (float)(mp & 0xFFu), m_hi = (float)((mp >> 8) & 0xFFu);
    const float d = half_bits_to_float(it.hdr.x & 0xFFFFu), dmin = half_bits_to_float(it.hdr.x >> 16);
#pragma unroll
    for (int b = 0; b < B; b++) {
        const uint4 *px = xs4 + (size_t)b * 8 * xstride + i;
        float raw_lo = 0.0f, raw_hi = 0.0f;
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const u32 w = dword_of(k < 4 ? it.q0 : it.q1, k & 3);
            const uint4 vl = px[(k >> 1) * xstride], vh = px[(4 + (k >> 1)) * xstride];
            const h2 xl02 = as_h2(dword_of(vl, (k & 1) * 2)), xl13 = as_h2(dword_of(vl, (k & 1) * 2 + 1));
            const h2 xh02 = as_h2(dword_of(vh, (k & 1) * 2)), xh13 = as_h2(dword_of(vh, (k & 1) * 2 + 1));
            const h2 l02 = as_h2(and_or(w << 4, 0x00F000F0u, 0x54005400u));
            const h2 l13 = as_h2(and_or(w >> 4, 0x00F000F0u, 0x54005400u));
            const h2 h02 = as_h2(and_or(w, 0x00F000F0u, 0x54005400u));
            const h2 h13 = as_h2(and_or(w >> 8, 0x00F000F0u, 0x54005400u));
            raw_lo = fdot2(l02, xl02, raw_lo);
            raw_lo = fdot2(l13, xl13, raw_lo);
            raw_hi = fdot2(h02, xh02, raw_hi);
            raw_hi = fdot2(h13, xh13, raw_hi);
        }
        const float2 xsp = *reinterpret_cast<const float2 *>(xsum + (size_t)b * (cols >> 5) + 2 * i);
        const float nx_lo = raw_lo - 64.0f * xsp.x, nx_hi = raw_hi - 64.0f * xsp.y;
        v[b] = d * (sc_lo * nx_lo + sc_hi * nx_hi) - dmin * (m_lo * xsp.x + m_hi * xsp.y);
    }
}

// IPR: items (64-weight chunks) per row when known at compile time, 0 = read from the arguments.
template <int B, int IPR>
__global__ __launch_bounds__(kThreads) void gemv_q4k_kernel(KernelArgs a) {
    extern __shared__ uint4 smem_raw[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int cols = IPR ? IPR * 64 : a.cols;
    const int ipr = IPR ? IPR : cols >> 6;   // items per row
    const int xstride = ipr | 1;             // 16-byte slots between consecutive k of one item
    constexpr int XSTRIDE = IPR ? (IPR | 1) : 0;
    const int total = 2 * ipr;               // items of the wavefront's row pair
    uint4 *xs4 = smem_raw;                                                        // [B][8][xstride] x 8 fp16, (x0,x2,x1,x3) order
    float *xsum = reinterpret_cast<float *>(smem_raw + (size_t)B * 8 * xstride);  // [B][cols/32] sub-block sums
    const int pair = blockIdx.x * kWaves + wave;
    const int row_a = 2 * pair < a.rows ? 2 * pair : a.rows - 1;          // clamped: loads stay inside the matrix
    const int row_b = 2 * pair + 1 < a.rows ? 2 * pair + 1 : a.rows - 1;
    const uint8_t *base_a = a.qs + (size_t)row_a * a.qs_row_bytes;
    const uint8_t *base_b = a.qs + (size_t)row_b * a.qs_row_bytes;

    Q4KLane L;
    {
        const int c = lane & 3, sh = (c & 1) * 16;
        L.upper = c >= 2;
        L.sh_sc = sh;
        L.sh_min = L.upper ? sh + 4 : sh;
        L.sh_top = sh + 2;
        L.mask_low = L.upper ? 0x0F0Fu : 0x3F3Fu;
        L.mask_top = L.upper ? 0x3030u : 0u;
    }

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
    auto stage_x = [&]() {
        // activations: 128-bit loads, middle elements of each group of four swapped, written to the
        // LDS layout [b][k][item] with an odd item stride (conflict-free for both the write and the
        // per-k reads of consecutive items); sub-block sums of 32 alongside
        const uint4 *xsrc = reinterpret_cast<const uint4 *>(a.x);
        const int n16 = B * cols / 8;
        for (int i = tid; i < n16; i += kThreads) {
            const uint4 v = xsrc[i];
            uint4 p;
            p.x = __builtin_amdgcn_perm(v.y, v.x, 0x05040100u);
            p.y = __builtin_amdgcn_perm(v.y, v.x, 0x07060302u);
            p.z = __builtin_amdgcn_perm(v.w, v.z, 0x05040100u);
            p.w = __builtin_amdgcn_perm(v.w, v.z, 0x07060302u);
            const int b = i / (cols / 8), g = i - b * (cols / 8);
            xs4[(size_t)b * 8 * xstride + (g & 7) * xstride + (g >> 3)] = p;
            float s = ((float)as_h2(v.x).x + (float)as_h2(v.x).y) + ((float)as_h2(v.y).x + (float)as_h2(v.y).y) +
                      ((float)as_h2(v.z).x + (float)as_h2(v.z).y) + ((float)as_h2(v.w).x + (float)as_h2(v.w).y);
            s += dpp_term<0xB1, 0xF>(s);
            s += dpp_term<0x4E, 0xF>(s);
            if ((lane & 3) == 0) xsum[i >> 2] = s;
        }
    };

    float acc_a[B], acc_b[B];
#pragma unroll
    for (int b = 0; b < B; b++) acc_a[b] = acc_b[b] = 0.0f;

    auto consume = [&](const Q4KItem &it, int t) {
        const bool valid = t < total;
        const int tt = valid ? t : 0;
        const bool second = tt >= ipr;
        const int i = tt - (second ? ipr : 0);
        float v[B];
        q4k_item_dots<B, XSTRIDE>(it, L, xs4, xsum, i, xstride, cols, v);
#pragma unroll
        for (int b = 0; b < B; b++) {
            const float vv = valid ? v[b] : 0.0f;
            acc_a[b] += second ? 0.0f : vv;
            acc_b[b] += second ? vv : 0.0f;
        }
    };

    if constexpr (IPR != 0) {
        constexpr int PASSES = (2 * IPR + 63) / 64;
        constexpr int NBUF = PASSES < 3 ? PASSES : 3;
        Q4KItem buf[NBUF];
#pragma unroll
        for (int p = 0; p < (PASSES > 2 ? 2 : PASSES); p++) buf[p] = load_item(p * 64 + lane);
        stage_x();
        __syncthreads();
#pragma unroll
        for (int p = 0; p < PASSES; p++) {
            if (PASSES > 2 && p + 2 < PASSES) buf[(p + 2) % NBUF] = load_item((p + 2) * 64 + lane);
            consume(buf[p % NBUF], p * 64 + lane);
        }
    } else {
        Q4KItem cur = load_item(lane);
        stage_x();
        __syncthreads();
        for (int t0 = 0; t0 < total; t0 += 64) {
            Q4KItem nxt = cur;
            if (t0 + 64 < total) nxt = load_item(t0 + 64 + lane);
            consume(cur, t0 + lane);
            cur = nxt;
        }
    }

#pragma unroll
    for (int b = 0; b < B; b++) {
        acc_a[b] = wave_sum(acc_a[b]);
        acc_b[b] = wave_sum(acc_b[b]);
    }
    if (lane == 0) pair_epilogue<B>(a, pair, acc_a, acc_b);
}

template <int B, int IPR>
hipError_t launch_q4k_ipr(const KernelArgs &a, hipStream_t stream) {
    const size_t lds = (size_t)B * 8 * ((a.cols / 64) | 1) * 16 + (size_t)B * (a.cols / 32) * 4;
    if (lds > 160 * 1024) return hipErrorInvalidValue;
    auto kernel = gemv_q4k_kernel<B, IPR>;
    static size_t configured_lds = 0;
    if (lds > 48 * 1024 && lds > configured_lds) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        configured_lds = lds;
    }
    const int pairs = (a.rows + 1) / 2;
    const int grid = (pairs + kWaves - 1) / kWaves;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(kThreads), lds, stream, a);
    return hipGetLastError();
}

template <int B>
hipError_t launch_q4k(const KernelArgs &a, hipStream_t stream) {
    if (a.cols == 4096) return launch_q4k_ipr<B, 64>(a, stream);
    if (a.cols == 14336) return launch_q4k_ipr<B, 224>(a, stream);
    return launch_q4k_ipr<B, 0>(a, stream);
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
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(kThreads), lds, stream, a);
    return hipGetLastError();
}

template <int FMT>
hipError_t launch_fmt(const KernelArgs &a, int batch, hipStream_t stream) {
    if (batch == 1) return launch_one<FMT, 1, 2>(a, stream);
    if (batch == 2) return launch_one<FMT, 2, 2>(a, stream);
    return hipErrorInvalidValue;
}

}  // namespace

hipError_t launch_gemv(const GemvParams &p, hipStream_t stream) {
    const DeviceMatrix &w = p.w;
    if (!w.qs || !p.x || w.rows <= 0 || w.cols <= 0 || p.batch <= 0) return hipErrorInvalidValue;
    if ((p.epilogue == EPI_STORE_F32 || p.epilogue == EPI_ADD_RESIDUAL) && !p.y) return hipErrorInvalidValue;
    if (p.epilogue == EPI_ADD_RESIDUAL && !p.residual) return hipErrorInvalidValue;
    if (p.epilogue == EPI_SWIGLU_F16 && (!p.out_f16 || w.rows % 2 != 0)) return hipErrorInvalidValue;
    if (p.epilogue == EPI_QKV_ROPE) {
        const QkvEpilogue &q = p.qkv;
        if (!q.rope_cos || !q.rope_sin || !q.pos || !q.seq || !q.q_out || !q.k_cache || !q.v_cache || q.head_dim % 2 != 0 ||
            w.rows != (q.n_head + 2 * q.n_kv_head) * q.head_dim)
            return hipErrorInvalidValue;
    }
    const int block = w.format == FMT_F16 ? 8 : w.format == FMT_F32 ? 4 : format_block_elems(w.format);
    if (w.cols % block != 0 || w.qs_row_bytes % 16 != 0) return hipErrorInvalidValue;
    if ((w.format == FMT_Q8_0 || w.format == FMT_Q4_0) && !w.scales) return hipErrorInvalidValue;

    // batches beyond 2 run as successive pairs (each pair re-reads the weights)
    for (int b0 = 0; b0 < p.batch; b0 += 2) {
        const int nb = p.batch - b0 >= 2 ? 2 : 1;
        KernelArgs a;
        a.qs = w.qs; a.scales = w.scales; a.qs_row_bytes = w.qs_row_bytes; a.rows = w.rows; a.cols = w.cols;
        a.x = p.x + (size_t)b0 * w.cols;
        a.y = p.y ? p.y + (size_t)b0 * w.rows : nullptr;
        a.residual = p.residual ? p.residual + (size_t)b0 * w.rows : nullptr;
        a.out_f16 = p.out_f16 ? p.out_f16 + (size_t)b0 * (w.rows / 2) : nullptr;
        a.qkv = p.qkv;
        if (p.epilogue == EPI_QKV_ROPE) {
            a.qkv.pos += b0;
            a.qkv.seq += b0;
            a.qkv.q_out += (size_t)b0 * p.qkv.n_head * p.qkv.head_dim;
        }
        a.epilogue = p.epilogue;
        hipError_t e;
        switch (w.format) {
        case FMT_Q4_K: e = nb == 1 ? launch_q4k<1>(a, stream) : launch_q4k<2>(a, stream); break;
        case FMT_Q4_0: e = launch_fmt<FMT_Q4_0>(a, nb, stream); break;
        case FMT_Q8_0: e = launch_fmt<FMT_Q8_0>(a, nb, stream); break;
        case FMT_F16: e = launch_fmt<FMT_F16>(a, nb, stream); break;
        case FMT_F32: e = launch_fmt<FMT_F32>(a, nb, stream); break;
        default: e = hipErrorInvalidValue;
        }
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

}  // namespace esp
