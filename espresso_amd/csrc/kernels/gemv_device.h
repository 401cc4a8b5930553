// Device-side building blocks shared by the GEMV kernels and the fused layer kernel (gfx950, wave64).
#pragma once

#include "../common.h"

namespace esp {
namespace detail {

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


// ---- activations -----------------------------------------------------------------------------
// Sum over the workgroup's four wavefronts; `red` holds kWaves floats that nobody else touches until
// the next barrier.  The same value, summed in the same order, reaches every thread.
__device__ __forceinline__ float workgroup_sum(float v, float *red) {
    v = wave_sum(v);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    return (red[0] + red[1]) + (red[2] + red[3]);
}
__device__ __forceinline__ float sum_squares(const float4 &a, const float4 &b) {
    return a.x * a.x + a.y * a.y + a.z * a.z + a.w * a.w + b.x * b.x + b.y * b.y + b.z * b.z + b.w * b.w;
}
__device__ __forceinline__ u32 pack_half2(float lo, float hi) {
    return (u32)__builtin_bit_cast(uint16_t, (_Float16)lo) | ((u32)__builtin_bit_cast(uint16_t, (_Float16)hi) << 16);
}
// Eight normalised activations as fp16:  fp16((x * inv) * w), the order of operations of rmsNorm
// (RealModelInferenceEngine.swift:6724-6743).
__device__ __forceinline__ uint4 normalized_group(const float4 &v0, const float4 &v1, const float4 &g0, const float4 &g1, float inv) {
    uint4 h;
    h.x = pack_half2(__fmul_rn(__fmul_rn(v0.x, inv), g0.x), __fmul_rn(__fmul_rn(v0.y, inv), g0.y));
    h.y = pack_half2(__fmul_rn(__fmul_rn(v0.z, inv), g0.z), __fmul_rn(__fmul_rn(v0.w, inv), g0.w));
    h.z = pack_half2(__fmul_rn(__fmul_rn(v1.x, inv), g1.x), __fmul_rn(__fmul_rn(v1.y, inv), g1.y));
    h.w = pack_half2(__fmul_rn(__fmul_rn(v1.z, inv), g1.z), __fmul_rn(__fmul_rn(v1.w, inv), g1.w));
    return h;
}

// The same eight values kept in fp32.
__device__ __forceinline__ void normalized_values(const float4 &v0, const float4 &v1, const float4 &g0, const float4 &g1, float inv, float (&c)[8]) {
    c[0] = __fmul_rn(__fmul_rn(v0.x, inv), g0.x); c[1] = __fmul_rn(__fmul_rn(v0.y, inv), g0.y);
    c[2] = __fmul_rn(__fmul_rn(v0.z, inv), g0.z); c[3] = __fmul_rn(__fmul_rn(v0.w, inv), g0.w);
    c[4] = __fmul_rn(__fmul_rn(v1.x, inv), g1.x); c[5] = __fmul_rn(__fmul_rn(v1.y, inv), g1.y);
    c[6] = __fmul_rn(__fmul_rn(v1.z, inv), g1.z); c[7] = __fmul_rn(__fmul_rn(v1.w, inv), g1.w);
}

// Split activations: an fp32 value v travels to the matrix cores as two fp16 numbers, hi = fp16(v) and
// lo = fp16((v - hi) * 2048), and a product with it is hi * w + (lo * w) / 2048.  The residue is scaled by 2^11 so that it
// stays a normal fp16 number wherever hi is one; v - hi is exact in fp32, so hi + lo / 2048 carries v to about 22 bits.
// The reference's CPU path feeds fp32 activations into every matrix product (RealModelInferenceEngine.swift:6674-6697);
// rounding them to fp16 costs 2^-12 relative per element and, over 32 layers of the 8B shape, 3e-2 on the logits.
constexpr float kSplitScale = 2048.0f, kSplitUnscale = 1.0f / 2048.0f;
struct SplitGroup { uint4 hi, lo; };
__device__ __forceinline__ void split_pair(float a, float b, u32 &hi, u32 &lo) {
    const _Float16 ha = (_Float16)a, hb = (_Float16)b;
    hi = (u32)__builtin_bit_cast(uint16_t, ha) | ((u32)__builtin_bit_cast(uint16_t, hb) << 16);
    lo = pack_half2(__fmul_rn(__fsub_rn(a, (float)ha), kSplitScale), __fmul_rn(__fsub_rn(b, (float)hb), kSplitScale));
}
__device__ __forceinline__ SplitGroup split_group(const float (&c)[8]) {
    SplitGroup g;
    split_pair(c[0], c[1], g.hi.x, g.lo.x);
    split_pair(c[2], c[3], g.hi.y, g.lo.y);
    split_pair(c[4], c[5], g.hi.z, g.lo.z);
    split_pair(c[6], c[7], g.hi.w, g.lo.w);
    return g;
}

// (x0,x1,x2,x3, x4,...) -> (x0,x2,x1,x3, x4,x6,x5,x7): the order the masked nibble / byte pairs meet
__device__ __forceinline__ uint4 swap_middle(const uint4 &v) {
    uint4 p;
    p.x = __builtin_amdgcn_perm(v.y, v.x, 0x05040100u);
    p.y = __builtin_amdgcn_perm(v.y, v.x, 0x07060302u);
    p.z = __builtin_amdgcn_perm(v.w, v.z, 0x05040100u);
    p.w = __builtin_amdgcn_perm(v.w, v.z, 0x07060302u);
    return p;
}

// ---------------------------------------------------------------------------------------------
// Q4_K.  A lane's item is one 64-weight chunk of a super-block: 32 bytes of nibbles (two 128-bit
// loads) whose low nibbles are sub-block 2c and whose high nibbles are sub-block 2c+1, plus the
// block's 16-byte header (d, dmin, twelve scale bytes; the four lanes of a block read the same
// 16 bytes).  The items of a row pair form one flat range of 2 * cols / 64 items.  Because rows hold
// a multiple of four items, a lane keeps the same chunk index c = lane & 3 for the whole kernel, so
// everything the 6-bit scale unpacking needs besides the header itself (shift counts, masks, which
// header word to read) is computed once.
//
// Nibbles are turned into fp16 with the exponent trick, without moving them: a low nibble (bits
// 0..3) under exponent 0x5400 reads as 64 + n/16, a high nibble (bits 4..7) under 0x4400 reads as
// 4 + n/16, both exactly.  v_dot2_f32_f16 accumulates sum (offset + n/16) x in fp32 with exact
// products, and the offset is removed once per sub-block with the precomputed sum of its 32
// activations:  sum n x = 16 * (raw - offset * sum x).  The same sums serve the dmin * m term.
//
// Two kernels: gemv_q4k_kernel for the column counts known at compile time (persistent workgroups,
// described there) and gemv_q4k_generic_kernel for any other multiple of 256.
struct Q4KItem {
    uint4 q0, q1, hdr;
};

struct Q4KLane {   // per-lane constants of the scale unpacking
    bool upper;    // sub-blocks 4..7: six-bit values are split over two header words
    u32 sh_sc, sh_min, sh_top, mask_low, mask_top;
    u32 magic_lo, magic_hi;   // kept in vector registers for v_and_or_b32
};

__device__ __forceinline__ Q4KLane q4k_chunk_constants(int c);
__device__ __forceinline__ Q4KLane q4k_lane_constants(int lane) { return q4k_chunk_constants(lane & 3); }
// c = which 64-weight chunk of a super-block the lane works on (0..3)
__device__ __forceinline__ Q4KLane q4k_chunk_constants(int c) {
    Q4KLane L;
    const int sh = (c & 1) * 16;
    L.upper = c >= 2;
    L.sh_sc = sh;
    L.sh_min = L.upper ? sh + 4 : sh;
    L.sh_top = sh + 2;
    L.mask_low = L.upper ? 0x0F0Fu : 0x3F3Fu;
    L.mask_top = L.upper ? 0x3030u : 0u;
    L.magic_lo = 0x54005400u;
    L.magic_hi = 0x44004400u;
    return L;
}

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
    const float d16 = 16.0f * half_bits_to_float(it.hdr.x & 0xFFFFu), dmin = half_bits_to_float(it.hdr.x >> 16);
#pragma unroll
    for (int b = 0; b < B; b++) {
        const uint4 *px = xs4 + (size_t)b * 8 * xstride + i;
        float raw_lo = 0.0f, raw_hi = 0.0f;
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const u32 w = dword_of(k < 4 ? it.q0 : it.q1, k & 3), w8 = w >> 8;
            const uint4 vl = px[(k >> 1) * xstride], vh = px[(4 + (k >> 1)) * xstride];
            const h2 xl02 = as_h2(dword_of(vl, (k & 1) * 2)), xl13 = as_h2(dword_of(vl, (k & 1) * 2 + 1));
            const h2 xh02 = as_h2(dword_of(vh, (k & 1) * 2)), xh13 = as_h2(dword_of(vh, (k & 1) * 2 + 1));
            const h2 l02 = as_h2(and_or(w, 0x000F000Fu, L.magic_lo));
            const h2 h02 = as_h2(and_or(w, 0x00F000F0u, L.magic_hi));
            const h2 l13 = as_h2(and_or(w8, 0x000F000Fu, L.magic_lo));
            const h2 h13 = as_h2(and_or(w8, 0x00F000F0u, L.magic_hi));
            raw_lo = fdot2(l02, xl02, raw_lo);
            raw_lo = fdot2(l13, xl13, raw_lo);
            raw_hi = fdot2(h02, xh02, raw_hi);
            raw_hi = fdot2(h13, xh13, raw_hi);
        }
        const float2 xsp = *reinterpret_cast<const float2 *>(xsum + (size_t)b * (cols >> 5) + 2 * i);
        const float nx_lo = raw_lo - 64.0f * xsp.x, nx_hi = raw_hi - 4.0f * xsp.y;
        v[b] = d16 * (sc_lo * nx_lo + sc_hi * nx_hi) - dmin * (m_lo * xsp.x + m_hi * xsp.y);
    }
}

// Activations into LDS for the Q4_K kernels: middle elements of each group of four swapped, written as
// [b][k][item] with an odd item stride (conflict-free for the write and for the per-k reads of
// consecutive items); sums of each 32 alongside.
__device__ __forceinline__ void q4k_store_group(const uint4 &v, int b, int g, int cols, int xstride, uint4 *xs4, float *xsum) {
    xs4[(size_t)b * 8 * xstride + (g & 7) * xstride + (g >> 3)] = swap_middle(v);
    float s = ((float)as_h2(v.x).x + (float)as_h2(v.x).y) + ((float)as_h2(v.y).x + (float)as_h2(v.y).y) +
              ((float)as_h2(v.z).x + (float)as_h2(v.z).y) + ((float)as_h2(v.w).x + (float)as_h2(v.w).y);
    s += dpp_term<0xB1, 0xF>(s);   // the four lanes of a quad hold the four groups of one 32
    s += dpp_term<0x4E, 0xF>(s);
    if ((threadIdx.x & 3) == 0) xsum[(size_t)b * (cols >> 5) + (g >> 2)] = s;
}

// The same for the matrix-core GEMV: groups of eight in their natural places, [b][cols / 8], sums of each 32 alongside.
// Q40: the term that removes the nibble offsets of a Q4_0 block instead, 1032 x (sum of the first sixteen) + 72 x (sum of the last
// sixteen): w = d (n - 8) with the low nibbles read as 64 + n / 16 and the high ones as 4 + n / 16.
template <bool Q40 = false>
__device__ __forceinline__ void q4k_store_group_natural(const uint4 &v, int b, int g, int cols, uint4 *xs4, float *xsum) {
    xs4[(size_t)b * (cols >> 3) + g] = swap_middle(v);
    float s = ((float)as_h2(v.x).x + (float)as_h2(v.x).y) + ((float)as_h2(v.y).x + (float)as_h2(v.y).y) +
              ((float)as_h2(v.z).x + (float)as_h2(v.z).y) + ((float)as_h2(v.w).x + (float)as_h2(v.w).y);
    if constexpr (Q40) s *= (g & 2) ? 72.0f : 1032.0f;
    s += dpp_term<0xB1, 0xF>(s);
    s += dpp_term<0x4E, 0xF>(s);
    if ((threadIdx.x & 3) == 0) xsum[(size_t)b * (cols >> 5) + (g >> 2)] = s;
}

__device__ __forceinline__ float sum_group(const uint4 &v) {
    return ((float)as_h2(v.x).x + (float)as_h2(v.x).y) + ((float)as_h2(v.y).x + (float)as_h2(v.y).y) +
           ((float)as_h2(v.z).x + (float)as_h2(v.z).y) + ((float)as_h2(v.w).x + (float)as_h2(v.w).y);
}
// Split activations in the matrix-core layout: logical row b occupies rows 2b (hi) and 2b + 1 (lo) of [rows][cols / 8]; the sums
// of each 32 are those of hi + lo / 2048, one per logical row.
__device__ __forceinline__ void q4k_store_split_natural(const SplitGroup &v, int b, int g, int cols, uint4 *xs4, float *xsum) {
    xs4[(size_t)(2 * b) * (cols >> 3) + g] = swap_middle(v.hi);
    xs4[(size_t)(2 * b + 1) * (cols >> 3) + g] = swap_middle(v.lo);
    float s = __builtin_fmaf(sum_group(v.lo), kSplitUnscale, sum_group(v.hi));
    s += dpp_term<0xB1, 0xF>(s);
    s += dpp_term<0x4E, 0xF>(s);
    if ((threadIdx.x & 3) == 0) xsum[(size_t)b * (cols >> 5) + (g >> 2)] = s;
}

}  // namespace detail
}  // namespace esp
