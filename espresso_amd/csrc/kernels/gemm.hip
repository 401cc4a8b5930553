// Dequant-fused MFMA GEMM for more than two activation rows (prompt prefill, batched verify, batch-8
// microbenchmarks):   y[m][n] = sum_k x[m][k] * dequant(W)[n][k],   fp16 operands, fp32 accumulation.
//
// Replaces the per-token vDSP_mmul calls the reference issues while it walks a prompt
// (RealModelInferenceEngine.swift:6674-6697 inside the prefill loop :6365-6375) by one pass over the
// packed weights per block of rows.
//
// Shape of the kernel (gfx950, wave64)
//   * a workgroup of four wavefronts owns 128 weight rows (n) x MT activation rows (m) and walks K in
//     tiles of 64;
//   * per K tile every thread fetches the packed bytes of (one weight row, one half of the tile) with
//     128-bit loads, turns them into 32 fp16 weights in registers (nibble / byte exponent tricks, one
//     packed fp16 multiply-add with the block's scale and minimum) and writes them to LDS; the fp16
//     activations of the tile are copied to LDS next to them;
//   * every weight reaches the matrix core as its dequantised value rounded to fp16 exactly once (Q4_K:
//     n * d*sc - dmin*m in fp32 first; Q4_0 / Q8_0: one exact packed fp16 product);
//   * the Q4_0 / Q8_0 exponent tricks yield elements in (0,2,1,3) order inside every group of four; the
//     activations are stored with the same swap, which costs nothing because a dot product does not care
//     about the order of k as long as both operands agree;
//   * v_mfma_f32_32x32x16_f16: activations are the A operand (rows m), weights the B operand (columns
//     n), so a lane's 16 accumulators belong to one weight row and 16 activation rows;
//   * the global loads of several tiles ahead are in flight while the matrix cores work on tile t;
//   * when the (n, m) grid is too small to fill the chip, K is split over grid.y and a small kernel
//     adds the partial sums in split order (deterministic, no atomics).
#include "../common.h"
#include "decode_ops.h"
#include <atomic>
#include <type_traits>

namespace esp {
namespace {

typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32;

constexpr int kThreads = 256;
constexpr int KT = 64;        // k per tile
constexpr int LDK = KT + 8;   // fp16 per LDS row: 144 bytes, so eight rows cover all banks
constexpr int NT = 128;       // weight rows per workgroup: two threads per row

struct GemmArgs {
    const uint8_t *qs;
    const uint16_t *scales;
    size_t qs_row_bytes;
    int N, K, M;
    const uint16_t *x;      // [M][K] fp16
    float *y;               // [M][N]
    const float *residual;  // [M][N] or null
    float *partial;         // [splits][M][N] when gridDim.y > 1
    int tiles_per_split;
    uint16_t *swiglu_out;   // tile kernel without split-K only: fp16 [M][N / 2] instead of y
};

__device__ __forceinline__ h2 as_h2(u32 v) { return __builtin_bit_cast(h2, v); }
__device__ __forceinline__ u32 as_u32(h2 v) { return __builtin_bit_cast(u32, v); }
__device__ __forceinline__ float half_bits_to_float(u32 bits16) { return (float)__builtin_bit_cast(_Float16, (uint16_t)bits16); }
__device__ __forceinline__ h2 splat(float v) { const _Float16 h = (_Float16)v; return h2{h, h}; }
__device__ __forceinline__ u32 dword_of(const uint4 &v, int k) { return k == 0 ? v.x : k == 1 ? v.y : k == 2 ? v.z : v.w; }
__device__ __forceinline__ uint4 swap_middle(const uint4 &v) {
    uint4 p;
    p.x = __builtin_amdgcn_perm(v.y, v.x, 0x05040100u);
    p.y = __builtin_amdgcn_perm(v.y, v.x, 0x07060302u);
    p.z = __builtin_amdgcn_perm(v.w, v.z, 0x05040100u);
    p.w = __builtin_amdgcn_perm(v.w, v.z, 0x07060302u);
    return p;
}

// The packed bytes one thread holds for (weight row, half h of a K tile), per format.
template <int FMT>
struct Raw;
template <>
struct Raw<FMT_Q4_K> { uint4 q, hdr; };          // 16 bytes of nibbles + the super-block header
template <>
struct Raw<FMT_Q4_0> { uint4 q; u32 d; };        // one block
template <>
struct Raw<FMT_Q8_0> { uint4 q0, q1; u32 d; };   // one block
template <>
struct Raw<FMT_F16> { uint4 v[4]; };

template <int FMT>
__device__ __forceinline__ Raw<FMT> fetch_raw(const GemmArgs &a, int row, int tile, int h) {
    Raw<FMT> r;
    const uint8_t *base = a.qs + (size_t)row * a.qs_row_bytes;
    if constexpr (FMT == FMT_Q4_K) {
        const uint8_t *blk = base + (size_t)(tile >> 2) * 144;
        r.hdr = *reinterpret_cast<const uint4 *>(blk);
        r.q = *reinterpret_cast<const uint4 *>(blk + 16 + (tile & 3) * 32 + h * 16);
    } else if constexpr (FMT == FMT_Q4_0) {
        const int block = tile * 2 + h;
        r.q = *reinterpret_cast<const uint4 *>(base + (size_t)block * 16);
        r.d = a.scales[(size_t)row * (a.K / 32) + block];
    } else if constexpr (FMT == FMT_Q8_0) {
        const int block = tile * 2 + h;
        const uint4 *q = reinterpret_cast<const uint4 *>(base + (size_t)block * 32);
        r.q0 = q[0];
        r.q1 = q[1];
        r.d = a.scales[(size_t)row * (a.K / 32) + block];
    } else {
        const uint4 *q = reinterpret_cast<const uint4 *>(base + ((size_t)tile * KT + h * 32) * 2);
#pragma unroll
        for (int i = 0; i < 4; i++) r.v[i] = q[i];
    }
    return r;
}

// Byte `idx` (0..11) of the twelve scale bytes that follow d and dmin in a Q4_K header.
__device__ __forceinline__ u32 scale_byte(const uint4 &hdr, int idx) {
    const u32 word = idx < 4 ? hdr.y : idx < 8 ? hdr.z : hdr.w;
    return (word >> ((idx & 3) * 8)) & 0xFFu;
}
// ggml's get_scale_min_k4
__device__ __forceinline__ void q4k_scale_min(const uint4 &hdr, int j, float &sc, float &m) {
    if (j < 4) {
        sc = (float)(scale_byte(hdr, j) & 63u);
        m = (float)(scale_byte(hdr, j + 4) & 63u);
    } else {
        sc = (float)((scale_byte(hdr, j + 4) & 0xFu) | ((scale_byte(hdr, j - 4) >> 6) << 4));
        m = (float)((scale_byte(hdr, j + 4) >> 4) | ((scale_byte(hdr, j) >> 6) << 4));
    }
}

// Four weights of dword `w` per call: nibbles at bits 0..3 (offset 1024) or 4..7 (offset 64) become exact
// fp16 integers, then w = n * s - dm in packed fp16 (one rounding per weight).
__device__ __forceinline__ uint2 nibbles_to_half(u32 w, bool high, h2 s, h2 dm) {
    const u32 mask = high ? 0x00F000F0u : 0x000F000Fu, magic = high ? 0x54005400u : 0x64006400u;
    const h2 off = high ? h2{(_Float16)64.0f, (_Float16)64.0f} : h2{(_Float16)1024.0f, (_Float16)1024.0f};
    const h2 n02 = as_h2((w & mask) | magic) - off, n13 = as_h2(((w >> 8) & mask) | magic) - off;
    return make_uint2(as_u32(__builtin_elementwise_fma(n02, s, -dm)), as_u32(__builtin_elementwise_fma(n13, s, -dm)));
}

// Q4_K: four nibbles spread over the bytes of `b` -> fp16(n * s - dm) with the product and the subtraction in
// fp32, so each weight is the dequantised value rounded to fp16 once (n * s and dm can both be several
// times larger than their difference; rounding them separately in fp16 would cost two more bits).
__device__ __forceinline__ uint2 q4k_bytes_to_half(u32 b, float s, float dm) {
    // The empty statement hides where `b` came from: otherwise the compiler folds the caller's nibble mask into four
    // bit-field extracts followed by byte conversions, two operations per weight where v_cvt_f32_ubyte0..3 on the masked
    // word need one.
    asm volatile("" : "+v"(b));
    const float w0 = __builtin_fmaf((float)(b & 0xFFu), s, -dm), w1 = __builtin_fmaf((float)((b >> 8) & 0xFFu), s, -dm);
    const float w2 = __builtin_fmaf((float)((b >> 16) & 0xFFu), s, -dm), w3 = __builtin_fmaf((float)(b >> 24), s, -dm);
    return make_uint2(as_u32(h2{(_Float16)w0, (_Float16)w1}), as_u32(h2{(_Float16)w2, (_Float16)w3}));
}

// Writes the thread's 32 fp16 weights into its LDS row (`wrow` points at k = 0 of the tile).
// Element order inside each group of four is (0,2,1,3) for Q4_0 and Q8_0, natural for Q4_K and F16.
// `c` = tile % 4, the pair of Q4_K sub-blocks the tile covers (a constant where the caller's loop is unrolled by four).
template <int FMT>
__device__ __forceinline__ void dequant_to_lds(const Raw<FMT> &r, int c, int h, _Float16 *wrow) {
    if constexpr (FMT == FMT_Q4_K) {
        // low nibbles: sub-block 2c, elements 16h..16h+15 (k = 16h..); high nibbles: sub-block 2c+1 (k = 32+16h..)
        const float d = half_bits_to_float(r.hdr.x & 0xFFFFu), dmin = half_bits_to_float(r.hdr.x >> 16);
        float sc_lo, m_lo, sc_hi, m_hi;
        q4k_scale_min(r.hdr, 2 * c, sc_lo, m_lo);
        q4k_scale_min(r.hdr, 2 * c + 1, sc_hi, m_hi);
        const float s_lo = d * sc_lo, dm_lo = dmin * m_lo, s_hi = d * sc_hi, dm_hi = dmin * m_hi;
        uint2 lo[4], hi[4];
#pragma unroll
        for (int k = 0; k < 4; k++) {
            lo[k] = q4k_bytes_to_half(dword_of(r.q, k) & 0x0F0F0F0Fu, s_lo, dm_lo);
            hi[k] = q4k_bytes_to_half((dword_of(r.q, k) >> 4) & 0x0F0F0F0Fu, s_hi, dm_hi);
        }
        uint4 *plo = reinterpret_cast<uint4 *>(wrow + 16 * h), *phi = reinterpret_cast<uint4 *>(wrow + 32 + 16 * h);
        plo[0] = make_uint4(lo[0].x, lo[0].y, lo[1].x, lo[1].y);
        plo[1] = make_uint4(lo[2].x, lo[2].y, lo[3].x, lo[3].y);
        phi[0] = make_uint4(hi[0].x, hi[0].y, hi[1].x, hi[1].y);
        phi[1] = make_uint4(hi[2].x, hi[2].y, hi[3].x, hi[3].y);
    } else if constexpr (FMT == FMT_Q4_0) {
        // byte j: low nibble = element j, high nibble = element j + 16; w = (n - 8) * d
        const h2 s = splat(half_bits_to_float(r.d)), dm = splat(8.0f * half_bits_to_float(r.d));
        uint2 lo[4], hi[4];
#pragma unroll
        for (int k = 0; k < 4; k++) {
            lo[k] = nibbles_to_half(dword_of(r.q, k), false, s, dm);
            hi[k] = nibbles_to_half(dword_of(r.q, k), true, s, dm);
        }
        uint4 *p = reinterpret_cast<uint4 *>(wrow + 32 * h);
        p[0] = make_uint4(lo[0].x, lo[0].y, lo[1].x, lo[1].y);
        p[1] = make_uint4(lo[2].x, lo[2].y, lo[3].x, lo[3].y);
        p[2] = make_uint4(hi[0].x, hi[0].y, hi[1].x, hi[1].y);
        p[3] = make_uint4(hi[2].x, hi[2].y, hi[3].x, hi[3].y);
    } else if constexpr (FMT == FMT_Q8_0) {
        const h2 s = splat(half_bits_to_float(r.d)), off = h2{(_Float16)1152.0f, (_Float16)1152.0f};   // 1024 + 128
        uint4 *p = reinterpret_cast<uint4 *>(wrow + 32 * h);
#pragma unroll
        for (int half = 0; half < 2; half++) {
            const uint4 &q = half ? r.q1 : r.q0;
            u32 out[8];
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const u32 t = dword_of(q, k) ^ 0x80808080u;   // signed -> biased
                const h2 f02 = as_h2(__builtin_amdgcn_perm(0x64646464u, t, 0x04020400u)) - off;
                const h2 f13 = as_h2(__builtin_amdgcn_perm(0x64646464u, t, 0x04030401u)) - off;
                out[2 * k] = as_u32(f02 * s);
                out[2 * k + 1] = as_u32(f13 * s);
            }
            p[2 * half] = make_uint4(out[0], out[1], out[2], out[3]);
            p[2 * half + 1] = make_uint4(out[4], out[5], out[6], out[7]);
        }
    } else {
        uint4 *p = reinterpret_cast<uint4 *>(wrow + 32 * h);
#pragma unroll
        for (int i = 0; i < 4; i++) p[i] = r.v[i];
    }
}

// WM x WN wavefronts, each TM x TN MFMA tiles of 32 x 32: the workgroup covers 32*WM*TM rows of x and
// 32*WN*TN = 128 weight rows.  DEPTH tiles of packed weights and activations are in flight in registers
// (a slot is refilled as soon as its tile has gone to LDS), and LDS holds two tiles so that one barrier
// per tile is enough: tile t+1 is written while other wavefronts still read tile t.
template <int FMT, int WM, int WN, int TM, int TN, int DEPTH>
__global__ __launch_bounds__(64 * WM * WN) void gemm_kernel(GemmArgs a) {
    constexpr int THREADS = 64 * WM * WN, NTILE = 32 * WN * TN;   // two threads per weight row dequantise
    static_assert(2 * NTILE == THREADS, "one (weight row, half tile) per thread");
    constexpr int MT = 32 * WM * TM;
    constexpr bool kSwap = FMT == FMT_Q4_0 || FMT == FMT_Q8_0;   // formats whose unpacking yields (0,2,1,3) order
    constexpr int XV = MT * KT / 8 / THREADS;   // 128-bit pieces of x per thread per tile
    static_assert(XV >= 1, "tile too small for the copy loop");
    __shared__ _Float16 xt[2][MT * LDK];
    __shared__ _Float16 wt[2][NTILE * LDK];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
    const int n0 = blockIdx.x * NTILE, m0 = blockIdx.z * MT;
    const int tiles = a.K / KT;
    const int t_begin = blockIdx.y * a.tiles_per_split;
    const int t_end = t_begin + a.tiles_per_split < tiles ? t_begin + a.tiles_per_split : tiles;

    // dequantisation role: weight row and half of the tile
    const int wr = tid >> 1, wh = tid & 1;
    const int w_row = n0 + wr < a.N ? n0 + wr : a.N - 1;   // clamped, the result is never stored

    floatx16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

    auto fetch_x = [&](int tile, uint4 (&xv)[XV]) {
#pragma unroll
        for (int i = 0; i < XV; i++) {
            const int piece = tid + i * THREADS, row = piece >> 3, part = piece & 7;   // eight pieces per row
            const int m = m0 + row < a.M ? m0 + row : a.M - 1;   // rows beyond M repeat the last one; their results are never stored
            xv[i] = reinterpret_cast<const uint4 *>(a.x + (size_t)m * a.K + (size_t)tile * KT)[part];
        }
    };

    // Slot j % DEPTH holds the packed bytes and activations of tile t_begin + j.  Staging a tile (dequantise into LDS,
    // copy the activations, refill the slot DEPTH tiles ahead) sits in the same barrier interval as the matrix-core work
    // on the tile before it, so the vector ALU and the LDS writes run in the shadow of the MFMAs of the same wavefront.
    // Tile indices beyond the last are clamped: the extra stage of the last interval is in bounds and never read.
    Raw<FMT> raw[DEPTH];
    uint4 xv[DEPTH][XV];
    const int t_last = t_end - 1;
#pragma unroll
    for (int d = 0; d < DEPTH; d++) {
        const int tile = t_begin + d < t_last ? t_begin + d : t_last;
        raw[d] = fetch_raw<FMT>(a, w_row, tile, wh);
        fetch_x(tile, xv[d]);
    }
    static_assert(4 % DEPTH == 0, "the main loop is unrolled by four");
    auto stage = [&](int S, int c, int tile, int buf) {   // S and c are constants after unrolling
        dequant_to_lds<FMT>(raw[S], c, wh, wt[buf] + wr * LDK);
#pragma unroll
        for (int i = 0; i < XV; i++) {
            const int piece = tid + i * THREADS, row = piece >> 3, part = piece & 7;
            *reinterpret_cast<uint4 *>(xt[buf] + row * LDK + part * 8) = kSwap ? swap_middle(xv[S][i]) : xv[S][i];
        }
        const int ahead = tile + DEPTH < t_last ? tile + DEPTH : t_last;
        raw[S] = fetch_raw<FMT>(a, w_row, ahead, wh);
        fetch_x(ahead, xv[S]);
    };
    stage(0, 0, t_begin, 0);   // t_begin is a multiple of four
    __syncthreads();
    for (int t0 = t_begin; t0 < t_end; t0 += 4) {
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int t = t0 + u, buf = u & 1;
            if (t < t_end) {
#pragma unroll
                for (int ks = 0; ks < KT / 16; ks++) {
                    const int kk = ks * 16 + 8 * (lane >> 5);
                    half8 af[TM], bf[TN];
#pragma unroll
                    for (int i = 0; i < TM; i++)
                        af[i] = *reinterpret_cast<const half8 *>(xt[buf] + ((wm * TM + i) * 32 + (lane & 31)) * LDK + kk);
#pragma unroll
                    for (int j = 0; j < TN; j++)
                        bf[j] = *reinterpret_cast<const half8 *>(wt[buf] + ((wn * TN + j) * 32 + (lane & 31)) * LDK + kk);
#pragma unroll
                    for (int i = 0; i < TM; i++)
#pragma unroll
                        for (int j = 0; j < TN; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], bf[j], acc[i][j], 0, 0, 0);
                }
                stage((u + 1) % DEPTH, (u + 1) & 3, t + 1, buf ^ 1);
                __syncthreads();
            }
        }
    }

    // accumulator r of lane l: row 8*(r/4) + 4*(l/32) + r%4, column l%32 of the 32 x 32 tile
    if (a.swiglu_out) {   // rows of W are (gate, up) pairs: even lanes hold gate, their right neighbours up (:6825-6827, :6337)
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++) {
                const int n = n0 + (wn * TN + j) * 32 + (lane & 31);
                // a pair of lanes holds (gate, up) of one unit for 16 rows; the even lane finishes the even accumulators, the
                // odd lane the odd ones, so that no lane idles through the tanh
                const bool odd = lane & 1;
#pragma unroll
                for (int k = 0; k < 8; k++) {
                    const float a0 = acc[i][j][2 * k], a1 = acc[i][j][2 * k + 1];
                    const float p0 = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, a0), 0xB1, 0xF, 0xF, false));   // quad_perm [1,0,3,2]
                    const float p1 = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, a1), 0xB1, 0xF, 0xF, false));
                    const float g = odd ? p1 : a0, u = odd ? a1 : p0;
                    const int r = 2 * k + (odd ? 1 : 0);
                    const int m = m0 + (wm * TM + i) * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                    if (m < a.M && (n | 1) < a.N) {
                        const float silu = g * __builtin_amdgcn_rcpf(1.0f + __expf(-g));   // = 0.5 g (1 + tanh(0.5 g)), a fifth of tanhf's instructions
                        a.swiglu_out[(size_t)m * (a.N / 2) + n / 2] = __builtin_bit_cast(uint16_t, (_Float16)__fmul_rn(silu, u));
                    }
                }
            }
        return;
    }
    const bool split = gridDim.y > 1;
    float *out = split ? a.partial + (size_t)blockIdx.y * a.M * a.N : a.y;
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int n = n0 + (wn * TN + j) * 32 + (lane & 31);
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int m = m0 + (wm * TM + i) * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                if (m < a.M && n < a.N) {
                    const size_t o = (size_t)m * a.N + n;
                    out[o] = (!split && a.residual) ? a.residual[o] + acc[i][j][r] : acc[i][j][r];
                }
            }
        }
}

// ---------------------------------------------------------------------------------------------
// Short M (at most 64 activation rows): the weights never touch LDS.  In v_mfma_f32_32x32x16_f16 a lane
// of the B operand holds eight consecutive k of ONE column, so a lane can load 16 packed bytes of its
// own weight row, dequantise them in registers and feed them to the matrix core directly; lanes 0..31
// and 32..63 of a wavefront take the two halves of each 64-k tile of the same 32 weight rows.  A
// wavefront owns 32 weight rows, a workgroup 128.  Only the activations go through LDS, 256 k at a
// time and double-buffered, so there is one barrier per 256 k.  Packed weights for DEPTH chunks of
// 256 k are in flight per lane.
constexpr int CK = 256;        // k per activation stage
constexpr int LDX = CK + 8;    // fp16 per LDS row of activations

template <int FMT>
struct RawChunk;
template <>
struct RawChunk<FMT_Q4_K> { uint4 hdr, q[4]; };
template <>
struct RawChunk<FMT_Q4_0> { uint4 q[4]; u32 d[4]; };
template <>
struct RawChunk<FMT_Q8_0> { uint4 q[8]; u32 d[4]; };

template <int FMT>
__device__ __forceinline__ RawChunk<FMT> fetch_chunk(const GemmArgs &a, int row, int chunk, int h) {
    RawChunk<FMT> r;
    const uint8_t *base = a.qs + (size_t)row * a.qs_row_bytes;
    if constexpr (FMT == FMT_Q4_K) {
        const uint8_t *blk = base + (size_t)chunk * 144;
        r.hdr = *reinterpret_cast<const uint4 *>(blk);
#pragma unroll
        for (int c = 0; c < 4; c++) r.q[c] = *reinterpret_cast<const uint4 *>(blk + 16 + c * 32 + h * 16);
    } else if constexpr (FMT == FMT_Q4_0) {
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const int block = chunk * 8 + t * 2 + h;
            r.q[t] = *reinterpret_cast<const uint4 *>(base + (size_t)block * 16);
            r.d[t] = a.scales[(size_t)row * (a.K / 32) + block];
        }
    } else {
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const int block = chunk * 8 + t * 2 + h;
            const uint4 *q = reinterpret_cast<const uint4 *>(base + (size_t)block * 32);
            r.q[2 * t] = q[0];
            r.q[2 * t + 1] = q[1];
            r.d[t] = a.scales[(size_t)row * (a.K / 32) + block];
        }
    }
    return r;
}

__device__ __forceinline__ half8 as_half8(const uint4 &v) { return __builtin_bit_cast(half8, v); }

// The four B fragments (eight fp16 each) a lane contributes to 64-k tile `t` of its chunk, and the k offset
// inside the tile at which the matching activations start.  Element order inside groups of four matches
// the activations' LDS copy (natural for Q4_K, (0,2,1,3) for Q4_0 and Q8_0).
template <int FMT>
__device__ __forceinline__ void tile_fragments(const RawChunk<FMT> &r, int t, int h, half8 frag[4], int koff[4]) {
    if constexpr (FMT == FMT_Q4_K) {
        const float d = half_bits_to_float(r.hdr.x & 0xFFFFu), dmin = half_bits_to_float(r.hdr.x >> 16);
        float sc_lo, m_lo, sc_hi, m_hi;
        q4k_scale_min(r.hdr, 2 * t, sc_lo, m_lo);
        q4k_scale_min(r.hdr, 2 * t + 1, sc_hi, m_hi);
        const float s_lo = d * sc_lo, dm_lo = dmin * m_lo, s_hi = d * sc_hi, dm_hi = dmin * m_hi;
        uint2 lo[4], hi[4];
#pragma unroll
        for (int k = 0; k < 4; k++) {
            lo[k] = q4k_bytes_to_half(dword_of(r.q[t], k) & 0x0F0F0F0Fu, s_lo, dm_lo);
            hi[k] = q4k_bytes_to_half((dword_of(r.q[t], k) >> 4) & 0x0F0F0F0Fu, s_hi, dm_hi);
        }
        frag[0] = as_half8(make_uint4(lo[0].x, lo[0].y, lo[1].x, lo[1].y));
        frag[1] = as_half8(make_uint4(lo[2].x, lo[2].y, lo[3].x, lo[3].y));
        frag[2] = as_half8(make_uint4(hi[0].x, hi[0].y, hi[1].x, hi[1].y));
        frag[3] = as_half8(make_uint4(hi[2].x, hi[2].y, hi[3].x, hi[3].y));
        koff[0] = 16 * h; koff[1] = 16 * h + 8; koff[2] = 32 + 16 * h; koff[3] = 40 + 16 * h;
    } else if constexpr (FMT == FMT_Q4_0) {
        const h2 s = splat(half_bits_to_float(r.d[t])), dm = splat(8.0f * half_bits_to_float(r.d[t]));
        uint2 lo[4], hi[4];
#pragma unroll
        for (int k = 0; k < 4; k++) {
            lo[k] = nibbles_to_half(dword_of(r.q[t], k), false, s, dm);
            hi[k] = nibbles_to_half(dword_of(r.q[t], k), true, s, dm);
        }
        frag[0] = as_half8(make_uint4(lo[0].x, lo[0].y, lo[1].x, lo[1].y));
        frag[1] = as_half8(make_uint4(lo[2].x, lo[2].y, lo[3].x, lo[3].y));
        frag[2] = as_half8(make_uint4(hi[0].x, hi[0].y, hi[1].x, hi[1].y));
        frag[3] = as_half8(make_uint4(hi[2].x, hi[2].y, hi[3].x, hi[3].y));
#pragma unroll
        for (int f = 0; f < 4; f++) koff[f] = 32 * h + 8 * f;
    } else {
        const h2 s = splat(half_bits_to_float(r.d[t])), off = h2{(_Float16)1152.0f, (_Float16)1152.0f};
#pragma unroll
        for (int half = 0; half < 2; half++) {
            const uint4 &q = r.q[2 * t + half];
            u32 out[8];
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const u32 b = dword_of(q, k) ^ 0x80808080u;
                const h2 f02 = as_h2(__builtin_amdgcn_perm(0x64646464u, b, 0x04020400u)) - off;
                const h2 f13 = as_h2(__builtin_amdgcn_perm(0x64646464u, b, 0x04030401u)) - off;
                out[2 * k] = as_u32(f02 * s);
                out[2 * k + 1] = as_u32(f13 * s);
            }
            frag[2 * half] = as_half8(make_uint4(out[0], out[1], out[2], out[3]));
            frag[2 * half + 1] = as_half8(make_uint4(out[4], out[5], out[6], out[7]));
        }
#pragma unroll
        for (int f = 0; f < 4; f++) koff[f] = 32 * h + 8 * f;
    }
}

template <int FMT, int TM, int DEPTH>
__global__ __launch_bounds__(kThreads) void gemm_skinny_kernel(GemmArgs a) {
    constexpr int MT = 32 * TM;
    constexpr int XV = MT * CK / 8 / kThreads;   // 128-bit pieces of x per thread per chunk (4 per 32 rows)
    __shared__ _Float16 xt[2][MT * LDX];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, h = lane >> 5;
    const int n = blockIdx.x * NT + wave * 32 + (lane & 31);
    const int w_row = n < a.N ? n : a.N - 1;     // clamped, the result is never stored
    const int chunks = a.K / CK;
    const int c_begin = blockIdx.y * a.tiles_per_split;   // split granularity is a chunk here
    const int c_end = c_begin + a.tiles_per_split < chunks ? c_begin + a.tiles_per_split : chunks;

    floatx16 acc[TM];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[i][r] = 0.0f;

    auto fetch_x = [&](int chunk, uint4 (&xv)[XV]) {
#pragma unroll
        for (int i = 0; i < XV; i++) {
            const int piece = tid + i * kThreads, row = piece >> 5, part = piece & 31;   // 32 pieces per row
            xv[i] = row < a.M ? reinterpret_cast<const uint4 *>(a.x + (size_t)row * a.K + (size_t)chunk * CK)[part] : make_uint4(0, 0, 0, 0);
        }
    };

    RawChunk<FMT> raw[DEPTH];
    uint4 xv[XV];
#pragma unroll
    for (int d = 0; d < DEPTH; d++)
        if (c_begin + d < c_end) raw[d] = fetch_chunk<FMT>(a, w_row, c_begin + d, h);
    if (c_begin < c_end) fetch_x(c_begin, xv);

    for (int c0 = c_begin; c0 < c_end; c0 += DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; d++) {
            const int c = c0 + d, buf = d & 1;   // DEPTH is even
            if (c < c_end) {
#pragma unroll
                for (int i = 0; i < XV; i++) {
                    const int piece = tid + i * kThreads, row = piece >> 5, part = piece & 31;
                    *reinterpret_cast<uint4 *>(xt[buf] + row * LDX + part * 8) = FMT == FMT_Q4_K ? xv[i] : swap_middle(xv[i]);
                }
                if (c + 1 < c_end) fetch_x(c + 1, xv);
            }
            __syncthreads();
            if (c < c_end) {
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    half8 frag[4];
                    int koff[4];
                    tile_fragments<FMT>(raw[d], t, h, frag, koff);
#pragma unroll
                    for (int f = 0; f < 4; f++)
#pragma unroll
                        for (int i = 0; i < TM; i++) {
                            const half8 af = *reinterpret_cast<const half8 *>(xt[buf] + (i * 32 + (lane & 31)) * LDX + t * KT + koff[f]);
                            acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af, frag[f], acc[i], 0, 0, 0);
                        }
                }
                if (c + DEPTH < c_end) raw[d] = fetch_chunk<FMT>(a, w_row, c + DEPTH, h);
            }
        }
    }

    const bool split = gridDim.y > 1;
    float *out = split ? a.partial + (size_t)blockIdx.y * a.M * a.N : a.y;
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int m = i * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
            if (m < a.M && n < a.N) {
                const size_t o = (size_t)m * a.N + n;
                out[o] = (!split && a.residual) ? a.residual[o] + acc[i][r] : acc[i][r];
            }
        }
}

// ---------------------------------------------------------------------------------------------
// Up to eight activation rows against Q4_K weights without dequantising them.  With so few rows the
// register-B kernel above is bound by the exact dequantisation (three vector operations per weight however few rows
// there are).  Here the B operand is the nibble itself under an fp16 exponent, as in the GEMV kernels: one
// v_and_or_b32 turns two low nibbles into (64 + n/16, 64 + n/16) and two high nibbles into (4 + n/16, 4 + n/16),
// exactly; two MFMAs contract a 32-weight sub-block into sum (offset + n/16) x with exact products, and scale and
// minimum of the sub-block are folded into the few accumulator registers that hold real rows afterwards:
//     sum_k (d sc n_k - dmin m) x_k = (16 d sc) raw - (16 d sc offset + dmin m) sum_k x_k,
// with the sums of the activations over each sub-block computed once per workgroup while they are staged.
// Lane mapping, loads, LDS staging of the activations (in (0,2,1,3) order inside fours, which is how the masked
// nibble pairs come out) are those of gemm_skinny_kernel; the rows 0..7 are accumulator registers 0..3 of a lane.
__device__ __forceinline__ float quad_sum(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, false));   // quad_perm [1,0,3,2]
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, false));   // quad_perm [2,3,0,1]
    return v;
}

// The workgroup owns 32 weight rows and its WAVES wavefronts split K between them, so a launch has one workgroup per 32 rows
// whatever K is, needs no split-K workspace and no reduce launch; the wavefronts' partial results meet in LDS and are added
// in wavefront order.  The activations are staged a span of SPAN chunks (of 256 k) at a time into one of two LDS buffers: the
// next span's are loaded into registers before the current span is computed and written after it, one barrier per span.
// Inside a span wavefront w takes chunks w, w + WAVES, ...; the packed weights of its chunks of the next two spans are always
// in flight (they do not wait for the staging).  Short spans measure faster than long ones (one chunk per wavefront and span:
// 15.7 us for 14336 x 4096 against 18.2 us with two and 17.9 us with all of K staged at once), and eight wavefronts
// faster than four when the rows fill no more than one workgroup per compute unit.
// Q4_0 takes the same route: a lane holds eight bytes of each block (low nibbles = elements 8h.., high = 16 + 8h..), the two
// MFMAs of a block share one accumulator, and w = d (n - 8) = 16 d pattern - (1032 | 72) d folds as
//     total += d (16 raw - (1032 sum of x over the block's first sixteen + 72 sum over its last sixteen)).
constexpr int kRowsMaxRows = 8;
template <int WAVES, int SPAN> constexpr size_t rows_lds_bytes() {
    return 2 * ((size_t)kRowsMaxRows * (SPAN * CK + 8) * 2 + (size_t)SPAN * 8 * kRowsMaxRows * 4) + (size_t)WAVES * 4 * 64 * 4;
}

template <int FMT>
struct RowsChunk;
template <>
struct RowsChunk<FMT_Q4_K> { RawChunk<FMT_Q4_K> r; };
template <>
struct RowsChunk<FMT_Q4_0> { uint2 q[8]; uint4 d; };   // eight bytes of each of the chunk's eight blocks, their eight fp16 scales

template <int FMT>
__device__ __forceinline__ RowsChunk<FMT> fetch_rows_chunk(const GemmArgs &a, int row, int chunk, int h) {
    RowsChunk<FMT> c;
    if constexpr (FMT == FMT_Q4_K) {
        c.r = fetch_chunk<FMT_Q4_K>(a, row, chunk, h);
    } else {
        const uint8_t *base = a.qs + (size_t)row * a.qs_row_bytes + (size_t)chunk * 128 + 8 * h;
#pragma unroll
        for (int b = 0; b < 8; b++) c.q[b] = *reinterpret_cast<const uint2 *>(base + 16 * b);
        c.d = *reinterpret_cast<const uint4 *>(a.scales + (size_t)row * (a.K / 32) + (size_t)chunk * 8);
    }
    return c;
}

template <int FMT, int WAVES, int SPAN>
__global__ __launch_bounds__(WAVES * 64, WAVES == 4 ? 2 : 1) void gemm_rows_kernel(GemmArgs a) {
    static_assert(FMT == FMT_Q4_K || FMT == FMT_Q4_0, "formats whose weights are nibbles");
    constexpr int MR = kRowsMaxRows, THREADS = WAVES * 64, LDW = SPAN * CK + 8;
    constexpr int CPW = SPAN / WAVES;                     // chunks per wavefront and span
    constexpr int PIECES = MR * SPAN * 32 / THREADS;      // 128-bit pieces of x per thread and span
    extern __shared__ uint4 rows_smem[];
    _Float16 *xt_base = reinterpret_cast<_Float16 *>(rows_smem);               // [2][MR][LDW]
    float *xsum_base = reinterpret_cast<float *>(xt_base + 2 * MR * LDW);      // [2][SPAN * 8 groups of 32][MR]
    float *red = xsum_base + 2 * SPAN * 8 * MR;                                // [WAVES][4][64]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, h = lane >> 5;
    const int n = blockIdx.x * 32 + (lane & 31);
    const int w_row = n < a.N ? n : a.N - 1;     // clamped, the result is never stored
    const int chunks = a.K / CK, spans = (chunks + SPAN - 1) / SPAN;
    // constants of the nibble trick, hidden from the optimiser so that (w & mask) | magic stays one v_and_or_b32
    u32 mask_lo = 0x000F000Fu, mask_hi = 0x00F000F0u, magic_lo = 0x54005400u, magic_hi = 0x44004400u;
    asm volatile("" : "+s"(mask_lo), "+s"(mask_hi));
    asm volatile("" : "+v"(magic_lo), "+v"(magic_hi));
    auto pattern_lo = [&](u32 w0, u32 w1) { return as_half8(make_uint4((w0 & mask_lo) | magic_lo, ((w0 >> 8) & mask_lo) | magic_lo, (w1 & mask_lo) | magic_lo, ((w1 >> 8) & mask_lo) | magic_lo)); };
    auto pattern_hi = [&](u32 w0, u32 w1) { return as_half8(make_uint4((w0 & mask_hi) | magic_hi, ((w0 >> 8) & mask_hi) | magic_hi, (w1 & mask_hi) | magic_hi, ((w1 >> 8) & mask_hi) | magic_hi)); };

    float total[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    auto chunk_of = [&](int sp, int j) { return sp * SPAN + j * WAVES + wave; };
    RowsChunk<FMT> ring[2 * CPW];
#pragma unroll
    for (int q = 0; q < 2 * CPW; q++)
        if (chunk_of(q / CPW, q % CPW) < chunks) ring[q] = fetch_rows_chunk<FMT>(a, w_row, chunk_of(q / CPW, q % CPW), h);

    uint4 xv[PIECES];
    auto load_x = [&](int sp) {
#pragma unroll
        for (int i = 0; i < PIECES; i++) {
            const int piece = tid + i * THREADS, row = piece / (SPAN * 32), part = piece % (SPAN * 32);
            const int k0 = sp * SPAN * CK + part * 8;
            xv[i] = row < a.M && k0 < a.K ? *reinterpret_cast<const uint4 *>(a.x + (size_t)row * a.K + k0) : make_uint4(0, 0, 0, 0);
        }
    };
    // (0,2,1,3) order inside fours; alongside, per group of 32: Q4_K the sum of the activations, Q4_0 1032 times the sum of
    // the first sixteen plus 72 times the sum of the last sixteen
    auto store_x = [&](int buf) {
        _Float16 *xt = xt_base + buf * MR * LDW;
        float *xsum = xsum_base + buf * SPAN * 8 * MR;
#pragma unroll
        for (int i = 0; i < PIECES; i++) {
            const int piece = tid + i * THREADS, row = piece / (SPAN * 32), part = piece % (SPAN * 32);
            *reinterpret_cast<uint4 *>(xt + row * LDW + part * 8) = swap_middle(xv[i]);
            const h2 p0 = as_h2(xv[i].x), p1 = as_h2(xv[i].y), p2 = as_h2(xv[i].z), p3 = as_h2(xv[i].w);
            float sum = (((float)p0.x + (float)p0.y) + ((float)p1.x + (float)p1.y)) + (((float)p2.x + (float)p2.y) + ((float)p3.x + (float)p3.y));
            if constexpr (FMT == FMT_Q4_0) sum *= (part & 2) ? 72.0f : 1032.0f;
            sum = quad_sum(sum);                 // the four pieces of a group of 32 sit in one quad of lanes
            if ((part & 3) == 0) xsum[(part >> 2) * MR + row] = sum;
        }
    };
    auto compute_span = [&](int sp, auto parity) {
        constexpr int P = decltype(parity)::value;
        const _Float16 *xt = xt_base + P * MR * LDW;
        const float *xsum = xsum_base + P * SPAN * 8 * MR;
#pragma unroll
        for (int j = 0; j < CPW; j++) {
            const int c = chunk_of(sp, j);
            if (c < chunks) {
                const RowsChunk<FMT> rc = ring[P * CPW + j];
                if (chunk_of(sp + 2, j) < chunks) ring[P * CPW + j] = fetch_rows_chunk<FMT>(a, w_row, chunk_of(sp + 2, j), h);
                const int local = j * WAVES + wave;   // chunk index inside the span
                // rows of x beyond MR alias real ones: they only reach accumulator registers that are never read
                const _Float16 *xchunk = xt + ((lane & 31) & (MR - 1)) * LDW + local * CK;
                if constexpr (FMT == FMT_Q4_K) {
                    const RawChunk<FMT_Q4_K> &r = rc.r;
                    const float dd = half_bits_to_float(r.hdr.x & 0xFFFFu), dmin = half_bits_to_float(r.hdr.x >> 16);
#pragma unroll
                    for (int t = 0; t < 4; t++) {
                        float sc_lo, m_lo, sc_hi, m_hi;
                        q4k_scale_min(r.hdr, 2 * t, sc_lo, m_lo);
                        q4k_scale_min(r.hdr, 2 * t + 1, sc_hi, m_hi);
                        const float a_lo = 16.0f * dd * sc_lo, b_lo = 64.0f * a_lo + dmin * m_lo;
                        const float a_hi = 16.0f * dd * sc_hi, b_hi = 4.0f * a_hi + dmin * m_hi;
                        const u32 w0 = r.q[t].x, w1 = r.q[t].y, w2 = r.q[t].z, w3 = r.q[t].w;
                        const half8 f0 = pattern_lo(w0, w1), f1 = pattern_lo(w2, w3), f2 = pattern_hi(w0, w1), f3 = pattern_hi(w2, w3);
                        const _Float16 *xrow = xchunk + t * KT;
                        floatx16 lo, hi;
#pragma unroll
                        for (int i = 0; i < 16; i++) lo[i] = hi[i] = 0.0f;
                        lo = __builtin_amdgcn_mfma_f32_32x32x16_f16(*reinterpret_cast<const half8 *>(xrow + 16 * h), f0, lo, 0, 0, 0);
                        hi = __builtin_amdgcn_mfma_f32_32x32x16_f16(*reinterpret_cast<const half8 *>(xrow + 32 + 16 * h), f2, hi, 0, 0, 0);
                        lo = __builtin_amdgcn_mfma_f32_32x32x16_f16(*reinterpret_cast<const half8 *>(xrow + 16 * h + 8), f1, lo, 0, 0, 0);
                        hi = __builtin_amdgcn_mfma_f32_32x32x16_f16(*reinterpret_cast<const half8 *>(xrow + 40 + 16 * h), f3, hi, 0, 0, 0);
                        const float4 xs_lo = *reinterpret_cast<const float4 *>(xsum + (local * 8 + 2 * t) * MR + 4 * h);
                        const float4 xs_hi = *reinterpret_cast<const float4 *>(xsum + (local * 8 + 2 * t + 1) * MR + 4 * h);
                        const float sl[4] = {xs_lo.x, xs_lo.y, xs_lo.z, xs_lo.w}, sh[4] = {xs_hi.x, xs_hi.y, xs_hi.z, xs_hi.w};
#pragma unroll
                        for (int i = 0; i < 4; i++) {   // accumulator registers 0..3 of a lane: rows 4 (lane / 32) + i
                            float acc = total[i];
                            acc = __builtin_fmaf(lo[i], a_lo, acc);
                            acc = __builtin_fmaf(-b_lo, sl[i], acc);
                            acc = __builtin_fmaf(hi[i], a_hi, acc);
                            acc = __builtin_fmaf(-b_hi, sh[i], acc);
                            total[i] = acc;
                        }
                        __builtin_amdgcn_sched_barrier(0);   // one sub-block pair at a time keeps the accumulators few
                    }
                } else {
                    const u32 dw[4] = {rc.d.x, rc.d.y, rc.d.z, rc.d.w};
#pragma unroll
                    for (int b = 0; b < 8; b++) {
                        const float d = half_bits_to_float((dw[b >> 1] >> (16 * (b & 1))) & 0xFFFFu);
                        const half8 f_lo = pattern_lo(rc.q[b].x, rc.q[b].y), f_hi = pattern_hi(rc.q[b].x, rc.q[b].y);
                        const _Float16 *xrow = xchunk + b * 32;
                        floatx16 raw;
#pragma unroll
                        for (int i = 0; i < 16; i++) raw[i] = 0.0f;
                        raw = __builtin_amdgcn_mfma_f32_32x32x16_f16(*reinterpret_cast<const half8 *>(xrow + 8 * h), f_lo, raw, 0, 0, 0);
                        raw = __builtin_amdgcn_mfma_f32_32x32x16_f16(*reinterpret_cast<const half8 *>(xrow + 16 + 8 * h), f_hi, raw, 0, 0, 0);
                        const float4 xs = *reinterpret_cast<const float4 *>(xsum + (local * 8 + b) * MR + 4 * h);
                        const float sx[4] = {xs.x, xs.y, xs.z, xs.w};
                        const float d16 = 16.0f * d;
#pragma unroll
                        for (int i = 0; i < 4; i++) total[i] = __builtin_fmaf(-d, sx[i], __builtin_fmaf(raw[i], d16, total[i]));
                        if (b & 1) __builtin_amdgcn_sched_barrier(0);
                    }
                }
            }
        }
    };
    auto span_step = [&](int sp, auto parity) {
        constexpr int P = decltype(parity)::value;
        const bool more = sp + 1 < spans;
        if (more) load_x(sp + 1);
        compute_span(sp, parity);
        if (more) store_x(1 - P);
        __syncthreads();
    };

    load_x(0);
    store_x(0);
    __syncthreads();
    for (int sp = 0; sp < spans; sp += 2) {
        span_step(sp, std::integral_constant<int, 0>{});
        if (sp + 1 < spans) span_step(sp + 1, std::integral_constant<int, 1>{});
    }

    // ---- the wavefronts' shares of K meet in LDS; wavefront 0 adds them in order and writes the rows ----
#pragma unroll
    for (int i = 0; i < 4; i++) red[(wave * 4 + i) * 64 + lane] = total[i];
    __syncthreads();
    if (wave == 0) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            float v = red[i * 64 + lane];
#pragma unroll
            for (int w = 1; w < WAVES; w++) v += red[(w * 4 + i) * 64 + lane];
            const int m = 4 * h + i;
            if (m < a.M && n < a.N) {
                const size_t o = (size_t)m * a.N + n;
                a.y[o] = a.residual ? a.residual[o] + v : v;
            }
        }
    }
}

// y = (residual +) sum over splits of partial, in split order
__global__ void gemm_reduce_kernel(const float *partial, int splits, size_t count, const float *residual, float *y) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= count) return;
    float s = partial[i];
    for (int k = 1; k < splits; k++) s += partial[(size_t)k * count + i];
    y[i] = residual ? residual[i] + s : s;
}

template <int FMT, int WM, int WN, int TM, int TN, int DEPTH>
hipError_t launch_tile(const GemmArgs &a, int splits, hipStream_t stream) {
    constexpr int MT = 32 * WM * TM;
    constexpr int NTILE = 32 * WN * TN;
    dim3 grid((a.N + NTILE - 1) / NTILE, splits, (a.M + MT - 1) / MT);
    hipLaunchKernelGGL((gemm_kernel<FMT, WM, WN, TM, TN, DEPTH>), grid, dim3(64 * WM * WN), 0, stream, a);
    return hipGetLastError();
}

hipError_t launch_reduce(const GemmArgs &a, int splits, hipStream_t stream) {
    const size_t count = (size_t)a.M * a.N;
    hipLaunchKernelGGL(gemm_reduce_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, stream, a.partial, splits, count, a.residual, a.y);
    return hipGetLastError();
}

// splits so that about `target` workgroups exist, each with at least `min_units` units of K
int choose_splits(int blocks, int units, int min_units, int target, const GemmArgs &a, size_t workspace_floats) {
    if (!a.partial || blocks >= target) return 1;
    int splits = (target + blocks - 1) / blocks;
    if (splits > units / min_units) splits = units / min_units;
    if (splits < 1) splits = 1;
    while (splits > 1 && (size_t)splits * a.M * a.N > workspace_floats) splits--;
    return splits;
}

// `swiglu_out` (may be null) is handed to the tile kernel when it runs without split-K; *fused tells the caller.
template <int FMT>
hipError_t launch_format(GemmArgs a, float *workspace, size_t workspace_floats, uint16_t *swiglu_out, bool *fused, int *deferred_splits, hipStream_t stream) {
    *fused = false;
    // split-K partial sums are added by gemm_reduce_kernel, or left to the caller's next kernel when it asked for that
    auto finish = [&](hipError_t err, int used_splits) {
        if (err != hipSuccess || used_splits == 1) return err;
        if (deferred_splits) { *deferred_splits = used_splits; return hipSuccess; }
        return launch_reduce(a, used_splits, stream);
    };
    const int n_blocks = (a.N + NT - 1) / NT;
    a.partial = workspace;
    hipError_t e;
    int splits;
    if constexpr (FMT == FMT_Q4_K || FMT == FMT_Q4_0) {
        // one workgroup per 32 weight rows, K split over its wavefronts (Q4_0 at 14336 columns measures 27 us here against 24 us
        // on the register-B kernel with split-K, so long rows of Q4_0 stay there)
        if (a.M <= kRowsMaxRows && a.K % CK == 0 && (FMT == FMT_Q4_K || a.K <= 8192)) {
            const int groups = (a.N + 31) / 32;
            // the kernels' LDS (above 64 KB) is dynamic: the limit is raised once per kernel and device
            auto go = [&](auto kernel, int waves, size_t lds, std::atomic<uint64_t> &raised) {
                int device = 0;
                hipError_t err = hipGetDevice(&device);
                if (err != hipSuccess) return err;
                const uint64_t bit = 1ull << (device & 63);
                if (!(raised.load(std::memory_order_acquire) & bit)) {
                    err = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
                    if (err != hipSuccess) return err;
                    raised.fetch_or(bit, std::memory_order_release);
                }
                hipLaunchKernelGGL(kernel, dim3(groups), dim3(waves * 64), lds, stream, a);
                return hipGetLastError();
            };
            static std::atomic<uint64_t> raised8{0}, raised4{0};   // one pair per format: this function is a template
            if (groups <= 256) return go(gemm_rows_kernel<FMT, 8, 8>, 8, rows_lds_bytes<8, 8>(), raised8);
            return go(gemm_rows_kernel<FMT, 4, 4>, 4, rows_lds_bytes<4, 4>(), raised4);
        }
    }
    if constexpr (FMT != FMT_F16) {
        if (a.M <= 64 && a.K % CK == 0) {
            const int chunks = a.K / CK;
            splits = choose_splits(n_blocks, chunks, 2, 1024, a, workspace_floats);
            a.tiles_per_split = (chunks + splits - 1) / splits;
            splits = (chunks + a.tiles_per_split - 1) / a.tiles_per_split;
            dim3 grid(n_blocks, splits, 1);
            if (a.M <= 32) hipLaunchKernelGGL((gemm_skinny_kernel<FMT, 1, 2>), grid, dim3(kThreads), 0, stream, a);
            else hipLaunchKernelGGL((gemm_skinny_kernel<FMT, 2, 2>), grid, dim3(kThreads), 0, stream, a);
            e = hipGetLastError();
            return finish(e, splits);
        }
    }
    const int tiles = a.K / KT;
    const int mt = a.M <= 32 ? 32 : a.M <= 64 ? 64 : 128;
    // (eight wavefronts on a 128 x 256 tile measure 2-5 % faster at 4096 and more weight rows and 10 % slower at 1024;
    //  a 256 x 256 tile is 25 % slower: not instantiated)
    splits = choose_splits(n_blocks * ((a.M + mt - 1) / mt), tiles, 8, 1024, a, workspace_floats);
    a.tiles_per_split = ((tiles + splits - 1) / splits + 3) & ~3;   // every split starts on a multiple of four tiles
    splits = (tiles + a.tiles_per_split - 1) / a.tiles_per_split;
    if (splits == 1 && swiglu_out && a.N % 2 == 0) { a.swiglu_out = swiglu_out; *fused = true; }
    if (mt == 32) e = launch_tile<FMT, 1, 4, 1, 1, 4>(a, splits, stream);
    else if (mt == 64) e = launch_tile<FMT, 1, 4, 2, 1, 4>(a, splits, stream);
    else e = launch_tile<FMT, 2, 2, 2, 2, 2>(a, splits, stream);
    return finish(e, splits);
}

}  // namespace

hipError_t launch_gemm(const GemmParams &p, hipStream_t stream) {
    const DeviceMatrix &w = p.w;
    if (!w.qs || !p.x || !p.y || p.rows <= 0 || w.rows <= 0 || w.cols <= 0 || w.cols % KT != 0 || w.qs_row_bytes % 16 != 0) return hipErrorInvalidValue;
    if ((w.format == FMT_Q8_0 || w.format == FMT_Q4_0) && !w.scales) return hipErrorInvalidValue;
    if (w.format == FMT_Q4_K && w.cols % 256 != 0) return hipErrorInvalidValue;
    GemmArgs a{};
    a.qs = w.qs; a.scales = w.scales; a.qs_row_bytes = w.qs_row_bytes; a.N = w.rows; a.K = w.cols; a.M = p.rows;
    a.x = p.x; a.y = p.y; a.residual = p.residual;
    bool fused = false;
    hipError_t e;
    if (p.deferred_splits) *p.deferred_splits = 1;
    switch (w.format) {
    case FMT_Q4_K: e = launch_format<FMT_Q4_K>(a, p.workspace, p.workspace_floats, p.swiglu_out, &fused, p.deferred_splits, stream); break;
    case FMT_Q4_0: e = launch_format<FMT_Q4_0>(a, p.workspace, p.workspace_floats, p.swiglu_out, &fused, p.deferred_splits, stream); break;
    case FMT_Q8_0: e = launch_format<FMT_Q8_0>(a, p.workspace, p.workspace_floats, p.swiglu_out, &fused, p.deferred_splits, stream); break;
    case FMT_F16: e = launch_format<FMT_F16>(a, p.workspace, p.workspace_floats, p.swiglu_out, &fused, p.deferred_splits, stream); break;
    default: return hipErrorInvalidValue;   // fp32 matrices stay on the GEMV path
    }
    if (e != hipSuccess || !p.swiglu_out || fused) return e;
    if (w.rows % 2 != 0 || p.residual) return hipErrorInvalidValue;
    return launch_swiglu(p.y, p.rows, w.rows / 2, p.swiglu_out, stream);
}

}  // namespace esp
