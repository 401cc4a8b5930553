// Q4_K prompt-block GEMM with exact weights and split activations:
//     y[m][n] = sum_k x[m][k] * dequant(W)[n][k]
// to about 22 bits of x and every bit of W, on the fp16 matrix cores with fp32 accumulation.
//
// The reference walks a prompt token by token with fp32 activations and fp32 dequantised weights
// (RealModelInferenceEngine.swift:6674-6697 inside :6365-6375).  Rounding either operand to fp16 costs 2^-12
// relative per product, which 32 layers of the 8B shape amplify to 3-4e-2 on the logits; this kernel keeps both.
//
//   * Weights.  A Q4_K weight is d * (sc_j * q) - dmin * m_j with a 4-bit q, 6-bit sc_j and m_j per sub-block of 32
//     and fp16 d, dmin per super-block of 256 and row.  sc_j * q <= 945 is an integer, exact in fp16: THAT is the B operand.
//     The sums over a super-block are then scaled by d in fp32 (one multiply-add per accumulator and super-block), and the
//     minimum term is dmin * sum_j m_j * S_j with S_j the activations' sum over sub-block j: one more MFMA per super-block
//     whose K is (8 x hi of S_j, 8 x lo of S_j scaled by 2048) against (m_0..m_7, m_0..m_7 / 2048).
//   * Activations.  v = hi + lo / 2048 with hi = fp16(v), lo = fp16((v - hi) * 2048) (SplitRowsView): two A operands against
//     the same B operand, two accumulator sets, joined in the per-super-block fold.
//
// Shape: a workgroup of four wavefronts (2 x 2) owns 128 activation rows x 128 weight rows, every wavefront 2 x 2 tiles of
// v_mfma_f32_32x32x16_f16; K walks in tiles of 64 (a pair of sub-blocks) through double-buffered LDS, one barrier per tile,
// with the packed weights and activations of the next tiles in flight in registers.  Two threads per weight row turn its 32
// bytes of nibbles into 64 fp16 integers per tile (one v_and_or_b32 and one packed fp16 multiply-add per two weights).
// Per 256 k a wavefront issues 128 + 4 MFMAs and about 200 fold operations.
#include "../common.h"
#include "decode_ops.h"
#include <atomic>
#include <mutex>
#include <cstdlib>
#include <type_traits>
#include <utility>

namespace esp {
namespace {

typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32;

constexpr int kThreads = 256;
constexpr int KT = 64;          // k per tile
constexpr int LDK = KT + 8;     // fp16 per LDS row
constexpr int NT = 128, MT = 128;
constexpr float kUnscale = 1.0f / 2048.0f, kScale = 2048.0f;

struct SplitGemmArgs {
    const uint8_t *qs;
    size_t qs_row_bytes;
    int N, K, M;
    const uint16_t *xh, *xl, *xs;   // [M][K], [M][K], [M][K / 256][16]
    float *y;
    const float *residual;
    float *partial;                 // [splits][M][N] when gridDim.y > 1
    int tiles_per_split;            // a multiple of four
    uint16_t *sw_hi, *sw_lo;        // SiLU(gate) * up as a split pair [M][N / 2] instead of y (no split-K)
    uint16_t *sw_sums;              // optional (gemm_q4k_split_regb_kernel, N / 2 a multiple of 32): the pair's sub-block sums, else split_sums_kernel follows
    const uint8_t *tiled;           // the matrix-core GEMV's tiled copy (gemm_q4k_split_regb_kernel reads its weights there)
    // shared K ranges (gemm_q4k_split_regb_kernel<.., true>): workgroup i owns K tiles [i * sk_units, (i + 1) * sk_units) of the
    // sequence (output tile 0: K tiles 0 .. K / 64 - 1, output tile 1: ...), output tile t = (t % sk_tiles_n, t / sk_tiles_n)
    int sk_units, sk_tiles_n;
    unsigned *sk_flags;             // [kStreamKFlags]: one word per workgroup, zero between launches
    unsigned sk_spin_limit;
    float *sk_partial;              // [workgroups][128 accumulators][256 threads]
};
constexpr int kStreamKFlags = 1024, kStreamKMaxWorkgroups = 256;
constexpr unsigned kStreamKReady = 1, kStreamKCancelled = 2;   // a flag word's states besides 0
constexpr unsigned kStreamKSpinLimit = 1u << 22;   // polls of the finisher (each at least a trip to memory) before it computes the rest itself

__device__ __forceinline__ h2 as_h2(u32 v) { return __builtin_bit_cast(h2, v); }
__device__ __forceinline__ u32 as_u32(h2 v) { return __builtin_bit_cast(u32, v); }
__device__ __forceinline__ float half_bits_to_float(u32 bits16) { return (float)__builtin_bit_cast(_Float16, (uint16_t)bits16); }
__device__ __forceinline__ u32 dword_of(const uint4 &v, int k) { return k == 0 ? v.x : k == 1 ? v.y : k == 2 ? v.z : v.w; }
__device__ __forceinline__ uint4 swap_middle(const uint4 &v) {
    uint4 p;
    p.x = __builtin_amdgcn_perm(v.y, v.x, 0x05040100u);
    p.y = __builtin_amdgcn_perm(v.y, v.x, 0x07060302u);
    p.z = __builtin_amdgcn_perm(v.w, v.z, 0x05040100u);
    p.w = __builtin_amdgcn_perm(v.w, v.z, 0x07060302u);
    return p;
}
__device__ __forceinline__ u32 scale_byte(const uint4 &hdr, int idx) {
    const u32 word = idx < 4 ? hdr.y : idx < 8 ? hdr.z : hdr.w;
    return (word >> ((idx & 3) * 8)) & 0xFFu;
}
// ggml's get_scale_min_k4, as integers
__device__ __forceinline__ void q4k_scale_min(const uint4 &hdr, int j, u32 &sc, u32 &m) {
    if (j < 4) {
        sc = scale_byte(hdr, j) & 63u;
        m = scale_byte(hdr, j + 4) & 63u;
    } else {
        sc = (scale_byte(hdr, j + 4) & 0xFu) | ((scale_byte(hdr, j - 4) >> 6) << 4);
        m = (scale_byte(hdr, j + 4) >> 4) | ((scale_byte(hdr, j) >> 6) << 4);
    }
}
__device__ __forceinline__ u32 pack_half2(float lo, float hi) {
    return (u32)__builtin_bit_cast(uint16_t, (_Float16)lo) | ((u32)__builtin_bit_cast(uint16_t, (_Float16)hi) << 16);
}

struct RawTile { uint4 q, hdr; };   // sixteen bytes of nibbles of (weight row, tile, half) and the super-block's header

// dynamic LDS: [2] weight tiles, [2] hi tiles, [2] lo tiles, [2] minimum rows, [2] sub-block sums, [2] (d, dmin)
constexpr size_t kTileHalfs = (size_t)128 * LDK;
constexpr size_t kLdsBytes = 6 * kTileHalfs * 2 + 2 * 128 * 16 * 2 + 2 * 128 * 16 * 2 + 2 * 128 * 8;

template <int DEPTH>
__global__ __launch_bounds__(kThreads) void gemm_q4k_split_kernel(SplitGemmArgs a) {
    constexpr int XV = MT * KT / 8 / kThreads;   // 128-bit pieces of a tile of one activation plane per thread (4)
    extern __shared__ uint4 smem_raw[];
    _Float16 *wt = reinterpret_cast<_Float16 *>(smem_raw);     // [2][128 * LDK]   sc * q, (0,2,1,3) order inside fours
    _Float16 *xh = wt + 2 * kTileHalfs;                          // [2][128 * LDK]
    _Float16 *xl = xh + 2 * kTileHalfs;                          // [2][128 * LDK]
    _Float16 *ms = xl + 2 * kTileHalfs;                          // [2][128][16]     m_0..m_7, then m_0..m_7 / 2048, of the weight row's super-block
    _Float16 *xs = ms + 2 * 128 * 16;                            // [2][128][16]     (hi of S_0..S_7, lo of S_0..S_7) of the row
    float2 *dd = reinterpret_cast<float2 *>(xs + 2 * 128 * 16);  // [2][128]         (d, dmin)
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int n0 = blockIdx.x * NT, m0 = blockIdx.z * MT;
    const int tiles = a.K / KT;
    const int t_begin = blockIdx.y * a.tiles_per_split;
    const int t_end = t_begin + a.tiles_per_split < tiles ? t_begin + a.tiles_per_split : tiles;
    const int t_last = t_end - 1;

    const int wr = tid >> 1, wh = tid & 1;                       // dequantisation role: weight row, half of the tile
    const int w_row = n0 + wr < a.N ? n0 + wr : a.N - 1;         // clamped, the result is never stored
    const uint8_t *w_base = a.qs + (size_t)w_row * a.qs_row_bytes;
    const int xs_row = m0 + (tid >> 1) < a.M ? m0 + (tid >> 1) : a.M - 1;
    const int sbs = a.K / 256;

    floatx16 tot[2][2], ah[2][2], al[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) tot[i][j][r] = ah[i][j][r] = al[i][j][r] = 0.0f;

    auto fetch_w = [&](int tile) __attribute__((always_inline)) {
        RawTile r;
        const uint8_t *blk = w_base + (size_t)(tile >> 2) * 144;
        r.hdr = *reinterpret_cast<const uint4 *>(blk);
        r.q = *reinterpret_cast<const uint4 *>(blk + 16 + (tile & 3) * 32 + wh * 16);
        return r;
    };
    // piece i of a thread: row (tid / 8) + 32 i of the tile, eight columns (tid % 8) * 8 .. of it; rows beyond M repeat the last
    // one (never stored).  Element offsets fit 32 bits (the host checks M * K).
    const unsigned x_col = (unsigned)(tid & 7) * 8;
    auto x_row_offset = [&](int i) __attribute__((always_inline)) {
        const int row = (tid >> 3) + 32 * i;
        return (unsigned)(m0 + row < a.M ? m0 + row : a.M - 1) * (unsigned)a.K + x_col;
    };
    const unsigned xo0 = x_row_offset(0), xo1 = x_row_offset(1), xo2 = x_row_offset(2), xo3 = x_row_offset(3);
    static_assert(XV == 4, "four pieces per thread and plane");
    struct XTile { uint4 h0, h1, h2, h3, l0, l1, l2, l3; };   // named members: the registers in flight must never look like an indexed array
    auto fetch_x = [&](int tile) __attribute__((always_inline)) {
        const unsigned t = (unsigned)tile * KT;
        XTile x;
        x.h0 = *reinterpret_cast<const uint4 *>(a.xh + (xo0 + t)); x.l0 = *reinterpret_cast<const uint4 *>(a.xl + (xo0 + t));
        x.h1 = *reinterpret_cast<const uint4 *>(a.xh + (xo1 + t)); x.l1 = *reinterpret_cast<const uint4 *>(a.xl + (xo1 + t));
        x.h2 = *reinterpret_cast<const uint4 *>(a.xh + (xo2 + t)); x.l2 = *reinterpret_cast<const uint4 *>(a.xl + (xo2 + t));
        x.h3 = *reinterpret_cast<const uint4 *>(a.xh + (xo3 + t)); x.l3 = *reinterpret_cast<const uint4 *>(a.xl + (xo3 + t));
        return x;
    };
    auto fetch_sums = [&](int sb) __attribute__((always_inline)) {
        return reinterpret_cast<const uint4 *>(a.xs + ((size_t)xs_row * sbs + (sb < sbs ? sb : sbs - 1)) * 16)[tid & 1];
    };

    static_assert(DEPTH == 2, "two tiles in flight: slots 0 and 1 below");
    const int t_second = t_begin + 1 < t_last ? t_begin + 1 : t_last;
    RawTile raw0 = fetch_w(t_begin), raw1 = fetch_w(t_second);
    XTile x0 = fetch_x(t_begin), x1 = fetch_x(t_second);
    uint4 sums_next = fetch_sums(t_begin >> 2);

    // Staging of tile `tile` (slot S of the registers in flight, c = tile % 4) into LDS buffer `buf` - and with the first tile of a
    // super-block that super-block's minimums, scales and activation sums into buffer (tile / 4) % 2 - cut into kPieces pieces of a few
    // instructions each.  A wavefront is alone on its SIMD (436 registers), so nothing overlaps unless its own instruction stream
    // interleaves: the main loop issues one piece behind every MFMA, fenced, and the piece runs while the matrix core works (counters
    // of the plain order: MFMA busy 31 %, vector ALU 30 %, waiting 38 % of the wavefront's cycles, adding up to all of them).
    struct StageRegs { h2 s_lo, s_hi, o_lo, o_hi; u32 lo[8], hi[8]; };
    constexpr int kPieces = 30;
    auto stage_piece = [&](auto piece_c, auto slot_c, auto chunk_c, int tile, int buf, StageRegs &sr) __attribute__((always_inline)) {
        constexpr int P = decltype(piece_c)::value, S = decltype(slot_c)::value, c = decltype(chunk_c)::value;
        RawTile &rs = S == 0 ? raw0 : raw1;
        XTile &xr = S == 0 ? x0 : x1;
        // low nibbles under 0x6400 read 1024 + q, high nibbles under 0x5400 read 64 + q; (offset + q) * sc - offset * sc is one
        // exact packed multiply-add: the result sc * q <= 945 is an integer
        if constexpr (P == 0) {
            u32 sc, m;
            q4k_scale_min(rs.hdr, 2 * c, sc, m);
            const _Float16 f = (_Float16)(float)sc, o = (_Float16)(-1024.0f * (float)sc);
            sr.s_lo = h2{f, f}; sr.o_lo = h2{o, o};
        } else if constexpr (P == 1) {
            u32 sc, m;
            q4k_scale_min(rs.hdr, 2 * c + 1, sc, m);
            const _Float16 f = (_Float16)(float)sc, o = (_Float16)(-64.0f * (float)sc);
            sr.s_hi = h2{f, f}; sr.o_hi = h2{o, o};
        } else if constexpr (P >= 2 && P < 6) {
            constexpr int k = P - 2;
            const u32 w = dword_of(rs.q, k), w8 = w >> 8;
            sr.lo[2 * k] = as_u32(__builtin_elementwise_fma(as_h2((w & 0x000F000Fu) | 0x64006400u), sr.s_lo, sr.o_lo));
            sr.lo[2 * k + 1] = as_u32(__builtin_elementwise_fma(as_h2((w8 & 0x000F000Fu) | 0x64006400u), sr.s_lo, sr.o_lo));
        } else if constexpr (P >= 6 && P < 10) {
            constexpr int k = P - 6;
            const u32 w = dword_of(rs.q, k), w8 = w >> 8;
            sr.hi[2 * k] = as_u32(__builtin_elementwise_fma(as_h2((w & 0x00F000F0u) | 0x54005400u), sr.s_hi, sr.o_hi));
            sr.hi[2 * k + 1] = as_u32(__builtin_elementwise_fma(as_h2((w8 & 0x00F000F0u) | 0x54005400u), sr.s_hi, sr.o_hi));
        } else if constexpr (P >= 10 && P < 14) {
            _Float16 *wrow = wt + buf * (int)kTileHalfs + wr * LDK;
            if constexpr (P == 10) *reinterpret_cast<uint4 *>(wrow + 16 * wh) = make_uint4(sr.lo[0], sr.lo[1], sr.lo[2], sr.lo[3]);
            if constexpr (P == 11) *reinterpret_cast<uint4 *>(wrow + 16 * wh + 8) = make_uint4(sr.lo[4], sr.lo[5], sr.lo[6], sr.lo[7]);
            if constexpr (P == 12) *reinterpret_cast<uint4 *>(wrow + 32 + 16 * wh) = make_uint4(sr.hi[0], sr.hi[1], sr.hi[2], sr.hi[3]);
            if constexpr (P == 13) *reinterpret_cast<uint4 *>(wrow + 32 + 16 * wh + 8) = make_uint4(sr.hi[4], sr.hi[5], sr.hi[6], sr.hi[7]);
        } else if constexpr (P >= 14 && P < 22) {
            // the planes already hold the (0,2,1,3) order the weights are unpacked in
            const int o = buf * (int)kTileHalfs + (tid >> 3) * LDK + (tid & 7) * 8;
            if constexpr (P == 14) *reinterpret_cast<uint4 *>(xh + o) = xr.h0;
            if constexpr (P == 15) *reinterpret_cast<uint4 *>(xl + o) = xr.l0;
            if constexpr (P == 16) *reinterpret_cast<uint4 *>(xh + o + 32 * LDK) = xr.h1;
            if constexpr (P == 17) *reinterpret_cast<uint4 *>(xl + o + 32 * LDK) = xr.l1;
            if constexpr (P == 18) *reinterpret_cast<uint4 *>(xh + o + 64 * LDK) = xr.h2;
            if constexpr (P == 19) *reinterpret_cast<uint4 *>(xl + o + 64 * LDK) = xr.l2;
            if constexpr (P == 20) *reinterpret_cast<uint4 *>(xh + o + 96 * LDK) = xr.h3;
            if constexpr (P == 21) *reinterpret_cast<uint4 *>(xl + o + 96 * LDK) = xr.l3;
        } else if constexpr (P == 22) {
            if constexpr (c == 0) {
                const int sbuf = (tile >> 2) & 1;
                u32 mm[4];
#pragma unroll
                for (int jj = 0; jj < 4; jj++) { u32 s_unused; q4k_scale_min(rs.hdr, 4 * wh + jj, s_unused, mm[jj]); }
                _Float16 *mrow = ms + sbuf * 128 * 16 + wr * 16 + 4 * wh;
                *reinterpret_cast<uint2 *>(mrow) = make_uint2(pack_half2((float)mm[0], (float)mm[1]), pack_half2((float)mm[2], (float)mm[3]));
                *reinterpret_cast<uint2 *>(mrow + 8) = make_uint2(pack_half2((float)mm[0] * kUnscale, (float)mm[1] * kUnscale),
                                                                  pack_half2((float)mm[2] * kUnscale, (float)mm[3] * kUnscale));
                // both threads of a weight row write the same (d, dmin): no branch
                dd[sbuf * 128 + wr] = make_float2(half_bits_to_float(rs.hdr.x & 0xFFFFu), half_bits_to_float(rs.hdr.x >> 16));
                *reinterpret_cast<uint4 *>(xs + sbuf * 128 * 16 + (tid >> 1) * 16 + 8 * (tid & 1)) = sums_next;
            }
        } else {
            // the slot is free: the tile DEPTH ahead goes into it (clamped past the end: fetched in bounds, never used)
            const int ahead = tile + DEPTH < t_last ? tile + DEPTH : t_last;
            const unsigned tk = (unsigned)ahead * KT;
            if constexpr (P == 23) {
                const uint8_t *blk = w_base + (size_t)(ahead >> 2) * 144;
                rs.hdr = *reinterpret_cast<const uint4 *>(blk);
                rs.q = *reinterpret_cast<const uint4 *>(blk + 16 + (ahead & 3) * 32 + wh * 16);
            }
            if constexpr (P == 24) { xr.h0 = *reinterpret_cast<const uint4 *>(a.xh + (xo0 + tk)); xr.l0 = *reinterpret_cast<const uint4 *>(a.xl + (xo0 + tk)); }
            if constexpr (P == 25) { xr.h1 = *reinterpret_cast<const uint4 *>(a.xh + (xo1 + tk)); xr.l1 = *reinterpret_cast<const uint4 *>(a.xl + (xo1 + tk)); }
            if constexpr (P == 26) { xr.h2 = *reinterpret_cast<const uint4 *>(a.xh + (xo2 + tk)); xr.l2 = *reinterpret_cast<const uint4 *>(a.xl + (xo2 + tk)); }
            if constexpr (P == 27) { xr.h3 = *reinterpret_cast<const uint4 *>(a.xh + (xo3 + tk)); xr.l3 = *reinterpret_cast<const uint4 *>(a.xl + (xo3 + tk)); }
            if constexpr (P == 28 && c == 0) sums_next = fetch_sums((tile >> 2) + 1);
        }
    };
    auto stage_all = [&](auto slot_c, auto chunk_c, int tile, int buf) __attribute__((always_inline)) {
        StageRegs sr;
        auto run = [&](auto... pc) __attribute__((always_inline)) { (stage_piece(pc, slot_c, chunk_c, tile, buf, sr), ...); };
        [&]<int... I>(std::integer_sequence<int, I...>) __attribute__((always_inline)) { run(std::integral_constant<int, I>{}...); }(std::make_integer_sequence<int, kPieces>{});
    };

    stage_all(std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{}, t_begin, 0);   // t_begin is a multiple of four
    __syncthreads();
    auto tile_step = [&](auto u_c, int t) __attribute__((always_inline)) {
            constexpr int u = decltype(u_c)::value, buf = u & 1;
            const _Float16 *xhb = xh + (size_t)buf * kTileHalfs, *xlb = xl + (size_t)buf * kTileHalfs, *wtb = wt + (size_t)buf * kTileHalfs;
            struct Frags { half8 h0, h1, l0, l1, b0, b1; };
            auto load_frags = [&](int ks) __attribute__((always_inline)) {
                const int kk = ks * 16 + 8 * (lane >> 5);
                const int ra = (wm * 64 + (lane & 31)) * LDK + kk, rb = (wn * 64 + (lane & 31)) * LDK + kk;
                Frags f;
                f.h0 = *reinterpret_cast<const half8 *>(xhb + ra);
                f.h1 = *reinterpret_cast<const half8 *>(xhb + ra + 32 * LDK);
                f.l0 = *reinterpret_cast<const half8 *>(xlb + ra);
                f.l1 = *reinterpret_cast<const half8 *>(xlb + ra + 32 * LDK);
                f.b0 = *reinterpret_cast<const half8 *>(wtb + rb);
                f.b1 = *reinterpret_cast<const half8 *>(wtb + rb + 32 * LDK);
                return f;
            };
            auto mfma_one = [&](const Frags &f, auto m_c) __attribute__((always_inline)) {
                constexpr int m = decltype(m_c)::value;
                if constexpr (m == 0) ah[0][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(f.h0, f.b0, ah[0][0], 0, 0, 0);
                if constexpr (m == 1) al[0][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(f.l0, f.b0, al[0][0], 0, 0, 0);
                if constexpr (m == 2) ah[0][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(f.h0, f.b1, ah[0][1], 0, 0, 0);
                if constexpr (m == 3) al[0][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(f.l0, f.b1, al[0][1], 0, 0, 0);
                if constexpr (m == 4) ah[1][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(f.h1, f.b0, ah[1][0], 0, 0, 0);
                if constexpr (m == 5) al[1][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(f.l1, f.b0, al[1][0], 0, 0, 0);
                if constexpr (m == 6) ah[1][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(f.h1, f.b1, ah[1][1], 0, 0, 0);
                if constexpr (m == 7) al[1][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(f.l1, f.b1, al[1][1], 0, 0, 0);
            };
            // the tile being staged behind the MFMAs: t + 1, from slot (u + 1) % 2 into the other LDS buffer
            constexpr int S = (u + 1) % DEPTH, c = (u + 1) & 3;
            StageRegs sr;
            // eight MFMAs of k step `ks` (fragments f), piece first + m behind MFMA m
            auto k_step = [&](const Frags &f, auto first_c) __attribute__((always_inline)) {
                constexpr int first = decltype(first_c)::value;
                [&]<int... M>(std::integer_sequence<int, M...>) __attribute__((always_inline)) {
                    ((mfma_one(f, std::integral_constant<int, M>{}),
                      stage_piece(std::integral_constant<int, (first + M < kPieces ? first + M : kPieces)>{}, std::integral_constant<int, S>{},
                                  std::integral_constant<int, c>{}, t + 1, buf ^ 1, sr),
                      __builtin_amdgcn_sched_barrier(0)), ...);
                }(std::make_integer_sequence<int, 8>{});
            };
            const Frags f0 = load_frags(0);
            stage_piece(std::integral_constant<int, 0>{}, std::integral_constant<int, S>{}, std::integral_constant<int, c>{}, t + 1, buf ^ 1, sr);
            stage_piece(std::integral_constant<int, 1>{}, std::integral_constant<int, S>{}, std::integral_constant<int, c>{}, t + 1, buf ^ 1, sr);
            const Frags f1 = load_frags(1);
            __builtin_amdgcn_sched_barrier(0);
            k_step(f0, std::integral_constant<int, 2>{});
            const Frags f2 = load_frags(2);
            __builtin_amdgcn_sched_barrier(0);
            k_step(f1, std::integral_constant<int, 10>{});
            const Frags f3 = load_frags(3);
            __builtin_amdgcn_sched_barrier(0);
            k_step(f2, std::integral_constant<int, 18>{});
            k_step(f3, std::integral_constant<int, 26>{});
            if (u == 3) {
                // the super-block is complete: total += d * (hi sums + lo sums / 2048) - dmin * sum_j m_j S_j
                const int sbuf = (t >> 2) & 1;
                half8 fs[2], fm[2];
                float2 dv[2];
#pragma unroll
                for (int i = 0; i < 2; i++) fs[i] = *reinterpret_cast<const half8 *>(xs + (size_t)sbuf * 128 * 16 + ((wm * 2 + i) * 32 + (lane & 31)) * 16 + 8 * (lane >> 5));
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    fm[j] = *reinterpret_cast<const half8 *>(ms + (size_t)sbuf * 128 * 16 + ((wn * 2 + j) * 32 + (lane & 31)) * 16 + 8 * (lane >> 5));
                    dv[j] = dd[sbuf * 128 + (wn * 2 + j) * 32 + (lane & 31)];
                }
#pragma unroll
                for (int i = 0; i < 2; i++)
#pragma unroll
                    for (int j = 0; j < 2; j++) {
                        floatx16 am;
#pragma unroll
                        for (int r = 0; r < 16; r++) am[r] = 0.0f;
                        am = __builtin_amdgcn_mfma_f32_32x32x16_f16(fs[i], fm[j], am, 0, 0, 0);
#pragma unroll
                        for (int r = 0; r < 16; r++) {
                            const float main = __builtin_fmaf(al[i][j][r], kUnscale, ah[i][j][r]);
                            tot[i][j][r] = __builtin_fmaf(-dv[j].y, am[r], __builtin_fmaf(dv[j].x, main, tot[i][j][r]));
                        }
                        ah[i][j] = floatx16{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                        al[i][j] = ah[i][j];
                    }
            }
            __syncthreads();
    };
    for (int t0 = t_begin; t0 < t_end; t0 += 4) {
        tile_step(std::integral_constant<int, 0>{}, t0);
        tile_step(std::integral_constant<int, 1>{}, t0 + 1);
        tile_step(std::integral_constant<int, 2>{}, t0 + 2);
        tile_step(std::integral_constant<int, 3>{}, t0 + 3);
    }

    // accumulator r of lane l: row 8 (r / 4) + 4 (l / 32) + r % 4, column l % 32 of the 32 x 32 tile
    if (a.sw_hi) {   // rows of W are (gate, up) pairs: even lanes hold gate, their right neighbours up (:6825-6827, :6337)
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const int n = n0 + (wn * 2 + j) * 32 + (lane & 31);
                const bool odd = lane & 1;
#pragma unroll
                for (int k = 0; k < 8; k++) {
                    const float a0 = tot[i][j][2 * k], a1 = tot[i][j][2 * k + 1];
                    const float p0 = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, a0), 0xB1, 0xF, 0xF, false));
                    const float p1 = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, a1), 0xB1, 0xF, 0xF, false));
                    const float g = odd ? p1 : a0, up = odd ? a1 : p0;
                    const int r = 2 * k + (odd ? 1 : 0);
                    const int m = m0 + (wm * 2 + i) * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                    if (m < a.M && (n | 1) < a.N) {
                        const float silu = g * __builtin_amdgcn_rcpf(1.0f + __expf(-g));   // = 0.5 g (1 + tanh(0.5 g)), a fifth of tanhf's instructions
                        const float act = __fmul_rn(silu, up);
                        const _Float16 hi = (_Float16)act;
                        const int unit = n / 2, slot = unit & 3;   // the planes' order inside fours: (0, 2, 1, 3)
                        const size_t o = (size_t)m * (a.N / 2) + (unit & ~3) + (slot == 1 ? 2 : slot == 2 ? 1 : slot);
                        a.sw_hi[o] = __builtin_bit_cast(uint16_t, hi);
                        a.sw_lo[o] = __builtin_bit_cast(uint16_t, (_Float16)__fmul_rn(__fsub_rn(act, (float)hi), kScale));
                    }
                }
            }
        return;
    }
    const bool split = gridDim.y > 1;
    float *out = split ? a.partial + (size_t)blockIdx.y * a.M * a.N : a.y;
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int n = n0 + (wn * 2 + j) * 32 + (lane & 31);
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int m = m0 + (wm * 2 + i) * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                if (m < a.M && n < a.N) {
                    const size_t o = (size_t)m * a.N + n;
                    out[o] = (!split && a.residual) ? a.residual[o] + tot[i][j][r] : tot[i][j][r];
                }
            }
        }
}

// ---- the same product with the weights kept out of LDS -------------------------------------------------------------------------
// Counters and timing-only builds of the kernel above say where its time goes: the 64 x 64 tile of a wavefront reads 6 KB of
// fragments per eight MFMAs (LDS busier than the matrix cores), a quarter of the time is the weights' way through LDS (dequantise,
// write, barrier, read back) and a sixth is the barrier itself.  Here a wavefront builds its B fragments in registers, straight from
// the tiled copy the GEMV reads (lane (n, kg) of a 32-column block fetches bytes 8 kg .. 8 kg + 7 of the first and of the second half
// of its row's 32-byte chunk: eight-byte loads that cover whole 256-byte runs of the tile), so only the activations go through LDS
// and a wavefront can own 64 activation rows x 128 weight rows: four A fragments per sixteen MFMAs.  The lo plane accumulates into
// the same registers as the hi plane, against the B operand scaled by 2^-11 (sc * q / 2048 is exact in fp16 too), so one accumulator
// set of 128 registers and one of totals suffice.  Workgroup = four wavefronts = 128 activation rows x 256 weight rows.
// Counters of this kernel: a wavefront's vector-ALU instructions and its MFMAs take turns (39 % + 44 % of its cycles; forcing an MFMA /
// vector interleave in the instruction order changes nothing, a second wavefront per SIMD with half the tile is slower), so what counts
// is the vector work per MFMA: with every wavefront on all 128 rows and 64 weight rows (RB x CB = 4 x 2) a B fragment serves eight
// MFMAs instead of four: gate|up of a 512-row block 356 -> 324 us (the kernel above: 421 on the same boxes).  The activation tiles
// rotate through four LDS buffers so that one barrier serves two tiles (318 -> 313 us, old and new alternating on one box).
__device__ __forceinline__ void store_subblock_sum(uint16_t *sums, size_t row, int cols, int group, float s);
constexpr int NT2 = 256;
constexpr int kRegBBufs = 4;   // activation tiles in LDS: with four, one barrier serves two tiles
constexpr size_t kLdsBytesRegB = 2 * kRegBBufs * kTileHalfs * 2 + 2 * 128 * 16 * 2;

// RB x CB = 32-row blocks of activations x 32-row blocks of weights per wavefront (eight in all: 128 accumulator registers).
//
// SK (shared K ranges): the SiLU(gate) * up launch of a 512-row block is 448 output tiles on 256 compute units, a full round and one
// that is three quarters full.  With SK the grid is one workgroup per compute unit and workgroup i takes K tiles [i u, (i + 1) u) of
// the sequence "all K tiles of output tile 0, then of output tile 1, ..." (u = all K tiles / workgroups, at least one output tile's
// worth, a multiple of four): the rest of the output tile its predecessor began, whole output tiles, and the beginning of one more.
// A workgroup that ends inside an output tile finishes it: its successor, whose first piece that tile's rest is, leaves its 128
// totals per lane in `sk_partial` and then writes the launch's number into its flag word; the finisher adds them and runs the
// epilogue.  The successor's piece is the first thing it does and waits for nothing, so whatever the order in which workgroups
// become resident the finisher's wait ends; it is bounded all the same (sk_spin_limit polls), and a finisher whose wait runs out
// computes the rest of the tile itself.  A flag word is 0 between launches: the successor moves it 0 -> ready, the finisher back to 0 once
// it has the totals; a finisher that gives up moves it 0 -> cancelled and the successor, finding that, back to 0 (both by compare-and-swap,
// so whichever comes first the word ends at 0 and the totals are taken at most once): a replay under a captured graph starts clean.
// `sk_partial` and `sk_flags` are uncached device memory: with ordinary memory the hand-over needs a release that writes the die's
// L2 back (10 us per workgroup, measured) and an acquire that invalidates the finisher's.
// Measured on gate|up of a 512-row block, workgroup by workgroup (wall-clock stamps): 2.2 us per K tile, 4.7 us per epilogue, 3.7 us to
// hand the totals over, 6.3 us to take them; the launch 295 against 310 us for the plain grid on the same box.
template <int RB, int CB, bool SK = false>
__global__ __launch_bounds__(kThreads) void gemm_q4k_split_regb_kernel(SplitGemmArgs a) {
    static_assert(RB * CB == 8 && (RB == 2 || RB == 4), "a wavefront owns eight 32 x 32 tiles");
    __shared__ int sk_flag_seen;
    constexpr int THREADS = kThreads, XP = 1024 / THREADS;   // sixteen-byte pieces of a plane's tile per thread
    constexpr int NW = 8 / CB;                               // wavefronts along the weight rows
    extern __shared__ uint4 smem_raw[];
    _Float16 *xh = reinterpret_cast<_Float16 *>(smem_raw);     // [kRegBBufs][128 * LDK]
    _Float16 *xl = xh + kRegBBufs * kTileHalfs;                  // [kRegBBufs][128 * LDK]
    _Float16 *xs = xl + kRegBBufs * kTileHalfs;                        // [2][128][16]   (hi of S_0..S_7, lo of S_0..S_7) of the row
    const int tiles = a.K / KT, sbs = a.K / 256;
    floatx16 tot[RB][CB], acc[RB][CB];   // acc starts every super-block from the zero C operand of its first MFMAs
    int sk_unit = SK ? (int)blockIdx.x * a.sk_units : 0;
    const int sk_unit_end = sk_unit + a.sk_units;
    int sk_resume_from = 0;   // > 0: the previous pass ended at this K tile of the same output tile and the totals stay
  for (;;) {   // one pass per piece of an output tile with SK, a single pass otherwise (the body keeps a function body's indentation)
    // The thread's coordinates are formed anew for every output tile piece: taken from outside the loop, every LDS and row offset
    // derived from them would be kept in registers across the pieces, and the kernel has none to spare.
    int tid = threadIdx.x;
    if constexpr (SK) asm volatile("" : "+v"(tid));
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave / NW, wn = wave % NW;            // wm: which 32 RB activation rows of the tile, wn: which 32 CB weight rows
    const int bn = lane & 31, kg = lane >> 5;
    int n0, m0, t_begin, t_end;
    if constexpr (SK) {
        const int out_tile = sk_unit / tiles, first = sk_resume_from ? sk_resume_from : sk_unit % tiles;
        const int room = sk_resume_from ? tiles - first : sk_unit_end - sk_unit;
        n0 = (out_tile % a.sk_tiles_n) * NT2; m0 = (out_tile / a.sk_tiles_n) * MT;
        t_begin = first; t_end = first + room < tiles ? first + room : tiles;
    } else {
        n0 = blockIdx.x * NT2; m0 = blockIdx.z * MT;
        t_begin = blockIdx.y * a.tiles_per_split;
        t_end = t_begin + a.tiles_per_split < tiles ? t_begin + a.tiles_per_split : tiles;
    }
    const int t_last = t_end - 1;

    // weights: column block cb of this wavefront = weight rows n0 + 32 CB wn + 32 cb + (0..31); this lane's row of it, clamped (never stored)
    const uint8_t *wrow[4];
#pragma unroll
    for (int cb = 0; cb < 4; cb++) {
        const int want = n0 + 32 * CB * wn + 32 * (cb < CB ? cb : 0) + bn;
        const int row = want < a.N ? want : a.N - 1;
        wrow[cb] = a.tiled + (size_t)(row >> 4) * sbs * 2304 + 16 * (row & 15);
    }
    struct WRaw { uint2 a0, a1, a2, a3, b0, b1, b2, b3; };   // per column block: eight bytes of the chunk's first / second sixteen
    auto fetch_w = [&](int tile) __attribute__((always_inline)) {
        WRaw r;
        const size_t o = (size_t)(tile >> 2) * 2304 + 256 + 256 * (tile & 3) + 8 * kg;
        r.a0 = *reinterpret_cast<const uint2 *>(wrow[0] + o); r.b0 = *reinterpret_cast<const uint2 *>(wrow[0] + o + 1024);
        r.a1 = *reinterpret_cast<const uint2 *>(wrow[1] + o); r.b1 = *reinterpret_cast<const uint2 *>(wrow[1] + o + 1024);
        if constexpr (CB > 2) {
            r.a2 = *reinterpret_cast<const uint2 *>(wrow[2] + o); r.b2 = *reinterpret_cast<const uint2 *>(wrow[2] + o + 1024);
            r.a3 = *reinterpret_cast<const uint2 *>(wrow[3] + o); r.b3 = *reinterpret_cast<const uint2 *>(wrow[3] + o + 1024);
        } else { r.a2 = r.a3 = r.a0; r.b2 = r.b3 = r.b0; }
        return r;
    };
    struct Hdrs { uint4 h0, h1, h2, h3; };
    auto fetch_hdr = [&](int sb) __attribute__((always_inline)) {
        Hdrs h;
        const size_t o = (size_t)(sb < sbs ? sb : sbs - 1) * 2304;
        h.h0 = *reinterpret_cast<const uint4 *>(wrow[0] + o); h.h1 = *reinterpret_cast<const uint4 *>(wrow[1] + o);
        if constexpr (CB > 2) { h.h2 = *reinterpret_cast<const uint4 *>(wrow[2] + o); h.h3 = *reinterpret_cast<const uint4 *>(wrow[3] + o); }
        else { h.h2 = h.h3 = h.h0; }
        return h;
    };

    // activations: piece i of a thread = row (tid / 8) + 32 i of the tile, eight columns (tid % 8) * 8 .. of it (as in the kernel above)
    const unsigned x_col = (unsigned)(tid & 7) * 8;
    constexpr int XSTEP = THREADS / 8;   // rows between a thread's pieces
    auto x_row_offset = [&](int i) __attribute__((always_inline)) {
        const int row = (tid >> 3) + XSTEP * i;
        return (unsigned)(m0 + row < a.M ? m0 + row : a.M - 1) * (unsigned)a.K + x_col;
    };
    const unsigned xo0 = x_row_offset(0), xo1 = x_row_offset(1), xo2 = x_row_offset(XP > 2 ? 2 : 0), xo3 = x_row_offset(XP > 2 ? 3 : 0);
    struct XTile { uint4 h0, h1, h2, h3, l0, l1, l2, l3; };
    auto fetch_x = [&](int tile) __attribute__((always_inline)) {
        const unsigned t = (unsigned)tile * KT;
        XTile x;
        x.h0 = *reinterpret_cast<const uint4 *>(a.xh + (xo0 + t)); x.l0 = *reinterpret_cast<const uint4 *>(a.xl + (xo0 + t));
        x.h1 = *reinterpret_cast<const uint4 *>(a.xh + (xo1 + t)); x.l1 = *reinterpret_cast<const uint4 *>(a.xl + (xo1 + t));
        if constexpr (XP > 2) {
            x.h2 = *reinterpret_cast<const uint4 *>(a.xh + (xo2 + t)); x.l2 = *reinterpret_cast<const uint4 *>(a.xl + (xo2 + t));
            x.h3 = *reinterpret_cast<const uint4 *>(a.xh + (xo3 + t)); x.l3 = *reinterpret_cast<const uint4 *>(a.xl + (xo3 + t));
        }
        return x;
    };
    const int xs_row = m0 + ((tid & 255) >> 1) < a.M ? m0 + ((tid & 255) >> 1) : a.M - 1;
    auto fetch_sums = [&](int sb) __attribute__((always_inline)) {
        return reinterpret_cast<const uint4 *>(a.xs + ((size_t)xs_row * sbs + (sb < sbs ? sb : sbs - 1)) * 16)[tid & 1];
    };
    auto store_x = [&](const XTile &x, int buf) __attribute__((always_inline)) {
        const int o = buf * (int)kTileHalfs + (tid >> 3) * LDK + (tid & 7) * 8;
        *reinterpret_cast<uint4 *>(xh + o) = x.h0; *reinterpret_cast<uint4 *>(xl + o) = x.l0;
        *reinterpret_cast<uint4 *>(xh + o + XSTEP * LDK) = x.h1; *reinterpret_cast<uint4 *>(xl + o + XSTEP * LDK) = x.l1;
        if constexpr (XP > 2) {
            *reinterpret_cast<uint4 *>(xh + o + 64 * LDK) = x.h2; *reinterpret_cast<uint4 *>(xl + o + 64 * LDK) = x.l2;
            *reinterpret_cast<uint4 *>(xh + o + 96 * LDK) = x.h3; *reinterpret_cast<uint4 *>(xl + o + 96 * LDK) = x.l3;
        }
    };
    auto store_sums = [&](const uint4 &v, int sb) __attribute__((always_inline)) {   // with 512 threads both halves write the same values
        *reinterpret_cast<uint4 *>(xs + (sb & 1) * 128 * 16 + ((tid & 255) >> 1) * 16 + 8 * (tid & 1)) = v;
    };

    if (!SK || !sk_resume_from) {
#pragma unroll
        for (int i = 0; i < RB; i++)
#pragma unroll
            for (int j = 0; j < CB; j++)
#pragma unroll
                for (int r = 0; r < 16; r++) tot[i][j][r] = 0.0f;
    }
    const floatx16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    // constants of the nibble trick, hidden from the optimiser so that (w & mask) | magic stays one v_and_or_b32
    u32 mask_lo = 0x000F000Fu, mask_hi = 0x00F000F0u, magic_lo = 0x64006400u, magic_hi = 0x54005400u;
    asm volatile("" : "+s"(mask_lo), "+s"(mask_hi));
    asm volatile("" : "+v"(magic_lo), "+v"(magic_hi));

    // prologue: tiles t_begin and t_begin + 1 staged, t_begin + 2 in registers, weights of the first two in registers
    const int t_second = t_begin + 1 < t_last ? t_begin + 1 : t_last;
    WRaw w0 = fetch_w(t_begin), w1 = fetch_w(t_second);
    Hdrs hdr = fetch_hdr(t_begin >> 2);
    {
        const XTile xfirst = fetch_x(t_begin);
        store_sums(fetch_sums(t_begin >> 2), t_begin >> 2);
        store_x(xfirst, 0);
        const XTile xsecond = fetch_x(t_second);
        store_x(xsecond, 1);
    }
    XTile xn = fetch_x(t_begin + 2 < t_last ? t_begin + 2 : t_last);
    uint4 sums_next = fetch_sums((t_begin >> 2) + 1);
    Hdrs hdr_next = fetch_hdr((t_begin >> 2) + 1);
    __syncthreads();

    const h2 kTwoM11 = {(_Float16)kUnscale, (_Float16)kUnscale};
    auto tile_step = [&](auto u_c, int t) __attribute__((always_inline)) {
        constexpr int u = decltype(u_c)::value;
        const _Float16 *xhb = xh + (size_t)u * kTileHalfs, *xlb = xl + (size_t)u * kTileHalfs;
        WRaw &w = (u & 1) == 0 ? w0 : w1;
        const uint4 hd[4] = {hdr.h0, hdr.h1, hdr.h2, hdr.h3};
        const uint2 wa[4] = {w.a0, w.a1, w.a2, w.a3}, wb[4] = {w.b0, w.b1, w.b2, w.b3};
        // scale constants of the tile's two sub-blocks per column block: (offset + q) * sc - offset * sc, and the same / 2048
        h2 s_lo[CB], o_lo[CB], s_hi[CB], o_hi[CB];
#pragma unroll
        for (int cb = 0; cb < CB; cb++) {
            u32 sc, m;
            q4k_scale_min(hd[cb], 2 * u, sc, m);
            const _Float16 f0 = (_Float16)(unsigned short)sc;
            s_lo[cb] = h2{f0, f0}; o_lo[cb] = s_lo[cb] * h2{(_Float16)-1024.0f, (_Float16)-1024.0f};
            q4k_scale_min(hd[cb], 2 * u + 1, sc, m);
            const _Float16 f1 = (_Float16)(unsigned short)sc;
            s_hi[cb] = h2{f1, f1}; o_hi[cb] = s_hi[cb] * h2{(_Float16)-64.0f, (_Float16)-64.0f};
        }
        // the tile two ahead goes to its LDS buffer (fetched during the previous tile), then its successor is fetched.  A tile's buffer
        // was last read two tiles ago and is read again two tiles on, and a barrier closes every odd tile: one lies in between either way.
        store_x(xn, (u + 2) & 3);
        if (u == 3) store_sums(sums_next, (t >> 2) + 1);
        {
            const int ahead = t + 3 < t_last ? t + 3 : t_last;
            xn = fetch_x(ahead);
            if (u == 3) sums_next = fetch_sums((t >> 2) + 2);
        }
        struct Frags { half8 h[RB], l[RB]; };
        auto load_frags = [&](int ks) __attribute__((always_inline)) {
            const int ra = (wm * 32 * RB + bn) * LDK + ks * 16 + 8 * kg;
            Frags f;
#pragma unroll
            for (int i = 0; i < RB; i++) {
                f.h[i] = *reinterpret_cast<const half8 *>(xhb + ra + 32 * i * LDK);
                f.l[i] = *reinterpret_cast<const half8 *>(xlb + ra + 32 * i * LDK);
            }
            return f;
        };
        // the super-block's fold, per column block, right behind that block's last MFMAs (the other blocks' MFMAs run meanwhile):
        // total += d * sums - dmin * sum_j m_j S_j (one MFMA: K = (8 x hi of S_j, 8 x lo of S_j * 2048) against (m_0..m_7, m_0..m_7 / 2048))
        half8 fs[RB];
        if (u == 3) {
            const int sbuf = (t >> 2) & 1;
#pragma unroll
            for (int i = 0; i < RB; i++) fs[i] = *reinterpret_cast<const half8 *>(xs + (size_t)sbuf * 128 * 16 + ((wm * RB + i) * 32 + bn) * 16 + 8 * kg);
        }
        auto fold = [&](int cb) __attribute__((always_inline)) {
            const float mscale = kg ? kUnscale : 1.0f;
            float mv[8];
#pragma unroll
            for (int j = 0; j < 8; j++) { u32 sc, m; q4k_scale_min(hd[cb], j, sc, m); mv[j] = (float)m * mscale; }
            const uint4 mq = make_uint4(pack_half2(mv[0], mv[1]), pack_half2(mv[2], mv[3]), pack_half2(mv[4], mv[5]), pack_half2(mv[6], mv[7]));
            const float d = half_bits_to_float(hd[cb].x & 0xFFFFu), dmin = half_bits_to_float(hd[cb].x >> 16);
#pragma unroll
            for (int i = 0; i < RB; i++) {
                const floatx16 am = __builtin_amdgcn_mfma_f32_32x32x16_f16(fs[i], __builtin_bit_cast(half8, mq), zero16, 0, 0, 0);
#pragma unroll
                for (int r = 0; r < 16; r++) tot[i][cb][r] = __builtin_fmaf(-dmin, am[r], __builtin_fmaf(d, acc[i][cb][r], tot[i][cb][r]));
            }
        };
        Frags fnext = load_frags(0);
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
            const Frags f = fnext;
            if (ks < 3) fnext = load_frags(ks + 1);
#pragma unroll
            for (int cb = 0; cb < CB; cb++) {
                const uint2 q = (ks & 1) ? wb[cb] : wa[cb];   // k 0..15 and 32..47 of the tile: the chunk's first sixteen bytes; 16..31, 48..63: its second
                const u32 x0 = q.x, x1 = q.y, x08 = x0 >> 8, x18 = x1 >> 8;
                uint4 bq, bs;
                if (ks < 2) {
                    const h2 v0 = as_h2((x0 & mask_lo) | magic_lo), v1 = as_h2((x08 & mask_lo) | magic_lo);
                    const h2 v2 = as_h2((x1 & mask_lo) | magic_lo), v3 = as_h2((x18 & mask_lo) | magic_lo);
                    const h2 p0 = __builtin_elementwise_fma(v0, s_lo[cb], o_lo[cb]), p1 = __builtin_elementwise_fma(v1, s_lo[cb], o_lo[cb]);
                    const h2 p2 = __builtin_elementwise_fma(v2, s_lo[cb], o_lo[cb]), p3 = __builtin_elementwise_fma(v3, s_lo[cb], o_lo[cb]);
                    bq = make_uint4(as_u32(p0), as_u32(p1), as_u32(p2), as_u32(p3));
                    bs = make_uint4(as_u32(p0 * kTwoM11), as_u32(p1 * kTwoM11), as_u32(p2 * kTwoM11), as_u32(p3 * kTwoM11));
                } else {
                    const h2 v0 = as_h2((x0 & mask_hi) | magic_hi), v1 = as_h2((x08 & mask_hi) | magic_hi);
                    const h2 v2 = as_h2((x1 & mask_hi) | magic_hi), v3 = as_h2((x18 & mask_hi) | magic_hi);
                    const h2 p0 = __builtin_elementwise_fma(v0, s_hi[cb], o_hi[cb]), p1 = __builtin_elementwise_fma(v1, s_hi[cb], o_hi[cb]);
                    const h2 p2 = __builtin_elementwise_fma(v2, s_hi[cb], o_hi[cb]), p3 = __builtin_elementwise_fma(v3, s_hi[cb], o_hi[cb]);
                    bq = make_uint4(as_u32(p0), as_u32(p1), as_u32(p2), as_u32(p3));
                    bs = make_uint4(as_u32(p0 * kTwoM11), as_u32(p1 * kTwoM11), as_u32(p2 * kTwoM11), as_u32(p3 * kTwoM11));
                }
                const half8 fb = __builtin_bit_cast(half8, bq), fbs = __builtin_bit_cast(half8, bs);
#pragma unroll
                for (int i = 0; i < RB; i++)
                    acc[i][cb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(f.h[i], fb, (u == 0 && ks == 0) ? zero16 : acc[i][cb], 0, 0, 0);
#pragma unroll
                for (int i = 0; i < RB; i++) acc[i][cb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(f.l[i], fbs, acc[i][cb], 0, 0, 0);
                if (u == 3 && ks == 3 && cb > 0) fold(cb - 1);
            }
        }
        if (u == 3) fold(CB - 1);
        // this slot's weights are used up: the tile two ahead goes into it
        {
            const int ahead = t + 2 < t_last ? t + 2 : t_last;
            w = fetch_w(ahead);
        }
        if (u == 3) {
            hdr = hdr_next;
            hdr_next = fetch_hdr((t >> 2) + 2);
        }
        if (u & 1) __syncthreads();
    };
    for (int t0 = t_begin; t0 < t_end; t0 += 4) {
        tile_step(std::integral_constant<int, 0>{}, t0);
        tile_step(std::integral_constant<int, 1>{}, t0 + 1);
        tile_step(std::integral_constant<int, 2>{}, t0 + 2);
        tile_step(std::integral_constant<int, 3>{}, t0 + 3);
    }

    if constexpr (SK) {
        const bool resumed = sk_resume_from != 0;
        if (!resumed) sk_unit += t_end - t_begin;
        sk_resume_from = 0;
        if (!resumed && t_begin > 0) {
            // the rest of an output tile that the previous workgroup began: hand the totals over and go on
            // (uncached memory: once the stores are acknowledged and the wavefronts have met, the flag may follow)
            float4 *slot = reinterpret_cast<float4 *>(a.sk_partial + (size_t)blockIdx.x * 128 * THREADS) + tid;
            asm volatile("" : "+v"(slot));   // formed here, not ahead of the loop: 32 addresses kept in registers would spill
#pragma unroll
            for (int i = 0; i < RB; i++)
#pragma unroll
                for (int j = 0; j < CB; j++)
#pragma unroll
                    for (int q = 0; q < 4; q++)
                        slot[(size_t)((i * CB + j) * 4 + q) * THREADS] = make_float4(tot[i][j][4 * q], tot[i][j][4 * q + 1], tot[i][j][4 * q + 2], tot[i][j][4 * q + 3]);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // every store of this wavefront acknowledged
            __syncthreads();
            if (tid == 0) {   // 0 -> ready; a finisher that gave up left "cancelled": nobody will take the totals, back to 0
                unsigned expected = 0;
                if (!__hip_atomic_compare_exchange_strong(a.sk_flags + blockIdx.x, &expected, kStreamKReady, __ATOMIC_RELAXED, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))
                    __hip_atomic_store(a.sk_flags + blockIdx.x, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            if (sk_unit >= sk_unit_end) return;
            continue;
        }
        if (t_end < tiles) {
            // this workgroup began the output tile: the next one has (or will have) the rest
            if (tid == 0) {
                unsigned *flag = a.sk_flags + blockIdx.x + 1;
                int seen = 0;
                for (unsigned polls = 0; polls < a.sk_spin_limit; polls++) {
                    if (__hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == kStreamKReady) { seen = 1; break; }
                    __builtin_amdgcn_s_sleep(8);
                }
                if (!seen && a.sk_spin_limit != 0) {   // give up: 0 -> cancelled, unless the successor got there first
                    unsigned expected = 0;
                    if (!__hip_atomic_compare_exchange_strong(flag, &expected, kStreamKCancelled, __ATOMIC_RELAXED, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) seen = 1;
                } else if (!seen) {                    // no polls at all (tests): never take the totals, even if they are there
                    if (__hip_atomic_exchange(flag, kStreamKCancelled, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == kStreamKReady)
                        __hip_atomic_store(flag, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
                sk_flag_seen = seen;
            }
            __syncthreads();
            const bool seen = sk_flag_seen != 0;
            __syncthreads();
            if (!seen) { sk_resume_from = t_end; continue; }
            // (issued behind the barrier that follows thread 0's sight of the flag)
            const float4 *slot = reinterpret_cast<const float4 *>(a.sk_partial + (size_t)(blockIdx.x + 1) * 128 * THREADS) + tid;
            asm volatile("" : "+v"(slot));
            // all loads in flight at once, into the accumulators (free between two super-blocks), then one pass of additions
#pragma unroll
            for (int i = 0; i < RB; i++)
#pragma unroll
                for (int j = 0; j < CB; j++)
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        const float4 v = slot[(size_t)((i * CB + j) * 4 + q) * THREADS];
                        acc[i][j][4 * q] = v.x; acc[i][j][4 * q + 1] = v.y; acc[i][j][4 * q + 2] = v.z; acc[i][j][4 * q + 3] = v.w;
                    }
#pragma unroll
            for (int i = 0; i < RB; i++)
#pragma unroll
                for (int j = 0; j < CB; j++)
#pragma unroll
                    for (int r = 0; r < 16; r++) tot[i][j][r] += acc[i][j][r];
            __syncthreads();   // every wavefront has its share of the totals
            if (tid == 0) __hip_atomic_store(a.sk_flags + blockIdx.x + 1, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    // accumulator r of lane l: row 8 (r / 4) + 4 (l / 32) + r % 4, column l % 32 of the 32 x 32 tile
    if (a.sw_hi) {
        // SiLU(gate) * up of the workgroup's 128 x 128 units as the two fp16 planes, through LDS (free now) so that the planes leave
        // in whole 16-byte pieces of a row: [plane][128 rows][kActLd].  SiLU as g / (1 + exp(-g)) (the form of Sources/CPUOps/SiLU.swift:5-8):
        // the same function as the 0.5 g (1 + tanh(0.5 g)) of RealModelInferenceEngine.swift:6825-6827 that the single-row kernels keep, a fifth of the instructions (this epilogue measured 10 us per
        // output tile with tanhf and two-byte stores, a fifteenth of the tile's time).
        constexpr int kActLd = 144;   // halfs per staged row: consecutive rows eight LDS banks apart
        uint16_t *act_hi = reinterpret_cast<uint16_t *>(smem_raw), *act_lo = act_hi + 128 * kActLd;
        const bool odd = lane & 1;
#pragma unroll
        for (int i = 0; i < RB; i++)
#pragma unroll
            for (int j = 0; j < CB; j++) {
                const int unit = (32 * CB * wn + 32 * j + bn) >> 1, slot = unit & 3;   // the planes' order inside fours: (0, 2, 1, 3)
                const int col = (unit & ~3) + (slot == 1 ? 2 : slot == 2 ? 1 : slot);
                const int row0 = (wm * RB + i) * 32 + 4 * kg + (odd ? 1 : 0);
#pragma unroll
                for (int k = 0; k < 8; k++) {
                    const float a0 = tot[i][j][2 * k], a1 = tot[i][j][2 * k + 1];
                    const float p0 = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, a0), 0xB1, 0xF, 0xF, false));
                    const float p1 = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, a1), 0xB1, 0xF, 0xF, false));
                    const float g = odd ? p1 : a0, up = odd ? a1 : p0;
                    const float silu = g * __builtin_amdgcn_rcpf(1.0f + __expf(-g));
                    const float act = __fmul_rn(silu, up);
                    const _Float16 hi = (_Float16)act;
                    const int o = (row0 + 8 * (k >> 1) + 2 * (k & 1)) * kActLd + col;   // row 8 (r / 4) + r % 4 of the block, r = 2 k (+ 1)
                    act_hi[o] = __builtin_bit_cast(uint16_t, hi);
                    act_lo[o] = __builtin_bit_cast(uint16_t, (_Float16)__fmul_rn(__fsub_rn(act, (float)hi), kScale));
                }
            }
        __syncthreads();
        const int units_n = a.N / 2, unit0 = n0 / 2;
        const bool whole_pieces = units_n % 8 == 0;
#pragma unroll
        for (int q = 0; q < 8; q++) {
            const int piece = q * THREADS + tid, row = piece >> 4, c8 = (piece & 15) * 8;
            const int m = m0 + row;
            if (m >= a.M || unit0 + c8 >= units_n) continue;
            const size_t o = (size_t)m * units_n + unit0 + c8;
            if (whole_pieces) {   // units_n and unit0 + c8 are multiples of eight: the piece is whole and 16-byte aligned
                const uint4 h = *reinterpret_cast<const uint4 *>(act_hi + row * kActLd + c8), l = *reinterpret_cast<const uint4 *>(act_lo + row * kActLd + c8);
                *reinterpret_cast<uint4 *>(a.sw_hi + o) = h;
                *reinterpret_cast<uint4 *>(a.sw_lo + o) = l;
                if (a.sw_sums) {   // the sums split_sums_kernel would form, in its order; four consecutive lanes hold one sub-block of a row
                    float sum = 0.0f;
#pragma unroll
                    for (int pp = 0; pp < 4; pp++) {
                        const h2 hp = as_h2(dword_of(h, pp)), lp = as_h2(dword_of(l, pp));
                        sum += __builtin_fmaf((float)lp.x, kUnscale, (float)hp.x) + __builtin_fmaf((float)lp.y, kUnscale, (float)hp.y);
                    }
                    store_subblock_sum(a.sw_sums, (size_t)m, units_n, (unit0 + c8) >> 3, sum);
                }
            } else {
                for (int e = 0; e < 8 && unit0 + c8 + e < units_n; e++) {
                    a.sw_hi[o + e] = act_hi[row * kActLd + c8 + e];
                    a.sw_lo[o + e] = act_lo[row * kActLd + c8 + e];
                }
            }
        }
        __syncthreads();   // the next output tile's prologue writes the same LDS
        if (SK && sk_unit < sk_unit_end) continue;
        return;
    }
    const bool split = gridDim.y > 1;
    float *out = split ? a.partial + (size_t)blockIdx.y * a.M * a.N : a.y;
#pragma unroll
    for (int i = 0; i < RB; i++)
#pragma unroll
        for (int j = 0; j < CB; j++) {
            const int n = n0 + 32 * CB * wn + 32 * j + bn;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int m = m0 + (wm * RB + i) * 32 + 8 * (r >> 2) + 4 * kg + (r & 3);
                if (m < a.M && n < a.N) {
                    const size_t o = (size_t)m * a.N + n;
                    out[o] = (!split && a.residual) ? a.residual[o] + tot[i][j][r] : tot[i][j][r];
                }
            }
        }
    if (SK && sk_unit < sk_unit_end) continue;
    return;
  }
}

// y = (residual +) sum over splits of partial, in split order
__global__ void split_gemm_reduce_kernel(const float *partial, int splits, size_t count, const float *residual, float *y) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= count) return;
    float s = partial[i];
    for (int k = 1; k < splits; k++) s += partial[(size_t)k * count + i];
    y[i] = residual ? residual[i] + s : s;
}

// ---- producers of split rows -------------------------------------------------------------------------------------------------
// Eight fp32 values -> hi and lo groups; returns their sum (of hi + lo / 2048)
__device__ __forceinline__ float split_eight(const float (&c)[8], uint4 &hi, uint4 &lo) {
    u32 h[4], l[4];
    float s = 0.0f;
#pragma unroll
    for (int p = 0; p < 4; p++) {
        // pairs (c0, c2), (c1, c3), (c4, c6), (c5, c7): the planes' order inside fours
        const int ia = 4 * (p >> 1) + (p & 1), ib = ia + 2;
        const _Float16 ha = (_Float16)c[ia], hb = (_Float16)c[ib];
        const _Float16 la = (_Float16)__fmul_rn(__fsub_rn(c[ia], (float)ha), kScale), lb = (_Float16)__fmul_rn(__fsub_rn(c[ib], (float)hb), kScale);
        h[p] = (u32)__builtin_bit_cast(uint16_t, ha) | ((u32)__builtin_bit_cast(uint16_t, hb) << 16);
        l[p] = (u32)__builtin_bit_cast(uint16_t, la) | ((u32)__builtin_bit_cast(uint16_t, lb) << 16);
        s += __builtin_fmaf((float)la, kUnscale, (float)ha) + __builtin_fmaf((float)lb, kUnscale, (float)hb);
    }
    hi = make_uint4(h[0], h[1], h[2], h[3]);
    lo = make_uint4(l[0], l[1], l[2], l[3]);
    return s;
}
// The sum S of a sub-block (held by the first of each four lanes after the quad reduction) as the pair the GEMM's extra MFMA reads:
// sums[(row, super-block)][j] = fp16(S), [8 + j] = fp16((S - fp16(S)) * 2048).
__device__ __forceinline__ void store_subblock_sum(uint16_t *sums, size_t row, int cols, int group, float s) {
    s += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, s), 0xB1, 0xF, 0xF, false));
    s += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, s), 0x4E, 0xF, 0xF, false));
    if ((group & 3) == 0) {
        const int sub = group >> 2;   // sub-block of 32 columns
        uint16_t *p = sums + (row * (size_t)(cols / 256) + (sub >> 3)) * 16 + (sub & 7);
        const _Float16 h = (_Float16)s;
        p[0] = __builtin_bit_cast(uint16_t, h);
        p[8] = __builtin_bit_cast(uint16_t, (_Float16)__fmul_rn(__fsub_rn(s, (float)h), kScale));
    }
}

// rows of fp32 values -> split rows; optional RMSNorm ((x * inv) * w, RealModelInferenceEngine.swift:6724-6743) and optional sum of
// split-K partial planes (+ residual) first, in which case the sums are also written to y.  One workgroup of 256 threads per row;
// cols % 256 == 0 and cols <= 8192 with the norm (the row is held in registers), any multiple of 256 without.
struct SplitRowsArgs {
    const float *x;          // [splits][rows][cols]
    int splits;
    size_t plane;
    const float *residual;   // optional
    float *y;                // optional: the summed rows
    const float *norm_w;     // optional
    float eps;
    int cols;
    uint16_t *hi, *lo, *sums;
};
template <bool NORM>
__global__ __launch_bounds__(256) void split_rows_kernel(SplitRowsArgs a) {
    __shared__ float red[4];
    const int m = blockIdx.x, tid = threadIdx.x;
    const int groups = a.cols / 8;   // groups of eight columns; consecutive threads take consecutive groups
    constexpr int KV = NORM ? 4 : 1; // groups per thread held in registers with the norm
    const size_t row = (size_t)m * a.cols;
    auto load_group = [&](int g, float (&c)[8]) {
        const float4 *p = reinterpret_cast<const float4 *>(a.x + row + (size_t)g * 8);
        float4 v0 = p[0], v1 = p[1];
        for (int sp = 1; sp < a.splits; sp++) {
            const float4 *q = reinterpret_cast<const float4 *>(a.x + (size_t)sp * a.plane + row + (size_t)g * 8);
            const float4 t0 = q[0], t1 = q[1];
            v0.x += t0.x; v0.y += t0.y; v0.z += t0.z; v0.w += t0.w; v1.x += t1.x; v1.y += t1.y; v1.z += t1.z; v1.w += t1.w;
        }
        if (a.residual) {
            const float4 *q = reinterpret_cast<const float4 *>(a.residual + row + (size_t)g * 8);
            const float4 t0 = q[0], t1 = q[1];
            v0.x = t0.x + v0.x; v0.y = t0.y + v0.y; v0.z = t0.z + v0.z; v0.w = t0.w + v0.w;
            v1.x = t1.x + v1.x; v1.y = t1.y + v1.y; v1.z = t1.z + v1.z; v1.w = t1.w + v1.w;
        }
        if (a.y) {
            float4 *o = reinterpret_cast<float4 *>(a.y + row + (size_t)g * 8);
            o[0] = v0; o[1] = v1;
        }
        c[0] = v0.x; c[1] = v0.y; c[2] = v0.z; c[3] = v0.w; c[4] = v1.x; c[5] = v1.y; c[6] = v1.z; c[7] = v1.w;
    };
    auto emit = [&](int g, const float (&c)[8]) {
        uint4 hi, lo;
        const float s = split_eight(c, hi, lo);
        reinterpret_cast<uint4 *>(a.hi + row)[g] = hi;
        reinterpret_cast<uint4 *>(a.lo + row)[g] = lo;
        store_subblock_sum(a.sums, (size_t)m, a.cols, g, s);
    };
    if constexpr (NORM) {
        float c[KV][8];
        float ss = 0.0f;
#pragma unroll
        for (int k = 0; k < KV; k++) {
            const int g = tid + k * 256;
            if (g < groups) load_group(g, c[k]);
            else
#pragma unroll
                for (int e = 0; e < 8; e++) c[k][e] = 0.0f;
#pragma unroll
            for (int e = 0; e < 8; e++) ss += c[k][e] * c[k][e];
        }
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) ss += __shfl_xor(ss, off);
        if ((tid & 63) == 0) red[tid >> 6] = ss;
        __syncthreads();
        const float inv = 1.0f / sqrtf(((red[0] + red[1]) + (red[2] + red[3])) / (float)a.cols + a.eps);
#pragma unroll
        for (int k = 0; k < KV; k++) {
            const int g = tid + k * 256;   // whole quads of threads are in or out together: groups is a multiple of four
            if (g < groups) {
                const float4 *wp = reinterpret_cast<const float4 *>(a.norm_w + (size_t)g * 8);
                const float4 w0 = wp[0], w1 = wp[1];
                const float w[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
                float n[8];
#pragma unroll
                for (int e = 0; e < 8; e++) n[e] = __fmul_rn(__fmul_rn(c[k][e], inv), w[e]);
                emit(g, n);
            }
        }
    } else {
        for (int g = tid; g < groups; g += 256) {
            float c[8];
            load_group(g, c);
            emit(g, c);
        }
    }
}

// sums of rows that exist as hi / lo planes already (the SiLU(gate) * up epilogue writes those)
__global__ __launch_bounds__(256) void split_sums_kernel(const uint16_t *hi, const uint16_t *lo, int cols, uint16_t *sums) {
    const int m = blockIdx.x;
    const size_t row = (size_t)m * cols;
    for (int g = threadIdx.x; g < cols / 8; g += 256) {
        const uint4 h = reinterpret_cast<const uint4 *>(hi + row)[g], l = reinterpret_cast<const uint4 *>(lo + row)[g];
        float s = 0.0f;
#pragma unroll
        for (int p = 0; p < 4; p++) {
            const h2 hp = as_h2(dword_of(h, p)), lp = as_h2(dword_of(l, p));
            s += __builtin_fmaf((float)lp.x, kUnscale, (float)hp.x) + __builtin_fmaf((float)lp.y, kUnscale, (float)hp.y);
        }
        store_subblock_sum(sums, (size_t)m, cols, g, s);
    }
}

}  // namespace

// 1 (default): shared K ranges where they apply; 0: never; 2: as 1, but a finishing workgroup does not wait for its successor's
// totals and always computes the rest of its output tile itself (the path a wait that runs out takes; for tests).
// Initial value from ESPRESSO_HIP_SPLIT_GEMM_SHARED_K.
static int g_shared_k_mode = -1;
static int shared_k_mode() {
    if (g_shared_k_mode < 0) { const char *e = getenv("ESPRESSO_HIP_SPLIT_GEMM_SHARED_K"); g_shared_k_mode = e ? atoi(e) : 1; }
    return g_shared_k_mode;
}
// One pool per device for the process's lifetime (uncached device memory is never given back once a kernel has read it).
hipError_t gemm_split_shared_k_pool(GemmSplitSharedK *out) {
    static std::atomic<void *> pools[64];
    int device = 0;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess) return e;
    const size_t partial_floats = (size_t)kStreamKMaxWorkgroups * 128 * kThreads, bytes = partial_floats * 4 + kStreamKFlags * 4;
    void *p = pools[device & 63].load(std::memory_order_acquire);
    if (!p) {
        static std::mutex m;
        std::lock_guard<std::mutex> lock(m);
        p = pools[device & 63].load(std::memory_order_acquire);
        if (!p) {
            e = hipExtMallocWithFlags(&p, bytes, hipDeviceMallocUncached);
            if (e != hipSuccess) return e;
            e = hipMemset(p, 0, bytes);
            if (e == hipSuccess) e = hipDeviceSynchronize();
            if (e != hipSuccess) return e;   // (the allocation stays: see above)
            pools[device & 63].store(p, std::memory_order_release);
        }
    }
    out->partial = static_cast<float *>(p);
    out->partial_floats = partial_floats;
    out->flags = reinterpret_cast<unsigned *>(static_cast<float *>(p) + partial_floats);
    return hipSuccess;
}
void gemm_split_set_shared_k(int mode) { g_shared_k_mode = mode < 0 ? 1 : mode; }

bool gemm_split_supported(const DeviceMatrix &w) { return w.format == FMT_Q4_K && w.qs && w.cols % 256 == 0 && w.qs_row_bytes % 16 == 0; }

hipError_t launch_gemm_split(const GemmSplitParams &p, hipStream_t stream) {
    const DeviceMatrix &w = p.w;
    if (!gemm_split_supported(w) || !p.x.hi || !p.x.lo || !p.x.sums || p.rows <= 0 || w.rows <= 0) return hipErrorInvalidValue;
    if ((uint64_t)p.rows * (uint64_t)w.cols >= (1ull << 32)) return hipErrorInvalidValue;   // the kernel's activation offsets are 32-bit
    const bool swiglu = p.swiglu.hi != nullptr;
    if (swiglu ? (!p.swiglu.lo || w.rows % 2 != 0 || p.residual) : !p.y) return hipErrorInvalidValue;
    SplitGemmArgs a{};
    a.qs = w.qs; a.qs_row_bytes = w.qs_row_bytes; a.N = w.rows; a.K = w.cols; a.M = p.rows;
    a.xh = p.x.hi; a.xl = p.x.lo; a.xs = p.x.sums; a.y = p.y; a.residual = p.residual; a.partial = p.workspace;
    a.tiled = w.tiled;
    // weights in registers (workgroups of 128 x 256) wherever the matrix keeps the tiled copy; ESPRESSO_HIP_SPLIT_GEMM_LDS_WEIGHTS=1
    // restores the kernel that stages them
    static const bool lds_weights = [] { const char *e = getenv("ESPRESSO_HIP_SPLIT_GEMM_LDS_WEIGHTS"); return e && atoi(e) != 0; }();
    const bool regb = w.tiled != nullptr && !lds_weights;
    const int nt = regb ? NT2 : NT;
    const int tiles = a.K / KT, blocks = ((a.N + nt - 1) / nt) * ((a.M + MT - 1) / MT);
    // split K until the grid fills the chip (one workgroup per compute unit is resident), whole super-blocks per split
    int splits = 1;
    if (!swiglu && p.workspace) {
        const int target = 256;
        splits = blocks >= target ? 1 : (target + blocks - 1) / blocks;
        if (splits > tiles / 16) splits = tiles / 16;
        if (splits < 1) splits = 1;
        while (splits > 1 && (size_t)splits * a.M * a.N > p.workspace_floats) splits--;
    }
    a.tiles_per_split = ((tiles + splits - 1) / splits + 3) & ~3;
    splits = (tiles + a.tiles_per_split - 1) / a.tiles_per_split;
    if (swiglu) { a.sw_hi = p.swiglu.hi; a.sw_lo = p.swiglu.lo; a.sw_sums = regb && (a.N / 2) % 32 == 0 ? p.swiglu.sums : nullptr; }
    static std::atomic<uint64_t> raised{0};
    int device = 0;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess) return e;
    const uint64_t bit = 1ull << (device & 63);
    static const int regb_shape = [] { const char *e = getenv("ESPRESSO_HIP_SPLIT_GEMM_SHAPE"); return e ? atoi(e) : 4; }();
    // Shared K ranges for the SiLU(gate) * up launch when its output tiles do not fill whole rounds of the chip: one workgroup
    // per compute unit, each with the same number of K tiles.
    const int shared_k = shared_k_mode();
    int shared_k_workgroups = 0;
    if (swiglu && regb && regb_shape == 4 && shared_k != 0 && p.shared_k && p.shared_k->flags && p.shared_k->partial) {
        static std::atomic<int> cus[64];
        int n = cus[device & 63].load(std::memory_order_relaxed);
        if (n == 0) {
            e = hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, device);
            if (e != hipSuccess) return e;
            cus[device & 63].store(n, std::memory_order_relaxed);
        }
        const long long units = (long long)blocks * tiles;
        if (n > 0 && n <= kStreamKMaxWorkgroups && blocks > n && blocks % n != 0 && units % n == 0 && (units / n) % 4 == 0 && units / n >= tiles &&
            (size_t)n * 128 * kThreads <= p.shared_k->partial_floats) {
            shared_k_workgroups = n;
            a.sk_units = (int)(units / n); a.sk_tiles_n = (a.N + nt - 1) / nt;
            a.sk_flags = p.shared_k->flags; a.sk_partial = p.shared_k->partial;
            a.sk_spin_limit = shared_k == 2 ? 0u : kStreamKSpinLimit;
        }
    }
    if (!(raised.load(std::memory_order_acquire) & bit)) {
        e = hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_q4k_split_kernel<2>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsBytes);
        if (e == hipSuccess)
            e = hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_q4k_split_regb_kernel<2, 4>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsBytesRegB);
        if (e == hipSuccess)
            e = hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_q4k_split_regb_kernel<4, 2>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsBytesRegB);
        if (e == hipSuccess)
            e = hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_q4k_split_regb_kernel<4, 2, true>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsBytesRegB);
        if (e != hipSuccess) return e;
        raised.fetch_or(bit, std::memory_order_release);
    }
    dim3 grid((a.N + nt - 1) / nt, splits, (a.M + MT - 1) / MT);
    if (shared_k_workgroups) hipLaunchKernelGGL((gemm_q4k_split_regb_kernel<4, 2, true>), dim3(shared_k_workgroups), dim3(kThreads), kLdsBytesRegB, stream, a);
    else if (regb && regb_shape == 4) hipLaunchKernelGGL((gemm_q4k_split_regb_kernel<4, 2>), grid, dim3(kThreads), kLdsBytesRegB, stream, a);
    else if (regb) hipLaunchKernelGGL((gemm_q4k_split_regb_kernel<2, 4>), grid, dim3(kThreads), kLdsBytesRegB, stream, a);
    else hipLaunchKernelGGL(gemm_q4k_split_kernel<2>, grid, dim3(kThreads), kLdsBytes, stream, a);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    if (swiglu) {
        if (a.sw_sums) return hipSuccess;   // the GEMM's epilogue wrote the sums
        hipLaunchKernelGGL(split_sums_kernel, dim3(a.M), dim3(256), 0, stream, p.swiglu.hi, p.swiglu.lo, a.N / 2, p.swiglu.sums);
        return hipGetLastError();
    }
    if (splits > 1) {
        if (p.deferred_splits) { *p.deferred_splits = splits; return hipSuccess; }
        const size_t count = (size_t)a.M * a.N;
        hipLaunchKernelGGL(split_gemm_reduce_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, stream, a.partial, splits, count, a.residual, a.y);
        return hipGetLastError();
    }
    if (p.deferred_splits) *p.deferred_splits = 1;
    return hipSuccess;
}

hipError_t launch_split_rows(const SplitRowsParams &p, hipStream_t stream) {
    if (!p.x || !p.out.hi || !p.out.lo || !p.out.sums || p.rows <= 0 || p.cols <= 0 || p.cols % 256 != 0 || p.splits < 1) return hipErrorInvalidValue;
    if (p.norm_w && p.cols > 8192) return hipErrorInvalidValue;
    SplitRowsArgs a{p.x, p.splits, p.plane, p.residual, p.y, p.norm_w, p.norm_eps, p.cols, p.out.hi, p.out.lo, p.out.sums};
    if (p.norm_w) hipLaunchKernelGGL(split_rows_kernel<true>, dim3(p.rows), dim3(256), 0, stream, a);
    else hipLaunchKernelGGL(split_rows_kernel<false>, dim3(p.rows), dim3(256), 0, stream, a);
    return hipGetLastError();
}

}  // namespace esp
