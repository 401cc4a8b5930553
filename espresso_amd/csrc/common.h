// Shared declarations for the HIP side of the library (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace esp {

// GGUF tensor type ids (public ggml numbering) for the formats this library runs.
enum Format : int { FMT_F32 = 0, FMT_F16 = 1, FMT_Q4_0 = 2, FMT_Q8_0 = 8, FMT_Q4_K = 12 };

inline bool format_supported(int f) {
    return f == FMT_F32 || f == FMT_F16 || f == FMT_Q4_0 || f == FMT_Q8_0 || f == FMT_Q4_K;
}
// elements per quantisation block and bytes per block in the GGUF file layout
inline int format_block_elems(int f) { return f == FMT_Q4_K ? 256 : (f == FMT_Q8_0 || f == FMT_Q4_0) ? 32 : 1; }
inline int format_block_bytes(int f) {
    switch (f) {
    case FMT_F32: return 4;
    case FMT_F16: return 2;
    case FMT_Q4_0: return 18;
    case FMT_Q8_0: return 34;
    case FMT_Q4_K: return 144;
    default: return 0;
    }
}
inline size_t format_bytes(int f, size_t elems) { return elems / format_block_elems(f) * format_block_bytes(f); }

// A weight matrix resident in HBM, laid out for the GEMV kernels.
//   Q4_K : `qs` holds the GGUF 144-byte super-blocks unchanged, row-major (16-byte aligned rows).
//   Q8_0 : split planes — `qs` = int8 quants [rows][cols], `scales` = fp16 d [rows][cols/32].
//   Q4_0 : split planes — `qs` = packed nibbles [rows][cols/2] (16 bytes per block, GGUF nibble
//          order), `scales` = fp16 d [rows][cols/32].
//   F16  : `qs` = fp16 values [rows][cols].
// The split planes carry exactly the bits of the GGUF blocks (34 / 18 bytes per 32 weights); they
// exist because 34- and 18-byte blocks cannot be read with aligned 128-bit loads.
struct DeviceMatrix {
    int format = 0;
    int rows = 0, cols = 0;
    uint8_t *qs = nullptr;
    uint16_t *scales = nullptr;
    // Q4_K and Q4_0 matrices of 4096 or 14336 columns: a second copy tiled by (block of sixteen rows, 256 or 512 columns) for
    // the matrix-core GEMV (layouts: kernels/gemv.hip); rows padded to a multiple of sixteen with zero blocks.  Null when not built.
    uint8_t *tiled = nullptr;
    size_t tiled_bytes() const {
        if (!tiled) return 0;
        if (format == FMT_Q8_0) return (size_t)((rows + 15) / 16) * (cols / 256) * 4352;
        if (format == FMT_F16) return (size_t)((rows + 15) / 16) * (cols / 256) * 8192;
        return format == FMT_Q4_K ? (size_t)((rows + 15) / 16) * (cols / 256) * 2304 : (size_t)((rows + 15) / 16) * (cols / 512) * 4608;
    }
    size_t qs_row_bytes = 0;
    size_t bytes() const {  // algorithmic bytes: what one GEMV must read
        return (size_t)rows * qs_row_bytes + (scales ? (size_t)rows * (cols / 32) * 2 : 0);
    }
    size_t resident_bytes() const { return bytes() + tiled_bytes(); }   // what the matrix holds in HBM
};

// GEMV epilogues (what happens to the fp32 row sums)
enum Epilogue : int {
    EPI_STORE_F32 = 0,     // y[b][r] = acc
    EPI_ADD_RESIDUAL = 1,  // y[b][r] = residual[b][r] + acc
    EPI_SWIGLU_F16 = 2,    // rows interleaved (gate_i, up_i): out_f16[b][i] = fp16(silu(gate_i) * up_i)
    EPI_QKV_ROPE = 3,      // fused q|k|v rows: RoPE, q -> q_out, k/v -> KV caches
    EPI_ARGMAX = 4,        // output head: no logits are stored; every workgroup leaves (largest row sum, lowest row index holding it)
};

// Destination of the fused q|k|v GEMV (EPI_QKV_ROPE).  The matrix rows are q and k as RoPE pairs
// (j, j + head_dim/2) side by side, then v in natural order.
struct QkvEpilogue {
    int n_head = 0, n_kv_head = 0, head_dim = 0, max_seq = 0;
    const float *rope_cos = nullptr, *rope_sin = nullptr;  // [max_seq][head_dim/2]
    const int *pos = nullptr, *seq = nullptr;              // [batch]
    float *q_out = nullptr;                                // [batch][attnDim]
    void *k_cache = nullptr, *v_cache = nullptr;           // this layer: [seq][max_seq][kvDim]
    size_t cache_seq_stride = 0;
    int kv_f16 = 0;
};

struct GemvParams {
    DeviceMatrix w;
    const uint16_t *x = nullptr;  // fp16 activations [batch][cols]
    // fused RMSNorm: when norm_x is set the activations are fp16((norm_x * inv_rms) * norm_w), computed
    // while staging, and `x` is ignored.  norm_x: fp32 [batch][cols]; norm_w: fp32 [cols].
    const float *norm_x = nullptr, *norm_w = nullptr;
    float norm_eps = 0.0f;
    // attention context merged while staging: when merge_partials is set (see gemv_merges_attention_partials)
    // the activations are the per-head partial states of launch_attention_partials, merged and rounded to
    // fp16; `x` and `norm_x` are ignored.  [batch][cols / head_dim][kAttentionHeadSplits][head_dim + 4] floats.
    const float *merge_partials = nullptr;
    int merge_head_dim = 0;
    float *y = nullptr;           // fp32 out [batch][rows]
    const float *residual = nullptr;
    uint16_t *out_f16 = nullptr;  // EPI_SWIGLU_F16: [batch][rows/2]
    QkvEpilogue qkv;              // EPI_QKV_ROPE
    // EPI_ARGMAX: per-workgroup partial results, [batch][*argmax_blocks] (value, index) pairs; `argmax_capacity` slots per
    // batch row are available and the launch fails if the kernel's grid is larger.  *argmax_blocks receives the grid size.
    float *argmax_value = nullptr;
    int *argmax_index = nullptr;
    int argmax_capacity = 0;
    int *argmax_blocks = nullptr;
    // split activations (gemv_splits_activations says where): `x` holds two fp16 rows per activation row, hi = fp16(v) and
    // lo = fp16((v - hi) * 2048), [2 * batch][cols]; with norm_x or merge_partials the staging makes both from the fp32 values.
    // The products then carry the activations to about 22 bits instead of 11.  split_out: EPI_SWIGLU_F16 writes such row pairs,
    // out_f16 = [2 * batch][rows / 2].
    bool split_x = false, split_out = false;
    // measurement only: device buffer of four wall-clock stamps (100 MHz) per wavefront of the launch, room for stamp_capacity
    // wavefronts (matrix-core Q4_K kernel, fp16 activations given, one or two rows)
    unsigned long long *stamps = nullptr;
    int stamp_capacity = 0;
    int batch = 1;
    int epilogue = EPI_STORE_F32;
    // optional (batch <= 2): events that take the kernel's own start and end times
    hipEvent_t start_event = nullptr, stop_event = nullptr;
};

// y[rows][w.rows] = x[rows][w.cols] * dequant(w)^T (+ residual) for more than two rows, on the matrix cores.
struct GemmParams {
    DeviceMatrix w;
    const uint16_t *x = nullptr;      // fp16 activations [rows][cols]
    float *y = nullptr;               // fp32 out [rows][w.rows]
    const float *residual = nullptr;  // optional [rows][w.rows], may alias y
    int rows = 0;
    float *workspace = nullptr;       // split-K partial sums for short row counts (optional)
    size_t workspace_floats = 0;
    // optional fp16 [rows][w.rows / 2]: silu(y[2i]) * y[2i + 1] for a matrix whose rows are (gate, up) pairs; y is then
    // scratch (written only when the SwiGLU could not be done in the GEMM's own epilogue)
    uint16_t *swiglu_out = nullptr;
    // optional: when the GEMM runs split-K, leave the partial sums [splits][rows][w.rows] in `workspace` for the caller's
    // next kernel to add (launch_rmsnorm_reduce) and report the split count here; 1 = y is complete
    int *deferred_splits = nullptr;
};

// Rows of activations split for the matrix cores: v = hi + lo / 2048 with hi = fp16(v), lo = fp16((v - hi) * 2048), both
// [rows][cols] fp16 with the middle two of every four columns exchanged (c0, c2, c1, c3: the order in which the GEMM unpacks nibbles), and per (row, super-block of 256 columns) sixteen fp16 `sums`: the sums S_j of the row over the eight
// sub-blocks of 32 columns as fp16(S_j), j = 0..7, then fp16((S_j - fp16(S_j)) * 2048).
struct SplitRowsView {
    uint16_t *hi = nullptr, *lo = nullptr, *sums = nullptr;
};

// y[rows][w.rows] = x * dequant(w)^T (+ residual) for a Q4_K matrix with exact weights and split activations
// (kernels/gemm_split.hip): prompt blocks of models whose logits must stay within 2e-2 of the fp32 CPU path over many layers.
struct GemmSplitParams {
    DeviceMatrix w;
    SplitRowsView x;                  // read only
    float *y = nullptr;               // fp32 out [rows][w.rows] (unused with `swiglu`)
    const float *residual = nullptr;  // optional, may alias y
    int rows = 0;
    float *workspace = nullptr;       // split-K partial sums when the grid would not fill the chip (optional)
    size_t workspace_floats = 0;
    SplitRowsView swiglu;             // optional: silu(y[2i]) * y[2i + 1] as split rows [rows][w.rows / 2] instead of y
    int *deferred_splits = nullptr;   // optional: leave split-K partial sums [splits][rows][w.rows] in workspace, report the count
    // optional, with `swiglu`: the device's hand-over pool (gemm_split_shared_k_pool).  Given it, a launch whose output tiles do not
    // fill whole rounds of the chip runs one workgroup per compute unit with equal shares of K tiles; workgroups that share an output
    // tile hand partial totals over through the pool.  One launch at a time per device.
    const struct GemmSplitSharedK *shared_k = nullptr;
};
struct GemmSplitSharedK {
    unsigned *flags = nullptr;
    float *partial = nullptr;
    size_t partial_floats = 0;
};
hipError_t gemm_split_shared_k_pool(GemmSplitSharedK *out);   // allocated on first use, kept until the process ends; not during a capture
void gemm_split_set_shared_k(int mode);
void attention_prompt_set_key_sets(int sets);   // prompt attention: 0 = sets of wavefronts by block size (default), 1 or 2 = always that many   // 0 off, 1 on (default), 2 on with the finisher never waiting (tests)
bool gemm_split_supported(const DeviceMatrix &w);
hipError_t launch_gemm_split(const GemmSplitParams &p, hipStream_t stream);

// fp32 rows -> split rows, optionally summing split-K partial planes (+ residual, sums also to y) and applying RMSNorm first.
struct SplitRowsParams {
    const float *x = nullptr;         // [splits][rows][cols], planes `plane` floats apart
    int splits = 1;
    size_t plane = 0;
    const float *residual = nullptr;
    float *y = nullptr;
    const float *norm_w = nullptr;    // RMSNorm weights (cols <= 8192) or null
    float norm_eps = 0.0f;
    int rows = 0, cols = 0;           // cols % 256 == 0
    SplitRowsView out;
};
hipError_t launch_split_rows(const SplitRowsParams &p, hipStream_t stream);

// kernels/gemv.hip
hipError_t launch_gemv(const GemvParams &p, hipStream_t stream);
bool gemv_splits_activations(const DeviceMatrix &w, int batch);
bool gemv_wants_tiled_copy(int format, int cols);
unsigned gemv_tuning_epoch();   // bumped by every gemv_set_tuning call
// Slices of the prefix per query head that launch_attention_partials writes and the merging GEMV reads.
#ifndef ESP_ATTENTION_HEAD_SPLITS
#define ESP_ATTENTION_HEAD_SPLITS 4
#endif
constexpr int kAttentionHeadSplits = ESP_ATTENTION_HEAD_SPLITS;
// Kernel-selection switches (also read from the environment at first use): "q4k_mfma" (ESPRESSO_HIP_Q4K_MFMA) and
// "q4k_mfma_ks" (ESPRESSO_HIP_Q4K_MFMA_KS).  False for an unknown key.
bool gemv_set_tuning(const char *key, int value);
// True when launch_gemv handles `batch` rows without re-reading the weights per pair of rows (always for one or two rows).
bool gemv_takes_rows(const DeviceMatrix &w, int batch);
// True when launch_gemv has the EPI_ARGMAX epilogue for this matrix (every format; Q4_K rows of 8192 or more columns, which
// several wavefronts share, keep the separate argmax launches).
bool gemv_supports_argmax(const DeviceMatrix &w);
// True when launch_gemv can take its input as attention partial states (batch <= 2, head size 64 or 128).
bool gemv_merges_attention_partials(const DeviceMatrix &w, int batch, int head_dim);
// kernels/gemm.hip
hipError_t launch_gemm(const GemmParams &p, hipStream_t stream);
// kernels/dequant.hip — GGUF-layout blocks -> fp32, bit-exact to the block definitions
hipError_t launch_dequant(int format, const uint8_t *blocks, size_t elems, float *out, hipStream_t stream);
// GGUF-layout blocks -> DeviceMatrix planes (device to device)
hipError_t launch_repack(int format, const uint8_t *blocks, int rows, int cols, const DeviceMatrix &dst,
                         hipStream_t stream);
// Q4_K super-blocks, row-major [rows][cols / 256][144 bytes] -> the tiled copy ((rows + 15) / 16 * cols / 256 tiles of 2304 bytes)
hipError_t launch_q4k_tile(const uint8_t *blocks, int rows, int cols, uint8_t *tiled, hipStream_t stream);
// Q4_0 planes -> the tiled copy ((rows + 15) / 16 * cols / 512 tiles of 4608 bytes)
hipError_t launch_q40_tile(const uint8_t *qs, const uint16_t *scales, int rows, int cols, uint8_t *tiled, hipStream_t stream);
// Q8_0 planes -> the tiled copy ((rows + 15) / 16 * cols / 256 tiles of 4352 bytes)
hipError_t launch_q80_tile(const uint8_t *qs, const uint16_t *scales, int rows, int cols, uint8_t *tiled, hipStream_t stream);
// fp16 weights -> the tiled copy ((rows + 15) / 16 * cols / 256 tiles of 8192 bytes)
hipError_t launch_f16_tile(const uint8_t *weights, int rows, int cols, uint8_t *tiled, hipStream_t stream);
// DeviceMatrix -> fp32 [rows][cols] (used to check the planes carry the same bits)
hipError_t launch_dequant_matrix(const DeviceMatrix &m, float *out, hipStream_t stream);

// kernels/int4_classifier.hip — logits of the per-row 4-bit output head (fp32 input, fp32 logits)
hipError_t launch_int4_matvec(const uint8_t *packed, const float *scales, const float *biases, const float *input, int vocab, int dim,
                              float *logits, hipStream_t stream);

// kernels/probe.hip — plain streaming read of `bytes` (a multiple of 16)
hipError_t launch_stream_read(const void *src, size_t bytes, unsigned *sink, hipStream_t stream);
// the same with the persistent Q4_K GEMV's grid and loads: `grid` workgroups of four wavefronts over pairs of rows of `pair_bytes`
hipError_t launch_stream_read_pairs(const void *src, size_t bytes, int pair_bytes, int grid, int wavefronts, unsigned *sink, hipStream_t stream);

// kernels/synth.hip — seeded N(0, std) weights quantised into GGUF-layout blocks on the GPU
hipError_t launch_synth(int format, uint64_t seed, float std_dev, size_t elems, uint8_t *out, hipStream_t stream);

}  // namespace esp
