/*
 * espresso_oracle.h — CPU restatement of the reference's quantized-decode path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library links, loads or
 * calls this code.  Only tests/, __graft_entry__.smoke() and the cpu_baseline
 * leg of bench.py may use it, and only as the checker / reported baseline.
 *
 * Every function names the reference lines it restates (paths relative to the
 * reference checkout).  The GGUF block arithmetic is NOT in the reference: it
 * lives in the un-vendored package "Edgerunner" (Package.swift:24, a local
 * path dependency with no pinned version) and is restated here from the
 * public ggml block definitions (block_q8_0, block_q4_0, block_q4_K and
 * dequantize_row_* / quantize_row_*_ref in ggml-quants.c).
 *
 * Pinning status (what checks each function against something other than
 * itself is listed in tests/test_oracle_*.py):
 *   - fp16 conversion, BLOBFILE, rmsNorm, per-head rmsNorm, RoPE, attention,
 *     SiLU, argmax, tiny-llama forward, two-token loop: pinned by the
 *     reference's own known-answer tests and closed forms.
 *   - GGUF block dequantization (Q8_0, Q4_0, Q4_K): the reference holds no
 *     vector for it ("parity unpinned" by the reference).  Pinned instead by an
 *     independent numpy restatement, exhaustive (sc, m, nibble) enumeration
 *     and the quantize->dequantize error bound of each format.
 *
 * Arithmetic is IEEE binary32 with no fused multiply-add (build with
 * -ffp-contract=off) so results do not depend on the host's vector ISA.
 */
#ifndef ESPRESSO_ORACLE_H
#define ESPRESSO_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- fp16 <-> fp32 (IEEE round-to-nearest-even, subnormals kept) ---------
 * Swift `Float16(x)` / `Float(Float16)` as used by roundFloat16Vector
 * (RealModelInferenceEngine.swift:6720-6722), BlobWeightLoader.swift:52 and
 * WeightBlob.swift:35,60. */
uint16_t orc_f32_to_f16(float value);
float orc_f16_to_f32(uint16_t bits);
void orc_round_f16_vector(float *values, size_t count);

/* ---- GGUF block codecs (public ggml definitions) ------------------------ */
#define ORC_Q8_0_BLOCK_BYTES 34
#define ORC_Q4_0_BLOCK_BYTES 18
#define ORC_Q4_K_BLOCK_BYTES 144
#define ORC_QK 32
#define ORC_QK_K 256

enum { ORC_FMT_F32 = 0, ORC_FMT_F16 = 1, ORC_FMT_Q4_0 = 2, ORC_FMT_Q8_0 = 8, ORC_FMT_Q4_K = 12 };

/* element count must be a multiple of the block length */
void orc_dequant_q8_0(const uint8_t *blocks, size_t elements, float *out);
void orc_dequant_q4_0(const uint8_t *blocks, size_t elements, float *out);
void orc_dequant_q4_k(const uint8_t *blocks, size_t elements, float *out);
void orc_quantize_q8_0(const float *x, size_t elements, uint8_t *blocks);
void orc_quantize_q4_0(const float *x, size_t elements, uint8_t *blocks);
void orc_quantize_q4_k(const float *x, size_t elements, uint8_t *blocks);
/* format-dispatching forms; return 0 on success, -1 on an unknown format */
size_t orc_format_bytes(int format, size_t elements);
int orc_dequantize(int format, const uint8_t *blocks, size_t elements, float *out);
int orc_quantize(int format, const float *x, size_t elements, uint8_t *blocks);
/* Q4_K 6-bit scale/min unpack for sub-block j (0..7) of a 12-byte table */
void orc_q4_k_scale_min(int j, const uint8_t *scales12, uint8_t *sc, uint8_t *m);

/* ---- math helpers of the CPU-exact llama path ---------------------------
 * RealModelInferenceEngine.swift:6648-6827 */
void orc_rmsnorm(const float *x, const float *weight, float eps, int n, float *out);
void orc_per_head_rmsnorm(float *values, const float *weights, int heads, int head_dim, float eps);
void orc_matvec(const float *matrix, int rows, int cols, const float *x, float *y);
/* Threads used by orc_matvec on large matrices (default 1; results do not depend on it). */
void orc_set_threads(int threads);
int orc_get_threads(void);
void orc_rope_half_split(float *values, int heads, int head_dim, int position, float theta);
void orc_attention_decode(const float *q, const float *k_cache, const float *v_cache, int heads,
                          int kv_heads, int head_dim, int visible, int cache_stride, float *context);
float orc_silu_tanh(float value);
/* RealModelInferenceEngine.swift:8182-8275; block_max_norms may be NULL (computed on the fly) */
int orc_partitioned_argmax(const float *classifier, const float *input, int vocab, int dim,
                           int block_size, int *blocks_pruned);
int orc_naive_argmax(const float *values, int count);

/* ---- BLOBFILE (WeightBlob.swift:6-38, BlobWeightLoader.swift:25-90) ----- */
size_t orc_blob_bytes(size_t elements);
void orc_blob_build(const float *weights, size_t elements, uint8_t *out);
/* returns element count, or a negative BlobWeightLoaderError ordinal:
 * -1 truncatedHeader, -2 invalidMagic, -3 invalidDataOffset,
 * -4 truncatedPayload, -5 invalidPayloadSize */
long orc_blob_parse(const uint8_t *data, size_t bytes, float *out, size_t out_capacity);

/* ---- stateful runtime (CPUExactLlamaRuntime, :548-850) ------------------ */
typedef struct {
    int n_layer, n_head, n_kv_head, d_model, head_dim, hidden_dim, vocab, max_seq;
    float norm_eps, rope_theta;
    int eos_token;                 /* -1 = none */
    /* rounding switches */
    int round_intermediates_fp16;  /* the reference's own flag (:289-301, :682-684) */
    int gemv_inputs_fp16;          /* 1: round every GEMV input vector to fp16 (what the GPU path did before it split them);
                                      other non-zero values: a mask of the inputs that are rounded (see gemv_input) */
    int kv_fp16;                   /* round k (post-RoPE) and v to fp16 at cache write */
} orc_llama_config;

typedef struct orc_llama_runtime orc_llama_runtime;

/* Weight slots.  Matrices are row-major [rows, cols] fp32, already dequantized. */
enum {
    ORC_W_TOKEN_EMBEDDING = 0, ORC_W_FINAL_NORM = 1, ORC_W_LM_HEAD = 2,
    ORC_W_RMS_ATT = 10, ORC_W_WQ = 11, ORC_W_WK = 12, ORC_W_WV = 13, ORC_W_WO = 14,
    ORC_W_RMS_FFN = 15, ORC_W_W1 = 16, ORC_W_W2 = 17, ORC_W_W3 = 18,
    ORC_W_Q_NORM = 19, ORC_W_K_NORM = 20
};

orc_llama_runtime *orc_llama_create(const orc_llama_config *config);
void orc_llama_free(orc_llama_runtime *rt);
/* copies `count` floats; layer ignored for the three top-level slots. 0 on success. */
int orc_llama_set_weight(orc_llama_runtime *rt, int layer, int slot, const float *data, size_t count);
/* A matrix slot (embedding, head, wq..w3) from GGUF blocks of `format`, `count` elements. */
int orc_llama_set_weight_blocks(orc_llama_runtime *rt, int layer, int slot, int format, const uint8_t *blocks, size_t count);
void orc_llama_set_gemv_inputs_fp16(orc_llama_runtime *rt, int enabled);
void orc_llama_reset(orc_llama_runtime *rt);
/* 0 ok; -1 empty prompt; -2 position beyond max_seq; -3 token outside vocab */
int orc_llama_prefill(orc_llama_runtime *rt, const uint32_t *tokens, int count);
int orc_llama_advance(orc_llama_runtime *rt, uint32_t token);
uint32_t orc_llama_select_greedy(orc_llama_runtime *rt);
int orc_llama_visible(const orc_llama_runtime *rt);
void orc_llama_set_visible(orc_llama_runtime *rt, int visible); /* rollback without a copy */
const float *orc_llama_last_hidden(const orc_llama_runtime *rt);
/* full-vocab logits of the current last hidden state (naive GEMV, fp32) */
void orc_llama_logits(orc_llama_runtime *rt, float *logits);
/* top-1 minus top-2 logit of the current state */
float orc_llama_top2_margin(orc_llama_runtime *rt);

typedef struct orc_llama_checkpoint orc_llama_checkpoint;
orc_llama_checkpoint *orc_llama_capture(const orc_llama_runtime *rt);   /* :647-654 */
void orc_llama_rollback(orc_llama_runtime *rt, const orc_llama_checkpoint *ck); /* :656-661 */
void orc_llama_checkpoint_free(orc_llama_checkpoint *ck);

/* generateIncrementalExactCPULlama, temperature 0 (:6192-6431).
 * Returns the number of generated tokens or a negative error as above. */
int orc_llama_generate(orc_llama_runtime *rt, const uint32_t *prompt, int prompt_count,
                       int max_tokens, uint32_t *out_tokens, float *out_min_margin);

/* generateIncrementalExactTwoTokenDraftLlama (:6014-6190). */
typedef struct {
    int passes;
    int committed_total;
    int accepted_total;
} orc_two_token_stats;
int orc_llama_generate_two_token(orc_llama_runtime *full, orc_llama_runtime *draft,
                                 const uint32_t *prompt, int prompt_count, int max_tokens,
                                 uint32_t *out_tokens, orc_two_token_stats *stats);

/* ---- temperature sampling -----------------------------------------------------------------
 * sampleToken (RealModelInferenceEngine.swift:8036-8068): temperature <= 0 -> first maximum; otherwise
 * weights exp(double((logit - max) / T)) (the division in float, the exponential in double), total in index
 * order, threshold = unit * total, first index at which the running remainder drops to <= 0; a total that is
 * not finite or not positive falls back to the first maximum.  `unit` in [0, 1) stands for Swift's
 * Double.random(in: 0..<total) / total. */
int orc_sample_token(const float *logits, int count, float temperature, double unit);

/* ---- INT4 classifier --------------------------------------------------------------------
 * TensorBufferINT4(quantizing:rows:cols:) (Sources/ANETypes/TensorBufferINT4.swift:53-135): per-row
 * min-max 4-bit, scale = (max - min) / 15 (1.0 when max - min < 1e-10), bias = min,
 * q = clamp(roundf((v - min) / scale), 0, 15), two nibbles per byte with the HIGH nibble first,
 * (cols + 1) / 2 bytes per row, trailing low nibble zero. */
void orc_int4_quantize(const float *src, int rows, int cols, uint8_t *packed, float *scales, float *biases);
/* INT4Classifier.rowDotProduct / int4Matvec / int4MatvecArgmax (Sources/Espresso/INT4Classifier.swift:40-160):
 * logit = scale * sum(nibble * x) + bias * sum(x); argmax with strict '>' (lowest index wins ties). */
float orc_int4_input_sum(const float *input, int dim);
void orc_int4_matvec(const uint8_t *packed, const float *scales, const float *biases, const float *input,
                     int vocab, int dim, float *out);
int orc_int4_argmax(const uint8_t *packed, const float *scales, const float *biases, const float *input,
                    int vocab, int dim);

#ifdef __cplusplus
}
#endif
#endif
