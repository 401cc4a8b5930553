/*
 * espresso_hip.h — C ABI of the MI355X (gfx950) implementation of Espresso's quantized
 * transformer decode path.  One header, plain pointers and sizes, no C++ or framework types:
 * it is meant to sit behind a Swift module map exactly like the reference's ANEInterop target
 * (Package.swift:27-41, Sources/ANEInterop/include/ane_interop.h).
 *
 * File references in comments are paths inside the reference checkout.
 *
 * Threading: one library-wide HIP stream; calls are synchronous (results valid on return) unless
 * a comment says otherwise.  A handle must not be used from two threads at once (the reference has
 * the same rule, Sources/ANERuntime/ANEKernel.swift:611-616).
 *
 * Errors: int-returning functions return 0 on success and a negative ESP_ERR_* code otherwise;
 * pointer-returning functions return NULL; esp_last_error() then holds a message for the calling
 * thread.  No function falls back to a CPU implementation: without a usable GPU every compute entry
 * point fails with ESP_ERR_NO_DEVICE.
 */
#ifndef ESPRESSO_HIP_H
#define ESPRESSO_HIP_H

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ESP_OK 0
#define ESP_ERR_INVALID_ARGUMENT (-1)
#define ESP_ERR_NO_DEVICE (-2)
#define ESP_ERR_OUT_OF_MEMORY (-3)
#define ESP_ERR_LAUNCH_FAILED (-4)
#define ESP_ERR_UNSUPPORTED (-5)
#define ESP_ERR_FORCED_FAILURE (-6)
#define ESP_ERR_OUT_OF_RANGE (-7)
#define ESP_ERR_IO (-8)

/* GGUF tensor type ids (public ggml numbering) of the weight formats the kernels consume. */
#define ESP_FORMAT_F32 0
#define ESP_FORMAT_F16 1
#define ESP_FORMAT_Q4_0 2
#define ESP_FORMAT_Q8_0 8
#define ESP_FORMAT_Q4_K 12

/* ---- library -------------------------------------------------------------------------- */

/* Selects GPU 0 and creates the library stream.  Idempotent.  (ane_interop_init, ane_interop.h:15) */
int esp_init(void);
/* Message of the calling thread's most recent failure ("" if none). */
const char *esp_last_error(void);
/* Name, compute-unit count and HBM bytes of the GPU in use. */
int esp_device_info(char *name, size_t name_capacity, int *compute_units, size_t *hbm_bytes);
/* Bytes of one tensor in the GGUF block layout; 0 for an unknown format or a ragged element count. */
size_t esp_format_bytes(int format, size_t elements);

/* ---- GGUF block dequantisation --------------------------------------------------------- *
 * Replaces Edgerunner's DequantDispatcher.dequantize(tensor:device:) -> [Float]
 * (Sources/EspressoGGUF/GGUFModelLoader.swift:359-372).  Host pointers in and out; the blocks are
 * decoded on the GPU.  Bit-exact to the ggml block definitions. */
int esp_dequantize(int format, const void *blocks, size_t elements, float *out);

/* ---- weight matrices resident in HBM ---------------------------------------------------- *
 * A row-major [rows, cols] linear-layer weight (wq [attnDim,d], w1 [hidden,d], lm_head [vocab,d] ...;
 * Sources/ModelSupport/BlobWeightLoader.swift:25-60 documents the orientation).  The bytes are copied
 * in, as ane_interop_compile copies its weight blobs (ane_interop.h:24-28). */
typedef struct ESPMatrix ESPMatrix;
ESPMatrix *esp_matrix_create(int format, const void *gguf_blocks, int rows, int cols);
void esp_matrix_free(ESPMatrix *matrix);
/* Bytes one GEMV must read from HBM for this matrix (packed weights incl. scales). */
size_t esp_matrix_bytes(const ESPMatrix *matrix);
/* Bytes the matrix holds in HBM: the packed weights plus, for the Q4_K / Q4_0 widths the matrix-core GEMVs are built for (Q4_K:
 * 1024, 2048, 3072, 4096, 8192, 14336 columns; Q4_0: 4096, 14336), a second copy tiled for those kernels (about as large again).
 * ESPRESSO_HIP_TILED_COPIES=0 in the environment keeps matrices at their packed size; the dot-product GEMVs then run everywhere. */
size_t esp_matrix_resident_bytes(const ESPMatrix *matrix);
/* Decode the resident copy back to fp32 [rows*cols] (checks the HBM layout carries the same bits). */
int esp_matrix_dequantize(const ESPMatrix *matrix, float *out);

/* ---- dequant-fused GEMV ----------------------------------------------------------------- *
 * y[b][r] = (residual ? residual[b][r] : 0) + sum_c dequant(W)[r][c] * x[b][c]
 * Replaces multiplyRowMajorMatrix (Sources/RealModelInference/RealModelInferenceEngine.swift:6674-6718).
 * x: fp16 bit patterns [batch][cols]; y, residual: fp32 [batch][rows]; host pointers.
 * batch 1 and 2 run the wave-per-row-pair GEMV; batch > 2 (prompt blocks, batched verify; any count) runs
 * the dequant-fused MFMA kernel, which rounds each dequantised weight to fp16 once (the GEMV does not). */
int esp_gemv(const ESPMatrix *matrix, const uint16_t *x_f16, int batch, float *y, const float *residual);
/* The same product for fp32 activations, as the reference's CPU path feeds them (multiplyRowMajorMatrix,
 * RealModelInferenceEngine.swift:6674-6718, called per prompt token at :6365-6375): y[r][n] = (residual +) sum_c x[r][c] *
 * dequant(W)[n][c] for a block of `rows` rows, x fp32 [rows][cols], y and residual fp32 [rows][matrix rows]; host pointers.
 * Q4_K matrices with a multiple of 256 columns.  The matrix cores take fp16 operands: each activation goes in as two fp16 numbers
 * (hi = fp16(v), lo = fp16((v - hi) * 2048)) and each weight as the exact integer sc * q of its sub-block, with d, dmin and the
 * sub-block minimums applied in fp32, so no operand is rounded. */
int esp_matmul_f32(const ESPMatrix *matrix, const float *x, int rows, float *y, const float *residual);
/* esp_gemv for callers that cannot allocate device memory (tight serving loops, harnesses that forbid hipMalloc, code that runs
 * between the captures of its own HIP graphs).  No counterpart in the reference.  x, y and residual are DEVICE pointers
 * (fp16 [batch][cols], fp32 [batch][rows], fp32 [batch][rows] or NULL); the call makes no hipMalloc / hipFree: the
 * split-K partial sums of the matrix-core kernels (batch > 2) live in a fixed 16 MiB array inside the library, one
 * copy per GPU, held until the process ends.  Limits: batch 1..64 and, for batch > 2, 2 * batch * rows <= 4 Mi floats
 * (whether or not the kernel ends up splitting K); beyond them the call fails with ESP_ERR_OUT_OF_RANGE.  It runs on the
 * library's stream and returns when the result is there, like esp_gemv, so it cannot itself sit inside a caller's stream
 * capture.  esp_gemv sizes its own workspace the same, so the two return the same bits.  All calls on a GPU share that
 * GPU's array: calls that overlap on one GPU race. */
int esp_gemv_device_noalloc(const ESPMatrix *matrix, const uint16_t *x_f16_device, int batch, float *y_device,
                            const float *residual_device_or_null);

/* ---- INT4 output head ---------------------------------------------------------------------------- *
 * INT4Classifier (Sources/Espresso/INT4Classifier.swift:40-160) over TensorBufferINT4
 * (Sources/ANETypes/TensorBufferINT4.swift:53-135).  create quantises fp32 [rows][cols] per row exactly as
 * TensorBufferINT4(quantizing:rows:cols:) does (scale = (max-min)/15, bias = min, high nibble first) and
 * uploads the result; export returns those bytes ((cols+1)/2 per row), scales and biases for inspection.
 * matvec_argmax = int4Matvec (all logits, optional) and int4MatvecArgmax (lowest index wins ties) on the GPU:
 * logit = scale * sum(nibble * x) + bias * sum(x), fp32 input. */
typedef struct ESPInt4Classifier ESPInt4Classifier;
ESPInt4Classifier *esp_int4_classifier_create(const float *weights_f32, int rows, int cols);
void esp_int4_classifier_free(ESPInt4Classifier *classifier);
int esp_int4_classifier_export(const ESPInt4Classifier *classifier, uint8_t *packed, float *scales, float *biases);
int esp_int4_classifier_matvec_argmax(ESPInt4Classifier *classifier, const float *input, float *logits_or_null, int *index_or_null);

/* ---- llama decoder state resident on the GPU -------------------------------------------- *
 * Replaces CPUExactLlamaRuntime (Sources/RealModelInference/RealModelInferenceEngine.swift:548-850):
 * create = init(config:weightDirURL:) :562-614, reset :616-635, prefill :637-645, advance :672-680,
 * select_greedy_token :663-670 + :825-849.  captureCheckpoint/rollback (:647-661) copy every KV
 * cache in the reference; here a rollback is esp_llama_set_visible_token_count with a smaller count,
 * because columns beyond the visible length are never read. */
typedef struct ESPLlamaRuntime ESPLlamaRuntime;

/* MultiModelConfig (Sources/ModelSupport/MultiModelConfig.swift:3-55) plus the two storage choices
 * this implementation adds. */
typedef struct ESPLlamaConfig {
    int32_t n_layer, n_head, n_kv_head, d_model, head_dim, hidden_dim, vocab, max_seq;
    float norm_eps, rope_theta;
    int32_t eos_token;      /* -1: none */
    int32_t kv_format;      /* ESP_FORMAT_F32 (the reference's caches) or ESP_FORMAT_F16 */
    int32_t max_sequences;  /* independent KV caches (1..16) */
} ESPLlamaConfig;

/* Weight slots, named after LayerWeightPaths (Sources/ModelSupport/LayerWeightPaths.swift:22-84):
 * embeddings/token.bin, rms_final.bin, lm_head.bin and layers/<i>/{rms_att,wq,wk,wv,wo,rms_ffn,w1,w2,w3,
 * q_norm,k_norm}.bin (w1 = gate, w3 = up, w2 = down). */
#define ESP_SLOT_TOKEN_EMBEDDING 0
#define ESP_SLOT_FINAL_NORM 1
#define ESP_SLOT_LM_HEAD 2
#define ESP_SLOT_RMS_ATT 10
#define ESP_SLOT_WQ 11
#define ESP_SLOT_WK 12
#define ESP_SLOT_WV 13
#define ESP_SLOT_WO 14
#define ESP_SLOT_RMS_FFN 15
#define ESP_SLOT_W1 16
#define ESP_SLOT_W2 17
#define ESP_SLOT_W3 18
#define ESP_SLOT_Q_NORM 19
#define ESP_SLOT_K_NORM 20

ESPLlamaRuntime *esp_llama_create(const ESPLlamaConfig *config);
void esp_llama_free(ESPLlamaRuntime *runtime);
/* Copies `bytes` of one tensor.  Projections and lm_head: GGUF block layout of `format`, row-major
 * [rows, cols]; norm vectors and the embedding table: f32 or f16.  `layer` is ignored for the three
 * top-level slots.  q_norm/k_norm are optional and used only when both are given
 * (RealModelInferenceEngine.swift:6585-6607). */
int esp_llama_set_weight(ESPLlamaRuntime *runtime, int layer, int slot, int format, const void *data, size_t bytes);
/* Lays the weights out in HBM; required once, before any of the calls below. */
int esp_llama_finalize(ESPLlamaRuntime *runtime);
/* Packed weight bytes one decoded token reads (all projections plus lm_head). */
size_t esp_llama_weight_bytes(const ESPLlamaRuntime *runtime);
/* Bytes the weights hold in HBM (packed matrices, their tiled copies, the embedding table): see esp_matrix_resident_bytes. */
size_t esp_llama_resident_weight_bytes(const ESPLlamaRuntime *runtime);
int esp_llama_reset(ESPLlamaRuntime *runtime);
int esp_llama_prefill(ESPLlamaRuntime *runtime, int sequence, const uint32_t *tokens, int count);
int esp_llama_advance(ESPLlamaRuntime *runtime, int sequence, uint32_t token);
int esp_llama_select_greedy_token(ESPLlamaRuntime *runtime, int sequence, uint32_t *token);
/* visibleTokenCount; returns -1 for a sequence out of range. */
int esp_llama_visible_token_count(const ESPLlamaRuntime *runtime, int sequence);
int esp_llama_set_visible_token_count(ESPLlamaRuntime *runtime, int sequence, int count);
/* lastHidden [d_model] and the full-vocabulary logits of the current state [vocab], fp32. */
int esp_llama_read_last_hidden(ESPLlamaRuntime *runtime, int sequence, float *out);
int esp_llama_read_logits(ESPLlamaRuntime *runtime, int sequence, float *out);

typedef struct ESPGenerationStats {
    int32_t generated;
    double prefill_ms, decode_ms, first_token_latency_ms, tokens_per_second;
} ESPGenerationStats;

/* generateIncrementalExactCPULlama at temperature 0 (RealModelInferenceEngine.swift:6192-6431).
 * Writes at most max_tokens ids; *out_count receives how many.  token_latencies_ms may be NULL,
 * else it receives one latency per generated token (GenerationResult.tokenLatenciesMs, :17-55). */
int esp_llama_generate(ESPLlamaRuntime *runtime, const uint32_t *prompt, int prompt_count, int max_tokens,
                       uint32_t *out_tokens, int *out_count, ESPGenerationStats *stats, double *token_latencies_ms);

typedef struct ESPTwoTokenStats {
    /* one pass = one batched verify of [current token, proposed token] by the target model; committed
     * is 1 or 2 per pass and accepted 0 or 1 (ExactTwoTokenPassMetrics, GenerationHarness.swift:104-131) */
    int32_t passes, committed_total, accepted_total;
    /* the reference CPU loop's accounting of the same stream (committedExactTokensPerPass /
     * acceptedFutureTokensPerPass, RealModelInferenceEngine.swift:6109-6175); accepted is -1 when
     * reference_accounting was 0 */
    int32_t reference_passes, reference_committed_total, reference_accepted_total;
} ESPTwoTokenStats;

/* generateIncrementalExactTwoTokenDraftLlama (RealModelInferenceEngine.swift:6014-6190) with the
 * target model verifying both tokens of a pass in one batched step.  The emitted stream equals
 * esp_llama_generate on `target`. */
int esp_llama_generate_two_token(ESPLlamaRuntime *target, ESPLlamaRuntime *draft, const uint32_t *prompt,
                                 int prompt_count, int max_tokens, int reference_accounting,
                                 uint32_t *out_tokens, int *out_count, ESPGenerationStats *stats,
                                 ESPTwoTokenStats *two_token_stats);

/* `n_seq` independent sequences (sequence s uses KV cache s; create the runtimes with max_sequences >= n_seq,
 * at most 16) decoded greedily in lock step for a fixed budget; steps of more than two rows run on the matrix
 * cores.  With a draft runtime the exact two-token loop (RealModelInferenceEngine.swift:6014-6190) runs over
 * all sequences at once: one target pass verifies (current, proposed) of every sequence.  Each sequence's stream
 * is the same with and without the draft.  out_tokens: [n_seq][max_tokens]; the reference's nearest notion of a
 * batch is lane/stream packing (ane_interop.h:270-289).  two_token_stats sums over sequences. */
int esp_llama_generate_batch(ESPLlamaRuntime *target, ESPLlamaRuntime *draft_or_null, const uint32_t *const *prompts,
                             const int *prompt_counts, int n_seq, int max_tokens, uint32_t *out_tokens, int *out_counts,
                             ESPTwoTokenStats *two_token_stats, double *decode_ms);

/* Continues greedy decoding of `sequence` from its current state for `steps` tokens: select, then
 * advance, per token (the body of the loop at RealModelInferenceEngine.swift:6365-6413 without the
 * EOS test).  Fails with ESP_ERR_OUT_OF_RANGE if the context would overflow. */
int esp_llama_continue_greedy(ESPLlamaRuntime *runtime, int sequence, int steps, uint32_t *out_tokens);
/* esp_llama_continue_greedy replays captured HIP graphs (head, argmax, trunk per token; eight tokens per graph while eight
 * are left, then one) and synchronises once at the end; 0 switches it to one kernel launch at a time with a host read of
 * every token (same results).  Default: enabled. */
int esp_llama_set_graph_replay(ESPLlamaRuntime *runtime, int enabled);
/* Prompts of 32 tokens or more are prefilled in blocks of up to 512 rows with every projection as one
 * dequant-fused MFMA GEMM (fp16 weights after dequantisation, fp32 accumulation), instead of the
 * reference's token-by-token walk (RealModelInferenceEngine.swift:6365-6375).  enabled = 0 restores the
 * per-token path, whose arithmetic keeps the dequantised weights in fp32.  Default: enabled. */
int esp_llama_set_matrix_prefill(ESPLlamaRuntime *runtime, int enabled);
/* Decode steps of one or two rows run attention (decodeContextFromCaches, :6774-6823) as one launch that leaves
 * per-head partial softmax states, and the wo GEMV merges them while it stages its input, where the shapes allow
 * (head size 128, Q4_K wo of 2048 or 4096 columns).  enabled = 0 restores the split kernel plus the merge kernel
 * everywhere.  Returns 1 when the merged form is in use after the call, 0 when not, negative on error. */
int esp_llama_set_merged_attention(ESPLlamaRuntime *runtime, int enabled);
/* The reference's CPU path feeds fp32 activations into every matrix product (RealModelInferenceEngine.swift:6674-6697,
 * :6221-6347).  The matrix cores take fp16, so decode steps of one or two rows hand every layer GEMV that has the form (Q4_K
 * matrices of 4096 or 14336 columns) each activation as two fp16 numbers, hi = fp16(v) and lo = fp16((v - hi) * 2048), and
 * add the two products: about 22 bits of the activation instead of 11, which is what keeps a 32-layer model's logits inside
 * 2e-2 of the CPU path.  enabled = 0 rounds activations to fp16 once (faster by the cost of staging the second row).
 * Default: enabled. */
int esp_llama_set_split_activations(ESPLlamaRuntime *runtime, int enabled);

/* ---- seeded synthetic weights ------------------------------------------------------------- *
 * Fills `out_blocks` (host memory, esp_format_bytes(format, elements) bytes) with N(0, std_dev) draws
 * quantised into GGUF-layout blocks; element i of stream `seed` is the same value on every call.
 * elements must be a multiple of 256.  Formats: F16, Q8_0, Q4_0, Q4_K. */
int esp_synth_weights(int format, uint64_t seed, float std_dev, size_t elements, void *out_blocks);

/* ---- weight files ------------------------------------------------------------------------------- *
 * BLOBFILE: 128-byte header + little-endian fp16 payload (Sources/ANETypes/WeightBlob.swift:6-38,
 * Sources/ModelSupport/BlobWeightLoader.swift:25-90).  Pure host code; no GPU needed. */
size_t esp_weight_blob_bytes(size_t element_count);
/* WeightBlob.build(from:rows:cols:): fp32 -> fp16 round-to-nearest-even.  `out` holds esp_weight_blob_bytes(count). */
int esp_weight_blob_build(const float *weights, size_t element_count, uint8_t *out);
/* BlobWeightLoader.load(from:): returns the element count, or -(1 + BlobWeightLoaderError ordinal):
 * -1 truncatedHeader, -2 invalidMagic, -3 invalidDataOffset, -4 truncatedPayload, -5 invalidPayloadSize, -6 file unreadable.
 * `out` may be NULL to query the count. */
long esp_blob_weight_load(const char *path, float *out, size_t capacity);
/* LayerWeightPaths.forLayer(_:config:blobDir:) for one ESP_SLOT_* of a llama layer
 * (Sources/ModelSupport/LayerWeightPaths.swift:56-84).  Returns the length written, or ESP_ERR_*. */
int esp_layer_weight_path(int layer, const char *blob_dir, int slot, char *out, size_t capacity);

/* MultiModelConfig (Sources/ModelSupport/MultiModelConfig.swift:3-55). */
typedef struct ESPModelConfig {
    char name[64];
    int32_t n_layer, n_head, n_kv_head, d_model, head_dim, hidden_dim, vocab, max_seq;
    float norm_eps, rope_theta;
    int32_t eos_token;     /* -1: none */
    int32_t architecture;  /* 0 gpt2, 1 llama */
} ESPModelConfig;
/* metadata.json as GGUFModelLoader writes it (GGUFModelLoader.swift:203-222) and the engine validates it
 * (RealModelInferenceEngine.swift:7658-7694). */
int esp_model_config_load_metadata(const char *metadata_json_path, ESPModelConfig *out);
int esp_model_config_write_metadata(const ESPModelConfig *config, const char *metadata_json_path);

/* ModelRegistry (Sources/ModelSupport/ModelRegistry.swift): esp_model_registry_count() named configurations in name
 * order; esp_model_registry_config(name, &out) = ModelRegistry.config(named:), ESP_ERR_INVALID_ARGUMENT when unknown. */
int esp_model_registry_count(void);
int esp_model_registry_at(int index, ESPModelConfig *out);
int esp_model_registry_config(const char *name, ESPModelConfig *out);
/* ClassifierStrategy.select(for:hasExactFloat32LMHead:) (Sources/RealModelInference/ClassifierStrategy.swift:46-69):
 * returns 0 ane, 1 cpuPartitionedFP32, 2 cpuFP16Tiled and writes exactHeadBackendLabel (:31-40) when out_label is given.
 * All three return the first maximum of the same logits; the GPU head does too. */
int esp_classifier_strategy_select(const ESPModelConfig *config, int has_exact_float32_lm_head, char *out_label, size_t label_bytes);

/* ---- GGUF front door ---------------------------------------------------------------------------- *
 * GGUFModelLoader.prepare(ggufURL:options:) -> PreparedModel (GGUFModelLoader.swift:273-405): parses
 * the GGUF container, maps its metadata to a MultiModelConfig (:297-326) and writes a weight directory:
 * fp16 BLOBFILEs for norms and the embedding, exact float32 sidecars for F32/BF16 tensors, and for each
 * quantised projection a packed sidecar "<stem>.<q8_0|q4_0|q4_k>.bin" holding the GGUF blocks unchanged,
 * which esp_engine_build uploads as they are.  emit_dequantized_blobs != 0 additionally writes the fp16
 * BLOBFILE of every quantised projection (the artefact the reference's own engine reads).
 * qk_layout: -1 by architecture, 0 keep rows as stored, 1 undo the GGUF llama Q/K row interleave. */
typedef struct ESPPrepareOptions {
    int32_t emit_dequantized_blobs;
    int32_t emit_float32_sidecars;
    int32_t qk_layout;
} ESPPrepareOptions;
int esp_gguf_prepare(const char *gguf_path, const char *output_dir, const ESPPrepareOptions *options_or_null,
                     ESPModelConfig *out_config, int *out_tensor_count);

/* The prepared-artifact cache of GGUFModelLoader.prepare(ggufURL:options:) (GGUFModelLoader.swift:38-127, :273-296,
 * :408-453, :472-566).  Options come from environment pairs as PrepareOptions.environment(_:) reads them
 * (ESPRESSO_GGUF_FORCE_FRESH_PREPARE, ESPRESSO_GGUF_PREPARE_CACHE, ESPRESSO_GGUF_PREPARE_CACHE_ROOT,
 * ESPRESSO_GGUF_SIDECAR_POLICY, ESPRESSO_GGUF_SELECTED_SIDECARS); the converter switches among the pairs enter the
 * cache key (:595-605). */
enum { ESP_SIDECAR_AUTOMATIC = 0, ESP_SIDECAR_NONE = 1, ESP_SIDECAR_ESSENTIAL = 2, ESP_SIDECAR_SELECTED = 3, ESP_SIDECAR_FULL = 4 };
typedef struct ESPPrepareCacheOptions {
    int32_t cache_enabled;            /* PrepareOptions.artifactCacheMode */
    int32_t sidecar_mode;             /* ESP_SIDECAR_* */
    char cache_root[1024];            /* "" = the default root */
    char selected_sidecars[2048];     /* sorted tensor names, comma separated (sidecar_mode == ESP_SIDECAR_SELECTED) */
} ESPPrepareCacheOptions;
int esp_gguf_prepare_options_from_environment(const char *const *env_keys, const char *const *env_values, int env_count,
                                              ESPPrepareCacheOptions *out);
/* 64 hexadecimal digits + NUL into out_key (artifactCacheKey, :424-447). */
int esp_gguf_artifact_cache_key(const char *gguf_path, const ESPPrepareCacheOptions *options, const char *const *env_keys,
                                const char *const *env_values, int env_count, char *out_key, size_t out_key_bytes);
/* prepare(ggufURL:options:): the cached directory when one matches, else a conversion into <cache root>/<key> (cache
 * on) or a fresh temporary directory (cache off).  out_weight_dir receives the directory. */
int esp_gguf_prepare_cached(const char *gguf_path, const ESPPrepareCacheOptions *options, const ESPPrepareOptions *convert_or_null,
                            const char *const *env_keys, const char *const *env_values, int env_count, ESPModelConfig *out_config,
                            int *out_tensor_count, char *out_weight_dir, size_t out_weight_dir_bytes);
/* GGUFModelLoader.cleanup(weightDir:) (:408-412): removes the directory unless it is a managed cache entry. */
int esp_gguf_cleanup(const char *weight_dir);
int esp_gguf_default_cache_root(char *out, size_t out_bytes);

/* ---- engine -------------------------------------------------------------------------------------- *
 * RealModelInferenceEngine.build(config:weightDir:tokenizerDir:) (RealModelInferenceEngine.swift:1377):
 * loads the weight directory into HBM (per tensor: packed sidecar, else float32 sidecar, else fp16
 * BLOBFILE).  Environment entries are passed as parallel key/value arrays, as the reference's functions
 * take an `environment:` dictionary.  Recognised: ESPRESSO_BUNDLE_DRAFT_KIND / _HORIZON / _ARTIFACT_REF
 * (:5324-5390), ESPRESSO_HIP_KV_CACHE=f16. */
typedef struct ESPEngine ESPEngine;
ESPEngine *esp_engine_build(const ESPModelConfig *config, const char *weight_dir, const char *tokenizer_dir_or_null,
                            const char *const *env_keys, const char *const *env_values, int env_count);
void esp_engine_free(ESPEngine *engine);

/* GenerationResult (:17-55) without text. */
typedef struct ESPGenerationResult {
    int32_t token_count;
    double tokens_per_second, compile_time_ms, first_token_latency_ms;
    int32_t has_two_token_stats;
    double committed_exact_tokens_per_pass, accepted_future_tokens_per_pass;
    char exact_head_backend[48];
} ESPGenerationResult;
/* generate(prompt:maxTokens:temperature:) in its token-id form (:1405-1493): greedy decode, or the exact
 * two-token draft loop when the environment names a draft.  out_tokens holds max_tokens ids. */
int esp_engine_generate(ESPEngine *engine, const uint32_t *prompt_tokens, int prompt_count, int max_tokens, float temperature,
                        const char *const *env_keys, const char *const *env_values, int env_count,
                        uint32_t *out_tokens, ESPGenerationResult *result);
/* The runtime inside the engine (owned by the engine). */
ESPLlamaRuntime *esp_engine_runtime(ESPEngine *engine);

/* generate(prompt:maxTokens:temperature:) on text (:1405-1437): the prompt is encoded by the tokenizer found in the
 * tokenizer directory given to esp_engine_build (encodePrompt, :5404-5418), generation runs as in
 * esp_engine_generate, and the text of prompt + generated tokens is written to out_text (UTF-8, not terminated;
 * *out_text_bytes = its full length, of which at most text_capacity bytes are written).  Fails with
 * ESP_ERR_INVALID_ARGUMENT when the engine has no tokenizer or the prompt encodes to nothing. */
int esp_engine_generate_text(ESPEngine *engine, const char *prompt_utf8, size_t prompt_bytes, int max_tokens, float temperature,
                             const char *const *env_keys, const char *const *env_values, int env_count,
                             uint32_t *out_tokens, char *out_text, size_t text_capacity, size_t *out_text_bytes,
                             ESPGenerationResult *result);

/* RunGGUF.main(ggufPath:tokenizerDir:prompt:maxTokens:) (Sources/EspressoGGUF/RunGGUF.swift:68-113, the body of the
 * runner's `<gguf> <tokenizer-dir> <prompt> [max]` form, Sources/EspressoGGUFRunner/main.swift:43-57): prepare with
 * PrepareOptions.environment, build the engine with the tokenizer directory, generate greedily from the prompt text,
 * then GGUFModelLoader.cleanup unless ESPRESSO_GGUF_KEEP_WEIGHT_DIR=1 (a managed cache entry is kept either way).
 * The environment pairs stand for the process environment the reference reads.  Text output as in
 * esp_engine_generate_text; out_tokens holds max_tokens ids.  The verify-qwen form needs the Qwen3 model file and its
 * golden tokens (RunGGUF.swift:115-214) and is not part of this library. */
typedef struct ESPRunGGUFInfo {
    ESPModelConfig config;
    int32_t tensor_count;
    int32_t kept_weight_dir;      /* 1: the directory still exists after the call */
    double prepare_ms, build_ms;
    char weight_dir[1024];
} ESPRunGGUFInfo;
int esp_run_gguf(const char *gguf_path, const char *tokenizer_dir, const char *prompt_utf8, size_t prompt_bytes, int max_tokens,
                 const char *const *env_keys, const char *const *env_values, int env_count, uint32_t *out_tokens, char *out_text,
                 size_t text_capacity, size_t *out_text_bytes, ESPGenerationResult *result, ESPRunGGUFInfo *info);

/* ---- tokenizers ----------------------------------------------------------------------------------- *
 * The Tokenizer protocol (Sources/ModelSupport/Tokenizer.swift:1-5: encode, decode, vocabSize) and its two
 * implementations, on the host.
 *   esp_tokenizer_load_sentencepiece    SentencePieceTokenizer(modelURL:)  SentencePieceTokenizer.swift:19-66
 *   esp_tokenizer_load_gpt2             GPT2BPETokenizer(vocabURL:mergesURL:)  GPT2BPETokenizer.swift:30-45
 *   esp_tokenizer_load_tokenizer_json   GPT2BPETokenizer(tokenizerJSONURL:)    GPT2BPETokenizer.swift:47-77
 *   esp_tokenizer_load_dir              loadTokenizer(config:tokenizerDirURL:) RealModelInferenceEngine.swift:7558-7613
 * A loader returns NULL on failure; esp_tokenizer_last_error then holds the case of
 * SentencePieceTokenizerError / GPT2BPETokenizerError (this thread's last load). */
typedef struct ESPTokenizer ESPTokenizer;
enum {
    ESP_TOK_OK = 0,
    ESP_TOK_UNREADABLE_FILE = 1,
    ESP_TOK_SP_TRUNCATED_MODEL = 10,
    ESP_TOK_SP_INVALID_MAX_TOKEN_LENGTH = 11,      /* detail = the value */
    ESP_TOK_SP_TRUNCATED_ENTRY = 12,               /* detail = entry index */
    ESP_TOK_SP_INVALID_UTF8_ENTRY = 13,            /* detail = entry index */
    ESP_TOK_SP_EMPTY_VOCABULARY = 14,
    ESP_TOK_BPE_MALFORMED_VOCABULARY = 20,
    ESP_TOK_BPE_EMPTY_VOCABULARY = 21,
    ESP_TOK_BPE_NON_CONTIGUOUS_TOKEN_IDS = 22,     /* detail = expectedCount, detail2 = actualMaxTokenID */
    ESP_TOK_BPE_MALFORMED_TOKENIZER_JSON = 23,
    ESP_TOK_BPE_UNSUPPORTED_TOKENIZER_MODEL = 24,  /* text = model type */
    ESP_TOK_BPE_INVALID_PRE_TOKENIZER_PATTERN = 25,/* text = pattern */
    ESP_TOK_MISSING_PATH = 30                      /* text = what was looked for */
};
typedef struct ESPTokenizerError {
    int32_t code;
    int64_t detail, detail2;
    char text[256];
} ESPTokenizerError;
ESPTokenizer *esp_tokenizer_load_sentencepiece(const char *model_path);
ESPTokenizer *esp_tokenizer_load_gpt2(const char *vocab_json_path, const char *merges_txt_path);
ESPTokenizer *esp_tokenizer_load_tokenizer_json(const char *tokenizer_json_path);
ESPTokenizer *esp_tokenizer_load_dir(const ESPModelConfig *config, const char *tokenizer_dir);
void esp_tokenizer_last_error(ESPTokenizerError *out);
void esp_tokenizer_free(ESPTokenizer *tokenizer);
int esp_tokenizer_vocab_size(const ESPTokenizer *tokenizer);
/* "sentencePiece" or "gpt2" (the cases of LoadedTokenizer) */
const char *esp_tokenizer_kind(const ESPTokenizer *tokenizer);
/* Returns the number of tokens of the text and writes the first `capacity` of them. */
long esp_tokenizer_encode(const ESPTokenizer *tokenizer, const char *text_utf8, size_t text_bytes, int32_t *out_tokens, size_t capacity);
/* The split GPT2BPETokenizer.encode applies before BPE (preTokenizer.matches(in:range:), GPT2BPETokenizer.swift:80-82):
 * non-overlapping matches of `pattern_utf8` (NULL = the GPT-2 default pattern, :13-14) from left to right, as byte
 * offsets [begin, end) into the text, two entries per match, the first `capacity_pairs` matches written.  Returns the
 * number of matches, or ESP_ERR_INVALID_ARGUMENT for a pattern outside the supported ICU subset. */
long esp_pretokenize(const char *pattern_utf8, const char *text_utf8, size_t text_bytes, int64_t *out_ranges, size_t capacity_pairs);
/* Returns the UTF-8 length of the decoded text and writes its first `capacity` bytes (not terminated). */
long esp_tokenizer_decode(const ESPTokenizer *tokenizer, const int32_t *tokens, size_t count, char *out_utf8, size_t capacity);

/* ---- .esp bundles ---------------------------------------------------------------------------------- *
 * The bridge from a bundle to the engine: ESPBundleArchive.open (Sources/ESPBundle/ESPBundle.swift:563-590: the
 * manifest, the ten top-level directories, the SHA-256 catalog signatures/content-hashes.json, referenced artefacts),
 * ESPManifest.parseTOML / validate / renderTOML (:219-394), ESPRuntimeResolver.selectBackend
 * (Sources/ESPRuntime/ESPRuntimeContracts.swift:77-138) and ESPRuntimeRunner.generate with environmentOverrides
 * (Sources/ESPRuntime/ESPBundledRuntime.swift:49-180): a [draft] section selects the exact two-token path, an
 * [output_head] section is passed on in the environment (the engine here always runs the dense head).
 * Both of the reference's backends ("ane-private", "cpu-safe") run the same GPU engine here.
 * Loaders return NULL / negative on failure; esp_bundle_last_error then holds the case of
 * ESPBundleValidationError or ESPRuntimeSelectionError (this thread's last call). */
typedef struct ESPBundle ESPBundle;
enum {
    ESP_BUNDLE_OK = 0, ESP_BUNDLE_EMPTY_FIELD = 1, ESP_BUNDLE_INVALID_MAX_CONTEXT = 2, ESP_BUNDLE_INVALID_CONTEXT_TARGET = 3,
    ESP_BUNDLE_INVALID_ADAPTER_SLOTS = 4, ESP_BUNDLE_MISSING_BACKENDS = 5, ESP_BUNDLE_MISSING_PROFILES = 6,
    ESP_BUNDLE_INVALID_WEIGHT_BITS = 7, ESP_BUNDLE_INVALID_ACTIVATION_BITS = 8, ESP_BUNDLE_MISSING_TOP_LEVEL_ENTRY = 9,
    ESP_BUNDLE_MISSING_MANIFEST = 10, ESP_BUNDLE_MALFORMED_LINE = 11, ESP_BUNDLE_MALFORMED_SECTION = 12,
    ESP_BUNDLE_UNSUPPORTED_VALUE = 13, ESP_BUNDLE_INVALID_OUTPUT_HEAD = 14, ESP_BUNDLE_INVALID_DRAFT = 15,
    ESP_BUNDLE_INVALID_REFERENCED_PATH = 16, ESP_BUNDLE_MISSING_REFERENCED_FILE = 17, ESP_BUNDLE_SIGNATURE_MISMATCH = 18,
    ESP_BUNDLE_UNREADABLE_FILE = 19, ESP_BUNDLE_NO_COMPATIBLE_BACKEND = 30, ESP_BUNDLE_NO_COMPATIBLE_PROFILE = 31,
    ESP_BUNDLE_REQUESTED_CONTEXT_EXCEEDS_TARGET = 32   /* detail = requested, detail2 = supported */
};
typedef struct ESPBundleError {
    int32_t code;
    int64_t detail, detail2;
    char text[256];
} ESPBundleError;
typedef struct ESPRuntimeSelectionInfo {   /* ESPRuntimeSelection (ESPRuntimeContracts.swift:43-69) */
    char backend[16];                      /* "ane-private" | "cpu-safe" */
    char profile[16];                      /* "prefill_256" | "prefill_2048" | "decode_1" | "decode_2" */
    int64_t context_target_tokens;
    int32_t has_output_head, has_draft;
    char reason[64];
} ESPRuntimeSelectionInfo;
void esp_bundle_last_error(ESPBundleError *out);
/* ESPManifest.parseTOML(text) then renderTOML(): 0 and the canonical text (its length in *out_bytes, the first
 * `capacity` bytes written), or ESP_ERR_INVALID_ARGUMENT with esp_bundle_last_error set. */
int esp_manifest_parse_toml(const char *text, size_t text_bytes, char *out_toml, size_t capacity, size_t *out_bytes);
/* ESPBundleArchive.writeSignatureCatalog for a bundle directory. */
int esp_bundle_write_signature_catalog(const char *bundle_dir);
/* ESPRuntimeBundle.open(at:) (ESPBundledRuntime.swift:17-23): archive + config from weights/metadata.json. */
ESPBundle *esp_bundle_open(const char *bundle_dir, int verify_signatures);
void esp_bundle_free(ESPBundle *bundle);
int esp_bundle_model_config(const ESPBundle *bundle, ESPModelConfig *out);
/* selectBackend; requested_context_tokens < 0 = none.  supports_ane_private mirrors ESPDeviceCapabilities. */
int esp_bundle_resolve(const ESPBundle *bundle, long requested_context_tokens, int supports_ane_private, ESPRuntimeSelectionInfo *out);
/* environmentOverrides(for:) of that selection as "KEY=VALUE\n" lines; returns the text length. */
long esp_bundle_environment_overrides(const ESPBundle *bundle, long requested_context_tokens, int supports_ane_private, char *out,
                                      size_t capacity);
/* ESPRuntimeRunner.generate(bundle:prompt:maxTokens:temperature:); outputs as esp_engine_generate_text. */
int esp_bundle_generate(const ESPBundle *bundle, const char *prompt_utf8, size_t prompt_bytes, int max_tokens, float temperature,
                        const char *const *env_keys, const char *const *env_values, int env_count, uint32_t *out_tokens,
                        char *out_text, size_t text_capacity, size_t *out_text_bytes, ESPGenerationResult *result,
                        ESPRuntimeSelectionInfo *selection);

/* sampleToken (RealModelInferenceEngine.swift:8036-8068) on the host: temperature <= 0 -> first maximum; else
 * weights exp(double((logit - max) / T)), threshold = unit * total, first index whose running remainder is <= 0.
 * `unit` in [0, 1) stands for Double.random(in: 0..<total) / total; esp_splitmix64_unit draws it from a SplitMix64
 * state (53 high bits * 2^-53) and advances the state.  esp_engine_generate with temperature > 0 reads the full
 * logits back every token and samples this way, seeded by ESPRESSO_HIP_SAMPLING_SEED (default 0x5EED5EED5EED);
 * the reference draws from the system generator, so only the distribution, not the stream, is comparable.
 * Returns the index (>= 0) or ESP_ERR_INVALID_ARGUMENT. */
int esp_sample_token(const float *logits, int count, float temperature, double unit);
double esp_splitmix64_unit(uint64_t *state);

/* ---- exact two-token harness ---------------------------------------------------------------------- *
 * ExactTwoTokenBranchPromotionPlan.make (Sources/Espresso/GenerationHarness.swift:149-180). */
typedef struct ESPPromotionPlan {
    uint32_t committed_tokens[2];
    int32_t committed_exact_token_count, accepted_future_token_count, promoted_step_count;
    uint32_t next_current_token;
} ESPPromotionPlan;
void esp_exact_two_token_promotion_plan(uint32_t current_token, uint32_t proposed_future_token, uint32_t exact_next_token,
                                        uint32_t exact_future_token, int remaining_token_budget, ESPPromotionPlan *out);

/* ExactTwoTokenPassMetrics / ExactTwoTokenPassResult (:104-147) */
typedef struct ESPPassResult {
    uint32_t committed_tokens[2];
    int32_t committed_count;
    uint32_t next_current_token;
    double proposer_latency_ms, verifier_trunk_latency_ms, verifier_logits_latency_ms, state_advance_latency_ms;
    int32_t accepted_future_token_count, committed_exact_token_count;
} ESPPassResult;
/* ExactTwoTokenGeneratingLanguageModel (:239-252) as a table of callbacks; each returns 0 on success. */
typedef struct ESPExactTwoTokenModel {
    void *context;
    int (*reset)(void *context);
    int (*prefill_selected_token)(void *context, const uint32_t *prompt_tokens, int count, uint32_t *selected);
    int (*perform_exact_two_token_pass)(void *context, uint32_t current_token, int remaining_token_budget, ESPPassResult *result);
} ESPExactTwoTokenModel;
/* ExactTwoTokenGenerationHarness.generate (:612-686): drives `model`, enforcing the pass invariants.
 * out_tokens holds max_new_tokens + 1 ids; pass arrays hold max_new_tokens entries.  `model` NULL with
 * target/draft runtimes given runs the GPU model (batched verify of [current, proposed]). */
int esp_exact_two_token_harness_generate(const ESPExactTwoTokenModel *model, ESPLlamaRuntime *target, ESPLlamaRuntime *draft,
                                         const uint32_t *prompt_tokens, int prompt_count, int max_new_tokens,
                                         uint32_t *out_tokens, int *out_token_count, int32_t *out_committed_per_pass,
                                         int32_t *out_accepted_per_pass, int *out_pass_count);

/* ================================================================================================== *
 * Kernel handles and surfaces: the call shape of the reference's ANEInterop module
 * (Sources/ANEInterop/include/ane_interop.h), one esp_interop_* function per ane_interop_* function
 * the decode path uses, same argument order and return conventions (NULL / false on failure, the
 * cause in esp_interop_last_compile_error()).  Swift's ANEKernel (Sources/ANERuntime/ANEKernel.swift:
 * 65-745) and SurfaceIO (Sources/ANETypes/SurfaceIO.swift) bind to these one for one.
 *
 * A surface is a flat fp16 buffer read as channel-first [channels, spatial], element (c, s) at
 * c * spatial + s (ane_interop.h:171-174).  It lives in HBM with a host shadow; the io functions work
 * on the shadow and eval moves what changed, so "lock, copy, unlock" keeps its meaning.
 * ================================================================================================== */
typedef struct ESPHandle ESPHandle;          /* ANEHandle, ane_interop.h:13 */
typedef struct ESPSurface *ESPSurfaceRef;    /* stands in for IOSurfaceRef; reference counted */

void esp_interop_init(void);                                     /* :15 */
ESPSurfaceRef esp_interop_create_surface(size_t bytes);          /* :16, returns +1 retained */
ESPSurfaceRef esp_surface_retain(ESPSurfaceRef surface);         /* CFRetain / CFRelease of the reference's surfaces */
void esp_surface_release(ESPSurfaceRef surface);
size_t esp_surface_bytes(ESPSurfaceRef surface);                 /* IOSurfaceGetAllocSize */

#define ESP_INTEROP_COMPILE_ERROR_NONE 0                          /* :18-22, same values */
#define ESP_INTEROP_COMPILE_ERROR_INVALID_ARGUMENTS 1
#define ESP_INTEROP_COMPILE_ERROR_DUPLICATE_WEIGHT_PATH 2
#define ESP_INTEROP_COMPILE_ERROR_SURFACE_ALLOCATION_FAILED 3
#define ESP_INTEROP_COMPILE_ERROR_COMPILER_FAILURE 4

/* ane_interop_compile (:24-28).  `program` is a text description of one HIP kernel set instead of MIL
 * text: "key: value" lines, e.g.
 *     program: espresso.hip/1
 *     kernel: gemv            (gemv | rmsnorm_classifier | decode_ffn | decode_qkv | decode_projection)
 *     format: q8_0            (f32 | f16 | q4_0 | q8_0 | q4_k; weight matrices)
 *     rows: 768  cols: 768    (gemv)   dim / hidden (decode_ffn)   dim / vocab (rmsnorm_classifier)
 *     spatial: 32             (surface width S; a decode token lives in column 0, DecodeKernelSet.swift:10)
 *     lanes: 1                (how many leading columns are computed, 1..16)
 *     norm_eps: 1e-5
 * Weights are matched by the file name at the end of their path ("@model_path/weights/w.bin" -> "w"):
 * gemv: w; rmsnorm_classifier: rms_final, classifier; decode_ffn: rms_ffn, w1, w3, w2.  Matrices are GGUF
 * blocks of `format`, or a BLOBFILE when format is f16; norm vectors are BLOBFILEs.  The bytes are copied
 * during the call.  Surfaces: gemv in [cols,S] -> out [rows,S]; rmsnorm_classifier in [dim,S] -> logits
 * [vocab,S], max [1,S] (GenerationRMSNormClassifierGenerator.swift:27-63); decode_ffn in [dim,S] -> [dim,S]
 * computing x + W2(silu(W1 n) * W3 n), n = rmsnorm(x) (DecodeFFNGenerator.swift:40-91).
 * decode_qkv (dim, q_dim, kv_dim; weights rms_att, wq, wk, wv): in [dim,S] -> k [kv_dim,S] @ 0, q [q_dim,S] @ 1, v [kv_dim,S] @ 2,
 * the output order of the reference's decodeQKVOnly kernel (DecodeForwardPass.swift:374-377; DecodeAttentionQKVGenerator.swift:86-131):
 * rmsnorm and the three projections, no RoPE.  decode_projection (dim, q_dim; weight wo): context [q_dim,S] @ 0 and residual
 * [dim,S] @ 1 -> residual + Wo context [dim,S]; the reference rebinds input 1 to the layer's input surface
 * (DecodeForwardPass.swift:383,396).  Together with decode_ffn and the three calls below these run one layer of
 * HybridDecodeKernelSet (Sources/ANERuntime/HybridDecodeKernelSet.swift:30-56) handle by handle. */
ESPHandle *esp_interop_compile(const uint8_t *program, size_t program_len,
                               const char **weight_paths, const uint8_t **weight_datas,
                               const size_t *weight_lens, int weight_count,
                               int n_inputs, const size_t *input_sizes,
                               int n_outputs, const size_t *output_sizes);
bool esp_interop_eval(ESPHandle *handle);                                   /* :30, synchronous */
ESPSurfaceRef esp_interop_get_input(ESPHandle *handle, int index);          /* :31, not retained */
ESPSurfaceRef esp_interop_get_output(ESPHandle *handle, int index);         /* :32, not retained */
ESPSurfaceRef esp_interop_copy_input(ESPHandle *handle, int index);         /* :33, +1 retained */
ESPSurfaceRef esp_interop_copy_output(ESPHandle *handle, int index);        /* :34, +1 retained */
void esp_interop_free(ESPHandle *handle);                                   /* :35 */
int esp_interop_compile_count(void);                                        /* :37 */
void esp_interop_set_compile_count(int value);                              /* :38 */
int esp_interop_last_compile_error(void);                                   /* :39 */
void esp_interop_set_force_eval_failure(bool value);                        /* :40, host-side fault injection */
int esp_interop_live_handle_count(void);                                    /* :41 */
uint64_t esp_interop_last_hw_execution_time_ns(ESPHandle *handle);          /* :42, HIP-event time of the last eval */
bool esp_interop_has_perf_stats(ESPHandle *handle);                         /* :43 */
bool esp_interop_rebind_input(ESPHandle *handle, int index, ESPSurfaceRef new_surface);   /* :50 */

/* Between the kernel evaluations of a hybrid decode layer the reference runs Metal kernels on the same surfaces
 * (Sources/Espresso/MetalAttentionKernel.swift); these are their counterparts on surfaces resident in HBM, synchronous:
 *   rope_decode       :1756-1795  half-split RoPE in place on lane 0 of q [heads*D, S] and k [kvHeads*D, S]
 *   kv_cache_scatter  :1805-1820  lane 0 of k / v into column token_index of the caches [kvDim, cacheStride]
 *   decode_sdpa       :1824-1886  fused_decode_sdpa: softmax(q K / sqrt(D)) V over columns token_base .. +visible of the caches into
 *                                 lane 0 of the context surface [heads*D, S] (fp16; kvHead = head / (heads / kvHeads), the
 *                                 reference's groupedContiguous mapping, :146-153; its moduloInterleaved mapping is not offered;
 *                                 at most 12032 visible tokens; the reference keeps this context in an fp32 buffer, there is no
 *                                 vector of it in the reference's tests to compare the fp16 rounding with)
 * A call that fails leaves every surface as it was. */
bool esp_interop_rope_decode(ESPSurfaceRef q, ESPSurfaceRef k, int n_heads, int n_kv_heads, int head_dim, int position, float theta, int lane_spatial);
bool esp_interop_kv_cache_scatter(ESPSurfaceRef k_src, ESPSurfaceRef v_src, ESPSurfaceRef k_cache, ESPSurfaceRef v_cache, int kv_dim, int token_index,
                                  int cache_stride, int lane_spatial);
bool esp_interop_decode_sdpa(ESPSurfaceRef q, ESPSurfaceRef k_cache, ESPSurfaceRef v_cache, ESPSurfaceRef context, int heads, int kv_heads, int head_dim,
                             int visible_tokens, int token_base, int cache_stride, int lane_spatial);

void esp_interop_cvt_f32_to_f16(void *dst, const float *src, int count);    /* :143, round to nearest even */
void esp_interop_cvt_f16_to_f32(float *dst, const void *src, int count);    /* :144 */
/* First-max argmax over fp16 values: lowest index wins ties (:146-156, neon_convert.c:36-101). */
void esp_interop_argmax_f16(const void *src, int count, int *out_index, float *out_value);
void esp_interop_argmax_f16_strided(const void *src, int count, int stride, int *out_index, float *out_value);
void esp_interop_gather_f16_to_f32(float *dst, const void *src, int count, int stride);      /* :160 */
void esp_interop_scatter_f32_to_f16(void *dst, const float *src, int count, int stride);     /* :165 */

/* Surface I/O (:168-348): fp32 on the caller's side, fp16 on the surface; all return false on a
 * range error instead of touching memory. */
bool esp_interop_io_copy(ESPSurfaceRef dst, int dst_ch_off, ESPSurfaceRef src, int src_ch_off, int channels, int spatial);   /* :168 */
bool esp_interop_io_copy_fp16_spatial_slice(ESPSurfaceRef dst, int dst_ch_off, int dst_spatial_index, int dst_spatial,
                                            ESPSurfaceRef src, int src_ch_off, int src_spatial_index, int src_spatial,
                                            int channels);                                                                 /* :175 */
bool esp_interop_io_write_fp16_spatial_slice(ESPSurfaceRef surface, int ch_off, int spatial_index, int spatial,
                                             const float *data, int channels);                                             /* :202 */
bool esp_interop_io_read_fp16_spatial_slice(ESPSurfaceRef surface, int ch_off, int spatial_index, int spatial,
                                            float *data, int channels);                                                    /* :208 */
bool esp_interop_io_argmax_fp16_spatial_slice(ESPSurfaceRef surface, int ch_off, int spatial_index, int spatial,
                                              int channels, int *out_index, float *out_value);                             /* :214 */
bool esp_interop_io_write_fp16(ESPSurfaceRef surface, const float *data, int channels, int spatial);                       /* :235 */
bool esp_interop_io_read_fp16(ESPSurfaceRef surface, int ch_off, float *data, int channels, int spatial);                  /* :237 */
bool esp_interop_io_read_fp16_batched(ESPSurfaceRef surface, int spatial, float *const *destinations,
                                      const int *channel_offsets, const int *channels, int region_count);                  /* :239 */
bool esp_interop_io_write_fp16_at(ESPSurfaceRef surface, int ch_off, const float *data, int channels, int spatial);        /* :244 */
bool esp_interop_io_write_embedding_batch_fp16(ESPSurfaceRef surface, int ch_off, int spatial, const float *embedding_table,
                                               int vocab_size, int dim, const uint16_t *token_ids, int stream_count);      /* :270 */
bool esp_interop_io_argmax_batch_fp16_spatial(ESPSurfaceRef surface, int ch_off, int spatial, int channels, int stream_count,
                                              int *out_indices, float *out_values);                                        /* :282 */
bool esp_interop_io_copy_two_fp16_spatial_slices(ESPSurfaceRef dst0, int dst0_ch_off, int dst0_spatial_index, int dst0_spatial, ESPSurfaceRef src0,
                                                 int src0_ch_off, int src0_spatial_index, int src0_spatial, ESPSurfaceRef dst1, int dst1_ch_off,
                                                 int dst1_spatial_index, int dst1_spatial, ESPSurfaceRef src1, int src1_ch_off, int src1_spatial_index,
                                                 int src1_spatial, int channels);                                              /* :184 */
bool esp_interop_io_argmax_fp16_spatial_slice_with_hint(ESPSurfaceRef surface, int ch_off, int spatial_index, int spatial, int channels,
                                                        ESPSurfaceRef hint_surface, int hint_spatial_index, int hint_spatial, int *out_index,
                                                        float *out_value);                                                    /* :224 */
bool esp_interop_io_write_fp16_at_batched(ESPSurfaceRef surface, const int *channel_offsets, const float *const *sources, const int *channels,
                                          int region_count, int spatial);                                                     /* :246 */
bool esp_interop_io_copy_batched(ESPSurfaceRef dst, ESPSurfaceRef src, const int *dst_channel_offsets, const int *src_channel_offsets,
                                 const int *channels, int region_count, int spatial);                                         /* :252 */
bool esp_interop_io_copy_multi_src(ESPSurfaceRef dst, const ESPSurfaceRef *sources, const int *dst_channel_offsets, const int *src_channel_offsets,
                                   const int *channels, int region_count, int spatial);                                       /* :259 */
bool esp_interop_io_argmax_batch_fp16_spatial_parallel(ESPSurfaceRef surface, int ch_off, int spatial, int channels, int stream_count,
                                                       int *out_indices, float *out_values, int n_blocks);                    /* :294 */
bool esp_interop_io_argmax_batch_fp16_spatial_nolock(ESPSurfaceRef surface, int ch_off, int spatial, int channels, int stream_count,
                                                     int *out_indices, float *out_values, int n_blocks);                      /* :306 */
/* :320; the factored output head's expansion + argmax on the host: fp16 fused multiply-adds in channel order, first maximum,
 * vocab <= 65535, spatial a multiple of 8 (surface_io.c:1438-1700).  Parity unpinned: the reference holds no vector for it. */
bool esp_interop_fused_expansion_argmax_fp16(ESPSurfaceRef proj_surface, int proj_ch_off, int spatial, int bottleneck, int groups,
                                             const void *expansion_weights_fp16, int vocab_size, int stream_count, int *out_indices,
                                             float *out_values, int n_blocks);
/* The same head resident on the GPU, in the shape of the reference's Metal twin (Sources/Espresso/MetalExpansionArgmax.swift:966-1186,
 * FusedExpansionArgmax: init(wExpand:bottleneck:vocabSize:spatial:) uploads the expansion weights once, run(projectedSurface:) returns one
 * token per spatial lane, no logits are stored).  create copies vocab_size x (bottleneck / groups) fp16 weights into HBM (groups = 1 is the
 * Metal twin's dense expansion; grouped weights as in surface_io.c).  argmax reads lanes 0 .. stream_count - 1 of the projected surface
 * where it lives on the device and runs one kernel over (vocab, lane): every logit is one chain of fused multiply-adds in k order, in fp16
 * (fp32_sums = 0: bit-identical to esp_interop_fused_expansion_argmax_fp16, including its argument checks) or in fp32 (fp32_sums = 1: the
 * Metal shader's arithmetic, first maximum on ties where the shader's reduction order is unspecified). */
typedef struct ESPExpansionHead *ESPExpansionHeadRef;
ESPExpansionHeadRef esp_interop_expansion_head_create(const void *expansion_weights_fp16, int bottleneck, int groups, int vocab_size);
bool esp_interop_expansion_head_argmax(ESPExpansionHeadRef head, ESPSurfaceRef proj_surface, int proj_ch_off, int spatial, int stream_count,
                                       int fp32_sums, int *out_indices, float *out_values);
void esp_interop_expansion_head_free(ESPExpansionHeadRef head);
bool esp_interop_io_lock_write(ESPSurfaceRef surface);                                                                     /* :335 */
bool esp_interop_io_unlock_write(ESPSurfaceRef surface);
bool esp_interop_io_lock_read(ESPSurfaceRef surface);
bool esp_interop_io_unlock_read(ESPSurfaceRef surface);
bool esp_interop_io_write_fp16_unlocked(ESPSurfaceRef surface, const float *data, int channels, int spatial);              /* :342 */
bool esp_interop_io_read_fp16_unlocked(ESPSurfaceRef surface, int ch_off, float *data, int channels, int spatial);         /* :347 */

#ifdef __cplusplus
}
#endif
#endif
