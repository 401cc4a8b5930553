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
/* Decode the resident copy back to fp32 [rows*cols] (checks the HBM layout carries the same bits). */
int esp_matrix_dequantize(const ESPMatrix *matrix, float *out);

/* ---- dequant-fused GEMV ----------------------------------------------------------------- *
 * y[b][r] = (residual ? residual[b][r] : 0) + sum_c dequant(W)[r][c] * x[b][c]
 * Replaces multiplyRowMajorMatrix (Sources/RealModelInference/RealModelInferenceEngine.swift:6674-6718).
 * x: fp16 bit patterns [batch][cols]; y, residual: fp32 [batch][rows]; host pointers. */
int esp_gemv(const ESPMatrix *matrix, const uint16_t *x_f16, int batch, float *y, const float *residual);
/* Times the GEMV kernel alone on buffers already resident in HBM: `warmup` untimed launches, then
 * `iters` launches bracketed by HIP events on the library stream.  Reports the mean and the best
 * per-launch time in microseconds.  rotate > 1 cycles through that many copies of the matrix so
 * that no launch finds its weights in the last-level cache. */
int esp_gemv_time(const ESPMatrix *matrix, int batch, int warmup, int iters, int rotate,
                  double *mean_us, double *best_us);

#ifdef __cplusplus
}
#endif
#endif
