/*
 * espresso_hip_bench.h — measurement and tuning entry points of libespresso_hip.so.
 *
 * Nothing here has a counterpart in the reference and no integration needs it: these calls exist for
 * bench.py and for the tests that pin kernel variants (timed launch trains, per-wavefront stamps,
 * bandwidth probes, kernel-selection switches).  The drop-in boundary is espresso_hip.h alone.
 */
#ifndef ESPRESSO_HIP_BENCH_H
#define ESPRESSO_HIP_BENCH_H

#include "espresso_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Times the GEMV kernel alone on buffers already resident in HBM: `warmup` untimed launches, then
 * `iters` launches bracketed by HIP events on the library stream.  Reports the mean and the best
 * per-launch time in microseconds.  rotate > 1 cycles through that many copies of the matrix so
 * that no launch finds its weights in the last-level cache. */
int esp_gemv_time(const ESPMatrix *matrix, int batch, int warmup, int iters, int rotate,
                  double *mean_us, double *best_us);

/* Measurement aid (no counterpart in the reference): runs the Q4_K GEMV back to back over copies of the matrix that together
 * exceed the caches (at least `launches` - 1 times and once through all copies: weights from HBM, code and activations warm,
 * the state a decode step finds); every wavefront of one launch inside that train records four 100 MHz wall-clock stamps:
 * start, activations staged, first weights consumed, end.  out_stamps receives [wavefront][4]; *out_wavefronts how many
 * wavefronts wrote (at most capacity_wavefronts); *out_period_us (may be null) the time from the first wavefront start of
 * that launch to the first wavefront start of the next one: the launch's share of the train, which exceeds its last
 * wavefront's end by the time in which no wavefront of either kernel runs. */
int esp_gemv_stamps(const ESPMatrix *matrix, int batch, int launches, uint64_t *out_stamps, int capacity_wavefronts, int *out_wavefronts,
                    double *out_period_us);
/* Kernel-selection switches for measurements and tests (no counterpart in the reference); the same switches are read from
 * the environment when first needed.  "q4k_mfma" (ESPRESSO_HIP_Q4K_MFMA): 1 = Q4_K GEMVs of 4096 / 14336 columns run on the
 * matrix cores (one to eight activation rows per pass over the weights), 0 = never, -1 = the library's own choice.
 * "q40_mfma" (ESPRESSO_HIP_Q40_MFMA): the same for Q4_0 (one to four rows).
 * "q4k_mfma_ks" / "q4k_mfma_waves" (ESPRESSO_HIP_Q4K_MFMA_KS / _WAVES): wavefronts that share a block of sixteen rows and
 * wavefronts per workgroup, 0 = by shape; combinations without a compiled kernel fall back to the dot-product kernels.
 * "q4k_mfma_ragged": 0 = every workgroup runs the same number of rounds.
 * "q4k_long_row_waves" (ESPRESSO_HIP_Q4K_LONG_ROW_WAVES): one activation row at 14336 columns: 0 (default) = the matrix-core
 * kernel, 8 or 4 = the dot-product kernel with that many wavefronts per workgroup (one or three workgroups per compute unit).
 * Runtimes that captured a step graph keep the kernels they captured. */
int esp_set_tuning(const char *key, int value);
/* Measurement aid with no counterpart in the reference: a kernel that only streams `bytes` (>= 1 MiB, a
 * multiple of 16) from HBM with 128-bit loads, `iters` times; reports GB/s.  bench.py prints it next to the
 * GEMV bandwidth so that fractions of the published peak can be read against what a plain reader gets. */
/* Diagnostic: copies the matrix's tiled copy (the second resident format, read by the matrix-core GEMVs) to `out`; returns the number of
 * bytes (esp_matrix_resident_bytes - esp_matrix_bytes; 0 when the matrix keeps none) or a negative ESP_ERR_* code.  tests/ rebuild the tiles
 * from the GGUF blocks with numpy and compare byte for byte. */
long long esp_matrix_read_tiled(const ESPMatrix *matrix, void *out, size_t capacity);
/* Test aid: the exact Q4_K product of esp_matmul_f32 with the epilogue the feed-forward block uses.  The matrix holds gate and up rows
 * interleaved (row 2i = gate_i, 2i + 1 = up_i; `matrix rows` a multiple of 8); act[r][i] = SiLU(x[r] . gate_i) * (x[r] . up_i) as the pair of
 * fp16 planes the kernel writes, added back together (hi + lo / 2048), fp32 [rows][matrix rows / 2]; host pointers.  The launch is made
 * twice on the same flag words; the sub-block sums the kernel writes beside the planes are checked against the planes on the host
 * (a mismatch fails the call); tuning key split_gemm_shared_k selects how
 * workgroups share an output tile's K range (0 never, 1 where it applies, 2 as 1 with the finishing workgroup never waiting). */
int esp_matmul_f32_swiglu(const ESPMatrix *matrix, const float *x, int rows, float *act);
int esp_hbm_read_probe(size_t bytes, int iters, double *gb_per_s);
/* The ceiling for ONE GEMV launch: a kernel with a persistent Q4_K GEMV's grid (`workgroups` of `wavefronts` = 4 or 8) and its
 * loads (a wavefront takes items of `pair_bytes`, a 2304-byte weight tile of the matrix-core kernel or a pair of rows of the
 * dot-product kernel, the next item's 128-bit loads in flight while the current one is consumed) that does nothing else, launched back to back `launches` times over `copies` buffers of `bytes_per_launch` in
 * turn (so that no launch finds its bytes in a cache).  Reports the mean time per launch, which includes what a dependent
 * launch costs on this machine, and the resulting GB/s. */
int esp_hbm_read_probe_pairs(size_t bytes_per_launch, int pair_bytes, int workgroups, int wavefronts, int copies, int launches, double *mean_us,
                             double *gb_per_s);

/* Per-kernel timing with HIP events on the library stream.  While enabled every launch of the GEMV
 * and attention kernels of a step is bracketed by an event pair; esp_llama_kernel_times synchronises
 * and reports, per kernel class, the summed elapsed microseconds, the launch count and the
 * algorithmic bytes of one batch-1 launch (packed weights + fp16 input + fp32 output).  Class
 * ESP_KERNEL_EVENT_PAIR brackets nothing, once per step: its mean is what an event pair itself adds to
 * every other class's mean. */
#define ESP_KERNEL_QKV 0
#define ESP_KERNEL_WO 1
#define ESP_KERNEL_GATE_UP 2
#define ESP_KERNEL_DOWN 3
#define ESP_KERNEL_HEAD 4
#define ESP_KERNEL_ATTENTION 5
#define ESP_KERNEL_EVENT_PAIR 6
#define ESP_KERNEL_CLASS_COUNT 7
int esp_llama_set_kernel_timing(ESPLlamaRuntime *runtime, int enabled);
int esp_llama_kernel_times(ESPLlamaRuntime *runtime, double *total_us, int64_t *launches, uint64_t *bytes_per_launch,
                           int reset);
/* The GEMV of one class (ESP_KERNEL_QKV .. ESP_KERNEL_HEAD) launched for every layer in turn, `iters` rounds,
 * between two HIP events: the mean duration of back-to-back dependent launches at the model's real shapes over
 * its real weights (a round moves more bytes than any cache holds).  No per-launch event overhead, so the mean
 * is directly comparable with a rocprofv3 kernel trace.  The epilogues write into live buffers: reset the
 * runtime before decoding again. */
int esp_llama_time_kernel(ESPLlamaRuntime *runtime, int kernel_class, int iters, double *mean_us);
/* The same launches twice: back to back between two events (back_to_back_us, as above) and then with a pair of
 * events attached to every launch, which take the kernel's own start and end (kernel_us: the mean kernel duration,
 * the figure a rocprofv3 kernel trace reports for the kernel).  Measurement only; no counterpart in the reference. */
int esp_llama_time_kernel_dispatch(ESPLlamaRuntime *runtime, int kernel_class, int iters, double *back_to_back_us, double *kernel_us);

#ifdef __cplusplus
}
#endif

#endif /* ESPRESSO_HIP_BENCH_H */
