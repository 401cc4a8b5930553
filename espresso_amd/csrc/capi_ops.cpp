// C ABI: library set-up, GGUF block dequantisation, resident matrices and the GEMV entry points.
#include <cstring>
#include <vector>

#include <cmath>
#include <cstring>

#include "context.h"
#include "host/model_support.h"
#include "kernels/decode_ops.h"

using namespace esp;

// ---- scratch of the entry point that allocates nothing (esp_gemv_device_noalloc) ---------------------------
// Split-K partial sums of the matrix-core kernels, [splits][batch][rows] floats, live in a file-scope device array
// instead of a hipMalloc'ed workspace.  The array's name is a host-side stand-in, not a device address: the
// address comes from hipGetSymbolAddress, once per device, at library set-up, and only that pointer is handed
// to kernels.  Every GPU holds its own 16 MiB copy until the process ends.
namespace {
constexpr size_t kNoAllocScratchFloats = (size_t)4 << 20;
constexpr int kNoAllocMaxBatch = 64;
constexpr int kNoAllocMaxDevices = 16;
static __device__ __align__(256) float scratch[kNoAllocScratchFloats];
float *g_scratch_ptr[kNoAllocMaxDevices] = {};
}  // namespace

namespace esp {
int noalloc_setup(int device) {
    if (device < 0 || device >= kNoAllocMaxDevices) return fail(ESP_ERR_INVALID_ARGUMENT, "device %d outside 0..%d", device, kNoAllocMaxDevices - 1);
    if (g_scratch_ptr[device]) return ESP_OK;
    float *ptr = nullptr;
    hipError_t e = hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch));   // `device` is the current device here
    if (e != hipSuccess || !ptr) return fail_hip(e == hipSuccess ? hipErrorInvalidSymbol : e, "hipGetSymbolAddress(scratch)");
    g_scratch_ptr[device] = ptr;
    return ESP_OK;
}
}  // namespace esp

extern "C" {

int esp_init(void) { return ensure_init(); }

int esp_device_info(char *name, size_t name_capacity, int *compute_units, size_t *hbm_bytes) {
    int rc = ensure_init();
    if (rc != ESP_OK) return rc;
    const Context &c = context();
    if (name && name_capacity) {
        std::strncpy(name, c.props.gcnArchName, name_capacity - 1);
        name[name_capacity - 1] = 0;
    }
    if (compute_units) *compute_units = c.props.multiProcessorCount;
    if (hbm_bytes) *hbm_bytes = c.props.totalGlobalMem;
    return ESP_OK;
}

size_t esp_format_bytes(int format, size_t elements) {
    if (!format_supported(format) || elements % format_block_elems(format) != 0) return 0;
    return format_bytes(format, elements);
}

int esp_dequantize(int format, const void *blocks, size_t elements, float *out) {
    if (!format_supported(format)) return fail(ESP_ERR_UNSUPPORTED, "dequantize: unknown format %d", format);
    if (elements % format_block_elems(format) != 0)
        return fail(ESP_ERR_INVALID_ARGUMENT, "dequantize: %zu elements is not a whole number of blocks", elements);
    if (elements == 0) return ESP_OK;
    if (!blocks || !out) return fail(ESP_ERR_INVALID_ARGUMENT, "dequantize: null pointer");
    int rc = ensure_init();
    if (rc != ESP_OK) return rc;
    Context &c = context();
    const size_t bytes = format_bytes(format, elements);
    uint8_t *d_blocks = nullptr;
    float *d_out = nullptr;
    if ((rc = device_alloc(&d_blocks, bytes)) != ESP_OK) return rc;
    if ((rc = device_alloc(&d_out, elements)) != ESP_OK) { (void)hipFree(d_blocks); return rc; }
    hipError_t e = hipMemcpyAsync(d_blocks, blocks, bytes, hipMemcpyHostToDevice, c.stream);
    if (e == hipSuccess) e = launch_dequant(format, d_blocks, elements, d_out, c.stream);
    if (e == hipSuccess) e = hipMemcpyAsync(out, d_out, elements * sizeof(float), hipMemcpyDeviceToHost, c.stream);
    if (e == hipSuccess) e = hipStreamSynchronize(c.stream);
    (void)hipFree(d_blocks);
    (void)hipFree(d_out);
    return e == hipSuccess ? ESP_OK : fail_hip(e, "dequantize");
}

ESPMatrix *esp_matrix_create(int format, const void *gguf_blocks, int rows, int cols) {
    DeviceMatrix m;
    if (matrix_upload(format, gguf_blocks, rows, cols, &m) != ESP_OK) return nullptr;
    ESPMatrix *h = new ESPMatrix();
    h->m = m;
    return h;
}

void esp_matrix_free(ESPMatrix *matrix) {
    if (!matrix) return;
    matrix_release(&matrix->m);
    delete matrix;
}

size_t esp_matrix_bytes(const ESPMatrix *matrix) { return matrix ? matrix->m.bytes() : 0; }
size_t esp_matrix_resident_bytes(const ESPMatrix *matrix) { return matrix ? matrix->m.resident_bytes() : 0; }

long long esp_matrix_read_tiled(const ESPMatrix *matrix, void *out, size_t capacity) {
    if (!matrix || !out) return fail(ESP_ERR_INVALID_ARGUMENT, "matrix_read_tiled: null pointer");
    const size_t bytes = matrix->m.tiled ? matrix->m.tiled_bytes() : 0;
    if (bytes == 0) return 0;
    if (capacity < bytes) return fail(ESP_ERR_OUT_OF_RANGE, "matrix_read_tiled: %zu bytes needed", bytes);
    int rc = ensure_init();
    if (rc != ESP_OK) return rc;
    const hipError_t e = hipMemcpy(out, matrix->m.tiled, bytes, hipMemcpyDeviceToHost);
    if (e != hipSuccess) return fail_hip(e, "matrix_read_tiled");
    return (long long)bytes;
}

int esp_matrix_dequantize(const ESPMatrix *matrix, float *out) {
    if (!matrix || !out) return fail(ESP_ERR_INVALID_ARGUMENT, "matrix_dequantize: null pointer");
    int rc = ensure_init();
    if (rc != ESP_OK) return rc;
    Context &c = context();
    const size_t elems = (size_t)matrix->m.rows * matrix->m.cols;
    float *d_out = nullptr;
    if ((rc = device_alloc(&d_out, elems)) != ESP_OK) return rc;
    hipError_t e = launch_dequant_matrix(matrix->m, d_out, c.stream);
    if (e == hipSuccess) e = hipMemcpyAsync(out, d_out, elems * sizeof(float), hipMemcpyDeviceToHost, c.stream);
    if (e == hipSuccess) e = hipStreamSynchronize(c.stream);
    (void)hipFree(d_out);
    return e == hipSuccess ? ESP_OK : fail_hip(e, "matrix_dequantize");
}

namespace {
// More than two rows of activations go to the matrix-core kernel (fp32 matrices stay on the GEMV path).
bool use_gemm(const DeviceMatrix &m, int batch) { return batch > 2 && m.format != FMT_F32 && m.cols % 64 == 0 && !gemv_takes_rows(m, batch); }
// 16 MiB of split-K partial sums: the size of the fixed scratch of esp_gemv_device_noalloc, so that both entry points always pick
// the same split count and add in the same order
constexpr size_t kGemmWorkspaceFloats = kNoAllocScratchFloats;

hipError_t run_matvec(const DeviceMatrix &m, const uint16_t *d_x, int batch, float *d_y, const float *d_res, float *workspace, hipStream_t s) {
    if (use_gemm(m, batch)) {
        GemmParams g;
        g.w = m; g.x = d_x; g.y = d_y; g.residual = d_res; g.rows = batch; g.workspace = workspace; g.workspace_floats = workspace ? kGemmWorkspaceFloats : 0;
        return launch_gemm(g, s);
    }
    GemvParams p;
    p.w = m; p.x = d_x; p.y = d_y; p.residual = d_res; p.batch = batch;
    p.epilogue = d_res ? EPI_ADD_RESIDUAL : EPI_STORE_F32;
    return launch_gemv(p, s);
}
}  // namespace

int esp_gemv(const ESPMatrix *matrix, const uint16_t *x_f16, int batch, float *y, const float *residual) {
    if (!matrix || !x_f16 || !y) return fail(ESP_ERR_INVALID_ARGUMENT, "gemv: null pointer");
    if (batch <= 0) return fail(ESP_ERR_INVALID_ARGUMENT, "gemv: batch %d", batch);
    int rc = ensure_init();
    if (rc != ESP_OK) return rc;
    Context &c = context();
    const DeviceMatrix &m = matrix->m;
    const size_t nx = (size_t)batch * m.cols, ny = (size_t)batch * m.rows;
    uint16_t *d_x = nullptr;
    float *d_y = nullptr, *d_res = nullptr, *d_ws = nullptr;
    if ((rc = device_alloc(&d_x, nx)) != ESP_OK) return rc;
    if ((rc = device_alloc(&d_y, ny)) != ESP_OK) { (void)hipFree(d_x); return rc; }
    if (residual && (rc = device_alloc(&d_res, ny)) != ESP_OK) { (void)hipFree(d_x); (void)hipFree(d_y); return rc; }
    if (use_gemm(m, batch) && (rc = device_alloc(&d_ws, kGemmWorkspaceFloats)) != ESP_OK) {
        (void)hipFree(d_x); (void)hipFree(d_y); if (d_res) (void)hipFree(d_res);
        return rc;
    }
    hipError_t e = hipMemcpyAsync(d_x, x_f16, nx * 2, hipMemcpyHostToDevice, c.stream);
    if (e == hipSuccess && residual) e = hipMemcpyAsync(d_res, residual, ny * 4, hipMemcpyHostToDevice, c.stream);
    if (e == hipSuccess) e = run_matvec(m, d_x, batch, d_y, d_res, d_ws, c.stream);
    if (e == hipSuccess) e = hipMemcpyAsync(y, d_y, ny * 4, hipMemcpyDeviceToHost, c.stream);
    if (e == hipSuccess) e = hipStreamSynchronize(c.stream);
    (void)hipFree(d_x); (void)hipFree(d_y);
    if (d_res) (void)hipFree(d_res);
    if (d_ws) (void)hipFree(d_ws);
    return e == hipSuccess ? ESP_OK : fail_hip(e, "gemv");
}

int esp_matmul_f32(const ESPMatrix *matrix, const float *x, int rows, float *y, const float *residual) {
    if (!matrix || !x || !y) return fail(ESP_ERR_INVALID_ARGUMENT, "matmul_f32: null pointer");
    if (rows <= 0) return fail(ESP_ERR_INVALID_ARGUMENT, "matmul_f32: rows %d", rows);
    int rc = ensure_init();
    if (rc != ESP_OK) return rc;
    Context &c = context();
    const DeviceMatrix &m = matrix->m;
    if (!gemm_split_supported(m)) return fail(ESP_ERR_UNSUPPORTED, "matmul_f32: Q4_K matrices with a multiple of 256 columns");
    const size_t nx = (size_t)rows * m.cols, ny = (size_t)rows * m.rows;
    float *d_x = nullptr, *d_y = nullptr, *d_res = nullptr, *d_ws = nullptr;
    SplitRowsView v;
    auto release = [&] {
        void *ptrs[] = {d_x, d_y, d_res, d_ws, v.hi, v.lo, v.sums};
        for (void *p : ptrs) if (p) (void)hipFree(p);
    };
    if ((rc = device_alloc(&d_x, nx)) != ESP_OK || (rc = device_alloc(&d_y, ny)) != ESP_OK || (rc = device_alloc(&v.hi, nx)) != ESP_OK ||
        (rc = device_alloc(&v.lo, nx)) != ESP_OK || (rc = device_alloc(&v.sums, nx / 16)) != ESP_OK ||
        (residual && (rc = device_alloc(&d_res, ny)) != ESP_OK) || (rc = device_alloc(&d_ws, kGemmWorkspaceFloats)) != ESP_OK) {
        release();
        return rc;
    }
    hipError_t e = hipMemcpyAsync(d_x, x, nx * 4, hipMemcpyHostToDevice, c.stream);
    if (e == hipSuccess && residual) e = hipMemcpyAsync(d_res, residual, ny * 4, hipMemcpyHostToDevice, c.stream);
    if (e == hipSuccess) {
        SplitRowsParams sp;
        sp.x = d_x; sp.rows = rows; sp.cols = m.cols; sp.out = v;
        e = launch_split_rows(sp, c.stream);
    }
    if (e == hipSuccess) {
        GemmSplitParams g;
        g.w = m; g.x = v; g.y = d_y; g.residual = d_res; g.rows = rows; g.workspace = d_ws; g.workspace_floats = kGemmWorkspaceFloats;
        e = launch_gemm_split(g, c.stream);
    }
    if (e == hipSuccess) e = hipMemcpyAsync(y, d_y, ny * 4, hipMemcpyDeviceToHost, c.stream);
    if (e == hipSuccess) e = hipStreamSynchronize(c.stream);
    release();
    return e == hipSuccess ? ESP_OK : fail_hip(e, "matmul_f32");
}

int esp_matmul_f32_swiglu(const ESPMatrix *matrix, const float *x, int rows, float *act) {
    if (!matrix || !x || !act) return fail(ESP_ERR_INVALID_ARGUMENT, "matmul_f32_swiglu: null pointer");
    if (rows <= 0) return fail(ESP_ERR_INVALID_ARGUMENT, "matmul_f32_swiglu: rows %d", rows);
    int rc = ensure_init();
    if (rc != ESP_OK) return rc;
    Context &c = context();
    const DeviceMatrix &m = matrix->m;
    if (!gemm_split_supported(m) || m.rows % 8 != 0) return fail(ESP_ERR_UNSUPPORTED, "matmul_f32_swiglu: Q4_K matrices with a multiple of 256 columns and of 8 rows");
    const size_t nx = (size_t)rows * m.cols, units = (size_t)m.rows / 2, na = (size_t)rows * units;
    float *d_x = nullptr;
    GemmSplitSharedK pool;
    SplitRowsView v, out;
    auto release = [&] {
        void *ptrs[] = {d_x, v.hi, v.lo, v.sums, out.hi, out.lo, out.sums};
        for (void *p : ptrs) if (p) (void)hipFree(p);
    };
    if ((rc = device_alloc(&d_x, nx)) != ESP_OK || (rc = device_alloc(&v.hi, nx)) != ESP_OK || (rc = device_alloc(&v.lo, nx)) != ESP_OK ||
        (rc = device_alloc(&v.sums, nx / 16)) != ESP_OK || (rc = device_alloc(&out.hi, na)) != ESP_OK || (rc = device_alloc(&out.lo, na)) != ESP_OK ||
        (rc = device_alloc(&out.sums, na / 16 + 16)) != ESP_OK) {
        release();
        return rc;
    }
    std::vector<uint16_t> hi(na), lo(na);
    hipError_t e = hipMemcpyAsync(d_x, x, nx * 4, hipMemcpyHostToDevice, c.stream);
    if (e == hipSuccess) e = gemm_split_shared_k_pool(&pool);
    if (e == hipSuccess) {
        SplitRowsParams sp;
        sp.x = d_x; sp.rows = rows; sp.cols = m.cols; sp.out = v;
        e = launch_split_rows(sp, c.stream);
    }
    // twice: the second launch runs under the next launch number and finds the first one's flags in place
    for (int pass = 0; pass < 2 && e == hipSuccess; pass++) {
        GemmSplitParams g;
        g.w = m; g.x = v; g.rows = rows; g.swiglu = out; g.shared_k = &pool;
        if (pass == 1) e = hipMemsetAsync(out.hi, 0xff, na * 2, c.stream);
        if (e == hipSuccess) e = launch_gemm_split(g, c.stream);
    }
    if (e == hipSuccess) e = hipMemcpyAsync(hi.data(), out.hi, na * 2, hipMemcpyDeviceToHost, c.stream);
    if (e == hipSuccess) e = hipMemcpyAsync(lo.data(), out.lo, na * 2, hipMemcpyDeviceToHost, c.stream);
    std::vector<uint16_t> sums(na / 16);
    if (e == hipSuccess) e = hipMemcpyAsync(sums.data(), out.sums, sums.size() * 2, hipMemcpyDeviceToHost, c.stream);
    if (e == hipSuccess) e = hipStreamSynchronize(c.stream);
    release();
    if (e != hipSuccess) return fail_hip(e, "matmul_f32_swiglu");
    // the sub-block sums that accompany the planes ([row][super-block][hi of S_0..7, lo of S_0..7]) must be the planes' own, to rounding
    // (checked where the units fill whole super-blocks of the next matrix, as a model's do)
    for (int r = 0; r < rows && units % 256 == 0; r++)
        for (size_t sub = 0; sub < units / 32; sub++) {
            double want = 0.0;
            for (size_t k = 0; k < 32; k++) want += (double)half_to_float(hi[(size_t)r * units + 32 * sub + k]) + (double)half_to_float(lo[(size_t)r * units + 32 * sub + k]) / 2048.0;
            const uint16_t *p = sums.data() + ((size_t)r * (units / 256) + (sub >> 3)) * 16 + (sub & 7);
            const double got = (double)half_to_float(p[0]) + (double)half_to_float(p[8]) / 2048.0;
            if (std::fabs(got - want) > 1e-5 * (1.0 + std::fabs(want)))
                return fail(ESP_ERR_LAUNCH_FAILED, "matmul_f32_swiglu: sub-block sum of row %d, sub-block %zu is %.9g, the planes give %.9g", r, sub, got, want);
        }
    // the planes keep the units of every four in the order (0, 2, 1, 3)
    for (int r = 0; r < rows; r++)
        for (size_t u = 0; u < units; u++) {
            const size_t slot = u & 3, o = (size_t)r * units + (u & ~(size_t)3) + (slot == 1 ? 2 : slot == 2 ? 1 : slot);
            act[(size_t)r * units + u] = half_to_float(hi[o]) + half_to_float(lo[o]) * (1.0f / 2048.0f);
        }
    return ESP_OK;
}

int esp_gemv_device_noalloc(const ESPMatrix *matrix, const uint16_t *x_f16_device, int batch, float *y_device,
                            const float *residual_device_or_null) {
    if (!matrix || !x_f16_device || !y_device) return fail(ESP_ERR_INVALID_ARGUMENT, "gemv_device_noalloc: null pointer");
    if (batch <= 0 || batch > kNoAllocMaxBatch)
        return fail(ESP_ERR_OUT_OF_RANGE, "gemv_device_noalloc: batch %d outside 1..%d", batch, kNoAllocMaxBatch);
    int rc = ensure_init();   // allocates nothing once the library is initialised
    if (rc != ESP_OK) return rc;
    Context &c = context();
    const DeviceMatrix &m = matrix->m;
    float *workspace = c.device >= 0 && c.device < kNoAllocMaxDevices ? g_scratch_ptr[c.device] : nullptr;
    if (!workspace) return fail(ESP_ERR_LAUNCH_FAILED, "gemv_device_noalloc: no scratch address for device %d", c.device);
    if (use_gemm(m, batch) && (size_t)2 * batch * m.rows > kNoAllocScratchFloats)
        return fail(ESP_ERR_OUT_OF_RANGE, "gemv_device_noalloc: batch %d x %d rows needs %zu floats of split-K scratch for two splits, the fixed scratch holds %zu",
                    batch, m.rows, (size_t)2 * batch * m.rows, kNoAllocScratchFloats);
    // Partial planes are written whole by every split before they are added: nothing has to start at zero.
    hipError_t e;
    if (use_gemm(m, batch)) {
        GemmParams g;
        g.w = m; g.x = x_f16_device; g.y = y_device; g.residual = residual_device_or_null; g.rows = batch;
        g.workspace = workspace; g.workspace_floats = kNoAllocScratchFloats;
        e = launch_gemm(g, c.stream);
    } else {
        e = run_matvec(m, x_f16_device, batch, y_device, residual_device_or_null, nullptr, c.stream);
    }
    if (e == hipSuccess) e = hipStreamSynchronize(c.stream);
    return e == hipSuccess ? ESP_OK : fail_hip(e, "gemv_device_noalloc");
}

namespace {
// Copies of one matrix in separate allocations, so that back-to-back launches that walk through them find no weights in a
// cache: the state a decode step finds, which streams every other matrix of the model between two uses of this one.
struct RotatingCopies {
    std::vector<DeviceMatrix> copies;
    int make(const DeviceMatrix &m, int rotate, hipStream_t stream) {
        copies.assign(rotate < 1 ? 1 : rotate, m);
        const size_t qs_bytes = (size_t)m.rows * m.qs_row_bytes, sc_count = m.scales ? (size_t)m.rows * (m.cols / 32) : 0;
        const size_t tiled_bytes = m.tiled_bytes();
        for (size_t i = 1; i < copies.size(); i++) { copies[i].qs = nullptr; copies[i].scales = nullptr; copies[i].tiled = nullptr; }
        for (size_t i = 1; i < copies.size(); i++) {
            int rc = device_alloc(&copies[i].qs, qs_bytes);
            if (rc == ESP_OK && tiled_bytes) rc = device_alloc(&copies[i].tiled, tiled_bytes);
            if (rc == ESP_OK && sc_count) rc = device_alloc(&copies[i].scales, sc_count);
            if (rc != ESP_OK) return rc;
            hipError_t e = hipMemcpyAsync(copies[i].qs, m.qs, qs_bytes, hipMemcpyDeviceToDevice, stream);
            if (e == hipSuccess && tiled_bytes) e = hipMemcpyAsync(copies[i].tiled, m.tiled, tiled_bytes, hipMemcpyDeviceToDevice, stream);
            if (e == hipSuccess && sc_count) e = hipMemcpyAsync(copies[i].scales, m.scales, sc_count * 2, hipMemcpyDeviceToDevice, stream);
            if (e != hipSuccess) return fail_hip(e, "copy of the matrix");
        }
        return ESP_OK;
    }
    const DeviceMatrix &operator[](size_t i) const { return copies[i % copies.size()]; }
    ~RotatingCopies() {
        for (size_t i = 1; i < copies.size(); i++) {
            if (copies[i].qs) (void)hipFree(copies[i].qs);
            if (copies[i].scales) (void)hipFree(copies[i].scales);
            if (copies[i].tiled) (void)hipFree(copies[i].tiled);
        }
    }
};
}  // namespace

int esp_gemv_time(const ESPMatrix *matrix, int batch, int warmup, int iters, int rotate,
                  double *mean_us, double *best_us) {
    if (!matrix || batch <= 0 || iters <= 0 || warmup < 0) return fail(ESP_ERR_INVALID_ARGUMENT, "gemv_time: bad argument");
    if (rotate < 1) rotate = 1;
    int rc = ensure_init();
    if (rc != ESP_OK) return rc;
    Context &c = context();
    const DeviceMatrix &m = matrix->m;
    const size_t nx = (size_t)batch * m.cols, ny = (size_t)batch * m.rows;

    RotatingCopies copies;
    uint16_t *d_x = nullptr;
    float *d_y = nullptr, *d_ws = nullptr;
    std::vector<hipEvent_t> marks;
    hipError_t e = hipSuccess;
    rc = copies.make(m, rotate, c.stream);
    if (rc == ESP_OK) rc = device_alloc(&d_x, nx);
    if (rc == ESP_OK) rc = device_alloc(&d_y, ny);
    if (rc == ESP_OK && use_gemm(m, batch)) rc = device_alloc(&d_ws, kGemmWorkspaceFloats);
    if (rc == ESP_OK) {
        // activations ~ small deterministic values; the kernel's timing does not depend on them
        std::vector<uint16_t> hx(nx);
        for (size_t i = 0; i < nx; i++) hx[i] = (uint16_t)(0x3000u + (i * 37u) % 0x0C00u);
        e = hipMemcpyAsync(d_x, hx.data(), nx * 2, hipMemcpyHostToDevice, c.stream);
        if (e == hipSuccess) e = hipStreamSynchronize(c.stream);
        if (e != hipSuccess) rc = fail_hip(e, "gemv_time upload");
    }
    if (rc == ESP_OK) {
        auto launch = [&](const DeviceMatrix &w) { return run_matvec(w, d_x, batch, d_y, nullptr, d_ws, c.stream); };
        for (int i = 0; i < warmup && e == hipSuccess; i++) e = launch(copies[i % rotate]);
        // mean: `iters` launches queued back to back between two events
        marks.resize(iters + 3, nullptr);
        for (auto &ev : marks) if (e == hipSuccess) e = hipEventCreate(&ev);
        hipEvent_t t0 = marks[iters + 1], t1 = marks[iters + 2];
        if (e == hipSuccess) e = hipEventRecord(t0, c.stream);
        for (int i = 0; i < iters && e == hipSuccess; i++) {
            e = launch(copies[(warmup + i) % rotate]);
        }
        if (e == hipSuccess) e = hipEventRecord(t1, c.stream);
        // best: every launch bracketed by its own events
        if (e == hipSuccess) e = hipEventRecord(marks[0], c.stream);
        for (int i = 0; i < iters && e == hipSuccess; i++) {
            e = launch(copies[(warmup + i) % rotate]);
            if (e == hipSuccess) e = hipEventRecord(marks[i + 1], c.stream);
        }
        if (e == hipSuccess) e = hipStreamSynchronize(c.stream);
        if (e == hipSuccess) {
            float total_ms = 0.0f;
            e = hipEventElapsedTime(&total_ms, t0, t1);
            double best = 1e30;
            for (int i = 0; i < iters && e == hipSuccess; i++) {
                float ms = 0.0f;
                e = hipEventElapsedTime(&ms, marks[i], marks[i + 1]);
                if (ms * 1e3 < best) best = ms * 1e3;
            }
            if (mean_us) *mean_us = (double)total_ms * 1e3 / iters;
            if (best_us) *best_us = best;
        }
        if (e != hipSuccess) rc = fail_hip(e, "gemv_time");
    }
    for (auto ev : marks) if (ev) (void)hipEventDestroy(ev);
    if (d_x) (void)hipFree(d_x);
    if (d_y) (void)hipFree(d_y);
    if (d_ws) (void)hipFree(d_ws);
    return rc;
}

// ---- INT4 classifier ------------------------------------------------------------------------------------
struct ESPInt4Classifier {
    int rows = 0, cols = 0;
    std::vector<uint8_t> h_packed;
    std::vector<float> h_scales, h_biases;
    uint8_t *packed = nullptr;
    float *scales = nullptr, *biases = nullptr, *input = nullptr, *logits = nullptr;
    int *token = nullptr;
    esp::ArgmaxScratch scratch;
};

ESPInt4Classifier *esp_int4_classifier_create(const float *weights, int rows, int cols) {
    if (!weights || rows <= 0 || cols <= 0) { fail(ESP_ERR_INVALID_ARGUMENT, "int4_classifier_create: bad argument"); return nullptr; }
    if (ensure_init() != ESP_OK) return nullptr;
    ESPInt4Classifier *h = new ESPInt4Classifier();
    h->rows = rows; h->cols = cols;
    const int bpr = (cols + 1) / 2;
    h->h_packed.assign((size_t)rows * bpr, 0);
    h->h_scales.resize(rows);
    h->h_biases.resize(rows);
    // TensorBufferINT4(quantizing:rows:cols:), TensorBufferINT4.swift:53-135
    auto q4 = [](float v, float row_min, float scale) { int q = (int)roundf((v - row_min) / scale); return q < 0 ? 0 : (q > 15 ? 15 : q); };
    for (int r = 0; r < rows; r++) {
        const float *row = weights + (size_t)r * cols;
        float row_min = row[0], row_max = row[0];
        for (int c = 1; c < cols; c++) { if (row[c] < row_min) row_min = row[c]; if (row[c] > row_max) row_max = row[c]; }
        const float range = row_max - row_min, scale = range < 1e-10f ? 1.0f : range / 15.0f;
        h->h_scales[r] = scale;
        h->h_biases[r] = row_min;
        uint8_t *out = h->h_packed.data() + (size_t)r * bpr;
        int c = 0, b = 0;
        for (; c + 1 < cols; c += 2) out[b++] = (uint8_t)((q4(row[c], row_min, scale) << 4) | q4(row[c + 1], row_min, scale));
        if (c < cols) out[b] = (uint8_t)(q4(row[c], row_min, scale) << 4);
    }
    bool ok = device_alloc(&h->packed, h->h_packed.size()) == ESP_OK && device_alloc(&h->scales, (size_t)rows) == ESP_OK &&
              device_alloc(&h->biases, (size_t)rows) == ESP_OK && device_alloc(&h->input, (size_t)cols) == ESP_OK &&
              device_alloc(&h->logits, (size_t)rows) == ESP_OK && device_alloc(&h->token, (size_t)1) == ESP_OK &&
              device_alloc(&h->scratch.part_value, (size_t)kArgmaxScratchSlots) == ESP_OK &&
              device_alloc(&h->scratch.part_index, (size_t)kArgmaxScratchSlots) == ESP_OK;
    ok = ok && hipMemcpy(h->packed, h->h_packed.data(), h->h_packed.size(), hipMemcpyHostToDevice) == hipSuccess &&
         hipMemcpy(h->scales, h->h_scales.data(), (size_t)rows * 4, hipMemcpyHostToDevice) == hipSuccess &&
         hipMemcpy(h->biases, h->h_biases.data(), (size_t)rows * 4, hipMemcpyHostToDevice) == hipSuccess;
    if (!ok) { esp_int4_classifier_free(h); fail(ESP_ERR_OUT_OF_MEMORY, "int4_classifier_create: device setup failed"); return nullptr; }
    return h;
}

void esp_int4_classifier_free(ESPInt4Classifier *h) {
    if (!h) return;
    void *ptrs[] = {h->packed, h->scales, h->biases, h->input, h->logits, h->token, h->scratch.part_value, h->scratch.part_index};
    for (void *p : ptrs) if (p) (void)hipFree(p);
    delete h;
}

int esp_int4_classifier_export(const ESPInt4Classifier *h, uint8_t *packed, float *scales, float *biases) {
    if (!h) return fail(ESP_ERR_INVALID_ARGUMENT, "int4_classifier_export: null handle");
    if (packed) std::memcpy(packed, h->h_packed.data(), h->h_packed.size());
    if (scales) std::memcpy(scales, h->h_scales.data(), h->h_scales.size() * 4);
    if (biases) std::memcpy(biases, h->h_biases.data(), h->h_biases.size() * 4);
    return ESP_OK;
}

int esp_int4_classifier_matvec_argmax(ESPInt4Classifier *h, const float *input, float *logits_or_null, int *index) {
    if (!h || !input) return fail(ESP_ERR_INVALID_ARGUMENT, "int4_classifier: null pointer");
    Context &c = context();
    hipError_t e = hipMemcpyAsync(h->input, input, (size_t)h->cols * 4, hipMemcpyHostToDevice, c.stream);
    if (e == hipSuccess) e = launch_int4_matvec(h->packed, h->scales, h->biases, h->input, h->rows, h->cols, h->logits, c.stream);
    if (e == hipSuccess && index) e = launch_argmax(h->logits, 1, h->rows, h->token, nullptr, h->scratch, c.stream);
    if (e == hipSuccess && logits_or_null) e = hipMemcpyAsync(logits_or_null, h->logits, (size_t)h->rows * 4, hipMemcpyDeviceToHost, c.stream);
    if (e == hipSuccess && index) e = hipMemcpyAsync(index, h->token, sizeof(int), hipMemcpyDeviceToHost, c.stream);
    if (e == hipSuccess) e = hipStreamSynchronize(c.stream);
    return e == hipSuccess ? ESP_OK : fail_hip(e, "int4_classifier");
}

int esp_gemv_stamps(const ESPMatrix *matrix, int batch, int launches, uint64_t *out_stamps, int capacity_wavefronts, int *out_wavefronts,
                    double *out_period_us) {
    if (!matrix || batch < 1 || batch > 2 || launches < 1 || !out_stamps || capacity_wavefronts < 1 || !out_wavefronts)
        return fail(ESP_ERR_INVALID_ARGUMENT, "gemv_stamps: bad argument");
    int rc = ensure_init();
    if (rc != ESP_OK) return rc;
    Context &c = context();
    const DeviceMatrix &m = matrix->m;
    if (m.format != FMT_Q4_K) return fail(ESP_ERR_UNSUPPORTED, "gemv_stamps: the stamped kernels are the persistent Q4_K ones");
    uint16_t *d_x = nullptr;
    float *d_y = nullptr;
    unsigned long long *d_s = nullptr;
    const size_t words = (size_t)capacity_wavefronts * 4;
    // enough copies that a walk through them passes more bytes than the last-level caches hold (8 x 4 MB of L2, 256 MB memory-side)
    const size_t bytes = (size_t)m.rows * m.qs_row_bytes;
    const int rotate = (int)std::min<size_t>(64, ((size_t)640 << 20) / bytes + 2);
    RotatingCopies copies;
    std::vector<unsigned long long> next(words);
    rc = copies.make(m, rotate, c.stream);
    if (rc == ESP_OK) rc = device_alloc(&d_x, (size_t)batch * m.cols);
    if (rc == ESP_OK) rc = device_alloc(&d_y, (size_t)batch * m.rows);
    if (rc == ESP_OK) rc = device_alloc(&d_s, 2 * words);
    hipError_t e = hipSuccess;
    if (rc == ESP_OK) {
        e = hipMemsetAsync(d_x, 0x3c, (size_t)batch * m.cols * 2, c.stream);
        if (e == hipSuccess) e = hipMemsetAsync(d_s, 0, 2 * words * 8, c.stream);
        GemvParams p;
        p.x = d_x; p.y = d_y; p.batch = batch; p.epilogue = EPI_STORE_F32;
        const int warm = std::max(launches - 1, rotate);   // at least one walk through the copies
        for (int i = 0; i < warm && e == hipSuccess; i++) { p.w = copies[i]; e = launch_gemv(p, c.stream); }
        // two stamped launches in a row, then two plain ones so that the stamped pair sits inside the train
        for (int k = 0; k < 4 && e == hipSuccess; k++) {
            p.w = copies[warm + k];
            p.stamps = k < 2 ? d_s + (size_t)k * words : nullptr;
            p.stamp_capacity = capacity_wavefronts;   // wavefronts beyond it leave no stamp
            e = launch_gemv(p, c.stream);
        }
        if (e == hipSuccess) e = hipMemcpyAsync(out_stamps, d_s, words * 8, hipMemcpyDeviceToHost, c.stream);
        if (e == hipSuccess) e = hipMemcpyAsync(next.data(), d_s + words, words * 8, hipMemcpyDeviceToHost, c.stream);
        if (e == hipSuccess) e = hipStreamSynchronize(c.stream);
    }
    int n = 0;
    if (rc == ESP_OK && e == hipSuccess) {
        unsigned long long first = ~0ull, first_next = ~0ull;
        for (n = 0; n < capacity_wavefronts && out_stamps[(size_t)n * 4] != 0; n++) {
            first = std::min<unsigned long long>(first, out_stamps[(size_t)n * 4]);
            if (next[(size_t)n * 4] != 0) first_next = std::min(first_next, next[(size_t)n * 4]);
        }
        if (out_period_us) *out_period_us = n > 0 && first_next != ~0ull ? (double)(first_next - first) / 100.0 : 0.0;
    }
    *out_wavefronts = n;
    (void)hipFree(d_x); (void)hipFree(d_y); (void)hipFree(d_s);
    if (rc != ESP_OK) return rc;
    return e == hipSuccess ? ESP_OK : fail_hip(e, "gemv_stamps");
}

int esp_set_tuning(const char *key, int value) {
    return gemv_set_tuning(key, value) ? ESP_OK : fail(ESP_ERR_INVALID_ARGUMENT, "set_tuning: unknown key %s", key ? key : "(null)");
}

int esp_hbm_read_probe(size_t bytes, int iters, double *gb_per_s) {
    if (bytes < (1u << 20) || bytes % 16 != 0 || iters <= 0 || !gb_per_s) return fail(ESP_ERR_INVALID_ARGUMENT, "hbm_read_probe: bad argument");
    int rc = ensure_init();
    if (rc != ESP_OK) return rc;
    Context &c = context();
    uint8_t *buf = nullptr;
    unsigned *sink = nullptr;
    if ((rc = device_alloc(&buf, bytes)) != ESP_OK) return rc;
    if ((rc = device_alloc(&sink, (size_t)4)) != ESP_OK) { (void)hipFree(buf); return rc; }
    hipEvent_t t0 = nullptr, t1 = nullptr;
    hipError_t e = hipMemsetAsync(buf, 1, bytes, c.stream);
    if (e == hipSuccess) e = hipEventCreate(&t0);
    if (e == hipSuccess) e = hipEventCreate(&t1);
    for (int i = 0; i < 3 && e == hipSuccess; i++) e = launch_stream_read(buf, bytes, sink, c.stream);
    if (e == hipSuccess) e = hipEventRecord(t0, c.stream);
    for (int i = 0; i < iters && e == hipSuccess; i++) e = launch_stream_read(buf, bytes, sink, c.stream);
    if (e == hipSuccess) e = hipEventRecord(t1, c.stream);
    if (e == hipSuccess) e = hipEventSynchronize(t1);
    float ms = 0.0f;
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, t0, t1);
    if (e == hipSuccess && ms > 0.0f) *gb_per_s = (double)bytes * iters / (ms * 1e-3) / 1e9;
    if (t0) (void)hipEventDestroy(t0);
    if (t1) (void)hipEventDestroy(t1);
    (void)hipFree(buf); (void)hipFree(sink);
    return e == hipSuccess ? ESP_OK : fail_hip(e, "hbm_read_probe");
}

int esp_hbm_read_probe_pairs(size_t bytes_per_launch, int pair_bytes, int workgroups, int wavefronts, int copies, int launches, double *mean_us, double *gb_per_s) {
    if (bytes_per_launch < 4096 || pair_bytes <= 0 || pair_bytes % 16 != 0 || bytes_per_launch % (size_t)pair_bytes != 0 || workgroups <= 0 ||
        (wavefronts != 4 && wavefronts != 8) ||
        copies < 1 || launches < 1 || !mean_us || !gb_per_s)
        return fail(ESP_ERR_INVALID_ARGUMENT, "hbm_read_probe_pairs: bad argument");
    int rc = ensure_init();
    if (rc != ESP_OK) return rc;
    Context &c = context();
    uint8_t *buf = nullptr;
    unsigned *sink = nullptr;
    if ((rc = device_alloc(&buf, bytes_per_launch * copies)) != ESP_OK) return rc;
    if ((rc = device_alloc(&sink, (size_t)4)) != ESP_OK) { (void)hipFree(buf); return rc; }
    hipEvent_t t0 = nullptr, t1 = nullptr;
    hipError_t e = hipMemsetAsync(buf, 1, bytes_per_launch * copies, c.stream);
    if (e == hipSuccess) e = hipEventCreate(&t0);
    if (e == hipSuccess) e = hipEventCreate(&t1);
    auto launch = [&](int i) { return launch_stream_read_pairs(buf + (size_t)(i % copies) * bytes_per_launch, bytes_per_launch, pair_bytes, workgroups, wavefronts, sink, c.stream); };
    for (int i = 0; i < copies && e == hipSuccess; i++) e = launch(i);
    if (e == hipSuccess) e = hipEventRecord(t0, c.stream);
    for (int i = 0; i < launches && e == hipSuccess; i++) e = launch(i);
    if (e == hipSuccess) e = hipEventRecord(t1, c.stream);
    if (e == hipSuccess) e = hipEventSynchronize(t1);
    float ms = 0.0f;
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, t0, t1);
    if (e == hipSuccess && ms > 0.0f) {
        *mean_us = (double)ms * 1e3 / launches;
        *gb_per_s = (double)bytes_per_launch * launches / (ms * 1e-3) / 1e9;
    }
    if (t0) (void)hipEventDestroy(t0);
    if (t1) (void)hipEventDestroy(t1);
    (void)hipFree(buf); (void)hipFree(sink);
    return e == hipSuccess ? ESP_OK : fail_hip(e, "hbm_read_probe_pairs");
}

}  // extern "C"
